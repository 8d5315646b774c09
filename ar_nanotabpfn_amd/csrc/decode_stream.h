// Decode-step buffer pass on the matrix pipe, as a light background stream (gfx950, head_dim 32).
//
// The context pass of a decode step is bound by the vector and matrix units and leaves HBM idle;
// the buffer pass streams B*H*n_buf*128 bytes and needs almost no arithmetic.  To run the two side
// by side the buffer pass has to fit in what the resident context-pass wavefronts leave on a SIMD
// (four of them at 96 registers leave 128: one wavefront) and must not compete for vector-ALU
// issue slots.  Hence:
//
//  * dot products on the matrix pipe with v_mfma_f32_4x4x4 (16 independent 4x4x4 products per
//    instruction): one block = four keys of one (trajectory, head) pair, lane 4p+i of a
//    wavefront is (block p, index i); described here for the chunk shape in which a block is a
//    pair (the other shape, four blocks per pair, is described at decode_stream_body).  Scores S^T[key i][query j] = K[key i] . Q[query j]: A operand = 4
//    head-dim elements of key row i (lane (p,i)), B operand = the same 4 elements of query j
//    (lane (p,j); zero for j >= Lq), result: lane (p,j) holds the 4 keys' scores of query j.
//    O^T[dim][query j] += V^T[dim][key] P^T[key][query j]: B operand = the lane's own four
//    probabilities, A operand = V[key 0..3][dim] fetched with the transposing LDS read
//    ds_read_b64_tr_b16; lane (p,j) accumulates all 32 output dims of query j.
//    Softmax state (max, sum) is one scalar per lane.  About 35 vector instructions, 16 MFMAs
//    (8 cycles each) and 16 LDS reads per 4 keys x 16 pairs.
//  * loads land in LDS, not in registers: every wavefront keeps a ring of three 8 KiB chunks (64
//    key rows, K and V: 4 keys x 16 pairs or 16 keys x 4 pairs) filled by direct global->LDS loads
//    (16 bytes per lane, lane l lands at chunk + 16 l): the chunk being read and the two behind
//    it, a slot being refilled as soon as its chunk has been read back lane-locally (K) or
//    transposed (V).  The wavefront is alone with its latencies, so the LDS
//    reads run one chunk ahead of the arithmetic that uses them.
//
// Output per (pair, query): normalised partial result in the input type + float32 LSE, i.e. one
// more "context slice" for the combine step; the new row is appended to the cache on the way.
#pragma once

#include <type_traits>

#include "common.h"
#include "decode_buffer.h"

namespace artab {

constexpr int kStreamChunks = 3;           // ring depth per wavefront
constexpr int kStreamShortRows = 32;       // buffers longer than this are read 16 rows x 4 pairs at a time
constexpr int kStreamChunkBytes = 8192;    // 64 key rows x (64 B of K + 64 B of V)
constexpr int kStreamQBytes = 4096;        // a region of query slots: 4 x (64 lanes x 16 B)
constexpr size_t kStreamLdsBytes = kStreamChunks * kStreamChunkBytes + 2 * kStreamQBytes;

// LDS reads of the ring go through inline assembly: the compiler must not see an LDS read that
// could alias the asynchronous fills, or it would drain every load before each read.
// A read is issued by one statement and waited for by another, with arithmetic in between: the
// wait names the registers as in/out operands, so every use of them is ordered behind it.
// Four 16-byte pieces of this lane's row (a K row of a chunk, a query row): pieces 1 KiB apart.
__device__ __forceinline__ void lds_issue_k(u32x4 (&k)[4], unsigned addr) {
    asm volatile(
        "ds_read_b128 %0, %4\n\t"
        "ds_read_b128 %1, %4 offset:1024\n\t"
        "ds_read_b128 %2, %4 offset:2048\n\t"
        "ds_read_b128 %3, %4 offset:3072"
        : "=&v"(k[0]), "=&v"(k[1]), "=&v"(k[2]), "=&v"(k[3])
        : "v"(addr)
        : "memory");
}
__device__ __forceinline__ void lds_read4x128(u32x4 (&k)[4], unsigned addr) {
    asm volatile(
        "ds_read_b128 %0, %4\n\t"
        "ds_read_b128 %1, %4 offset:1024\n\t"
        "ds_read_b128 %2, %4 offset:2048\n\t"
        "ds_read_b128 %3, %4 offset:3072\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(k[0]), "=&v"(k[1]), "=&v"(k[2]), "=&v"(k[3])
        : "v"(addr)
        : "memory");
}
__device__ __forceinline__ void lds_write128(unsigned addr, u32x4 v) {
    asm volatile("ds_write_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : : "v"(addr), "v"(v) : "memory");
}
// Eight transposing reads: the V operands of the eight 4-dim groups of one 4-key chunk.
// Address layout of a V chunk: sub-slot t (1 KiB) holds dims 8t..8t+7, so group u = 2t + half
// sits at t * 1024 + 8 * half.
__device__ __forceinline__ void lds_issue_v(u32x2 (&v)[8], unsigned addr) {
    asm volatile(
        "ds_read_b64_tr_b16 %0, %8\n\t"
        "ds_read_b64_tr_b16 %1, %8 offset:8\n\t"
        "ds_read_b64_tr_b16 %2, %8 offset:1024\n\t"
        "ds_read_b64_tr_b16 %3, %8 offset:1032\n\t"
        "ds_read_b64_tr_b16 %4, %8 offset:2048\n\t"
        "ds_read_b64_tr_b16 %5, %8 offset:2056\n\t"
        "ds_read_b64_tr_b16 %6, %8 offset:3072\n\t"
        "ds_read_b64_tr_b16 %7, %8 offset:3080"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
        : "v"(addr)
        : "memory");
}
__device__ __forceinline__ void lds_wait(u32x4 (&k)[4], u32x2 (&v)[8]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(k[0]), "+v"(k[1]), "+v"(k[2]), "+v"(k[3]), "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]),
                   "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])
                 :
                 : "memory");
}

// The value held by another lane of this lane's row of 16: the row rotated by N places.
template <int N>
__device__ __forceinline__ float row_ror(float v) {
    const int x = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(x, x, 0x120 + N, 0xf, 0xf, false));
}

template <typename T>
struct Mfma4;
template <>
struct Mfma4<bf16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x2 a, u32x2 b, f32x4 c) {
        typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
        return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(v4bf, a), __builtin_bit_cast(v4bf, b), c, 0,
                                                      0, 0);
    }
};
template <>
struct Mfma4<f16_t> {
    static __device__ __forceinline__ f32x4 mma(u32x2 a, u32x2 b, f32x4 c) {
        typedef _Float16 v4h __attribute__((ext_vector_type(4)));
        return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(v4h, a), __builtin_bit_cast(v4h, b), c, 0, 0, 0);
    }
};

// One wavefront per workgroup, KEYS rows of 64 / KEYS consecutive (trajectory, head) pairs per
// chunk; a task = those pairs over the whole buffer; tasks are dealt round-robin over the grid.
//
// KEYS = 4: 16 pairs per task, lane 4p + i loads row 4g + i of pair p.  Every lane group of four
//   is one pair: softmax state and output of (pair, query) live in one lane for the whole task.
//   A request touches 256 contiguous bytes per pair.
// KEYS = 16: 4 pairs per task, lane 16p + r loads row 16g + r of pair p: 1 KiB contiguous per pair
//   and request, which the memory system serves faster once the buffers outgrow the last-level
//   cache and, above all, with less delay for the loads of a kernel running next door.  The four
//   lane groups of a pair hold the keys 4k..4k+3 (k = 0..3) of a chunk and keep separate softmax
//   states; they are merged (rotations within the row of 16 lanes) when the task ends.  More
//   work per task: worth it only for buffers of some length.
// The LDS side is the same for both: lane l's row at chunk + 1024 t + 16 l, a 4x4x4 block = four
// consecutive lanes.  Only what a lane's row *is* differs.
template <typename T, int LQ, int KEYS>
__device__ __forceinline__ void decode_stream_body(const DecodeParams &P, unsigned char *stream_lds, int n_buf,
                                                   bool slot_fits) {
    constexpr int DH = 32;
    constexpr int S = kStreamChunks;
    constexpr int PP = 64 / KEYS;             // pairs per task
    constexpr int NKG = KEYS / 4;             // lane groups (of four keys each) per pair
    constexpr int QREG = KEYS == 16 ? 1 : 2;  // 4 KiB query regions in use
    constexpr int QS = QREG * NKG;            // query slots: lane group k of a region holds one task's queries
    static_assert(KEYS == 4 || KEYS == 16, "chunk shapes: 16 pairs x 4 rows or 4 pairs x 16 rows");
    static_assert(QS == 2 || QS == 4, "slot index is taken modulo a power of two");

    // Every argument the loop needs, as plain values: the inline assembly clobbers memory, and
    // anything still read through the argument block would be re-read after every such statement.
    const View vq = P.q, vkb = P.kb, vvb = P.vb, vkn = P.knew, vvn = P.vnew;
    const int H = P.H, has_new = P.has_new;
    const float qscale = P.qscale;
    T *const part_o = static_cast<T *>(P.buf_part_o);
    float *const part_lse = P.buf_part_lse;
    const int n_pairs = P.B * H;
    const int n_total = n_buf + (has_new ? 1 : 0);

    const int lane = threadIdx.x;
    const int n_tasks = (n_pairs + PP - 1) / PP;
    const int n_groups = (n_total + KEYS - 1) / KEYS;  // chunks per task

    const unsigned lds0 = static_cast<unsigned>(reinterpret_cast<uintptr_t>(stream_lds));
    const unsigned q_lds0 = lds0 + S * kStreamChunkBytes;
    // transposing read: within a 16-lane group lane L supplies LDS row 4 (L % 4) + L / 4 of the group
    const unsigned tr_off = 16u * (4u * (4u * (lane >> 4) + (lane & 3)) + ((lane & 15) >> 2));

    if (n_total == 0) {  // nothing to attend to: empty partials (weight 0 in the combine)
        for (int task = blockIdx.x; task < n_tasks; task += gridDim.x) {
            const int pair = PP * task + lane / KEYS;
            if (pair < n_pairs && lane % KEYS < LQ) {
                const int sub = lane % KEYS;
                part_lse[static_cast<long>(pair) * LQ + sub] = -INFINITY;
                u32x4 z = {0u, 0u, 0u, 0u};
                T *po = part_o + (static_cast<long>(pair) * LQ + sub) * DH;
#pragma unroll
                for (int e = 0; e < 4; ++e) *reinterpret_cast<u32x4 *>(po + 8 * e) = z;
            }
        }
        return;
    }

    // ---- producer: chunk `issue_g` of task `issue_task` into ring slot issue_slot.  Row pointers
    // are kept per task and advanced by KEYS rows per chunk; only a task's last chunk (clamped
    // rows, the new row) computes addresses the long way.
    const int my_tasks = blockIdx.x < n_tasks ? (n_tasks - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const int total_chunks = my_tasks * n_groups;
    const long chunk_step = KEYS * vkb.sn, chunk_step_v = KEYS * vvb.sn;  // elements from chunk g to g + 1
    int issued = 0, issue_task = blockIdx.x, issue_g = 0, issue_slot = 0;
    int issue_seq = 0, seq = 0;  // how many of this wavefront's tasks the producer / consumer have finished
    const T *p_k = nullptr, *p_v = nullptr;  // this lane's row of the chunk to be requested next
    auto issue_one = [&]() {
        const bool first = issue_g == 0, last = issue_g + 1 == n_groups;  // wavefront-uniform
        int p_b = 0, p_h = 0, kq = 0;
        if (first || last) {  // the (trajectory, head) of this lane's pair: twice per task at most
            const int ln = opaque(lane);
            kq = ln % KEYS;
            int pair = PP * issue_task + ln / KEYS;
            pair = pair < n_pairs ? pair : n_pairs - 1;  // a ragged last task re-reads the last pair; never stored
            p_b = pair / H;
            p_h = pair % H;
        }
        if (first) {
            p_k = view_row<T>(vkb, p_b, p_h, kq);
            p_v = view_row<T>(vvb, p_b, p_h, kq);
            // the task's queries, fetched by the lanes of one lane group per pair (which group:
            // the slot); the pieces of lanes that stand for no query stay zero (cleared once, below)
            const int qslot = issue_seq & (QS - 1);
            unsigned char *qd = stream_lds + S * kStreamChunkBytes + (qslot / NKG) * kStreamQBytes;
            const int j = kq - 4 * (qslot % NKG);
            if (j >= 0 && j < LQ) load_row64_to_lds(view_row<T>(vq, p_b, p_h, j), qd);
        }
        const T *kr = p_k, *vr = p_v;
        if (last) {
            int row = KEYS * issue_g + kq;
            row = row < n_total ? row : n_total - 1;  // keys past the end re-read the last one and are masked
            const bool is_new = has_new && row == n_buf;
            kr = is_new ? view_row<T>(vkn, p_b, p_h, 0) : view_row<T>(vkb, p_b, p_h, row);
            vr = is_new ? view_row<T>(vvn, p_b, p_h, 0) : view_row<T>(vvb, p_b, p_h, row);
        }
        unsigned char *cd = stream_lds + issue_slot * kStreamChunkBytes;
        load_row64_to_lds(kr, cd);
        load_row64_to_lds(vr, cd + 4096);
        p_k += chunk_step;
        p_v += chunk_step_v;
        ++issued;
        issue_slot = issue_slot + 1 == S ? 0 : issue_slot + 1;
        if (++issue_g == n_groups) {
            issue_g = 0;
            issue_task += gridDim.x;
            ++issue_seq;
        }
    };
    // Lanes that stand for no query (index within the lane group >= LQ) contribute zeros to the
    // score product: their pieces of every query region are cleared once and never written again.
    if ((lane & 3) >= LQ) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int t = 0; t < 4 * QREG; ++t) lds_write128(q_lds0 + 1024u * t + lane * 16u, zero);
    }
    // QS query slots: the producer may be at most QS - 1 tasks ahead of the consumer
    auto may_issue = [&]() { return issued < total_chunks && issue_seq <= seq + (QS - 1); };
    const int depth = S;
    for (int i = 0; i < depth; ++i)
        if (may_issue()) issue_one();

    // ---- consumer.  The LDS reads of a chunk are split in time so that no read is waited for right
    // after it is issued (the wavefront has nobody to hide a round trip behind but itself): the K
    // rows of chunk c + 1 and the V rows of chunk c are requested early in step c and arrive while
    // the softmax of chunk c (whose K rows came in during step c - 1) is computed; the queries sit
    // in registers for the whole task.
    float m = -INFINITY, mq = 0.f, l = 0.f;  // running maximum of the raw scores, and times qscale
    f32x4 o[8];  // output dims 4u..4u+3 of this lane's query
#pragma unroll
    for (int u = 0; u < 8; ++u) o[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    int task = blockIdx.x, g = 0, slot = 0;
    const int new_group = has_new && slot_fits ? n_buf / KEYS : -1;  // the chunk that holds the row to append
    u32x4 qr[4];  // this lane's query row (zero for lanes that stand for no query)
    u32x4 kr[4];  // the K rows of the chunk whose scores come next

    // chunk `c` must have landed; only the chunks requested after it (8 loads each: 4 for the K
    // rows, then 4 for the V rows) may be pending.  (A task's query loads sit in front of its
    // first chunk's: where they are in flight the wait is stricter than needed, never too lax.)
    auto wait_chunk = [&](int c) {
        switch (issued - c - 1) {
            case 3: __builtin_amdgcn_s_waitcnt(vmcnt_imm(24)); break;
            case 2: __builtin_amdgcn_s_waitcnt(vmcnt_imm(16)); break;
            case 1: __builtin_amdgcn_s_waitcnt(vmcnt_imm(8)); break;
            default: __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); break;
        }
    };
    // the same for the K rows of chunk `c` alone: its V rows may be pending as well
    auto wait_chunk_k = [&](int c) {
        switch (issued - c - 1) {
            case 3: __builtin_amdgcn_s_waitcnt(vmcnt_imm(28)); break;
            case 2: __builtin_amdgcn_s_waitcnt(vmcnt_imm(20)); break;
            case 1: __builtin_amdgcn_s_waitcnt(vmcnt_imm(12)); break;
            default: __builtin_amdgcn_s_waitcnt(vmcnt_imm(4)); break;
        }
    };
    // ---- the arithmetic of one chunk, shared by the two kinds of step below
    auto scores = [&]() {
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            s = Mfma4<T>::mma(u32x2{kr[e][0], kr[e][1]}, u32x2{qr[e][0], qr[e][1]}, s);
            s = Mfma4<T>::mma(u32x2{kr[e][2], kr[e][3]}, u32x2{qr[e][2], qr[e][3]}, s);
        }
        return s;
    };
    // online softmax of four raw dot products (qscale > 0 enters with the exponent); the rescale is
    // skipped (wavefront-uniformly) while no maximum moves.  Returns the packed probabilities.
    // A lane group that has seen no valid key yet (KEYS = 16, short buffers) keeps m = -inf and
    // mq = 0: its probabilities are exp2(-inf) = 0.
    auto softmax = [&](const float (&sc)[4]) {
        const float m_new = max3(max3(m, sc[0], sc[1]), sc[2], sc[3]);
        if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {
            const float alpha = m == -INFINITY ? 0.f : fast_exp2((m - m_new) * qscale);
            l *= alpha;
#pragma unroll
            for (int u = 0; u < 8; ++u) o[u] *= alpha;
            m = m_new;
            mq = KEYS > 4 && m_new == -INFINITY ? 0.f : m_new * qscale;
        }
        float p[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) p[r] = fast_exp2(fmaf(sc[r], qscale, -mq));
        l += (p[0] + p[1]) + (p[2] + p[3]);
        return u32x2{pack2<T>(p[0], p[1]), pack2<T>(p[2], p[3])};
    };

    // ---- a step in the middle of a task, for consumer and producer alike (no query fetch, no
    // ragged or new row, nothing to store, ring full): nothing is decided at run time, the waits
    // are constants.  D chunks are live at its start: c .. c + D - 1.
    auto steady_step = [&](auto depth_tag) {
        constexpr int D = decltype(depth_tag)::value;
        const unsigned chunk = lds0 + static_cast<unsigned>(slot) * kStreamChunkBytes;
        u32x2 vop[8];
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(8 * (D - 1)));  // chunk c has landed
        lds_issue_v(vop, chunk + 4096u + tr_off);
        const f32x4 s = scores();
        slot = slot + 1 == S ? 0 : slot + 1;
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(8 * (D - 2) + 4));  // and the K rows of chunk c + 1
        lds_issue_k(kr, lds0 + static_cast<unsigned>(slot) * kStreamChunkBytes + lane * 16u);
        const float sc[4] = {s[0], s[1], s[2], s[3]};
        const u32x2 pop = softmax(sc);
        lds_wait(kr, vop);
#pragma unroll
        for (int u = 0; u < 8; ++u) o[u] = Mfma4<T>::mma(vop[u], pop, o[u]);
        unsigned char *cd = stream_lds + issue_slot * kStreamChunkBytes;
        load_row64_to_lds(p_k, cd);
        load_row64_to_lds(p_v, cd + 4096);
        p_k += chunk_step;
        p_v += chunk_step_v;
        issue_slot = issue_slot + 1 == S ? 0 : issue_slot + 1;
    };

    if (total_chunks == 0) return;
    wait_chunk_k(0);
    lds_read4x128(kr, lds0 + lane * 16u);
    int c = 0;
    while (c < total_chunks) {
        // how many steady steps lie ahead: consumer and producer both strictly inside a task
        if (g >= 1 && issue_g >= 1 && issued - c == depth && issue_seq <= seq + (QS - 1)) {
            int run = n_groups - 1 - (g > issue_g ? g : issue_g);
            if (new_group >= g && new_group - g < run) run = new_group - g;
            if (run > 0) {
                for (int r = 0; r < run; ++r) steady_step(std::integral_constant<int, S>{});
                c += run;
                g += run;
                issue_g += run;
                issued += run;
                continue;
            }
        }
        const unsigned chunk = lds0 + static_cast<unsigned>(slot) * kStreamChunkBytes;
        const bool more = c + 1 < total_chunks;
        if (g == 0) {
            // the task's queries: those of the lane's pair and query index, from the lane group
            // that fetched them for this slot
            const int ln = opaque(lane), qslot = seq & (QS - 1);
            const int src = ln - 4 * ((ln % KEYS) >> 2) + 4 * (qslot % NKG);
            lds_read4x128(qr, q_lds0 + static_cast<unsigned>(qslot / NKG) * kStreamQBytes + src * 16u);
        }
        u32x2 vop[8];
        wait_chunk(c);
        lds_issue_v(vop, chunk + 4096u + tr_off);
        const f32x4 s = scores();
        // the products have taken their operands: the same registers receive the next chunk's rows
        if (more) {
            wait_chunk_k(c + 1);
            const int nslot = slot + 1 == S ? 0 : slot + 1;
            lds_issue_k(kr, lds0 + static_cast<unsigned>(nslot) * kStreamChunkBytes + lane * 16u);
        }
        float sc[4] = {s[0], s[1], s[2], s[3]};
        if (g + 1 == n_groups) {  // only a task's last chunk can hold keys past the end
            const int key0 = KEYS * g + ((opaque(lane) % KEYS) & ~3);  // first key of this lane group
#pragma unroll
            for (int r = 0; r < 4; ++r) sc[r] = key0 + r < n_total ? sc[r] : -INFINITY;
        }
        const u32x2 pop = softmax(sc);
        lds_wait(kr, vop);
#pragma unroll
        for (int u = 0; u < 8; ++u) o[u] = Mfma4<T>::mma(vop[u], pop, o[u]);

        if (g == new_group) {
            // in-place append (once per task): the lane that holds the new row copies it from the
            // chunk, lane-locally, into slot n_buf of the cache
            const int ln = opaque(lane);
            const int pair = PP * task + ln / KEYS;
            if (KEYS * g + ln % KEYS == n_buf && pair < n_pairs) {
                const int b = pair / H, h = pair % H;
                T *kd = view_row<T>(vkb, b, h, n_buf), *vd = view_row<T>(vvb, b, h, n_buf);
                u32x4 kk[4], vv[4];
                lds_read4x128(kk, chunk + lane * 16u);
                lds_read4x128(vv, chunk + 4096u + lane * 16u);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    *reinterpret_cast<u32x4 *>(kd + 8 * e) = kk[e];
                    *reinterpret_cast<u32x4 *>(vd + 8 * e) = vv[e];
                }
            }
        }
        // the chunk has been read: refill its slot (and any the producer had to leave empty)
        if (g + 1 == n_groups) ++seq;
        while (may_issue() && issued - c - 1 < depth) issue_one();

        slot = slot + 1 == S ? 0 : slot + 1;
        if (++g == n_groups) {
            // ---- task done
            if (NKG > 1) {
                // merge the lane groups of a pair: lanes l, l+4, l+8, l+12 of a row of 16 hold
                // states of the same (pair, query) over disjoint keys; afterwards each holds the sum
                float mt = fmaxf(m, row_ror<4>(m));
                mt = fmaxf(mt, row_ror<8>(mt));
                const float f = m == -INFINITY ? 0.f : fast_exp2((m - mt) * qscale);
                l *= f;
                l += row_ror<4>(l);
                l += row_ror<8>(l);
#pragma unroll
                for (int u = 0; u < 8; ++u)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float x = o[u][e] * f;
                        x += row_ror<4>(x);
                        x += row_ror<8>(x);
                        o[u][e] = x;
                    }
                mq = mt == -INFINITY ? 0.f : mt * qscale;
            }
            // write the partial of this lane's (pair, query): the first lane group of each pair,
            // lanes of real queries of real pairs
            const int ln = opaque(lane);
            const int pair = PP * task + ln / KEYS, sub = ln % KEYS;
            if (pair < n_pairs && sub < LQ) {
                const float inv = l > 0.f ? 1.f / l : 0.f;
                T *po = part_o + (static_cast<long>(pair) * LQ + sub) * DH;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    u32x4 val = {pack2<T>(o[2 * e][0] * inv, o[2 * e][1] * inv), pack2<T>(o[2 * e][2] * inv, o[2 * e][3] * inv),
                                 pack2<T>(o[2 * e + 1][0] * inv, o[2 * e + 1][1] * inv),
                                 pack2<T>(o[2 * e + 1][2] * inv, o[2 * e + 1][3] * inv)};
                    *reinterpret_cast<u32x4 *>(po + 8 * e) = val;
                }
                part_lse[static_cast<long>(pair) * LQ + sub] = l > 0.f ? (mq + fast_log2(l)) * kLn2 : -INFINITY;
            }
            m = -INFINITY;
            mq = 0.f;
            l = 0.f;
#pragma unroll
            for (int u = 0; u < 8; ++u) o[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            g = 0;
            task += gridDim.x;
        }
        ++c;
    }
}

// Buffers of at most `P.stream_short_rows` rows (committed + new) take the 16-pair chunks, longer
// ones the 4-pair chunks: one kernel, so that a recorded launch serves every length.  KEYS != 0
// pins the shape.  Dynamic LDS: kStreamLdsBytes.
template <typename T, int LQ, int PRIO = 3, int KEYS = 0>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4))) void decode_stream_kernel(DecodeParams P) {
    warm_kernel_arguments<sizeof(DecodeParams)>();
    extern __shared__ __attribute__((aligned(16))) unsigned char stream_lds[];
    bool slot_fits;
    const int n_buf = committed_rows(P, slot_fits);
    // This wavefront shares its SIMD with older, compute-bound ones; without a raised priority it
    // is only issued in their gaps.  It issues little: the priority costs them little — but not
    // nothing, so a buffer short enough to be done long before its neighbours stays at the base priority.
    if (n_buf + (P.has_new ? 1 : 0) > P.stream_calm_rows) __builtin_amdgcn_s_setprio(PRIO);
    if (KEYS == 4 || (KEYS == 0 && n_buf + (P.has_new ? 1 : 0) <= P.stream_short_rows))
        decode_stream_body<T, LQ, 4>(P, stream_lds, n_buf, slot_fits);
    else
        decode_stream_body<T, LQ, 16>(P, stream_lds, n_buf, slot_fits);
}

}  // namespace artab
