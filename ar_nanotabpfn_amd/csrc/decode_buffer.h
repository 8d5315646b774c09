// Decode-step buffer pass + log-sum-exp merge + in-place cache append (gfx950).
//
// One wavefront per (trajectory, head).  The buffer K/V rows of that pair are
// streamed once with 16-byte loads (HBM-bound: 2 flop per byte), each group of
// DH/8 lanes owning one key row at a time and keeping a private online-softmax
// state per query.  The lane-group states are then brought to a common maximum
// and summed through LDS together with the partial results of the split context
// pass, each weighted by its log-sum-exp (a wavefront-wide LSE merge in float32,
// one output element per lane).  The new buffer row is read from the
// projection and written to its cache slot by the same wavefront: no torch.cat,
// no second pass.
#pragma once

#include "common.h"

namespace artab {

struct DecodeParams {
    View q, kb, vb, knew, vnew, out;
    const void *part_o;     // [n_split][B*H*Lq][DH] normalised context partials, input type
    const float *part_lse;  // [n_split][B*H*Lq] natural-log LSE of each partial
    float *lse;             // optional final LSE [B,H,Lq]
    void *buf_part_o;       // streaming variant only: the buffer pass's own partial, [B*H*Lq][DH] input type,
    float *buf_part_lse;    // and its natural-log LSE [B*H*Lq]
    int B, H;
    int n_split;
    int n_buf;    // committed buffer rows
    const int *n_buf_dev;  // when set, the committed length is read from here at run time
    int stream_short_rows;  // streaming variant: buffers longer than this are read 16 rows x 4 pairs at a time
    int stream_calm_rows;   // streaming variant: buffers up to this length are streamed at the base wave priority
    int n_base;   // rows of kb/vb that precede the counted ones (a per-trajectory context stored in
                  // front of the buffer rows); 0 for a shared context
    int has_new;  // 1: row n_buf comes from knew/vnew, is attended and appended
    int capacity; // counted rows the cache holds (behind n_base); a length read from n_buf_dev is
                  // clamped to it, and a new row that would land behind it is not appended
    float qscale; // scale * log2(e)
};

// Committed length of a decode call.  A host value has been validated by the caller of the
// kernel; a value read from device memory (a recorded launch replayed more often than the
// cache has slots, a cell that was never reset) is clamped so that every access stays inside
// the cache.  `fits` tells whether slot n of the cache exists for the new row.
__device__ __forceinline__ int committed_rows(const DecodeParams &P, bool &fits) {
    fits = true;
    if (!P.n_buf_dev) return P.n_buf;
    const int raw = *P.n_buf_dev;
    const int hi = P.capacity - (P.has_new ? 1 : 0);
    fits = raw >= 0 && raw <= hi;
    return raw < 0 ? 0 : (raw > hi ? (hi > 0 ? hi : 0) : raw);
}

struct CommittedRows {
    int n;
    bool fits;
};
__device__ __forceinline__ CommittedRows read_committed_rows(const DecodeParams &P) {
    CommittedRows c;
    c.n = committed_rows(P, c.fits);
    return c;
}

constexpr int kDecodeWaves = 4;
constexpr int kDecodeUnroll = 4;
constexpr int kSplitBatch = 8;  // context partials fetched per round of the merge

// Where the buffer pass finds the context pass's partial results of its (trajectory, head) pair:
// in the split workspace in global memory (normalised outputs in the input type, natural-log LSE) ...
template <typename T, int DH, int LQ>
struct WorkspacePartials {
    const T *part_o;
    const float *part_lse;
    long total_rows, row0;  // rows per slot; the pair's first row (pair * LQ)
    int n;
    __device__ __forceinline__ int count() const { return n; }
    __device__ __forceinline__ float lse2(int sp, int i) const { return part_lse[sp * total_rows + row0 + i] * kLog2e; }
    __device__ __forceinline__ float o(int sp, int i, int d) const {
        return to_f32(part_o[(sp * total_rows + row0 + i) * DH + d]);
    }
};
// ... or in LDS, left there by the wavefronts of the same workgroup (float32, base-2 LSE).
template <int DH, int LQ>
struct LdsPartials {
    const float *part_o;     // [n][ld_cols][DH]
    const float *part_lse2;  // [n][ld_cols]
    int ld_cols, col0, n;    // columns per slot; the pair's first column
    __device__ __forceinline__ int count() const { return n; }
    __device__ __forceinline__ float lse2(int sp, int i) const { return part_lse2[sp * ld_cols + col0 + i]; }
    __device__ __forceinline__ float o(int sp, int i, int d) const { return part_o[(sp * ld_cols + col0 + i) * DH + d]; }
};

// What a wavefront asks for before it can start on a pair: its slice of the queries, the committed
// length and the first batch of buffer rows.  Requested by decode_buffer_request() — as early as
// the caller likes: the one-launch kernel does it in front of its context phase — and consumed by
// decode_buffer_pair().
template <typename T, int DH, int LQ>
struct BufferHead {
    u32x4 qraw[LQ];
    u32x4 kraw[kDecodeUnroll], vraw[kDecodeUnroll];
    int n_buf, n_total;
    bool slot_fits;
};

// ALL_LANES: every lane group loads, without a lane mask — one past the last row re-reads the last
// row, which the consumer masks by position.  Loads under a mask, merged with zeros, make the
// compiler wait for them where they are issued, so a batch requested ahead hides nothing: the
// streaming buffer kernel takes the unmasked form (2-7 % faster from 128 rows on).  The one-launch
// kernel keeps the masked one: at a handful of rows the 31 idle lane groups' loads cost more than
// the wait (11.4 against 11.9 us at one row).
template <typename T, int DH, int LQ, bool ALL_LANES = false>
__device__ __forceinline__ void decode_buffer_rows(const DecodeParams &P, long b, int h, int lane, int kv0, int n_buf,
                                                   int n_total, u32x4 (&kraw)[kDecodeUnroll],
                                                   u32x4 (&vraw)[kDecodeUnroll]) {
    constexpr int LPR = DH / 8, RPW = 64 / LPR;
    const int grp = lane / LPR, sub = lane % LPR;
#pragma unroll
    for (int u = 0; u < kDecodeUnroll; ++u) {
        const int kv_raw = kv0 + u * RPW + grp;
        if constexpr (ALL_LANES) {
            const int kv = kv_raw < n_total ? kv_raw : (n_total > 0 ? n_total - 1 : 0);
            const bool is_new = P.has_new && kv == n_buf;
            const T *kr = is_new ? view_row<T>(P.knew, b, h, 0) : view_row<T>(P.kb, b, h, kv);
            const T *vr = is_new ? view_row<T>(P.vnew, b, h, 0) : view_row<T>(P.vb, b, h, kv);
            kraw[u] = *reinterpret_cast<const u32x4 *>(kr + 8 * sub);
            vraw[u] = *reinterpret_cast<const u32x4 *>(vr + 8 * sub);
        } else {
            const int kv = kv_raw;
            kraw[u] = u32x4{0u, 0u, 0u, 0u};
            vraw[u] = u32x4{0u, 0u, 0u, 0u};
            if (kv < n_total) {
                const bool is_new = P.has_new && kv == n_buf;
                const T *kr = is_new ? view_row<T>(P.knew, b, h, 0) : view_row<T>(P.kb, b, h, kv);
                const T *vr = is_new ? view_row<T>(P.vnew, b, h, 0) : view_row<T>(P.vb, b, h, kv);
                kraw[u] = *reinterpret_cast<const u32x4 *>(kr + 8 * sub);
                vraw[u] = *reinterpret_cast<const u32x4 *>(vr + 8 * sub);
            }
        }
    }
}

// (`rows`: the committed length as read_committed_rows() gave it — to a caller that read it
// earlier, so that nothing here waits for it.)
template <typename T, int DH, int LQ, bool ALL_LANES = false>
__device__ __forceinline__ void decode_buffer_request(const DecodeParams &P, long b, int h, int lane,
                                                      BufferHead<T, DH, LQ> &hd, const CommittedRows &rows) {
    const int sub = lane % (DH / 8);
#pragma unroll
    for (int i = 0; i < LQ; ++i) hd.qraw[i] = *reinterpret_cast<const u32x4 *>(view_row<T>(P.q, b, h, i) + 8 * sub);
    hd.n_buf = P.n_base + rows.n;
    hd.slot_fits = rows.fits;
    hd.n_total = hd.n_buf + (P.has_new ? 1 : 0);
    if (ALL_LANES && hd.n_total <= 0) {
        // No row at all (an empty buffer and no new row: the call only merges context partials).
        // The unmasked form would re-read "the last row" of a cache that may have none, or be NULL.
#pragma unroll
        for (int u = 0; u < kDecodeUnroll; ++u) {
            hd.kraw[u] = u32x4{0u, 0u, 0u, 0u};
            hd.vraw[u] = u32x4{0u, 0u, 0u, 0u};
        }
        return;
    }
    decode_buffer_rows<T, DH, LQ, ALL_LANES>(P, b, h, lane, 0, hd.n_buf, hd.n_total, hd.kraw, hd.vraw);
}
template <typename T, int DH, int LQ, bool ALL_LANES = false>
__device__ __forceinline__ void decode_buffer_request(const DecodeParams &P, long b, int h, int lane,
                                                      BufferHead<T, DH, LQ> &hd) {
    decode_buffer_request<T, DH, LQ, ALL_LANES>(P, b, h, lane, hd, read_committed_rows(P));
}

// The buffer pass of one (trajectory, head) pair by one wavefront: streams the committed buffer
// rows, appends the new one, merges with the context partials `parts` and writes the final output.
// `wave` (0 .. NWAVES-1) selects the wavefront's private LDS region.
template <typename T, int DH, int LQ, int NWAVES, typename Parts, bool ALL_LANES = false>
__device__ __forceinline__ void decode_buffer_pair(const DecodeParams &P, long b, int h, int wave, int lane,
                                                   const Parts &parts, const BufferHead<T, DH, LQ> &hd) {
    constexpr int LPR = DH / 8;    // lanes per key row
    constexpr int RPW = 64 / LPR;  // key rows per wavefront load
    const long pair = b * P.H + h;
    const int grp = lane / LPR;  // which row of a load this lane works on
    const int sub = lane % LPR;  // which 8-element slice of the head dimension

    // the lane's query slice, scale * log2(e) folded in and rounded to the input type (the matrix
    // kernels round it at the same point, triton_kernels.py:120-121): packed pairs for v_dot2
    unsigned qp[LQ][4];
#pragma unroll
    for (int i = 0; i < LQ; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            qp[i][e] = pack2<T>(unpack_lo<T>(hd.qraw[i][e]) * P.qscale, unpack_hi<T>(hd.qraw[i][e]) * P.qscale);

    float m[LQ], l[LQ], acc[LQ][8];
#pragma unroll
    for (int i = 0; i < LQ; ++i) {
        m[i] = -INFINITY;
        l[i] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[i][e] = 0.f;
    }

    // maximum over the context partials' LSEs (log2 domain), requested before the key loop so
    // that its latency hides under it
    float M[LQ];
#pragma unroll
    for (int i = 0; i < LQ; ++i) M[i] = -INFINITY;
    const int n_parts = parts.count();
    for (int sp0 = 0; sp0 < n_parts; sp0 += kSplitBatch) {
        float v[kSplitBatch][LQ];  // a batch of loads in flight, then the maxima
#pragma unroll
        for (int u = 0; u < kSplitBatch; ++u) {
            const int sp = sp0 + u < n_parts ? sp0 + u : n_parts - 1;
#pragma unroll
            for (int i = 0; i < LQ; ++i) v[u][i] = parts.lse2(sp, i);
        }
#pragma unroll
        for (int u = 0; u < kSplitBatch; ++u)
#pragma unroll
            for (int i = 0; i < LQ; ++i) M[i] = fmaxf(M[i], v[u][i]);
    }

    const bool slot_fits = hd.slot_fits;
    const int n_buf = hd.n_buf, n_total = hd.n_total;
    const T *knew_row = P.has_new ? view_row<T>(P.knew, b, h, 0) : nullptr;
    const T *vnew_row = P.has_new ? view_row<T>(P.vnew, b, h, 0) : nullptr;

    // the batch after the one being worked on is always on its way
    u32x4 knext[kDecodeUnroll], vnext[kDecodeUnroll];
#pragma unroll
    for (int u = 0; u < kDecodeUnroll; ++u) {
        knext[u] = hd.kraw[u];
        vnext[u] = hd.vraw[u];
    }
    for (int kv0 = 0; kv0 < n_total; kv0 += RPW * kDecodeUnroll) {
        u32x4 kraw[kDecodeUnroll], vraw[kDecodeUnroll];
        bool ok[kDecodeUnroll];
#pragma unroll
        for (int u = 0; u < kDecodeUnroll; ++u) {
            ok[u] = kv0 + u * RPW + grp < n_total;
            kraw[u] = knext[u];
            vraw[u] = vnext[u];
        }
        if (kv0 + RPW * kDecodeUnroll < n_total)
            decode_buffer_rows<T, DH, LQ, ALL_LANES>(P, b, h, lane, kv0 + RPW * kDecodeUnroll, n_buf, n_total, knext, vnext);
        float s[LQ][kDecodeUnroll];
#pragma unroll
        for (int u = 0; u < kDecodeUnroll; ++u) {
            if (kv0 + u * RPW >= n_total) {  // wavefront-uniform: no lane group has a row in this sub-step
#pragma unroll
                for (int i = 0; i < LQ; ++i) s[i][u] = -INFINITY;
                continue;
            }
#pragma unroll
            for (int i = 0; i < LQ; ++i) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) d = dot2_acc<T>(qp[i][e], kraw[u][e], d);
#pragma unroll
                for (int o = 1; o < LPR; o <<= 1) d += __shfl_xor(d, o, 64);
                s[i][u] = ok[u] ? d : -INFINITY;
            }
        }
#pragma unroll
        for (int i = 0; i < LQ; ++i) {
            float cm = s[i][0];
#pragma unroll
            for (int u = 1; u < kDecodeUnroll; ++u) cm = fmaxf(cm, s[i][u]);
            const float m_new = fmaxf(m[i], cm);
            if (m_new == -INFINITY) continue;  // this lane group had no row in the chunk yet
            const float alpha = fast_exp2(m[i] - m_new);
            m[i] = m_new;
            l[i] *= alpha;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[i][e] *= alpha;
        }
#pragma unroll
        for (int u = 0; u < kDecodeUnroll; ++u) {
            if (kv0 + u * RPW >= n_total) continue;
            float vf[8];
            unpack8<T>(vraw[u], vf);
#pragma unroll
            for (int i = 0; i < LQ; ++i) {
                const float p = ok[u] ? fast_exp2(s[i][u] - m[i]) : 0.f;
                l[i] += p;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[i][e] = fmaf(p, vf[e], acc[i][e]);
            }
        }
    }

    // ---- merge of the RPW lane-group states and the context partials, through LDS.
    // (A register butterfly needs 4 dependent rounds of 20 cross-lane moves here; the LDS
    // version is two short phases of independent accesses.)  Every wavefront has its own region;
    // its LDS operations execute in issue order, wave_barrier keeps the compiler from moving
    // them across the phases.
    __shared__ float lds_m[NWAVES][RPW][LQ];
    __shared__ float lds_l[NWAVES][RPW][LQ];
    __shared__ __attribute__((aligned(16))) float lds_acc[NWAVES][RPW][LQ][DH];
    if (sub == 0) {
#pragma unroll
        for (int i = 0; i < LQ; ++i) lds_m[wave][grp][i] = m[i];
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int g = 0; g < RPW; ++g)
#pragma unroll
        for (int i = 0; i < LQ; ++i) M[i] = fmaxf(M[i], lds_m[wave][g][i]);
    // scale this group's state to the common maximum and publish it
#pragma unroll
    for (int i = 0; i < LQ; ++i) {
        const float w = m[i] == -INFINITY ? 0.f : fast_exp2(m[i] - M[i]);
        f32x4 a0 = {acc[i][0] * w, acc[i][1] * w, acc[i][2] * w, acc[i][3] * w};
        f32x4 a1 = {acc[i][4] * w, acc[i][5] * w, acc[i][6] * w, acc[i][7] * w};
        *reinterpret_cast<f32x4 *>(&lds_acc[wave][grp][i][8 * sub]) = a0;
        *reinterpret_cast<f32x4 *>(&lds_acc[wave][grp][i][8 * sub + 4]) = a1;
        if (sub == 0) lds_l[wave][grp][i] = l[i] * w;
    }
    __builtin_amdgcn_wave_barrier();
    // one output element per lane and round: column (i, d)
    for (int col = lane; col < LQ * DH; col += 64) {
        const int i = col / DH, d = col % DH;
        // M of row i: select without dynamic register indexing
        float Mi = M[0];
#pragma unroll
        for (int ii = 1; ii < LQ; ++ii) Mi = i == ii ? M[ii] : Mi;
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int g = 0; g < RPW; ++g) {
            num += lds_acc[wave][g][i][d];
            den += lds_l[wave][g][i];
        }
        for (int sp0 = 0; sp0 < n_parts; sp0 += kSplitBatch) {
            float lv[kSplitBatch], ov[kSplitBatch];
#pragma unroll
            for (int u = 0; u < kSplitBatch; ++u) {
                const int sp = sp0 + u < n_parts ? sp0 + u : n_parts - 1;
                lv[u] = parts.lse2(sp, i);
                ov[u] = parts.o(sp, i, d);
            }
#pragma unroll
            for (int u = 0; u < kSplitBatch; ++u) {
                const float lse2 = lv[u];
                const float w = (sp0 + u < n_parts && lse2 != -INFINITY) ? fast_exp2(lse2 - Mi) : 0.f;
                num = fmaf(w, ov[u], num);
                den += w;
            }
        }
        view_row<T>(P.out, b, h, i)[d] = from_f32<T>(den > 0.f ? num / den : 0.f);
        if (P.lse && d == 0) P.lse[pair * LQ + i] = den > 0.f ? (Mi + fast_log2(den)) * kLn2 : -INFINITY;
    }
    if (grp == 1 && P.has_new && slot_fits) {
        // In-place append: slot n_buf of the cache receives the new row.
        *reinterpret_cast<u32x4 *>(view_row<T>(P.kb, b, h, n_buf) + 8 * sub) =
            *reinterpret_cast<const u32x4 *>(knew_row + 8 * sub);
        *reinterpret_cast<u32x4 *>(view_row<T>(P.vb, b, h, n_buf) + 8 * sub) =
            *reinterpret_cast<const u32x4 *>(vnew_row + 8 * sub);
    }
}

template <typename T, int DH, int LQ>
__global__ __launch_bounds__(kDecodeWaves * 64) void decode_buffer_kernel(DecodeParams P) {
    warm_kernel_arguments<sizeof(DecodeParams)>();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long pair = static_cast<long>(blockIdx.x) * kDecodeWaves + wave;  // b*H + h
    if (pair >= static_cast<long>(P.B) * P.H) return;
    const WorkspacePartials<T, DH, LQ> parts{static_cast<const T *>(P.part_o), P.part_lse,
                                             static_cast<long>(P.B) * P.H * LQ, pair * LQ, P.n_split};
    const long b = pair / P.H;
    const int h = static_cast<int>(pair % P.H);
    BufferHead<T, DH, LQ> hd;
    decode_buffer_request<T, DH, LQ, true>(P, b, h, lane, hd);
    decode_buffer_pair<T, DH, LQ, kDecodeWaves, decltype(parts), true>(P, b, h, wave, lane, parts, hd);
}

}  // namespace artab
