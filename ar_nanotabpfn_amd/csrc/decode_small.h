// A whole decode attention call in one launch, for problems too small to be worth three
// (gfx950; bf16/f16; head_dim 32/64/128; shared context).
//
// At B*H*Lq of a few thousand query rows and a context of a thousand rows the split-context pass,
// the buffer pass and their merge are each a launch of a few microseconds of work: the call is
// bound by launch latency (23 us for 0.5 GFLOP at B=256, H=8, head_dim 64, N_ctx=1024).  Here one
// workgroup owns 8 trajectories of one head and does everything for them:
//
//   phase 1  the 8*Lq queries are columns of one 32-column MFMA tile (S^T = K Q^T, O^T = V^T P^T
//            as in mfma_flash.h); the 8 wavefronts deal the context's 32-key blocks among
//            themselves, each with its own online softmax, K operands straight from global
//            memory, V through a wavefront-private LDS tile for the transposing read; every
//            wavefront leaves a normalised partial (float32) and its base-2 LSE in LDS;
//   phase 2  wavefront w runs the buffer pass of trajectory w (decode_buffer_pair: streams the
//            committed rows, appends the new one) and merges with the 8 partials from LDS.
//
// No workspace, no second launch.  Every workgroup reads its head's whole context (N_ctx * Dh * 4
// bytes from L2), which is what limits the shapes it is used for (see small_decode_applies()).
#pragma once

#include "common.h"
#include "decode_buffer.h"
#include "mfma_flash.h"

namespace artab {

constexpr int kSmallWaves = 8;
constexpr int kSmallTraj = 8;  // trajectories per workgroup: one per wavefront in phase 2

// The context arrives as the kernel's leading scalar arguments (base pointers; head and row
// strides in elements, within 31 bits: the launcher checks; head count; length), which the
// command processor preloads into SGPRs: the first two key blocks of every wavefront are
// requested before the argument struct, a cold miss of 750 cycles, has been fetched.
template <typename T, int DH, int LQ>
__global__ __launch_bounds__(kSmallWaves * 64) void decode_small_kernel(const char *kc_p, const char *vc_p, int kc_sh,
                                                                        int kc_sn, int vc_sh, int vc_sn, int n_heads,
                                                                        int Nc, DecodeParams P) {
    KernelArgumentLines<40 + sizeof(DecodeParams)> arguments;
    arguments.request();
    typedef MfmaOps<T> Ops;
    typedef typename Ops::vec vec;
    constexpr int KS = DH / 16, DB = DH / 32, NW = kSmallWaves, NCOL = kSmallTraj * LQ;
    constexpr int VPAD = DH + 16;  // row stride = 32 or 96 bytes mod 128 for the transposing reads
    constexpr int CPR = DH / 8;    // 16-byte pieces per row
    constexpr int VP = 32 * CPR / 64;  // V pieces per lane and block
    static_assert(NCOL <= 32, "the queries of a workgroup are one MFMA tile");

    __shared__ __attribute__((aligned(16))) T v_lds[NW][32 * VPAD];
    __shared__ float part_lse2[NW][NCOL];
    __shared__ __attribute__((aligned(16))) float part_o[NW][NCOL][DH];

    const int h = blockIdx.x % n_heads;
    const long b0 = static_cast<long>(blockIdx.x / n_heads) * kSmallTraj;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int c = lane & 31, hb = lane >> 5;
    const T *const kc_h = reinterpret_cast<const T *>(kc_p) + static_cast<long>(h) * kc_sh;  // this head's context
    const T *const vc_h = reinterpret_cast<const T *>(vc_p) + static_cast<long>(h) * vc_sh;

    const int n_blocks = (Nc + 31) / 32;
    const int my_blocks = wave < n_blocks ? (n_blocks - wave + NW - 1) / NW : 0;
    // operands of a block as they come from global memory: K in MFMA order (row c, 8 elements at
    // 16 ks + 8 hb), V as 16-byte pieces of a row-major tile (piece lane + 64 x)
    struct Raw {
        u32x4 k[KS];
        u32x4 v[VP];
    };
    // Row pointers of the block to be requested next (blocks wave, wave + NW, ... in order): full
    // blocks advance them by NW * 32 rows; the context's ragged last block computes clamped rows the
    // long way (rows past the end re-read the last one: their scores are masked and their
    // probabilities are zero, only finite values are needed).
    const long k_step = static_cast<long>(NW) * 32 * kc_sn, v_step = static_cast<long>(NW) * 32 * vc_sn;
    const T *k_ptr = kc_h + static_cast<long>(min(32 * wave + c, Nc - 1)) * kc_sn + 8 * hb;
    const T *v_ptr[VP];
#pragma unroll
    for (int x = 0; x < VP; ++x)
        v_ptr[x] = vc_h + static_cast<long>(min(32 * wave + (lane + 64 * x) / CPR, Nc - 1)) * vc_sn + 8 * ((lane + 64 * x) % CPR);
    auto fetch = [&](int blk, Raw &r) {
        if (32 * blk + 32 <= Nc) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) r.k[ks] = *reinterpret_cast<const u32x4 *>(k_ptr + 16 * ks);
#pragma unroll
            for (int x = 0; x < VP; ++x) r.v[x] = *reinterpret_cast<const u32x4 *>(v_ptr[x]);
        } else {
            const T *kr = kc_h + static_cast<long>(min(32 * blk + c, Nc - 1)) * kc_sn + 8 * hb;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) r.k[ks] = *reinterpret_cast<const u32x4 *>(kr + 16 * ks);
#pragma unroll
            for (int x = 0; x < VP; ++x) {
                const int idx = lane + 64 * x;
                r.v[x] = *reinterpret_cast<const u32x4 *>(vc_h + static_cast<long>(min(32 * blk + idx / CPR, Nc - 1)) * vc_sn +
                                                          8 * (idx % CPR));
            }
        }
        k_ptr += k_step;
#pragma unroll
        for (int x = 0; x < VP; ++x) v_ptr[x] += v_step;
    };
    // blocks wave, wave + NW, ...: two requested ahead of the one being multiplied; the first two
    // right here, from the arguments that arrived in registers
    Raw r0, r1, r2;
    if (my_blocks > 0) fetch(wave, r0);
    if (my_blocks > 1) fetch(wave + NW, r1);
    arguments.await();

    // what phase 2 needs from global memory is requested early, so that its round trips (the
    // buffer rows come from HBM) run under phase 1 — but behind the first product: loads return
    // in the order they were requested, and the first product must not wait for the buffer rows
    const long b2 = b0 + wave;
    BufferHead<T, DH, LQ> head2;
    // (the committed length first of all: the form of phase 2's requests depends on it, and a
    // value requested here has arrived when they are made)
    const CommittedRows committed = read_committed_rows(P);

    // ---- phase 1: context.  Column c = (trajectory c / LQ, query c % LQ); columns past the end
    // carry zero queries (their results are never read).
    vec qreg[KS];
    {
        const long b = b0 + c / LQ;
        const bool live = c < NCOL && b < P.B;
        const T *qrow = view_row<T>(P.q, live ? b : 0, h, live ? c % LQ : 0);
        // Loaded without a lane mask (an idle column re-reads a valid row and is zeroed by its
        // scale): a masked load merged with zeros made the compiler wait for the queries on the
        // spot, and with them for the buffer rows of phase 2 requested just before.
        const float qs = live ? P.qscale : 0.f;
        u32x4 raw[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) raw[ks] = *reinterpret_cast<const u32x4 *>(qrow + 16 * ks + 8 * hb);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 sc;  // scale * log2(e) folded in and rounded to the input type (triton_kernels.py:120-121)
#pragma unroll
            for (int e = 0; e < 4; ++e) sc[e] = pack2<T>(unpack_lo<T>(raw[ks][e]) * qs, unpack_hi<T>(raw[ks][e]) * qs);
            qreg[ks] = __builtin_bit_cast(vec, sc);
        }
    }

    f32x16 o_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[db][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;  // per column: both lanes of a column hold the same maximum
    T *vt = v_lds[wave];
    T *v_wr = vt + (lane / CPR) * VPAD + 8 * (lane % CPR);  // piece lane + 64 x sits 64 / CPR rows further down
    const int v_rd = (4 * hb + ((lane & 15) >> 2)) * VPAD + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    auto compute = [&](int blk, const Raw &r) {
        // V tile of this block into the wavefront's LDS region (its previous reads were issued
        // earlier by the same wavefront: LDS operations of a wavefront execute in order)
#pragma unroll
        for (int x = 0; x < VP; ++x) *reinterpret_cast<u32x4 *>(v_wr + x * (64 / CPR) * VPAD) = r.v[x];
        f32x16 s;
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = Ops::mma(__builtin_bit_cast(vec, r.k[ks]), qreg[ks], s);
        const int key0 = 32 * blk;
        if (key0 + 32 > Nc) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
                if (key0 + 8 * (v >> 2) + 4 * hb + (v & 3) >= Nc) s[v] = -INFINITY;
        }
        float tmax = s[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) tmax = fmaxf(tmax, s[v]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);  // finite: the first key of a block always exists
        const float alpha = fast_exp2(m_run - m_new);  // 2^(-inf) = 0 on the first block
        if (__any(alpha != 1.f)) {
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o_acc[db][v] *= alpha;
        }
        m_run = m_new;
        u32x4 pb[2];
        float lsum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float p0 = fast_exp2(s[8 * t + 2 * e] - m_new), p1 = fast_exp2(s[8 * t + 2 * e + 1] - m_new);
                lsum += p0 + p1;
                pb[t][e] = pack2<T>(p0, p1);
            }
        l_run += lsum;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const T *vp_ = vt + (16 * t) * VPAD + 32 * db + v_rd;
                s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp_));
                s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) s16x4 *)(vp_ + 8 * VPAD));
                typedef short s16x8 __attribute__((ext_vector_type(8)));
                s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                o_acc[db] = Ops::mma(__builtin_bit_cast(vec, both), __builtin_bit_cast(vec, pb[t]), o_acc[db]);
            }
        __builtin_amdgcn_wave_barrier();
    };

    // phase 2's requests: a handful of rows under a lane mask (the idle lane groups' loads would
    // cost more than the wait that the masked form brings with it), from half a batch on every
    // lane loads and nothing waits
    constexpr int kBatch = kDecodeUnroll * 64 / (DH / 8);
    const int n_total2 = P.n_base + committed.n + (P.has_new ? 1 : 0);

    {
        // Phase 2's requests follow the first product: loads return in the order of their
        // requests, and the first product waits for everything requested before it.
        int i = 0;
        if (my_blocks > 0) {
            if (2 < my_blocks) fetch(wave + NW * 2, r2);
            compute(wave, r0);
            i = 1;
        }
        if (b2 < P.B) {
            if (n_total2 > kBatch / 2)
                decode_buffer_request<T, DH, LQ, true>(P, b2, h, lane, head2, committed);
            else
                decode_buffer_request<T, DH, LQ, false>(P, b2, h, lane, head2, committed);
        }
        while (i < my_blocks) {
            if (i + 2 < my_blocks) fetch(wave + NW * (i + 2), r0);
            compute(wave + NW * i, r1);
            if (++i >= my_blocks) break;
            if (i + 2 < my_blocks) fetch(wave + NW * (i + 2), r1);
            compute(wave + NW * i, r2);
            if (++i >= my_blocks) break;
            if (i + 2 < my_blocks) fetch(wave + NW * (i + 2), r2);
            compute(wave + NW * i, r0);
            ++i;
        }
    }

    // this wavefront's partial: normalised, with its base-2 LSE (-inf: it had no block)
    {
        const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (c < NCOL) {
            if (hb == 0) part_lse2[wave][c] = l_tot > 0.f ? m_run + fast_log2(l_tot) : -INFINITY;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const f32x4 val = {o_acc[db][4 * q4] * inv, o_acc[db][4 * q4 + 1] * inv, o_acc[db][4 * q4 + 2] * inv,
                                       o_acc[db][4 * q4 + 3] * inv};
                    *reinterpret_cast<f32x4 *>(&part_o[wave][c][32 * db + 8 * q4 + 4 * hb]) = val;
                }
        }
    }
    __syncthreads();

    // ---- phase 2: buffer rows of trajectory b0 + wave, merged with the eight partials
    if (b2 >= P.B) return;
    const LdsPartials<DH, LQ> parts{&part_o[0][0][0], &part_lse2[0][0], NCOL, wave * LQ, NW};
    decode_buffer_pair<T, DH, LQ, NW>(P, b2, h, wave, lane, parts, head2);
}

}  // namespace artab
