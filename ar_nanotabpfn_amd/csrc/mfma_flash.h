// MFMA flash-attention kernel for gfx950 (CDNA4), 16-bit inputs, float32 statistics.
//
// One kernel serves the three dense phases of the hot path:
//   * context pass   — queries of all trajectories stacked along the MFMA "N"
//                      dimension against one context K/V (optionally a slice of
//                      it: split-context partials with log-sum-exp),
//   * teacher forcing — context tiles unmasked, then buffer tiles under the
//                      structural mask (skip / diagonal / full per 32-key block),
//   * prefill        — dense self-attention plus the K/V cache write.
//
// Layout.  Everything is computed transposed so that softmax statistics are
// per-lane scalars and P never leaves registers:
//     S^T[kv, q] = K[kv, :] . Q[q, :]        (A = K tile from LDS, B = Q in registers)
//     O^T[d,  q] = V^T[d, kv] . P^T[kv, q]   (A = V^T tile from LDS, B = P in registers)
// With v_mfma_f32_32x32x16 a lane (c = lane % 32, hb = lane / 32) owns query
// column c and, in accumulator register v = 4g + r, row 8g + 4hb + r.  The 16
// scores a lane holds for one 32-key block are therefore keys {8g + 4hb + r};
// used directly as the B operand of the second product this enumerates the
// contraction index as e = 4(g mod 2) + r per 16-wide step t = g / 2.  V is
// staged into LDS transposed and with its key columns permuted to exactly that
// order, so one 16-byte LDS read yields the matching A operand.
#pragma once

#include "common.h"

namespace artab {

template <typename T>
struct MfmaOps;

template <>
struct MfmaOps<bf16_t> {
    typedef bf16x8 vec;
    static __device__ __forceinline__ f32x16 mma(vec a, vec b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(unsigned packed, float acc) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed),
                                               __builtin_bit_cast(bf16x2, 0x3f803f80u), acc, false);
    }
};

template <>
struct MfmaOps<f16_t> {
    typedef f16x8 vec;
    static __device__ __forceinline__ f32x16 mma(vec a, vec b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(unsigned packed, float acc) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), __builtin_bit_cast(f16x2, 0x3c003c00u),
                                      acc, false);
    }
};

enum FlashMode : int { kFlashContext = 0, kFlashTeacher = 1, kFlashPrefill = 2 };

struct FlashParams {
    View q, kc, vc, kb, vb, out;
    View kcache, vcache;
    int cache_batches;
    float *lse;       // [B,H,Lq] final log-sum-exp (natural log) or nullptr
    float *part_o;    // split partials: [n_split][B*H*Lq][DH] normalised float32
    float *part_lse;  // [n_split][B*H*Lq] natural log
    int B, H, Lq;
    int Nc, Nb, Nt;
    int G;                // query rows per group (B*Lq stacked, or Lq per batch entry)
    int tiles_per_group;  // ceil(G / BM)
    int n_groups;         // 1 (stacked) or B
    int n_split, kv_per_split;
    float qscale;  // softmax scale * log2(e), folded into Q
    int mode;
};

constexpr float kRescaleSum = 4096.0f;  // block probability sum (16 keys) that forces a refresh of the offset

// Largest teacher-forcing key limit over query rows [a, b] (inclusive).
__host__ __device__ inline int tf_range_max(int a, int b, int Nt) {
    int best = 0;
    if (a < Nt) best = tf_limit(b < Nt ? b : Nt - 1, Nt);
    if (b >= Nt) {
        int t = tf_limit(b, Nt);
        best = t > best ? t : best;
    }
    return best;
}
__host__ __device__ inline int tf_range_min(int a, int b, int Nt) {
    // tf_limit rises on [0,Nt) from 1 and on [Nt,2Nt) from 0.
    int best = tf_limit(a, Nt);
    if (a < Nt && b >= Nt) best = 0;
    return best;
}

template <typename T, int DH, int QB, int NW, int BN>
__global__ __launch_bounds__(NW * 64) void flash_kernel(FlashParams P) {
    typedef MfmaOps<T> Ops;
    typedef typename Ops::vec vec;
    constexpr int KS = DH / 16;
    constexpr int DB = DH / 32;
    constexpr int SB = BN / 32;
    constexpr int KPAD = DH + 8;
    constexpr int VPAD = BN + 8;
    constexpr int NT = NW * 64;
    constexpr int ROWS_W = 32 * QB;
    constexpr int BM = NW * ROWS_W;
    constexpr int K_CHUNKS = BN * DH / 8;         // 16-byte pieces of a K tile
    constexpr int V_TASKS = (BN / 4) * (DH / 4);  // 4 keys x 4 dims transposes of a V tile
    constexpr int KCH = (K_CHUNKS + NT - 1) / NT;
    constexpr int VTK = (V_TASKS + NT - 1) / NT;

    __shared__ __attribute__((aligned(16))) T k_lds[2][BN * KPAD];
    __shared__ __attribute__((aligned(16))) T v_lds[2][DH * VPAD];

    // ---- workgroup -> (kv-sharing group, q tile, context split); XCD-aware: the
    // hardware deals consecutive workgroup ids round-robin over the 8 XCDs, so all
    // workgroups that stream the same K/V are given ids congruent modulo 8.
    const int W = P.tiles_per_group * P.n_split;
    const int n_kvg = P.H * P.n_groups;
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int kvg = (slot / W) * 8 + xcd;
    if (kvg >= n_kvg) return;
    const int w_in = slot % W;
    const int split = w_in % P.n_split;
    const int tile = w_in / P.n_split;
    const int h = kvg % P.H;
    const int g = kvg / P.H;
    const long kvb = P.n_groups == 1 ? 0 : g;  // batch entry whose K/V this group reads

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int c = lane & 31, hb = lane >> 5;
    const int row0_wg = tile * BM;
    const int row0_w = row0_wg + wave * ROWS_W;

    // ---- Q fragments (B operand of S^T), pre-scaled by scale*log2e in float32 and
    // split into two 16-bit terms (hi + lo) so the scaling adds no rounding of its
    // own: scores carry ~16 mantissa bits of q, which keeps the log-sum-exp within
    // 1e-3 at unit-variance scores.  The extra MFMAs ride on a pipe that has slack.
    vec qhi[QB][KS], qlo[QB][KS];
    long orow_idx[QB];  // (b*H + h)*Lq + i of this lane's query per block, or -1
    int qi[QB];         // query index i within its batch entry
    long qb[QB];
#pragma unroll
    for (int j = 0; j < QB; ++j) {
        int r = row0_w + 32 * j + c;
        bool valid = r < P.G;
        long flat = static_cast<long>(g) * P.G + (valid ? r : 0);
        long b = flat / P.Lq;
        int i = static_cast<int>(flat % P.Lq);
        qb[j] = b;
        qi[j] = valid ? i : -1;
        orow_idx[j] = valid ? (b * P.H + h) * P.Lq + i : -1;
        const T *qrow = view_row<T>(P.q, b, h, i);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 raw = {0u, 0u, 0u, 0u};
            if (valid) raw = *reinterpret_cast<const u32x4 *>(qrow + 16 * ks + 8 * hb);
            u32x4 hi, lo;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a = unpack_lo<T>(raw[e]) * P.qscale, bq = unpack_hi<T>(raw[e]) * P.qscale;
                hi[e] = pack2<T>(a, bq);
                lo[e] = pack2<T>(a - unpack_lo<T>(hi[e]), bq - unpack_hi<T>(hi[e]));
            }
            qhi[j][ks] = __builtin_bit_cast(vec, hi);
            qlo[j][ks] = __builtin_bit_cast(vec, lo);
        }
    }

    // ---- prefill: this tile's own K/V rows go to the cache.
    if (P.mode == kFlashPrefill && P.kcache.p && g < P.cache_batches) {
        int nrows = min(BM, P.G - row0_wg);
        for (int idx = tid; idx < nrows * (DH / 8); idx += NT) {
            int rr = row0_wg + idx / (DH / 8), ch = idx % (DH / 8);
            *reinterpret_cast<u32x4 *>(view_row<T>(P.kcache, g, h, rr) + 8 * ch) =
                *reinterpret_cast<const u32x4 *>(view_row<T>(P.kc, kvb, h, rr) + 8 * ch);
            *reinterpret_cast<u32x4 *>(view_row<T>(P.vcache, g, h, rr) + 8 * ch) =
                *reinterpret_cast<const u32x4 *>(view_row<T>(P.vc, kvb, h, rr) + 8 * ch);
        }
    }

    // ---- key ranges: context slice of this split, then (teacher forcing) buffer keys.
    const int ctx_begin = split * P.kv_per_split;
    const int ctx_end = min(P.Nc, ctx_begin + P.kv_per_split);
    const int ctx_tiles = (ctx_end - ctx_begin + BN - 1) / BN;
    int buf_tiles = 0;
    int lim[QB];         // per-lane visible buffer keys
    int wave_lim_min = 0, wave_lim_max = 0;
    if (P.mode == kFlashTeacher) {
        int last = min(row0_wg + BM, P.G) - 1;
        int wg_max = min(P.Nb, tf_range_max(row0_wg, last, P.Nt));
        buf_tiles = (wg_max + BN - 1) / BN;
        int wlast = min(row0_w + ROWS_W, P.G) - 1;
        if (wlast >= row0_w) {
            wave_lim_max = min(P.Nb, tf_range_max(row0_w, wlast, P.Nt));
            wave_lim_min = min(P.Nb, tf_range_min(row0_w, wlast, P.Nt));
            if (wlast < row0_w + ROWS_W - 1) wave_lim_min = 0;  // padded rows see nothing
        }
#pragma unroll
        for (int j = 0; j < QB; ++j) lim[j] = qi[j] >= 0 ? min(P.Nb, tf_limit(qi[j], P.Nt)) : 0;
    } else {
#pragma unroll
        for (int j = 0; j < QB; ++j) lim[j] = 0;
    }
    const int n_tiles = ctx_tiles + buf_tiles;

    // ---- staging registers (global -> registers -> LDS, one tile ahead).
    u32x4 kst[KCH];
    u32x2 vst[VTK][4];

    auto fetch = [&](int it) {
        const bool is_ctx = it < ctx_tiles;
        const View &ks_ = is_ctx ? P.kc : P.kb;
        const View &vs_ = is_ctx ? P.vc : P.vb;
        const long bb = is_ctx ? kvb : g;
        const int kv0 = is_ctx ? ctx_begin + it * BN : (it - ctx_tiles) * BN;
        const int seg_end = is_ctx ? ctx_end : P.Nb;
#pragma unroll
        for (int x = 0; x < KCH; ++x) {
            int idx = tid + x * NT;
            int kvl = idx / (DH / 8), ch = idx % (DH / 8);
            u32x4 val = {0u, 0u, 0u, 0u};
            if (idx < K_CHUNKS && kv0 + kvl < seg_end)
                val = *reinterpret_cast<const u32x4 *>(view_row<T>(ks_, bb, h, kv0 + kvl) + 8 * ch);
            kst[x] = val;
        }
#pragma unroll
        for (int x = 0; x < VTK; ++x) {
            int idx = tid + x * NT;
            int kg4 = idx / (DH / 4), dq = idx % (DH / 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                u32x2 val = {0u, 0u};
                int kv = kv0 + 4 * kg4 + r;
                if (idx < V_TASKS && kv < seg_end)
                    val = *reinterpret_cast<const u32x2 *>(view_row<T>(vs_, bb, h, kv) + 4 * dq);
                vst[x][r] = val;
            }
        }
    };

    auto stash = [&](int buf) {
#pragma unroll
        for (int x = 0; x < KCH; ++x) {
            int idx = tid + x * NT;
            int kvl = idx / (DH / 8), ch = idx % (DH / 8);
            if (idx < K_CHUNKS) *reinterpret_cast<u32x4 *>(&k_lds[buf][kvl * KPAD + 8 * ch]) = kst[x];
        }
#pragma unroll
        for (int x = 0; x < VTK; ++x) {
            int idx = tid + x * NT;
            if (idx < V_TASKS) {
                int kg4 = idx / (DH / 4), dq = idx % (DH / 4);
                int kvl = 4 * kg4;
                int sbk = kvl >> 5, kl = kvl & 31;
                int pcol = sbk * 32 + ((kl >> 2) & 1) * 16 + (kl >> 3) * 4;
                // 4x4 transpose of 16-bit elements: rows = keys r, columns = dims dd.
                unsigned a0 = vst[x][0][0], a1 = vst[x][1][0], a2 = vst[x][2][0], a3 = vst[x][3][0];
                unsigned b0 = vst[x][0][1], b1 = vst[x][1][1], b2 = vst[x][2][1], b3 = vst[x][3][1];
                u32x2 d0 = {(a0 & 0xffffu) | (a1 << 16), (a2 & 0xffffu) | (a3 << 16)};
                u32x2 d1 = {(a0 >> 16) | (a1 & 0xffff0000u), (a2 >> 16) | (a3 & 0xffff0000u)};
                u32x2 d2 = {(b0 & 0xffffu) | (b1 << 16), (b2 & 0xffffu) | (b3 << 16)};
                u32x2 d3 = {(b0 >> 16) | (b1 & 0xffff0000u), (b2 >> 16) | (b3 & 0xffff0000u)};
                T *base = &v_lds[buf][(4 * dq) * VPAD + pcol];
                *reinterpret_cast<u32x2 *>(base) = d0;
                *reinterpret_cast<u32x2 *>(base + VPAD) = d1;
                *reinterpret_cast<u32x2 *>(base + 2 * VPAD) = d2;
                *reinterpret_cast<u32x2 *>(base + 3 * VPAD) = d3;
            }
        }
    };

    // ---- running softmax state.  m is the offset already subtracted from the
    // scores (log2 domain); it starts at 0, is set exactly on the first block and
    // afterwards only moves when a block's maximum exceeds it by the threshold.
    float m_run[QB], l_run[QB];
    f32x16 negm[QB];
    f32x16 o_acc[QB][DB];
#pragma unroll
    for (int j = 0; j < QB; ++j) {
        m_run[j] = 0.f;
        l_run[j] = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) negm[j][v] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[j][db][v] = 0.f;
    }
    bool first = true;

    if (n_tiles > 0) {
        fetch(0);
        stash(0);
    }
    __syncthreads();

    for (int it = 0; it < n_tiles; ++it) {
        const int cur = it & 1;
        if (it + 1 < n_tiles) fetch(it + 1);

        const bool is_ctx = it < ctx_tiles;
        const int kv0 = is_ctx ? ctx_begin + it * BN : (it - ctx_tiles) * BN;
        const int seg_end = is_ctx ? ctx_end : P.Nb;
        const int w_min = is_ctx ? seg_end : wave_lim_min;
        const int w_max = is_ctx ? seg_end : wave_lim_max;

#pragma unroll
        for (int sb = 0; sb < SB; ++sb) {
            const int blk0 = kv0 + 32 * sb;
            if (blk0 >= w_max) continue;  // wave-uniform: nothing visible to this wavefront
            const bool need_mask = blk0 + 32 > w_min;

            vec ak[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                ak[ks] = *reinterpret_cast<const vec *>(&k_lds[cur][(32 * sb + c) * KPAD + 16 * ks + 8 * hb]);

            f32x16 s[QB];
#pragma unroll
            for (int j = 0; j < QB; ++j) {
                s[j] = negm[j];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    s[j] = Ops::mma(ak[ks], qhi[j][ks], s[j]);
                    s[j] = Ops::mma(ak[ks], qlo[j][ks], s[j]);
                }
            }

            if (need_mask) {
#pragma unroll
                for (int j = 0; j < QB; ++j) {
                    const int lj = is_ctx ? seg_end : lim[j];
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        int kv = blk0 + 8 * (v >> 2) + 4 * hb + (v & 3);
                        if (kv >= lj) s[j][v] = -INFINITY;
                    }
                }
            }

            unsigned pk[QB][8];
#pragma unroll
            for (int j = 0; j < QB; ++j) {
                // Common path: the scores already carry -m (accumulator init), so
                // p = 2^s directly.  The running offset m is stale by design; it is
                // refreshed only when this block's probabilities sum past
                // 16 * 2^threshold (or overflow), which also covers any single
                // score more than `threshold` above m.
                float lsum = 0.f;
                if (!first) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        pk[j][e] = pack2<T>(fast_exp2(s[j][2 * e]), fast_exp2(s[j][2 * e + 1]));
                        lsum = Ops::dot2(pk[j][e], lsum);
                    }
                }
                const bool need = first || !(lsum <= kRescaleSum);
                if (__any(need)) {
                    float tmax = s[j][0];
#pragma unroll
                    for (int v = 1; v < 16; ++v) tmax = fmaxf(tmax, s[j][v]);
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
                    float delta = first ? tmax : fmaxf(tmax, 0.f);
                    if (delta == -INFINITY) delta = 0.f;
                    const float alpha = fast_exp2(-delta);
                    m_run[j] += delta;
                    l_run[j] *= alpha;
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int v = 0; v < 16; ++v) o_acc[j][db][v] *= alpha;
#pragma unroll
                    for (int v = 0; v < 16; ++v) negm[j][v] = -m_run[j];
                    lsum = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        pk[j][e] = pack2<T>(fast_exp2(s[j][2 * e] - delta), fast_exp2(s[j][2 * e + 1] - delta));
                        lsum = Ops::dot2(pk[j][e], lsum);
                    }
                }
                l_run[j] += lsum;
            }
            first = false;

#pragma unroll
            for (int db = 0; db < DB; ++db) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    vec av = *reinterpret_cast<const vec *>(
                        &v_lds[cur][(32 * db + c) * VPAD + 32 * sb + 16 * hb + 8 * t]);
#pragma unroll
                    for (int j = 0; j < QB; ++j) {
                        u32x4 pb = {pk[j][4 * t], pk[j][4 * t + 1], pk[j][4 * t + 2], pk[j][4 * t + 3]};
                        o_acc[j][db] = Ops::mma(av, __builtin_bit_cast(vec, pb), o_acc[j][db]);
                    }
                }
            }
        }

        if (it + 1 < n_tiles) stash(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: normalise, write output (final or split partial) and log-sum-exp.
    const long total_rows = static_cast<long>(P.B) * P.H * P.Lq;
#pragma unroll
    for (int j = 0; j < QB; ++j) {
        float l_tot = l_run[j] + __shfl_xor(l_run[j], 32, 64);
        if (orow_idx[j] < 0) continue;
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        const float lse = l_tot > 0.f ? (m_run[j] + fast_log2(l_tot)) * kLn2 : -INFINITY;
        if (P.part_o) {
            float *po = P.part_o + (static_cast<long>(split) * total_rows + orow_idx[j]) * DH;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    f32x4 val = {o_acc[j][db][4 * gq] * inv, o_acc[j][db][4 * gq + 1] * inv,
                                 o_acc[j][db][4 * gq + 2] * inv, o_acc[j][db][4 * gq + 3] * inv};
                    *reinterpret_cast<f32x4 *>(po + 32 * db + 8 * gq + 4 * hb) = val;
                }
            if (hb == 0) P.part_lse[static_cast<long>(split) * total_rows + orow_idx[j]] = lse;
        } else {
            T *orow = view_row<T>(P.out, qb[j], h, qi[j]);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    u32x2 val = {pack2<T>(o_acc[j][db][4 * gq] * inv, o_acc[j][db][4 * gq + 1] * inv),
                                 pack2<T>(o_acc[j][db][4 * gq + 2] * inv, o_acc[j][db][4 * gq + 3] * inv)};
                    *reinterpret_cast<u32x2 *>(orow + 32 * db + 8 * gq + 4 * hb) = val;
                }
            if (P.lse && hb == 0) P.lse[orow_idx[j]] = lse;
        }
    }
}

}  // namespace artab
