// Backward pass of the row attention of the training forward (gfx950).
//
// Rows are [context Nc | buffer Nb | target ...] and the mask is the tile schedule of the forward
// (row_mask_limit in common.h): row i sees keys [0, vis_end(i)) with
// vis_end(i) = Nc + row_mask_limit(i), nobody sees a target key.  With P = softmax(scale Q K^T)
// under that mask (recomputed from the forward's log-sum-exp), O = P V and dO given:
//
//     delta_i = sum_d dO[i,d] O[i,d]
//     dV = P^T dO            dP = dO V^T            dS = P o (dP - delta)
//     dQ = scale dS K        dK = scale dS^T Q
//
// Two launches, no atomics, results independent of the schedule:
//   * the dQ kernel walks the visible keys of a block of queries (and leaves delta in a
//     float32 workspace),
//   * the dK/dV kernel walks the queries that see a block of keys.
// Each recomputes S and dP for its tiles.
//
// Matrix-core form (16-bit inputs, head_dim 32 / 64), v_mfma_f32_32x32x16:
//   dQ kernel, transposed as in the forward so that the statistics of a query are per-lane scalars:
//       S^T[kv,q] = K[kv,:] . Q[q,:]      dP^T[kv,q] = V[kv,:] . dO[q,:]      (A from LDS, B in registers)
//       dQ^T[d,q] += K^T[d,kv] . dS^T[kv,q]                                  (A = transposing LDS read of the K tile)
//   dK/dV kernel, keys as columns (their K and V operands stay in registers for the whole walk):
//       S[q,kv] = Q[q,:] . K[kv,:]        dP[q,kv] = dO[q,:] . V[kv,:]        (A from LDS, B in registers)
//       dV^T[d,kv] += dO^T[d,q] . P[q,kv]     dK^T[d,kv] += Q^T[d,q] . dS[q,kv]   (A = transposing reads)
//   In both the accumulator of the first products is the B operand of the second as it stands
//   (lane = column, registers enumerate rows 8g + 4hb + r), and ds_read_b64_tr_b16 delivers the
//   A operand in the same enumeration.
//
// Portable form (any element type, float32 arithmetic): one wavefront per query row / key row.
#pragma once

#include "common.h"
#include "mfma_flash.h"
#include "portable_kernels.h"

namespace artab {

struct BackwardParams {
    View q, k, v, out, dout;  // [B,H,R,Dh]
    View dq, dk, dv;          // [B,H,R,Dh]
    const float *lse;         // [B,H,R] natural-log log-sum-exp of the forward
    float *delta;             // [B,H,R] workspace: written by the dQ kernel, read by the dK/dV kernel
    int B, H, R, Nc, Nb, attend;
    int Dh;
    float scale;
    int vec_ok;
};

// One past the last key row i sees (0 for rows past the end).
__device__ __forceinline__ int backward_vis_end(const BackwardParams &P, int i) {
    return i < P.R ? P.Nc + min(P.Nb, row_mask_limit(i, P.Nc, P.Nb, P.attend)) : 0;
}

// --------------------------------------------------------------------------- portable kernels

// dQ of one query row per wavefront (and delta of that row).  Lane l owns dq[l], dq[l + 64], ...
template <typename T, int DPL>
__global__ __launch_bounds__(kPortableWaves * 64) void backward_dq_portable_kernel(BackwardParams P) {
    __shared__ float q_s[kPortableWaves][kPortableMaxDh];
    __shared__ float do_s[kPortableWaves][kPortableMaxDh];
    __shared__ float ds_s[kPortableWaves][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long row = static_cast<long>(blockIdx.x) * kPortableWaves + wave;
    const long total = static_cast<long>(P.B) * P.H * P.R;
    if (row >= total) return;  // the wavefront leaves as a whole; no workgroup barrier below
    const int i = static_cast<int>(row % P.R);
    const int h = static_cast<int>((row / P.R) % P.H);
    const long b = row / (static_cast<long>(P.R) * P.H);
    const int Dh = P.Dh;
    float *q_lds = q_s[wave], *do_lds = do_s[wave], *ds_lds = ds_s[wave];

    const T *qrow = view_row<T>(P.q, b, h, i), *dorow = view_row<T>(P.dout, b, h, i), *orow = view_row<T>(P.out, b, h, i);
    float part = 0.f;
    for (int d = lane; d < Dh; d += 64) {
        const float g = to_f32<T>(dorow[d]);
        q_lds[d] = to_f32<T>(qrow[d]);
        do_lds[d] = g;
        part = fmaf(g, to_f32<T>(orow[d]), part);
    }
    const float delta = wave_sum(part);
    const float lse = P.lse[row];
    __builtin_amdgcn_wave_barrier();

    float acc[DPL];
#pragma unroll
    for (int x = 0; x < DPL; ++x) acc[x] = 0.f;
    const int vis_end = backward_vis_end(P, i);
    for (int kv0 = 0; kv0 < vis_end; kv0 += 64) {
        const int kv = kv0 + lane;
        const bool vis = kv < vis_end;
        float ds = 0.f;
        if (vis) {
            const float s = dot_row<T>(q_lds, view_row<T>(P.k, b, h, kv), Dh, P.vec_ok) * P.scale;
            const float dp = dot_row<T>(do_lds, view_row<T>(P.v, b, h, kv), Dh, P.vec_ok);
            ds = expf(s - lse) * (dp - delta);
        }
        ds_lds[lane] = ds;
        __builtin_amdgcn_wave_barrier();
        const int cnt = min(64, vis_end - kv0);
        for (int kk = 0; kk < cnt; ++kk) {
            const float w = ds_lds[kk];
            const T *krow = view_row<T>(P.k, b, h, kv0 + kk);
#pragma unroll
            for (int x = 0; x < DPL; ++x) {
                const int d = lane + 64 * x;
                if (d < Dh) acc[x] = fmaf(w, to_f32<T>(krow[d]), acc[x]);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    T *dqrow = view_row<T>(P.dq, b, h, i);
#pragma unroll
    for (int x = 0; x < DPL; ++x) {
        const int d = lane + 64 * x;
        if (d < Dh) dqrow[d] = from_f32<T>(acc[x] * P.scale);
    }
    if (lane == 0) P.delta[row] = delta;
}

// dK and dV of one key row per wavefront.  Key j < Nc is seen by every row; buffer key j by the
// rows from j on that the mask admits; target keys by nobody (their gradients are zero).
template <typename T, int DPL>
__global__ __launch_bounds__(kPortableWaves * 64) void backward_dkv_portable_kernel(BackwardParams P) {
    __shared__ float k_s[kPortableWaves][kPortableMaxDh];
    __shared__ float v_s[kPortableWaves][kPortableMaxDh];
    __shared__ float p_s[kPortableWaves][64];
    __shared__ float ds_s[kPortableWaves][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long row = static_cast<long>(blockIdx.x) * kPortableWaves + wave;
    const long total = static_cast<long>(P.B) * P.H * P.R;
    if (row >= total) return;
    const int j = static_cast<int>(row % P.R);
    const int h = static_cast<int>((row / P.R) % P.H);
    const long b = row / (static_cast<long>(P.R) * P.H);
    const int Dh = P.Dh;
    float *k_lds = k_s[wave], *v_lds = v_s[wave], *p_lds = p_s[wave], *ds_lds = ds_s[wave];

    const T *krow = view_row<T>(P.k, b, h, j), *vrow = view_row<T>(P.v, b, h, j);
    for (int d = lane; d < Dh; d += 64) {
        k_lds[d] = to_f32<T>(krow[d]);
        v_lds[d] = to_f32<T>(vrow[d]);
    }
    __builtin_amdgcn_wave_barrier();

    float acc_k[DPL], acc_v[DPL];
#pragma unroll
    for (int x = 0; x < DPL; ++x) acc_k[x] = acc_v[x] = 0.f;
    const long stat0 = (b * P.H + h) * static_cast<long>(P.R);
    const int i_begin = j < P.Nc ? 0 : j, i_end = j < P.Nc + P.Nb ? P.R : 0;
    for (int i0 = i_begin; i0 < i_end; i0 += 64) {
        const int i = i0 + lane;
        float p = 0.f, ds = 0.f;
        if (i < P.R && j < backward_vis_end(P, i)) {
            const float s = dot_row<T>(k_lds, view_row<T>(P.q, b, h, i), Dh, P.vec_ok) * P.scale;
            const float dp = dot_row<T>(v_lds, view_row<T>(P.dout, b, h, i), Dh, P.vec_ok);
            p = expf(s - P.lse[stat0 + i]);
            ds = p * (dp - P.delta[stat0 + i]);
        }
        p_lds[lane] = p;
        ds_lds[lane] = ds;
        __builtin_amdgcn_wave_barrier();
        const int cnt = min(64, P.R - i0);
        for (int ii = 0; ii < cnt; ++ii) {
            const float wp = p_lds[ii], ws = ds_lds[ii];
            if (wp == 0.f && ws == 0.f) continue;  // wave-uniform: a row that does not see this key
            const T *qr = view_row<T>(P.q, b, h, i0 + ii), *gr = view_row<T>(P.dout, b, h, i0 + ii);
#pragma unroll
            for (int x = 0; x < DPL; ++x) {
                const int d = lane + 64 * x;
                if (d < Dh) {
                    acc_v[x] = fmaf(wp, to_f32<T>(gr[d]), acc_v[x]);
                    acc_k[x] = fmaf(ws, to_f32<T>(qr[d]), acc_k[x]);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    T *dkrow = view_row<T>(P.dk, b, h, j), *dvrow = view_row<T>(P.dv, b, h, j);
#pragma unroll
    for (int x = 0; x < DPL; ++x) {
        const int d = lane + 64 * x;
        if (d < Dh) {
            dkrow[d] = from_f32<T>(acc_k[x] * P.scale);
            dvrow[d] = from_f32<T>(acc_v[x]);
        }
    }
}

// --------------------------------------------------------------------------- matrix-core kernels

constexpr int kBackwardWaves = 4;                      // wavefronts per workgroup, 32 rows each
constexpr int kBackwardRows = 32 * kBackwardWaves;     // query rows (dQ) / key rows (dK, dV) per workgroup
static_assert(kBackwardWaves == 4, "the four LDS tiles of a workgroup double as one staging tile per wavefront");

// A 32-row tile of a [.,.,rows,DH] tensor in LDS, filled by the whole workgroup (16-byte piece
// `tid`: row tid / CPR, piece tid % CPR; rows past the end re-read the last row: finite values that
// the mask keeps out of every result).  Layout: blocks of 16 columns, each block 32 rows of
// 32 bytes side by side (1 KiB).  Both kinds of operand reads are then free of bank conflicts: a
// row operand (lane = row c, half hb of the block) is 64 lanes x 16 bytes in one contiguous KiB,
// and the 16 lanes that a transposing read combines (4 rows x 4 groups of 4 columns) cover 128
// contiguous bytes.  (With padded whole rows, 96 bytes apart at head_dim 32, a third to a half of
// the LDS cycles of these kernels were bank conflicts; removing them was worth 1 %: the LDS pipe
// is not what the kernels wait for.)  The array is sized for the padded form, which the epilogue
// still uses to stage results (backward_store_rows).
template <typename T, int DH>
struct BackwardTile {
    static constexpr int PAD = DH + 16;
    static constexpr int CPR = DH / 8;
    static constexpr int PIECES = 32 * CPR;  // <= 256 = threads of the workgroup
    static constexpr int BLOCK = 32 * 16;    // elements of a 16-column block
    // (every thread loads, without a lane mask: threads beyond the tile's pieces re-read one of
    // them and never store it.  A masked load merged with zeros makes the compiler wait for the
    // load where it is issued, and the prefetch of the next tile would hide nothing.)
    static __device__ __forceinline__ u32x4 fetch(const View &src, long b, long h, int row0, int R, int tid) {
        const int piece = tid % PIECES;
        return *reinterpret_cast<const u32x4 *>(view_row<T>(src, b, h, min(row0 + piece / CPR, R - 1)) + 8 * (piece % CPR));
    }
    static __device__ __forceinline__ void stash(T *tile, int tid, const u32x4 &raw) {
        const int row = tid / CPR, piece = tid % CPR;
        if (tid < PIECES) *reinterpret_cast<u32x4 *>(tile + (piece >> 1) * BLOCK + row * 16 + 8 * (piece & 1)) = raw;
    }
    // operand of a product contracted over head_dim, for the lane's row c: 8 elements at 16 ks + 8 hb
    static __device__ __forceinline__ typename MfmaOps<T>::vec row_operand(const T *tile, int c, int hb, int ks) {
        return __builtin_bit_cast(typename MfmaOps<T>::vec,
                                  *reinterpret_cast<const u32x4 *>(tile + ks * BLOCK + c * 16 + 8 * hb));
    }
    // operand of a product contracted over the tile's rows (step t: rows 16 t .. 16 t + 15 in the
    // enumeration of an accumulator used as the other operand), for output dimension 32 db + c:
    // the lane hands the transposing read four consecutive elements of row 4 hb + (lane % 16) / 4
    // (+ 8 for the second read) at column 16 ((lane / 16) % 2) + 4 (lane % 4) of the 32-column block
    static __device__ __forceinline__ typename MfmaOps<T>::vec col_operand(const T *tile, int lane, int t, int db) {
        const int hb = lane >> 5;
        const int row = 16 * t + 4 * hb + ((lane & 15) >> 2);
        const T *p = tile + (2 * db + ((lane >> 4) & 1)) * BLOCK + row * 16 + 4 * (lane & 3);
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(p));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(p + 8 * 16));
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(typename MfmaOps<T>::vec, both);
    }
};

// 8 elements of row `c` of a global tensor at 16 ks + 8 hb (a register operand for the whole walk)
template <typename T>
__device__ __forceinline__ u32x4 backward_row_piece(const View &src, long b, long h, int row, int R, int ks, int hb) {
    return *reinterpret_cast<const u32x4 *>(view_row<T>(src, b, h, min(row, R - 1)) + 16 * ks + 8 * hb);
}

// A wavefront's transposed result (lane = row c of its 32 rows, accumulator registers = columns
// 8g + 4hb + r of each 32-column block) to rows in global memory, through a wavefront-private LDS
// tile, so that a row's DH elements leave as 16-byte pieces side by side instead of 8-byte pieces
// of 32 different rows per store.  (LDS operations of one wavefront execute in order.)
template <typename T, int DH>
__device__ __forceinline__ void backward_store_rows(T *tile, const f32x16 (&acc)[DH / 32], float mul, const View &dst,
                                                    long b, long h, int row0, int R, int lane) {
    typedef BackwardTile<T, DH> Tile;
    const int c = lane & 31, hb = lane >> 5;
#pragma unroll
    for (int db = 0; db < DH / 32; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 o;
            o[0] = pack2<T>(acc[db][4 * g] * mul, acc[db][4 * g + 1] * mul);
            o[1] = pack2<T>(acc[db][4 * g + 2] * mul, acc[db][4 * g + 3] * mul);
            *reinterpret_cast<u32x2 *>(tile + c * Tile::PAD + 32 * db + 8 * g + 4 * hb) = o;
        }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int pass = 0; pass < Tile::PIECES / 64; ++pass) {
        const int idx = lane + 64 * pass, row = idx / Tile::CPR, piece = idx % Tile::CPR;
        const u32x4 val = *reinterpret_cast<const u32x4 *>(tile + row * Tile::PAD + 8 * piece);
        if (row0 + row < R) *reinterpret_cast<u32x4 *>(view_row<T>(dst, b, h, row0 + row) + 8 * piece) = val;
    }
    __builtin_amdgcn_wave_barrier();
}

// (head_dim 32 is held to 128 registers, four wavefronts per SIMD: measured 6 % faster than the
// 130 the compiler takes unconstrained; the dK/dV kernel loses 12 % when held to the same)
template <typename T, int DH>
__global__ __launch_bounds__(kBackwardWaves * 64) __attribute__((amdgpu_waves_per_eu(DH == 32 ? 4 : 2)))
void backward_dq_mfma_kernel(BackwardParams P) {
    typedef MfmaOps<T> Ops;
    typedef typename Ops::vec vec;
    typedef BackwardTile<T, DH> Tile;
    constexpr int KS = DH / 16, DB = DH / 32;
    __shared__ __attribute__((aligned(16))) T k_tiles[2][32 * Tile::PAD];  // two tiles in turn: one barrier per tile
    __shared__ __attribute__((aligned(16))) T v_tiles[2][32 * Tile::PAD];

    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, c = lane & 31, hb = lane >> 5;
    const int blocks = (P.R + kBackwardRows - 1) / kBackwardRows;
    const int blk = blockIdx.x % blocks;
    const int h = (blockIdx.x / blocks) % P.H;
    const long b = blockIdx.x / (blocks * P.H);
    const int qi = blk * kBackwardRows + 32 * wave + c;  // this lane's query (column)
    const long stat = (b * P.H + h) * static_cast<long>(P.R) + min(qi, P.R - 1);

    vec qf[KS], gf[KS];
    float part = 0.f;
    const float c2 = P.scale * kLog2e;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const u32x4 qr = backward_row_piece<T>(P.q, b, h, qi, P.R, ks, hb);
        const u32x4 gr = backward_row_piece<T>(P.dout, b, h, qi, P.R, ks, hb);
        const u32x4 orw = backward_row_piece<T>(P.out, b, h, qi, P.R, ks, hb);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            part = fmaf(unpack_lo<T>(gr[e]), unpack_lo<T>(orw[e]), part);
            part = fmaf(unpack_hi<T>(gr[e]), unpack_hi<T>(orw[e]), part);
        }
        // scale * log2(e) folded into the queries and rounded to the input type, as the forward
        // does (the rounding model of the reference kernel, triton_kernels.py:120-121): the scores
        // come out of the matrix pipe in base-2 units and P is the forward's P
        u32x4 sc;
#pragma unroll
        for (int e = 0; e < 4; ++e) sc[e] = pack2<T>(unpack_lo<T>(qr[e]) * c2, unpack_hi<T>(qr[e]) * c2);
        qf[ks] = __builtin_bit_cast(vec, sc);
        gf[ks] = __builtin_bit_cast(vec, gr);
    }
    const float delta = part + __shfl_xor(part, 32, 64);
    const float lse2 = P.lse[stat] * kLog2e;
    const int vis_end = backward_vis_end(P, qi);
    if (qi < P.R && hb == 0) P.delta[stat] = delta;

    f32x16 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[db][v] = 0.f;

    // every workgroup walks the keys anybody can see; what its own rows do not see is masked
    const int n_tiles = (P.Nc + P.Nb + 31) / 32;
    // tile kt + 1 goes to LDS at the start of iteration kt (it was requested one iteration earlier), tile
    // kt + 2 is requested then: one barrier per tile, a whole iteration to cover the memory round trip
    u32x4 k_raw = Tile::fetch(P.k, b, h, 0, P.R, tid), v_raw = Tile::fetch(P.v, b, h, 0, P.R, tid);
    Tile::stash(k_tiles[0], tid, k_raw);
    Tile::stash(v_tiles[0], tid, v_raw);
    if (n_tiles > 1) {
        k_raw = Tile::fetch(P.k, b, h, 32, P.R, tid);
        v_raw = Tile::fetch(P.v, b, h, 32, P.R, tid);
    }
    for (int kt = 0; kt < n_tiles; ++kt) {
        __syncthreads();  // tile kt is complete; everyone has finished reading the other one
        const T *k_tile = k_tiles[kt & 1], *v_tile = v_tiles[kt & 1];
        if (kt + 1 < n_tiles) {
            Tile::stash(k_tiles[(kt + 1) & 1], tid, k_raw);
            Tile::stash(v_tiles[(kt + 1) & 1], tid, v_raw);
            if (kt + 2 < n_tiles) {
                k_raw = Tile::fetch(P.k, b, h, 32 * (kt + 2), P.R, tid);
                v_raw = Tile::fetch(P.v, b, h, 32 * (kt + 2), P.R, tid);
            }
        }
        f32x16 s, dp;  // dp starts at -delta: the product leaves dP - delta.  (Starting s at -lse2
                       // as well costs 16 more registers than four wavefronts per SIMD leave: measured slower.)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            s[v] = 0.f;
            dp[v] = -delta;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            s = Ops::mma(Tile::row_operand(k_tile, c, hb, ks), qf[ks], s);
            dp = Ops::mma(Tile::row_operand(v_tile, c, hb, ks), gf[ks], dp);
        }
        u32x4 dsb[2];
        if (32 * kt + 32 <= P.Nc) {
            // a tile of context keys: every row sees all of it (rows past the end are never stored)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int v = 8 * t + 2 * e;
                    dsb[t][e] = pack2<T>(fast_exp2(s[v] - lse2) * dp[v], fast_exp2(s[v + 1] - lse2) * dp[v + 1]);
                }
        } else {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float ds[2];
#pragma unroll
                    for (int x = 0; x < 2; ++x) {
                        const int v = 8 * t + 2 * e + x;
                        const bool vis = 32 * kt + 8 * (v >> 2) + 4 * hb + (v & 3) < vis_end;
                        ds[x] = vis ? fast_exp2(s[v] - lse2) * dp[v] : 0.f;
                    }
                    dsb[t][e] = pack2<T>(ds[0], ds[1]);
                }
        }
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int t = 0; t < 2; ++t)
                acc[db] = Ops::mma(Tile::col_operand(k_tile, lane, t, db), __builtin_bit_cast(vec, dsb[t]), acc[db]);
    }

    __syncthreads();  // the tiles are free: one per wavefront stages its rows
    T *stage = wave < 2 ? k_tiles[wave] : v_tiles[wave - 2];
    backward_store_rows<T, DH>(stage, acc, P.scale, P.dq, b, h, blk * kBackwardRows + 32 * wave, P.R, lane);
}

template <typename T, int DH>
__global__ __launch_bounds__(kBackwardWaves * 64) void backward_dkv_mfma_kernel(BackwardParams P) {
    typedef MfmaOps<T> Ops;
    typedef typename Ops::vec vec;
    typedef BackwardTile<T, DH> Tile;
    constexpr int KS = DH / 16, DB = DH / 32;
    __shared__ __attribute__((aligned(16))) T q_tiles[2][32 * Tile::PAD];  // two tiles in turn: one barrier per tile
    __shared__ __attribute__((aligned(16))) T g_tiles[2][32 * Tile::PAD];
    __shared__ __attribute__((aligned(16))) float lse2_t[2][32];
    __shared__ __attribute__((aligned(16))) float delta_t[2][32];
    __shared__ __attribute__((aligned(16))) int end_t[2][32];

    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, c = lane & 31, hb = lane >> 5;
    const int blocks = (P.R + kBackwardRows - 1) / kBackwardRows;
    const int blk = blockIdx.x % blocks;
    const int h = (blockIdx.x / blocks) % P.H;
    const long b = blockIdx.x / (blocks * P.H);
    const int key0 = blk * kBackwardRows;       // first key of the workgroup
    const int kj = key0 + 32 * wave + c;        // this lane's key (column)
    const long stat0 = (b * P.H + h) * static_cast<long>(P.R);

    if (key0 >= P.Nc + P.Nb) {
        // target keys only: nobody sees them.  Zero rows, 16 bytes per lane, whole rows side by side.
        constexpr int CPR = Tile::CPR;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        for (int piece = tid; piece < kBackwardRows * CPR; piece += kBackwardWaves * 64) {
            const int row = key0 + piece / CPR;
            if (row < P.R) {
                *reinterpret_cast<u32x4 *>(view_row<T>(P.dk, b, h, row) + 8 * (piece % CPR)) = zero;
                *reinterpret_cast<u32x4 *>(view_row<T>(P.dv, b, h, row) + 8 * (piece % CPR)) = zero;
            }
        }
        return;
    }

    vec kf[KS], vf[KS];
    const float c2 = P.scale * kLog2e;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        // scale * log2(e) folded into the keys (this kernel's register operand) and rounded to the
        // input type: scores in base-2 units straight from the matrix pipe.  The forward and the dQ
        // kernel round q * scale * log2(e) instead, so the P recomputed here is not bit for bit the
        // forward's: the two roundings differ by up to 2^-9 of a score, i.e. P by |s| * 2^-9
        // relative (about 1 % at |s| = 10 in base-2 units).  That is inside the 16-bit tolerance
        // the gradients are held to (2e-2 of the gradient's scale, against a float64 evaluation);
        // folding the factor into the Q tile instead would put it into the A operand of
        // dK^T += Q^T dS as well and cost a multiply per staged element.
        const u32x4 kr = backward_row_piece<T>(P.k, b, h, kj, P.R, ks, hb);
        u32x4 sc;
#pragma unroll
        for (int e = 0; e < 4; ++e) sc[e] = pack2<T>(unpack_lo<T>(kr[e]) * c2, unpack_hi<T>(kr[e]) * c2);
        kf[ks] = __builtin_bit_cast(vec, sc);
        vf[ks] = __builtin_bit_cast(vec, backward_row_piece<T>(P.v, b, h, kj, P.R, ks, hb));
    }

    f32x16 acc_k[DB], acc_v[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_k[db][v] = acc_v[db][v] = 0.f;

    // Queries that can see a key of this workgroup: everybody while it holds a context key, the
    // rows from the first buffer row on otherwise.
    const int t_end = (P.R + 31) / 32;
    const int t_begin = key0 < P.Nc ? 0 : P.Nc / 32;
    u32x4 q_raw = {0u, 0u, 0u, 0u}, g_raw = {0u, 0u, 0u, 0u};
    float st_lse2 = 0.f, st_delta = 0.f;
    int st_end = 0;
    auto fetch = [&](int qt) {
        q_raw = Tile::fetch(P.q, b, h, 32 * qt, P.R, tid);
        g_raw = Tile::fetch(P.dout, b, h, 32 * qt, P.R, tid);
        {   // (all threads, as above; threads 32.. hold copies that are never stored)
            const int i = 32 * qt + (tid & 31);
            // (as loaded: any arithmetic on them here would wait for the loads, and with them for
            // the tile requested just before; they are negated and scaled when they go to LDS)
            st_lse2 = P.lse[stat0 + min(i, P.R - 1)];
            st_delta = P.delta[stat0 + min(i, P.R - 1)];
            st_end = backward_vis_end(P, i);
        }
    };
    auto stash = [&](int slot) {
        Tile::stash(q_tiles[slot], tid, q_raw);
        Tile::stash(g_tiles[slot], tid, g_raw);
        if (tid < 32) {
            lse2_t[slot][tid] = -st_lse2 * kLog2e;  // negated: the accumulators start from them
            delta_t[slot][tid] = -st_delta;
            end_t[slot][tid] = st_end;
        }
    };
    // as in the dQ kernel: tile qt + 1 goes to LDS at the start of iteration qt, tile qt + 2 is requested then
    if (t_begin < t_end) {
        fetch(t_begin);
        stash(0);
        if (t_begin + 1 < t_end) fetch(t_begin + 1);
    }
    for (int qt = t_begin; qt < t_end; ++qt) {
        __syncthreads();
        const int slot = (qt - t_begin) & 1;
        const T *q_tile = q_tiles[slot], *g_tile = g_tiles[slot];
        const float *lse2_s = lse2_t[slot], *delta_s = delta_t[slot];
        const int *end_s = end_t[slot];
        if (qt + 1 < t_end) {
            stash(slot ^ 1);
            if (qt + 2 < t_end) fetch(qt + 2);
        }
        // rows of the accumulators are queries 8g + 4hb + r of the tile: the accumulators start at
        // -lse2 and -delta of their rows, read from LDS, so that the products leave log2 P and dP - delta
        f32x16 s, dp;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 l4 = *reinterpret_cast<const f32x4 *>(&lse2_s[8 * g + 4 * hb]);
            const f32x4 d4 = *reinterpret_cast<const f32x4 *>(&delta_s[8 * g + 4 * hb]);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                s[4 * g + r] = l4[r];
                dp[4 * g + r] = d4[r];
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            s = Ops::mma(Tile::row_operand(q_tile, c, hb, ks), kf[ks], s);
            dp = Ops::mma(Tile::row_operand(g_tile, c, hb, ks), vf[ks], dp);
        }
        u32x4 pb[2], dsb[2];
        // context keys under a full tile of rows: everything is visible.  One wavefront-uniform
        // branch around the whole block (`wave` is a scalar: the compiler must not turn the two
        // paths into lane masks and issue the exponentials of both).
        if (key0 + 32 * wave + 32 <= P.Nc && 32 * qt + 32 <= P.R) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float p[4], ds[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    p[r] = fast_exp2(s[4 * g + r]);
                    ds[r] = p[r] * dp[4 * g + r];
                }
                const int t = g >> 1, e = 2 * (g & 1);
                pb[t][e] = pack2<T>(p[0], p[1]);
                pb[t][e + 1] = pack2<T>(p[2], p[3]);
                dsb[t][e] = pack2<T>(ds[0], ds[1]);
                dsb[t][e + 1] = pack2<T>(ds[2], ds[3]);
            }
        } else {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int4 e4 = *reinterpret_cast<const int4 *>(&end_s[8 * g + 4 * hb]);
                const int ends[4] = {e4.x, e4.y, e4.z, e4.w};
                float p[4], ds[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool vis = kj < ends[r];
                    const float pr = fast_exp2(s[4 * g + r]);
                    p[r] = vis ? pr : 0.f;
                    ds[r] = vis ? pr * dp[4 * g + r] : 0.f;
                }
                const int t = g >> 1, e = 2 * (g & 1);
                pb[t][e] = pack2<T>(p[0], p[1]);
                pb[t][e + 1] = pack2<T>(p[2], p[3]);
                dsb[t][e] = pack2<T>(ds[0], ds[1]);
                dsb[t][e + 1] = pack2<T>(ds[2], ds[3]);
            }
        }
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                acc_v[db] = Ops::mma(Tile::col_operand(g_tile, lane, t, db), __builtin_bit_cast(vec, pb[t]), acc_v[db]);
                acc_k[db] = Ops::mma(Tile::col_operand(q_tile, lane, t, db), __builtin_bit_cast(vec, dsb[t]), acc_k[db]);
            }
    }

    __syncthreads();  // the tiles are free: one per wavefront stages its rows
    T *stage = wave < 2 ? q_tiles[wave] : g_tiles[wave - 2];
    backward_store_rows<T, DH>(stage, acc_k, P.scale, P.dk, b, h, key0 + 32 * wave, P.R, lane);
    backward_store_rows<T, DH>(stage, acc_v, 1.f, P.dv, b, h, key0 + 32 * wave, P.R, lane);
}

}  // namespace artab
