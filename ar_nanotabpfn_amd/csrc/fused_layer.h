// Fused transformer-layer glue around the attention call (gfx950, bf16/f16).
//
// A decode step touches only B*N token rows (2048 at B=1024), so the GEMMs of a layer
// are tiny and the step is dominated by the number of launches.  Two kernels replace
// the nine launches of a layer's non-attention part:
//
//   fused_pre_kernel :  y = LN1(x + x W_fo^T);  qkv = y W_qkv^T
//   fused_post_kernel:  x1 = LN2(y + attn W_o^T);  h = gelu(x1 W_1^T + b_1);
//                       out = LN3(x1 + h W_2^T + b_2)
//
// One workgroup owns 32 (or, for few rows, 16) token rows and all columns.  Products are
// computed transposed with v_mfma_f32_32x32x16 / v_mfma_f32_16x16x32
// (C^T[n, m] = sum_k W[n, k] A[m, k]): the weight rows are the
// A operand, read straight from global memory in a pre-packed operand order (weights are
// constants, packed once), so every wavefront load is one contiguous KiB; the
// activation rows are the B operand, staged once in LDS and re-read per 16 contraction
// elements; a lane then owns one token column, so LayerNorm statistics are per-lane sums
// plus one exchange between the four wavefronts.  Activations stay in LDS between the
// chained products.
#pragma once

#include "common.h"
#include "queue_order.h"
#include "mfma_flash.h"

namespace artab {


constexpr int kFusedRows = 32;       // token rows per workgroup ...
constexpr int kFusedRowsSmall = 16;  // ... or, when that leaves most of the chip idle, 16: a decode step has
                                     // 2048 rows = 64 workgroups of 32, and everything a workgroup does
                                     // per row (merge, LayerNorm, epilogues) is bound by its one CU's
                                     // instruction issue
constexpr long kFusedSmallMaxRows = 8192;  // up to here the 16-row tiles are used

// Stands in for an absent bias vector (1024 16-bit zeros; widths go up to 512).
static __device__ const unsigned int kZeroVector[512] = {0u};

// Wavefronts per workgroup: one 32-column output block each where the width allows, so that
// a wavefront has every weight fragment of a product in flight at once (the kernels are
// latency-bound at decode sizes: 64 workgroups for 2048 rows).
constexpr int fused_waves(int D) { return D >= 256 ? 8 : 4; }

struct FusedPreParams {
    const void *x;   long ldx;   // [rows, D]
    const void *w_fo;            // [D, D] packed
    const void *g1, *b1;         // LayerNorm 1
    const void *w_qkv;           // [3D, D] packed
    void *y;                     // [rows, D] contiguous
    void *qkv;                   // [rows, 3D] contiguous
    long rows;
    float eps;
};

struct FusedPostParams {
    const void *attn; long lda;  // [rows, D]; unused when the attention arrives as partials:
    const void *part_o;          // [n_slots][part_rows][D / H] partial outputs (input type), or NULL
    const float *part_lse;       // [n_slots][part_rows] their natural-log LSEs
    int n_slots;                 // partials per (trajectory, head, query)
    long part_rows;              // B * H * Lq
    int H, Lq;                   // token row r = b * Lq + i  <->  partial row (b * H + h) * Lq + i
    const void *y;    long ldy;  // [rows, D] residual stream (output of the pre kernel)
    const void *w_o;             // [D, D] packed
    const void *g2, *b2;         // LayerNorm 2
    const void *w_1, *bias_1;    // [F, D] packed, [F]
    const void *w_2, *bias_2;    // [D, F] packed, [D]
    const void *g3, *b3;         // LayerNorm 3
    void *out;                   // [rows, D] contiguous
    long rows;
    float eps2, eps3;
    unsigned *order_wait;        // queue-order state: wait for the side counter before the partials are read
    unsigned long long order_limit;  // ... for at most this many ticks of the 100 MHz wall clock
};

// Packed weight layout.  A torch.nn.Linear weight W [N, K] (row-major) is stored as
// [N/32][K/16][64 lanes][8]: element (blk, ks, lane, e) = W[32*blk + lane%32][16*ks + 8*(lane/32) + e],
// i.e. exactly the A operand of v_mfma_f32_32x32x16 for output block blk and contraction step ks,
// so that one wavefront load reads 1 KiB of consecutive memory.
template <typename T>
__global__ void pack_weight_kernel(const T *w, T *packed, int N, int K) {
    const long chunk = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;  // one 16-byte chunk each
    const long total = static_cast<long>(N) * K / 8;
    if (chunk >= total) return;
    const int lane = static_cast<int>(chunk % 64);
    const long t = chunk / 64;
    const int ks = static_cast<int>(t % (K / 16));
    const int blk = static_cast<int>(t / (K / 16));
    const T *src = w + static_cast<long>(32 * blk + (lane & 31)) * K + 16 * ks + 8 * (lane >> 5);
    *reinterpret_cast<u32x4 *>(packed + chunk * 8) = *reinterpret_cast<const u32x4 *>(src);
}

// Tile shapes.  TR = 32: v_mfma_f32_32x32x16, a lane owns token lane%32 and, per block of 32
// output features, 16 of them in four groups of four consecutive ones (group g of half
// s = lane/32 starts at 8g + 4s).  TR = 16: v_mfma_f32_16x16x32, token lane%16, blocks of 16
// features, one group of four starting at 4s with s = lane/16.  Both read the same packed weights:
// the A operand of the 16x16x32 shape for feature block nb and 32-wide contraction step KS is
// W[16 nb + lane%16][32 KS + 8 s ..], which the 32x32x16 packing holds at block nb/2, 16-wide step
// 2 KS + s/2, lane 16 (nb%2) + lane%16 + 32 (s%2) — runs of 256 contiguous bytes.
template <typename T>
struct Mfma16;
template <>
struct Mfma16<bf16_t> {
    static __device__ __forceinline__ f32x4 mma(bf16x8 a, bf16x8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mfma16<f16_t> {
    static __device__ __forceinline__ f32x4 mma(f16x8 a, f16x8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

template <typename T, int TR>
struct Tile;
template <typename T>
struct Tile<T, 32> {
    typedef f32x16 acc_t;
    typedef typename MfmaOps<T>::vec vec;
    static constexpr int kBlock = 32, kGroups = 4, kVals = 16, kStepK = 16;
    static constexpr long kStepStride = 512;  // packed elements from one contraction step to the next
    static __device__ __forceinline__ int token(int lane) { return lane & 31; }
    static __device__ __forceinline__ int sub(int lane) { return lane >> 5; }
    static __device__ __forceinline__ int col(int nb, int g, int s) { return 32 * nb + 8 * g + 4 * s; }
    static __device__ __forceinline__ long weight_offset(int nb, int K, int lane) {
        return (static_cast<long>(nb) * (K / 16) * 64 + lane) * 8;
    }
    static __device__ __forceinline__ acc_t mma(vec a, vec b, acc_t c) { return MfmaOps<T>::mma(a, b, c); }
    // sum over the lanes that hold the same token
    static __device__ __forceinline__ float over_token(float x) { return x + __shfl_xor(x, 32, 64); }
};
template <typename T>
struct Tile<T, 16> {
    typedef f32x4 acc_t;
    typedef typename MfmaOps<T>::vec vec;
    static constexpr int kBlock = 16, kGroups = 1, kVals = 4, kStepK = 32;
    static constexpr long kStepStride = 1024;
    static __device__ __forceinline__ int token(int lane) { return lane & 15; }
    static __device__ __forceinline__ int sub(int lane) { return lane >> 4; }
    static __device__ __forceinline__ int col(int nb, int, int s) { return 16 * nb + 4 * s; }
    static __device__ __forceinline__ long weight_offset(int nb, int K, int lane) {
        const int s = lane >> 4, c = lane & 15;
        return ((static_cast<long>(nb >> 1) * (K / 16) + (s >> 1)) * 64 + 16 * (nb & 1) + c + 32 * (s & 1)) * 8;
    }
    static __device__ __forceinline__ acc_t mma(vec a, vec b, acc_t c) { return Mfma16<T>::mma(a, b, c); }
    static __device__ __forceinline__ float over_token(float x) {
        x += __shfl_xor(x, 16, 64);
        return x + __shfl_xor(x, 32, 64);
    }
};

struct NoHook {
    __device__ __forceinline__ void operator()() const {}
    __device__ __forceinline__ void operator()(int) const {}
};

// One transposed product: acc[b][v] = sum_k W[32*nblk[b] + row(v)][k] * A[c][k] for NB blocks of
// 32 output columns; A is the [32, K] activation tile in LDS (row stride ld), W the packed weight.
// The weight fragments are fetched explicitly ahead of their use — start() issues the first PF
// contraction steps and is called long before run(), so that the memory round trips of chained
// products overlap.  (Left to itself the compiler issues each load right before the MFMA that
// needs it: one round trip per step.)  The memory pipeline of a compute
// unit takes about 1.75 us for one 128 KiB matrix and its request queue holds much less than a
// matrix: a wavefront that asks for the next matrix while the current one is still on its way
// blocks at the request until there is room, and does nothing else meanwhile.  Hence the rule
// every caller follows: request a matrix when the one before it has arrived — run() waits for
// its own fragments and then calls `on_arrival`, which requests the next stream — so that the
// pipeline always has one matrix to work on and no wavefront queues up behind it.  The rule is
// for matrices that fit the prefetch window (kWhole; widths up to 256): a deeper one is
// requested piecemeal inside its product, the next stream is then requested ahead of that
// product as before, and run() calls `on_arrival` without waiting.
template <typename T, int K, int NB, int TR = 32>
struct WeightStream {
    typedef Tile<T, TR> TL;
    typedef typename TL::vec vec;
    typedef typename TL::acc_t acc_t;
    static constexpr int KS = K / TL::kStepK;
    static constexpr int PFW = NB >= 4 ? 4 : (NB == 2 ? 8 : 16);
    static constexpr int PF = PFW < KS ? PFW : KS;
    static constexpr bool kWhole = PF >= KS;  // start() requests the whole matrix
    const T *wl[NB];
    vec wf[PF][NB];
    int rot;  // contraction step this workgroup starts with

    // start() = begin() + request(0 .. PF-1).  The requests of a wavefront are accepted at the pace
    // of the CU's address unit (64 B/clk: 1 us for a 128 KiB matrix over the eight wavefronts) and
    // the wavefront waits at each; run() can spread the requests of the NEXT stream over the steps
    // of its own product (`per_step`), so that its MFMAs execute while the requests queue.
    __device__ __forceinline__ void start(const T *wp, const int (&nblk)[NB], int lane, int tile = -1) {
        begin(wp, nblk, lane, tile);
#pragma unroll
        for (int p = 0; p < PF; ++p) request(p);
        __builtin_amdgcn_sched_barrier(0);  // the prefetch stays where it was written
    }

    __device__ __forceinline__ void request(int p) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
            wf[p][b] = *reinterpret_cast<const vec *>(wl[b] + ((p + rot) & (KS - 1)) * TL::kStepStride);
    }

    // A product offers the caller kPoints places for the requests of a later stream: one behind
    // each of its KS contraction steps (0 .. KS-1) and, in four groups (tail_points), KS more in
    // its epilogue, where the address unit would otherwise idle while the wavefronts exchange row
    // statistics.
    static constexpr int kTail = KS;  // (three times as many, i.e. a quarter of the requests at the steps: no difference)
    static constexpr int kPoints = KS + kTail;
    template <typename StepHook>
    static __device__ __forceinline__ void tail_points(int group, StepHook &steps) {
#pragma unroll
        for (int i = 0; i < kTail; ++i)
            if (i * 4 / kTail == group) steps(KS + i);
    }

    // The requests that fall to point `ks` of `n_steps` when this stream's PF requests are spread
    // evenly over them.
    __device__ __forceinline__ void request_share(int ks, int n_steps) {
#pragma unroll
        for (int p = 0; p < PF; ++p)
            if (p * n_steps / PF == ks) request(p);
    }

    // `tile`: index of this workgroup's tile in the launch that would process the same rows on
    // their own (default: the workgroup index).  A kernel that runs several bodies on differently
    // sized tiles passes it, so that a row's sums are taken in the same order wherever it is computed.
    __device__ __forceinline__ void begin(const T *wp, const int (&nblk)[NB], int lane, int tile = -1) {
#pragma unroll
        for (int b = 0; b < NB; ++b) wl[b] = wp + TL::weight_offset(nblk[b], K, lane);
        // Every workgroup streams the same matrix at about the same time, and the 16 of an XCD
        // would ask its L2 for the same lines at the same moment (measured: 1.5 us of a 19 us layer
        // kernel).  Each starts its contraction at a different step instead; a sum does not care.
        // Workgroup ids are dealt round-robin over the 8 XCDs, so id / 8 counts within an XCD.
        static_assert((KS & (KS - 1)) == 0, "contraction steps must be a power of two");
        rot = ((tile < 0 ? static_cast<int>(blockIdx.x) : tile) >> 3) & (KS - 1);
    }

    // `before` runs ahead of the product — the place to begin() a later stream —, `per_step(ks)`
    // behind the MFMAs of every contraction step — the place for that stream's
    // request_share(ks, kPoints); the fragment registers of step ks are free by then, so the later
    // stream may be this very object (the matrix two ahead goes where the current one was).  The
    // caller passes the same hook to tail_points() at four places of the product's epilogue for the
    // points KS .. kPoints-1.  For a stream deeper than its prefetch window all points run up
    // front, which is start() of the later stream ahead of this product.
    template <typename Hook = NoHook, typename StepHook = NoHook>
    __device__ __forceinline__ void run(acc_t (&acc)[NB], const T *a_lds, int ld, int c, int hb,
                                        Hook on_arrival = Hook{}, StepHook per_step = StepHook{}) {
        on_arrival();
        if (!kWhole) {
#pragma unroll
            for (int ks = 0; ks < kPoints; ++ks) per_step(ks);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < TL::kVals; ++v) acc[b][v] = 0.f;
        if (kWhole)
            multiply(acc, a_lds, ld, c, hb, per_step);
        else
            multiply(acc, a_lds, ld, c, hb);
    }

    // acc += W A^T over the whole contraction, without waiting for anything but the fragments used
    // (a matrix deeper than the prefetch window is requested step by step as fragments are used up)
    template <typename StepHook = NoHook>
    __device__ __forceinline__ void multiply(acc_t (&acc)[NB], const T *a_lds, int ld, int c, int hb,
                                             StepHook per_step = StepHook{}) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const vec af =
                *reinterpret_cast<const vec *>(a_lds + c * ld + TL::kStepK * ((ks + rot) & (KS - 1)) + 8 * hb);
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[b] = TL::mma(wf[ks % PF][b], af, acc[b]);
            if (ks + PF < KS) {
#pragma unroll
                for (int b = 0; b < NB; ++b)
                    wf[ks % PF][b] =
                        *reinterpret_cast<const vec *>(wl[b] + ((ks + PF + rot) & (KS - 1)) * TL::kStepStride);
            }
            per_step(ks);
        }
    }
};

// Column index of accumulator element (block nb, register v) for this lane.
__device__ __forceinline__ int col_of(int nb, int v, int hb) { return 32 * nb + 8 * (v >> 2) + 4 * hb + (v & 3); }

template <typename T>
__device__ __forceinline__ void load4f(const T *p, float *f) {
    u32x2 r = *reinterpret_cast<const u32x2 *>(p);
    f[0] = unpack_lo<T>(r[0]);
    f[1] = unpack_hi<T>(r[0]);
    f[2] = unpack_lo<T>(r[1]);
    f[3] = unpack_hi<T>(r[1]);
}
template <typename T>
__device__ __forceinline__ void store4f(T *p, float a, float b, float c, float d) {
    u32x2 r = {pack2<T>(a, b), pack2<T>(c, d)};
    *reinterpret_cast<u32x2 *>(p) = r;
}

// The entries of a length-N vector (bias, gamma, beta) at this lane's accumulator columns;
// a missing bias is read from a zero vector the caller substitutes.
template <typename T, int NB, int TR = 32>
__device__ __forceinline__ void load_cols(const T *vec, const int (&nblk)[NB], int hb,
                                          float (&out)[NB][Tile<T, TR>::kVals]) {
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g = 0; g < Tile<T, TR>::kGroups; ++g)
            load4f<T>(vec + Tile<T, TR>::col(nblk[b], g, hb), &out[b][4 * g]);
}

// The attention tile of 32 token rows built from partial results (context slices + buffer pass)
// instead of a finished matrix: out = sum_s w_s o_s / sum_s w_s with w_s = exp(lse_s - max lse),
// the same arithmetic, in the same order, as the stand-alone combine launch, rounded once to the
// storage type on its way into LDS.  One item = 8 output dims of one (row, head).
// Partial row and first dim of item (token row `tok`, 16-byte chunk `ch`): token = b*Lq + i, the
// chunk lies in head h at dim d0, and the partial row is (b*H + h)*Lq + i.  Decode has Lq in
// {1, 2} and a power-of-two head dim: those take shifts; anything else 32-bit divisions (a
// 64-bit division per item cost more than the loads it addressed).
struct PartialIndex {
    int lq, heads, dh, dh_shift;  // dh_shift < 0: head dim is not a power of two
    __device__ __forceinline__ PartialIndex(int Lq, int H, int Dh)
        : lq(Lq), heads(H), dh(Dh), dh_shift((Dh & (Dh - 1)) == 0 ? __builtin_ctz(static_cast<unsigned>(Dh)) : -1) {}
    __device__ __forceinline__ void locate(unsigned tok, int ch, unsigned &prow, int &d0) const {
        unsigned b, i;
        if (lq == 1) {
            b = tok; i = 0;
        } else if (lq == 2) {
            b = tok >> 1; i = tok & 1u;
        } else {
            b = tok / static_cast<unsigned>(lq); i = tok - b * static_cast<unsigned>(lq);
        }
        unsigned h;
        if (dh_shift >= 0) {
            h = static_cast<unsigned>(8 * ch) >> dh_shift; d0 = (8 * ch) & (dh - 1);
        } else {
            h = static_cast<unsigned>(8 * ch) / static_cast<unsigned>(dh); d0 = 8 * ch - static_cast<int>(h) * dh;
        }
        prow = (b * static_cast<unsigned>(heads) + h) * static_cast<unsigned>(lq) + i;
    }
};

constexpr int kMergeBatch = 9;  // partials fetched per round (8 context slices + the buffer pass)

// `on_arrival` runs once every load issued so far (the caller's and the partials') has come back
// and before the merge arithmetic — the place to begin() the next weight stream —, `per_slot(u)`,
// u = 0 .. kMergeBatch-1, between the slots of the merge arithmetic of the last item: the place for
// that stream's request_share(u, kMergeBatch), so that its requests queue while the merge computes.
template <typename T, int D, int NT, int TR, typename WaitHook, typename Hook, typename SlotHook>
__device__ __forceinline__ void stage_merged_attention(T *dst, int lds_ld, const FusedPostParams &P, long row0,
                                                       int valid, int tid, WaitHook before_last_slot, Hook on_arrival,
                                                       SlotHook per_slot) {
    const int dh = D / P.H;          // head dim, a multiple of 8
    const PartialIndex where(P.Lq, P.H, dh);
    const unsigned tok0 = static_cast<unsigned>(row0);  // the launcher keeps rows below 2^31
    constexpr int CPR = D / 8;       // 16-byte chunks per token row
    constexpr int ITEMS = TR * CPR / NT;
    static_assert(TR * CPR % NT == 0, "whole items per thread");
    const long o_step = P.part_rows * dh;
    if (P.n_slots <= kMergeBatch) {
        // Common case: every slot of two items is requested before anything is used, so the
        // thread pays one memory round trip per pair of items (rows beyond `valid` read the
        // last valid row and are zeroed afterwards: no divergent loads).  The last slot is the one
        // another queue may still be writing (the buffer pass's partial): `before_last_slot()` —
        // the caller's wait for that queue — runs between the requests for the slots in front of
        // it and the request for it, so the wait's own round trip travels with the former.
        constexpr int G = ITEMS % 2 == 0 ? 2 : 1;
        constexpr int NC = kMergeBatch - 1;  // slots in front of the last one, at most
        const int n_front = P.n_slots - 1;
#pragma unroll
        for (int it0 = 0; it0 < ITEMS; it0 += G) {
            float lv[G][kMergeBatch];
            u32x4 ov[G][kMergeBatch];
            const T *po_[G];
            const float *pl_[G];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int idx = tid + (it0 + g) * NT;
                const int r = idx / CPR, ch = idx % CPR;
                unsigned prow;
                int d0;
                where.locate(tok0 + (r < valid ? r : valid - 1), ch, prow, d0);
                po_[g] = static_cast<const T *>(P.part_o) + static_cast<long>(prow) * dh + d0;
                pl_[g] = P.part_lse + prow;
#pragma unroll
                for (int u = 0; u < NC; ++u) {
                    const int sl = u < n_front ? u : (n_front > 0 ? n_front - 1 : 0);  // repeats are never used
                    lv[g][u] = pl_[g][sl * P.part_rows];
                    ov[g][u] = *reinterpret_cast<const u32x4 *>(po_[g] + sl * o_step);
                }
            }
            if (it0 == 0) before_last_slot();
#pragma unroll
            for (int g = 0; g < G; ++g) {
                lv[g][NC] = pl_[g][n_front * P.part_rows];
                ov[g][NC] = *reinterpret_cast<const u32x4 *>(po_[g] + n_front * o_step);
            }
            if (it0 + G >= ITEMS) {  // the last round of loads
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
                __builtin_amdgcn_sched_barrier(0);
                on_arrival();
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int idx = tid + (it0 + g) * NT;
                const int r = idx / CPR, ch = idx % CPR;
                float mx = lv[g][NC];
#pragma unroll
                for (int u = 0; u < NC; ++u) mx = fmaxf(mx, lv[g][u]);  // repeats of a slot change nothing
                float wsum = 0.f, acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < kMergeBatch; ++u) {  // slots in their order; the last one last
                    if (u < n_front || u == NC) {
                        const float w = merge_weight(lv[g][u], mx);
                        wsum += w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            acc[2 * e] = fmaf(w, unpack_lo<T>(ov[g][u][e]), acc[2 * e]);
                            acc[2 * e + 1] = fmaf(w, unpack_hi<T>(ov[g][u][e]), acc[2 * e + 1]);
                        }
                    }
                    if (g == G - 1 && it0 + G >= ITEMS) {
                        per_slot(u);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                const float inv = 1.f / wsum;
                u32x4 packed = {0u, 0u, 0u, 0u};
                if (r < valid) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) packed[e] = pack2<T>(acc[2 * e] * inv, acc[2 * e + 1] * inv);
                }
                *reinterpret_cast<u32x4 *>(dst + r * lds_ld + 8 * ch) = packed;
            }
        }
        return;
    }
    before_last_slot();
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    on_arrival();
#pragma unroll
    for (int u = 0; u < kMergeBatch; ++u) per_slot(u);
    for (int idx = tid; idx < TR * CPR; idx += NT) {
        const int r = idx / CPR, ch = idx % CPR;
        u32x4 packed = {0u, 0u, 0u, 0u};
        if (r < valid) {
            unsigned prow;
            int d0;
            where.locate(tok0 + r, ch, prow, d0);
            const T *po = static_cast<const T *>(P.part_o) + static_cast<long>(prow) * dh + d0;
            const float *pl = P.part_lse + prow;
            float mx = -INFINITY;
            for (int s0 = 0; s0 < P.n_slots; s0 += kMergeBatch) {
                float lv[kMergeBatch];
#pragma unroll
                for (int u = 0; u < kMergeBatch; ++u) {
                    const int sl = s0 + u < P.n_slots ? s0 + u : P.n_slots - 1;
                    lv[u] = pl[sl * P.part_rows];
                }
#pragma unroll
                for (int u = 0; u < kMergeBatch; ++u) mx = fmaxf(mx, lv[u]);
            }
            float wsum = 0.f, acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int s0 = 0; s0 < P.n_slots; s0 += kMergeBatch) {
                float lv[kMergeBatch];
                u32x4 ov[kMergeBatch];
#pragma unroll
                for (int u = 0; u < kMergeBatch; ++u) {
                    const int sl = s0 + u < P.n_slots ? s0 + u : P.n_slots - 1;
                    lv[u] = pl[sl * P.part_rows];
                    ov[u] = *reinterpret_cast<const u32x4 *>(po + sl * o_step);
                }
#pragma unroll
                for (int u = 0; u < kMergeBatch; ++u) {
                    if (s0 + u < P.n_slots) {
                        const float w = merge_weight(lv[u], mx);
                        wsum += w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            acc[2 * e] = fmaf(w, unpack_lo<T>(ov[u][e]), acc[2 * e]);
                            acc[2 * e + 1] = fmaf(w, unpack_hi<T>(ov[u][e]), acc[2 * e + 1]);
                        }
                    }
                }
            }
            const float inv = 1.f / wsum;
#pragma unroll
            for (int e = 0; e < 4; ++e) packed[e] = pack2<T>(acc[2 * e] * inv, acc[2 * e + 1] * inv);
        }
        *reinterpret_cast<u32x4 *>(dst + r * lds_ld + 8 * ch) = packed;
    }
}

// Parameter vectors (LayerNorm gamma / beta, biases) are copied to LDS when the kernel starts:
// fetched from global memory right where they are used, each costs its phase a full memory
// round trip (the phases are far shorter than that).  A missing vector becomes zeros.
// Tiles and vectors are copied without registers: each wavefront sends whole rows (one vector) from global
// memory straight into LDS, so every load of a kernel's prologue is in flight at once instead of
// one round trip per copy.  The caller waits (vmcnt 0) before the barrier that publishes them.
template <typename T, int W, int NT, int TR>
__device__ __forceinline__ void dma_tile(T *dst, int lds_ld, const T *src, long ld, int valid, int tid) {
    constexpr int NW = NT / 64, CPR = W / 8;
    static_assert(CPR <= 64, "a row is at most one wavefront of 16-byte pieces");
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
#pragma unroll
    for (int r = wave; r < TR; r += NW) {
        if (lane < CPR) {
            if (r < valid) {
                load_to_lds_16(src + r * ld + 8 * lane, dst + r * lds_ld);
            } else {
                const u32x4 zero = {0u, 0u, 0u, 0u};
                *reinterpret_cast<u32x4 *>(dst + r * lds_ld + 8 * lane) = zero;
            }
        }
    }
}
// `turn` spreads the vectors of a prologue over the wavefronts.
template <typename T, int LEN, int NT>
__device__ __forceinline__ void dma_vector(T *dst, const void *src, int tid, int turn) {
    constexpr int NW = NT / 64;
    static_assert(LEN % 8 == 0 && LEN / 8 <= 64, "at most one wavefront of 16-byte pieces");
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    if (wave == turn % NW && lane < LEN / 8) {
        if (src) {
            load_to_lds_16(static_cast<const T *>(src) + 8 * lane, dst);
        } else {
            const u32x4 zero = {0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4 *>(dst + 8 * lane) = zero;
        }
    }
}
__device__ __forceinline__ void wait_all_loads() { __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); }

// LDS slots of the parameter vectors (each max(D, F) elements wide)
enum VecSlot : int { kVecG1 = 0, kVecB1, kVecG2, kVecB2, kVecBias1, kVecG3, kVecB3, kVecBias2, kVecSlots };

// Row statistics over all N = NB*32*NW columns of the tile: each lane holds, for its token column,
// the values of NB blocks.  A wavefront first reduces its own NB*32 values per row to (mean, sum of
// squared deviations) in registers; the wavefronts' pairs are combined after ONE exchange through
// red_a / red_b ([NW*32] each) by the pairwise update of Chan et al., which is as robust as the
// two-pass form.  Callers separate two calls by a barrier (the one that publishes the normalised
// tile does).
template <typename T, int NB, int NW, int TR, typename Hook = NoHook>
__device__ __forceinline__ void row_mean_rstd(const float (&v)[NB][Tile<T, TR>::kVals], float *red_a, float *red_b,
                                              int wave, int c, int hb, int N, float eps, float &mean, float &rstd,
                                              Hook at = Hook{}) {
    typedef Tile<T, TR> TL;
    at(0);
    constexpr float kLocal = NB * TL::kBlock;
    float s = 0.f;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int e = 0; e < TL::kVals; ++e) s += v[b][e];
    s = TL::over_token(s);
    const float lmean = s * (1.f / kLocal);
    float q = 0.f;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int e = 0; e < TL::kVals; ++e) {
            const float d = v[b][e] - lmean;
            q += d * d;
        }
    q = TL::over_token(q);
    if (hb == 0) {
        red_a[wave * TR + c] = lmean;
        red_b[wave * TR + c] = q;
    }
    at(1);
    __syncthreads();
    at(2);
    float lm[NW], tot = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        lm[w] = red_a[w * TR + c];
        tot += lm[w];
    }
    mean = tot * (1.f / NW);
    float m2 = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        const float d = lm[w] - mean;
        m2 += red_b[w * TR + c] + kLocal * d * d;
    }
    rstd = rsqrtf(m2 / N + eps);
}

// Cooperative copy of a [TR, W] tile between global memory (row stride ld) and LDS (row stride
// lds_ld) with 16-byte accesses along rows.  Loading zero-fills rows beyond `valid`.
template <typename T, int W, int NT, int TR = 32>
__device__ __forceinline__ void stage_tile(T *dst, int lds_ld, const T *src, long ld, int valid, int tid) {
    constexpr int CPR = W / 8;
#pragma unroll
    for (int idx = tid; idx < TR * CPR; idx += NT) {
        const int r = idx / CPR, ch = idx % CPR;
        u32x4 val = {0u, 0u, 0u, 0u};
        if (r < valid) val = *reinterpret_cast<const u32x4 *>(src + r * ld + 8 * ch);
        *reinterpret_cast<u32x4 *>(dst + r * lds_ld + 8 * ch) = val;
    }
}
template <typename T, int W, int NT, int TR>
__device__ __forceinline__ void unstage_tile(T *dst, long ld, const T *src, int lds_ld, int valid, int tid) {
    constexpr int CPR = W / 8;
#pragma unroll
    for (int idx = tid; idx < TR * CPR; idx += NT) {
        const int r = idx / CPR, ch = idx % CPR;
        if (r < valid)
            *reinterpret_cast<u32x4 *>(dst + r * ld + 8 * ch) = *reinterpret_cast<const u32x4 *>(src + r * lds_ld + 8 * ch);
    }
}

// LayerNorm over the tile rows of v (statistics across all wavefronts), result written as T
// into the LDS tile `dst` at this lane's (row c, accumulator columns).
template <typename T, int NB, int NW, int TR, typename Hook = NoHook>
__device__ __forceinline__ void layer_norm_to_lds(const float (&v)[NB][Tile<T, TR>::kVals],
                                                  const float (&gam)[NB][Tile<T, TR>::kVals],
                                                  const float (&bet)[NB][Tile<T, TR>::kVals], const int (&nblk)[NB],
                                                  T *dst, int ld, float *red_a, float *red_b, int wave, int c, int hb,
                                                  int N, float eps, Hook at = Hook{}) {
    typedef Tile<T, TR> TL;
    float mean, rstd;
    row_mean_rstd<T, NB, NW, TR>(v, red_a, red_b, wave, c, hb, N, eps, mean, rstd, at);
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g = 0; g < TL::kGroups; ++g) {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (v[b][4 * g + e] - mean) * rstd * gam[b][4 * g + e] + bet[b][4 * g + e];
            store4f<T>(dst + c * ld + TL::col(nblk[b], g, hb), o[0], o[1], o[2], o[3]);
        }
    at(3);
}

// Body of the pre kernel on one TR-row tile.  a0: x tile (row stride D + 8), staged here from
// P.x unless X_IN_LDS (then a finished tile is already there and the caller has synchronised);
// later the staging buffer of the qkv passes.  a1: y tile.
template <typename T, int D, int NT>
__device__ __forceinline__ void stage_pre_vectors(const FusedPreParams &P, T *vecs, int vec_ld, int tid) {
    dma_vector<T, D, NT>(vecs + kVecG1 * vec_ld, P.g1, tid, 6);
    dma_vector<T, D, NT>(vecs + kVecB1 * vec_ld, P.b1, tid, 7);
}

// 32/16-feature blocks per wavefront for N output features
template <typename T, int TR>
constexpr int fused_blocks(int N, int NW) { return (N / Tile<T, TR>::kBlock + NW - 1) / NW; }

template <typename T, int D, int TR, bool X_IN_LDS, bool Q_REQUESTED = false>
__device__ __forceinline__ void fused_pre_body(const FusedPreParams &P, T *a0, T *a1, float *red_a, float *red_b,
                                               long row0, int valid,
                                               WeightStream<T, D, fused_blocks<T, TR>(D, fused_waves(D)), TR> &w_a,
                                               WeightStream<T, D, fused_blocks<T, TR>(D, fused_waves(D)), TR> &w_b,
                                               T *vecs, int vec_ld, int tile = -1) {
    typedef Tile<T, TR> TL;
    constexpr int NW = fused_waves(D), NT = NW * 64;
    constexpr int LD = D + 8;
    constexpr int NB = fused_blocks<T, TR>(D, NW);  // feature blocks per wavefront per D columns
    constexpr int VB = TL::kVals, GB = TL::kGroups;
    static_assert(D % (TL::kBlock * NW) == 0, "D must be a multiple of block width * wavefronts");
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = TL::token(lane), hb = TL::sub(lane);

    int nblk[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) nblk[b] = wave + NW * b;

    // Weight order: W_fo (w_a), q (w_b), k (w_a again), v (w_b again).  With X_IN_LDS the caller has
    // requested W_fo and, with Q_REQUESTED, the q weights already.
    constexpr bool kWhole = WeightStream<T, D, NB, TR>::kWhole;
    if (!X_IN_LDS) {
        w_a.start(static_cast<const T *>(P.w_fo), nblk, lane, tile);
        dma_tile<T, D, NT, TR>(a0, LD, static_cast<const T *>(P.x) + row0 * P.ldx, P.ldx, valid, tid);
        stage_pre_vectors<T, D, NT>(P, vecs, vec_ld, tid);
        wait_all_loads();
        __syncthreads();
    }
    if (!Q_REQUESTED) w_b.start(static_cast<const T *>(P.w_qkv), nblk, lane, tile);  // q columns
    int nb_k[NB], nb_v[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        nb_k[b] = (D / TL::kBlock) + nblk[b];
        nb_v[b] = 2 * (D / TL::kBlock) + nblk[b];
    }
    float gam[NB][VB], bet[NB][VB];
    load_cols<T, NB, TR>(vecs + kVecG1 * vec_ld, nblk, hb, gam);
    load_cols<T, NB, TR>(vecs + kVecB1 * vec_ld, nblk, hb, bet);

    // ---- y = LN1(x + x W_fo^T)
    {
        typename TL::acc_t acc[NB];
        // whole-matrix streams: the k weights go where W_fo's fragments were, step by step
        auto k_steps = [&](int ks) { if (kWhole) w_a.request_share(ks, WeightStream<T, D, NB, TR>::kPoints); };
        w_a.run(acc, a0, LD, c, hb, [&]() { if (kWhole) w_a.begin(static_cast<const T *>(P.w_qkv), nb_k, lane, tile); },
                k_steps);
        float v[NB][VB];
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int g = 0; g < GB; ++g) {
                float r[4];
                load4f<T>(a0 + c * LD + TL::col(nblk[b], g, hb), r);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[b][4 * g + e] = acc[b][4 * g + e] + r[e];
            }
        layer_norm_to_lds<T, NB, NW, TR>(v, gam, bet, nblk, a1, LD, red_a, red_b, wave, c, hb, D, P.eps, [&](int e) {
            if (kWhole) WeightStream<T, D, NB, TR>::tail_points(e, k_steps);
        });
    }
    __syncthreads();  // y complete in a1; a0 no longer read
    unstage_tile<T, D, NT, TR>(static_cast<T *>(P.y) + row0 * D, D, a1, LD, valid, tid);

    // ---- qkv = y W_qkv^T, three passes of D columns, each staged through a0 for row-contiguous
    // stores; the weights of the next pass are requested before the current one is computed
#pragma unroll
    for (int part = 0; part < 3; ++part) {
        WeightStream<T, D, NB, TR> &cur = (part & 1) ? w_a : w_b, &nxt = (part & 1) ? w_b : w_a;
        typename TL::acc_t acc[NB];
        // whole-matrix streams: the v weights follow the q weights through w_b during the q pass (k
        // is on its way already); deeper ones: the next pass's weights ahead of this pass
        auto steps = [&](int ks) {
            if (kWhole) {
                if (part == 0) w_b.request_share(ks, WeightStream<T, D, NB, TR>::kPoints);
            } else if (part < 2) {
                nxt.request_share(ks, WeightStream<T, D, NB, TR>::kPoints);
            }
        };
        cur.run(acc, a1, LD, c, hb,
                [&]() {
                    if (kWhole) {
                        if (part == 0) w_b.begin(static_cast<const T *>(P.w_qkv), nb_v, lane, tile);
                    } else if (part < 2) {
                        nxt.begin(static_cast<const T *>(P.w_qkv), part == 0 ? nb_k : nb_v, lane, tile);
                    }
                },
                steps);
        if (kWhole) WeightStream<T, D, NB, TR>::tail_points(0, steps);
        if (part) __syncthreads();  // the previous pass has been copied out of a0
        if (kWhole) WeightStream<T, D, NB, TR>::tail_points(1, steps);
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int g = 0; g < GB; ++g)
                store4f<T>(a0 + c * LD + TL::col(nblk[b], g, hb), acc[b][4 * g], acc[b][4 * g + 1],
                           acc[b][4 * g + 2], acc[b][4 * g + 3]);
        if (kWhole) WeightStream<T, D, NB, TR>::tail_points(2, steps);
        __syncthreads();
        if (kWhole) WeightStream<T, D, NB, TR>::tail_points(3, steps);
        unstage_tile<T, D, NT, TR>(static_cast<T *>(P.qkv) + row0 * (3 * D) + part * D, 3 * D, a0, LD, valid, tid);
    }
}

template <typename T, int D, int TR>
__global__ __launch_bounds__(fused_waves(D) * 64) void fused_pre_kernel(FusedPreParams P) {
    warm_kernel_arguments<sizeof(FusedPreParams)>();
    constexpr int NW = fused_waves(D), LD = D + 8;
    __shared__ __attribute__((aligned(16))) T a0[TR * LD];
    __shared__ __attribute__((aligned(16))) T a1[TR * LD];
    __shared__ float red_a[NW * TR], red_b[NW * TR];
    const long row0 = static_cast<long>(blockIdx.x) * TR;
    const int valid = static_cast<int>(min(static_cast<long>(TR), P.rows - row0));
    __shared__ __attribute__((aligned(16))) T vecs[kVecSlots * D];
    WeightStream<T, D, fused_blocks<T, TR>(D, NW), TR> w_a, w_b;
    fused_pre_body<T, D, TR, false>(P, a0, a1, red_a, red_b, row0, valid, w_a, w_b, vecs, D);
}

// Body of the post kernel on one TR-row tile.  a0 (row stride max(D, F) + 8): attn tile, gelu
// output, finally the finished tile (row stride D + 8); a1: y tile, then x1 = LN2(...).  With
// WRITE_OUT the tile is stored to P.out; otherwise it is left in a0, synchronised, for the
// caller (the next layer's pre body).
// The caller's requests for what follows this body ride on its last two products:
// `mid_begin()` / `mid_steps(ks)` around the feed-forward product's contraction steps and in its
// epilogue, `last_begin()` / `last_steps(ks)` around the last product's (ks = 0 .. kPoints-1 of
// the product's stream, see WeightStream::run).  The fused layer boundary requests the next
// layer's first two matrices there.  `after_first_requests()` runs behind the requests for W_o,
// which need nothing of P but w_o: a kernel that receives that pointer in a register waits for
// the rest of its arguments there.
template <typename T, int D, int F, int TR, bool WRITE_OUT, typename MidBegin, typename MidSteps, typename LastBegin,
          typename LastSteps, typename First = NoHook>
__device__ __forceinline__ void fused_post_body(const FusedPostParams &P, T *a0, T *a1, float *red_a, float *red_b,
                                                long row0, int valid, MidBegin mid_begin, MidSteps mid_steps,
                                                LastBegin last_begin, LastSteps last_steps, T *vecs, int vec_ld,
                                                int tile = -1, First after_first_requests = First{}) {
    typedef Tile<T, TR> TL;
    constexpr int NW = fused_waves(D), NT = NW * 64;
    constexpr int LDD = D + 8, LDF = F + 8;
    constexpr int NBD = fused_blocks<T, TR>(D, NW);
    constexpr int NBF = fused_blocks<T, TR>(F, NW);  // with fewer blocks than wavefronts the upper ones sit the product out
    constexpr int VB = TL::kVals, GB = TL::kGroups;
    static_assert(D % (TL::kBlock * NW) == 0 && F % TL::kBlock == 0, "unsupported widths");
    static_assert(F / TL::kBlock >= NW ? (F / TL::kBlock) % NW == 0 : true, "unsupported widths");
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = TL::token(lane), hb = TL::sub(lane);

    int nbd[NBD], nbf[NBF];
#pragma unroll
    for (int b = 0; b < NBD; ++b) nbd[b] = wave + NW * b;
#pragma unroll
    for (int b = 0; b < NBF; ++b) nbf[b] = wave + NW * b;
    const bool ff_active = wave < F / TL::kBlock;  // wavefront-uniform

    WeightStream<T, D, NBD, TR> w_o;
    WeightStream<T, D, NBF, TR> w_1;
    WeightStream<T, F, NBD, TR> w_2;
    // whole-matrix streams follow the request-on-arrival rule of WeightStream
    constexpr bool kWhole = WeightStream<T, D, NBD, TR>::kWhole && WeightStream<T, D, NBF, TR>::kWhole &&
                            WeightStream<T, F, NBD, TR>::kWhole;
    // prologue: everything this tile needs from memory is requested before anything is waited for;
    // the first weights travel while the partials are waited for, fetched and merged
    if (kWhole) w_o.start(static_cast<const T *>(P.w_o), nbd, lane, tile);
    after_first_requests();
    dma_tile<T, D, NT, TR>(a1, LDD, static_cast<const T *>(P.y) + row0 * P.ldy, P.ldy, valid, tid);
    if (!P.part_o)
        dma_tile<T, D, NT, TR>(a0, LDD, static_cast<const T *>(P.attn) + row0 * P.lda, P.lda, valid, tid);
    dma_vector<T, D, NT>(vecs + kVecG2 * vec_ld, P.g2, tid, 0);
    dma_vector<T, D, NT>(vecs + kVecB2 * vec_ld, P.b2, tid, 1);
    dma_vector<T, F, NT>(vecs + kVecBias1 * vec_ld, P.bias_1, tid, 2);
    dma_vector<T, D, NT>(vecs + kVecG3 * vec_ld, P.g3, tid, 3);
    dma_vector<T, D, NT>(vecs + kVecB3 * vec_ld, P.b3, tid, 4);
    dma_vector<T, D, NT>(vecs + kVecBias2 * vec_ld, P.bias_2, tid, 5);
    if (P.part_o) {
        // (The order of these requests was measured both other ways round — the partials in front
        // of the weights, the wait in front of everything: the compute unit's address unit is what
        // the prologue queues for, 16 clocks per 16-byte-per-lane request of a wavefront, and either
        // change makes the first product wait longer for its weights than it gains on the merge.)
        stage_merged_attention<T, D, NT, TR>(
            a0, LDD, P, row0, valid, tid,
            [&]() {
                if (P.order_wait) {  // the buffer pass's partial (the last slot) comes from the other queue
                    if (tid == 0) order_wait_device(P.order_wait, 0, P.order_limit);
                    __syncthreads();
                }
            },
            [&]() { if (kWhole && ff_active) w_1.begin(static_cast<const T *>(P.w_1), nbf, lane, tile); },
            [&](int u) { if (kWhole && ff_active) w_1.request_share(u, kMergeBatch); });
        if (!kWhole) {
            w_o.start(static_cast<const T *>(P.w_o), nbd, lane, tile);
            wait_all_loads();
        }
    } else {
        if (!kWhole) w_o.start(static_cast<const T *>(P.w_o), nbd, lane, tile);
        wait_all_loads();
        if (kWhole && ff_active) w_1.start(static_cast<const T *>(P.w_1), nbf, lane, tile);
    }
    __syncthreads();
    if (!kWhole && ff_active) w_1.start(static_cast<const T *>(P.w_1), nbf, lane, tile);

    // ---- x1 = LN2(y + attn W_o^T); each lane replaces exactly the y entries it read
    {
        float gam[NBD][VB], bet[NBD][VB];
        load_cols<T, NBD, TR>(vecs + kVecG2 * vec_ld, nbd, hb, gam);
        load_cols<T, NBD, TR>(vecs + kVecB2 * vec_ld, nbd, hb, bet);
        typename TL::acc_t acc[NBD];
        auto w2_steps = [&](int ks) { if (kWhole) w_2.request_share(ks, WeightStream<T, D, NBD, TR>::kPoints); };
        {   // W_o arrived with the prologue; W_1 is on its way and must not be waited for here
            WeightStream<T, D, NBD, TR> &w = w_o;
#pragma unroll
            for (int b = 0; b < NBD; ++b)
#pragma unroll
                for (int q = 0; q < TL::kVals; ++q) acc[b][q] = 0.f;
            // W_2 goes where W_o's fragments were, half of it step by step and half from the
            // epilogue: two matrices (W_1, W_2) are on their way while the row statistics are
            // exchanged, and the address unit has requests to accept while the wavefronts wait
            if (kWhole) w_2.begin(static_cast<const T *>(P.w_2), nbd, lane, tile);
            w.multiply(acc, a0, LDD, c, hb, w2_steps);
        }
        if (!kWhole) w_2.start(static_cast<const T *>(P.w_2), nbd, lane, tile);
        float v[NBD][VB];
#pragma unroll
        for (int b = 0; b < NBD; ++b)
#pragma unroll
            for (int g = 0; g < GB; ++g) {
                float r[4];
                load4f<T>(a1 + c * LDD + TL::col(nbd[b], g, hb), r);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[b][4 * g + e] = acc[b][4 * g + e] + r[e];
            }
        layer_norm_to_lds<T, NBD, NW, TR>(v, gam, bet, nbd, a1, LDD, red_a, red_b, wave, c, hb, D, P.eps2, [&](int e) {
            if (kWhole) WeightStream<T, D, NBD, TR>::tail_points(e, w2_steps);
        });
    }
    __syncthreads();  // x1 complete in a1; every wavefront is done reading a0

    // ---- h = gelu(x1 W_1^T + b_1)  -> a0
    if (ff_active) {
        float bias[NBF][VB];
        load_cols<T, NBF, TR>(vecs + kVecBias1 * vec_ld, nbf, hb, bias);
        typename TL::acc_t acc[NBF];
        w_1.run(acc, a1, LDD, c, hb, mid_begin, mid_steps);
        if (kWhole) WeightStream<T, D, NBF, TR>::tail_points(0, mid_steps);
#pragma unroll
        for (int b = 0; b < NBF; ++b) {
#pragma unroll
            for (int g = 0; g < GB; ++g) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float t = acc[b][4 * g + e] + bias[b][4 * g + e];
                    o[e] = 0.5f * t * (1.f + erff(t * 0.70710678118654752f));
                }
                store4f<T>(a0 + c * LDF + TL::col(nbf[b], g, hb), o[0], o[1], o[2], o[3]);
            }
            // the rest of the caller's requests between the blocks of the activation
            if (kWhole) {
                if (NBF == 1 || b == 0) WeightStream<T, D, NBF, TR>::tail_points(1, mid_steps);
                if (NBF == 1 || b == NBF / 2) WeightStream<T, D, NBF, TR>::tail_points(2, mid_steps);
                if (b == NBF - 1) WeightStream<T, D, NBF, TR>::tail_points(3, mid_steps);
            }
        }
    } else {  // a wavefront that sits the feed-forward product out still makes the caller's requests
        mid_begin();
#pragma unroll
        for (int ks = 0; ks < WeightStream<T, D, NBF, TR>::kPoints; ++ks) mid_steps(ks);
    }
    float gam[NBD][VB], bet[NBD][VB], bias[NBD][VB];
    load_cols<T, NBD, TR>(vecs + kVecG3 * vec_ld, nbd, hb, gam);
    load_cols<T, NBD, TR>(vecs + kVecB3 * vec_ld, nbd, hb, bet);
    load_cols<T, NBD, TR>(vecs + kVecBias2 * vec_ld, nbd, hb, bias);
    __syncthreads();

    // ---- out = LN3(x1 + h W_2^T + b_2), staged through a0 for row-contiguous stores
    {
        typename TL::acc_t acc[NBD];
        w_2.run(acc, a0, LDF, c, hb, last_begin, last_steps);
        float v[NBD][VB];
#pragma unroll
        for (int b = 0; b < NBD; ++b)
#pragma unroll
            for (int g = 0; g < GB; ++g) {
                float r[4];
                load4f<T>(a1 + c * LDD + TL::col(nbd[b], g, hb), r);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[b][4 * g + e] = acc[b][4 * g + e] + r[e] + bias[b][4 * g + e];
            }
        // every wavefront must be done with its last read of a0 (the product above) before the
        // result is written into it: the barrier inside the statistics orders exactly that
        layer_norm_to_lds<T, NBD, NW, TR>(v, gam, bet, nbd, a0, LDD, red_a, red_b, wave, c, hb, D, P.eps3, [&](int e) {
            if (kWhole) WeightStream<T, F, NBD, TR>::tail_points(e, last_steps);
        });
    }
    __syncthreads();
    if (WRITE_OUT) unstage_tile<T, D, NT, TR>(static_cast<T *>(P.out) + row0 * D, D, a0, LDD, valid, tid);
}

template <typename T, int D, int F, int TR>
__global__ __launch_bounds__(fused_waves(D) * 64) void fused_post_kernel(FusedPostParams P) {
    warm_kernel_arguments<sizeof(FusedPostParams)>();
    constexpr int NW = fused_waves(D), LDD = D + 8, LDF = F + 8, LDM = LDD > LDF ? LDD : LDF;
    __shared__ __attribute__((aligned(16))) T a0[TR * LDM];
    __shared__ __attribute__((aligned(16))) T a1[TR * LDD];
    __shared__ float red_a[NW * TR], red_b[NW * TR];
    const long row0 = static_cast<long>(blockIdx.x) * TR;
    const int valid = static_cast<int>(min(static_cast<long>(TR), P.rows - row0));
    constexpr int VW = D > F ? D : F;
    __shared__ __attribute__((aligned(16))) T vecs[kVecSlots * VW];
    fused_post_body<T, D, F, TR, true>(P, a0, a1, red_a, red_b, row0, valid, NoHook{}, NoHook{}, NoHook{}, NoHook{},
                                       vecs, VW);
}

// Body of a fetcher workgroup: reads its share of the matrices w[0 .. N-1] (kib[i] KiB each) once
// into `junk` (1 KiB of LDS that nobody reads), which brings their lines into the L2 of the XCD it
// runs on.  Share `part` of `n_parts`, dealt in pieces of 1 KiB over the wavefronts.
//
// Between the decode step's layer kernels the context pass streams its keys and values through the
// L2s, so a layer kernel finds its weights in the memory-side cache at best.  Its weight streams
// request a matrix one product ahead, which hides that latency only in part: at 2048 rows a
// product with its epilogue takes 1.5 us, 1.3 us with the lines in L2 and 1.0 us with them in the
// compute unit's own cache.  A launch that leaves compute units idle therefore carries extra
// workgroups, behind those that own rows, which do nothing but fetch; each XCD gets its own (ids
// are dealt round-robin over the 8 XCDs).  Fetching from the workgroups that own rows instead,
// ahead of their own requests, gains half as much: the prologue's requests are then accepted
// 0.8 us later, whether the extra loads touch one word per line or read whole lines.
template <int N, int NT>
__device__ __forceinline__ void fetch_weights_to_l2(const void *const (&w)[N], const int (&kib)[N], void *junk,
                                                    int part, int n_parts) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    int total = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) total += kib[i];
    for (int g = part * (NT / 64) + wave; g < total; g += n_parts * (NT / 64)) {
        const char *p = static_cast<const char *>(w[0]);
        int l = g;
#pragma unroll
        for (int i = 1; i < N; ++i) {
            if (l < kib[i - 1]) break;
            l -= kib[i - 1];
            p = static_cast<const char *>(w[i]);
        }
        load_to_lds_16(p + (static_cast<long>(l) << 10) + 16 * lane, junk);
    }
}

// The post part of layer L and the pre part of layer L+1 on the same rows: the layer output
// never leaves LDS, and one launch (with its fixed cost) disappears per layer boundary.
template <typename T, int D, int F, int TR>
__global__ __launch_bounds__(fused_waves(D) * 64) void fused_post_pre_kernel(const void *w_o, long rows,
                                                                              FusedPostParams P0, FusedPreParams N) {
    // w_o and rows (= P0.w_o, P0.rows) arrive in registers: the requests for the first matrix go
    // out while the rest of the arguments is on its way from memory
    KernelArgumentLines<16 + sizeof(FusedPostParams) + sizeof(FusedPreParams)> arguments;
    arguments.request();
    FusedPostParams P = P0;
    P.w_o = w_o;
    P.rows = rows;
    constexpr int NW = fused_waves(D), LDD = D + 8, LDF = F + 8, LDM = LDD > LDF ? LDD : LDF;
    __shared__ __attribute__((aligned(16))) T a0[TR * LDM];
    __shared__ __attribute__((aligned(16))) T a1[TR * LDD];
    __shared__ float red_a[NW * TR], red_b[NW * TR];
    const long row0 = static_cast<long>(blockIdx.x) * TR;
    if (row0 >= P.rows) {
        // a fetcher (see fetch_weights_to_l2): workgroup `part` of the `n_parts` fetchers of its XCD
        arguments.await();
        const int n_tiles = static_cast<int>((P.rows + TR - 1) / TR), xcd = blockIdx.x & 7;
        const int first = n_tiles + ((xcd - n_tiles) & 7);  // this XCD's first fetcher
        const int part = (static_cast<int>(blockIdx.x) - first) >> 3;
        const int n_parts = (static_cast<int>(gridDim.x) - first + 7) >> 3;
        constexpr int KD = sizeof(T) * D * D / 1024, KF = sizeof(T) * D * F / 1024;  // KiB per matrix
        const char *w_q = static_cast<const char *>(N.w_qkv);
        const void *const w[7] = {P.w_o, P.w_1, P.w_2, N.w_fo, w_q, w_q + sizeof(T) * D * D, w_q + 2 * sizeof(T) * D * D};
        const int kib[7] = {KD, KF, KF, KD, KD, KD, KD};
        fetch_weights_to_l2<7, NW * 64>(w, kib, a0, part, n_parts);
        wait_all_loads();  // the LDS they land in is this workgroup's until it ends
        return;
    }
    const int valid = static_cast<int>(min(static_cast<long>(TR), P.rows - row0));
    constexpr int NB = fused_blocks<T, TR>(D, NW);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int nblk[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) nblk[b] = wave + NW * b;
    WeightStream<T, D, NB, TR> next_fo, next_q;
    constexpr int VW = D > F ? D : F;
    __shared__ __attribute__((aligned(16))) T vecs[kVecSlots * VW];
    // Whole-matrix streams: the next layer's W_fo is requested during the feed-forward product and
    // its q weights during the last product.  Deeper ones: W_fo ahead of the last product, the q
    // weights by the pre body (the order that measured best for them).
    constexpr int NBF = fused_blocks<T, TR>(F, NW);
    constexpr bool kWhole = WeightStream<T, D, NB, TR>::kWhole && WeightStream<T, D, NBF, TR>::kWhole &&
                            WeightStream<T, F, NB, TR>::kWhole;
    const T *w_fo = static_cast<const T *>(N.w_fo), *w_q = static_cast<const T *>(N.w_qkv);
    fused_post_body<T, D, F, TR, false>(
        P, a0, a1, red_a, red_b, row0, valid,
        [&]() { if (kWhole) next_fo.begin(w_fo, nblk, lane); },
        [&](int ks) { if (kWhole) next_fo.request_share(ks, WeightStream<T, D, NBF, TR>::kPoints); },
        [&]() {
            if (kWhole)
                next_q.begin(w_q, nblk, lane);
            else
                next_fo.begin(w_fo, nblk, lane);
        },
        [&](int ks) {
            if (kWhole)
                next_q.request_share(ks, WeightStream<T, F, NB, TR>::kPoints);
            else
                next_fo.request_share(ks, WeightStream<T, F, NB, TR>::kPoints);
        },
        vecs, VW, -1,
        [&]() {
            arguments.await();
            stage_pre_vectors<T, D, NW * 64>(N, vecs, VW, threadIdx.x);  // visible after the body's first barrier
        });
    fused_pre_body<T, D, TR, true, kWhole>(N, a0, a1, red_a, red_b, row0, valid, next_fo, next_q, vecs, VW);
}

// ---- end of a decode step: final norm + mixture head + one sample per trajectory + the
// embedding of the next step's [buffer, target] rows, in one launch.
//
// Replaces, for dim_y = 1, the chain  backbone.norm -> head MLP -> mixture parameters ->
// component pick -> normal draw -> write the prediction -> embed (x_t, y_t) as the next buffer
// row and x_{t+1} as the next target row.  The uniform and normal variates come from the
// caller (one pair per trajectory and step), the step index from device memory, so that the
// whole sampling loop can be replayed from one recorded graph.
struct SampleEmbedParams {
    const void *x_last; long ld_row;  // target row of trajectory b at x_last + b * ld_row, [D]
    const void *norm_g, *norm_b; float eps;
    const void *w_h1, *b_h1;          // head layer 1: packed [F, D], [F]
    const void *w_h2, *b_h2;          // head layer 2 padded to 32 outputs: packed [32, F], [32]
    const void *mean_bias, *std_bias, *weight_bias;  // [K]
    int K; float std_min, std_max;
    const float *rand_u, *rand_n;     // [Nt, B] uniform [0,1) / standard normal
    const void *x_mean;               // [B, Nt] feature mean of every target row
    const void *w_x, *b_x, *w_y, *b_y;  // embedder: Linear(1, D) weights as [D] vectors
    const void *markers;              // [3, D]: target, context, buffer
    const void *ar_tokens; int bs;    // [bs, D]
    const int *step;                  // device-side index t of the target being sampled
    int Nt;
    void *preds;                      // [B, Nt]
    void *emb;                        // [B, 2, D] rows of step t + 1
    int B;
    int *advance; int n_advance;      // loop counters to increment once per launch, or nullptr
    unsigned *ticket;                 // zero between launches: counts finished workgroups
};

constexpr int kMaxMixture = 10;  // 3 * K outputs must fit one 32-column block

// What a thread of the step tail needs from memory for itself: its trajectory's variates (threads
// 0 .. valid-1), the feature means of the rows its embedding items cover, and one of the 3 K
// mixture biases (threads 0 .. 3K-1: mean, std, weight biases in turn).  Loaded as early as the
// caller can afford the registers; used late.
template <typename T, int N>
struct StepTailRegs {
    float u, n, xv[N];
    T mix;
};
template <int D, int TR, bool FUSED>
constexpr int step_tail_items() { return (FUSED ? TR / 2 : TR) * 2 * (D / 8) / (fused_waves(D) * 64); }

template <typename T, int D, int TR, bool FUSED>
__device__ __forceinline__ StepTailRegs<T, step_tail_items<D, TR, FUSED>()> load_step_tail_regs(
    const SampleEmbedParams &P, int t, long row0, int valid) {
    constexpr int NT = fused_waves(D) * 64, CPR_E = D / 8, N = step_tail_items<D, TR, FUSED>();
    const int tid = threadIdx.x;
    StepTailRegs<T, N> r;
    r.u = r.n = 0.f;
    if (tid < valid) {
        r.u = P.rand_u[static_cast<long>(t) * P.B + row0 + tid];
        r.n = P.rand_n[static_cast<long>(t) * P.B + row0 + tid];
    }
    const T *xm = static_cast<const T *>(P.x_mean);
    const int tn = min(t + 1, P.Nt - 1);
#pragma unroll
    for (int k = 0; k < N; ++k) {
        const int idx = tid + k * NT;
        const int which = (idx / CPR_E) & 1, row = idx / (2 * CPR_E);
        r.xv[k] = row < valid ? to_f32(xm[(row0 + row) * P.Nt + (which == 0 ? t : tn)]) : 0.f;
    }
    r.mix = from_f32<T>(0.f);
    if (tid < 3 * P.K) {
        const T *src = static_cast<const T *>(tid < P.K ? P.mean_bias : (tid < 2 * P.K ? P.std_bias : P.weight_bias));
        r.mix = src[tid % P.K];
    }
    return r;
}

// Body of the step tail on the TR-row tile of trajectories row0 .. row0 + valid - 1.
// Stand-alone (FUSED = false): the target rows are staged from P.x_last into a0 here and the
// head's first matrix is requested here.  FUSED: a finished, synchronised tile is already in a0
// (row stride D + 8), `w_1` has been requested by the caller when W1_REQUESTED, and the two
// embedded rows of trajectory r are also left in `x_next` (an LDS tile, row stride D + 8, rows
// 2 r and 2 r + 1; valid <= TR / 2 then) for the pre body that follows.  `before_draw` runs after
// the first head product: the place to request what the caller needs next.
// a0: z = norm(x_last) [TR, D + 8]; a1: gelu(head layer 1) [TR, F + 8].
template <typename T, int D, int F, int TR, bool FUSED, bool W1_REQUESTED = false, typename Hook = NoHook>
__device__ __forceinline__ void sample_embed_body(
    const SampleEmbedParams &P, int t, T *a0, T *a1, float (*raw_s)[33], float *y_s, T *mix_s, long row0, int valid,
    const StepTailRegs<T, step_tail_items<D, TR, FUSED>()> &regs,
    WeightStream<T, D, fused_blocks<T, TR>(F, fused_waves(D)), TR> &w_1, T *x_next = nullptr, int tile = -1,
    Hook before_draw = Hook{}, const T *mk_target = nullptr, const T *mk_buffer = nullptr, const T *token = nullptr) {
    typedef Tile<T, TR> TL;
    constexpr int NW = fused_waves(D), NT = NW * 64;
    constexpr int LDD = D + 8, LDF = F + 8;
    constexpr int NBF = fused_blocks<T, TR>(F, NW);
    constexpr int NB2 = 32 / TL::kBlock;  // the second head layer is padded to 32 outputs: first wavefront
    constexpr int VB = TL::kVals, GB = TL::kGroups;
    constexpr int EPL = D / 64;  // elements per lane of one row in the row-wise norm
    constexpr int ROWS = FUSED ? TR / 2 : TR;  // rows of the tile that can hold a trajectory
    static_assert(F / TL::kBlock >= NW ? (F / TL::kBlock) % NW == 0 : true, "unsupported widths");
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = TL::token(lane), hb = TL::sub(lane);

    int nbf[NBF];
#pragma unroll
    for (int b = 0; b < NBF; ++b) nbf[b] = wave + NW * b;
    int nb0[NB2];
#pragma unroll
    for (int b = 0; b < NB2; ++b) nb0[b] = b;
    const bool ff_active = wave < F / TL::kBlock;
    WeightStream<T, F, NB2, TR> w_2;
    if (!W1_REQUESTED && ff_active) w_1.start(static_cast<const T *>(P.w_h1), nbf, lane, tile);
    if (wave == 0) w_2.start(static_cast<const T *>(P.w_h2), nb0, lane, tile);
    // Everything small that a later phase reads from memory is requested here, in one round trip
    // with the weights and the input tile: fetched where it is used, each costs its phase (all far
    // shorter than a memory access) a round trip of its own.
    float gam[EPL], bet[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
        gam[e] = to_f32(static_cast<const T *>(P.norm_g)[lane * EPL + e]);
        bet[e] = to_f32(static_cast<const T *>(P.norm_b)[lane * EPL + e]);
    }
    float bias1[NBF][VB], bias2[NB2][VB];
    if (ff_active)
        load_cols<T, NBF, TR>(P.b_h1 ? static_cast<const T *>(P.b_h1) : reinterpret_cast<const T *>(kZeroVector), nbf,
                              hb, bias1);
    if (wave == 0)
        load_cols<T, NB2, TR>(P.b_h2 ? static_cast<const T *>(P.b_h2) : reinterpret_cast<const T *>(kZeroVector), nb0,
                              hb, bias2);
    const float my_u = regs.u, my_n = regs.n;  // this trajectory's variates (threads 0 .. valid-1)
    // the model vectors of the embedding: a thread handles the same 8 columns in every item
    constexpr int CPR_E = D / 8;
    const int ch_e = tid % CPR_E;
    static_assert(NT % CPR_E == 0, "a thread's embedding items share their column chunk");
    u32x4 e_wx, e_bx, e_wy, e_by, e_mb, e_mt, e_tok;
    {
        // (copies the caller may have staged already: the markers "target" and "buffer", the token)
        const T *tok = token ? token : static_cast<const T *>(P.ar_tokens) + static_cast<long>((t + 1) % P.bs) * D;
        const T *mkt = mk_target ? mk_target : static_cast<const T *>(P.markers);
        const T *mkb = mk_buffer ? mk_buffer : static_cast<const T *>(P.markers) + 2 * D;
        e_wx = *reinterpret_cast<const u32x4 *>(static_cast<const T *>(P.w_x) + 8 * ch_e);
        e_bx = *reinterpret_cast<const u32x4 *>(static_cast<const T *>(P.b_x) + 8 * ch_e);
        e_wy = *reinterpret_cast<const u32x4 *>(static_cast<const T *>(P.w_y) + 8 * ch_e);
        e_by = *reinterpret_cast<const u32x4 *>(static_cast<const T *>(P.b_y) + 8 * ch_e);
        e_mb = *reinterpret_cast<const u32x4 *>(mkb + 8 * ch_e);
        e_mt = *reinterpret_cast<const u32x4 *>(mkt + 8 * ch_e);
        e_tok = *reinterpret_cast<const u32x4 *>(tok + 8 * ch_e);
    }
    constexpr int E_ITEMS = step_tail_items<D, TR, FUSED>();  // (trajectory, row, 8-column chunk) items per thread
    static_assert(ROWS * 2 * CPR_E % NT == 0 && E_ITEMS >= 1, "whole embedding items per thread");
    // the mixture biases go through LDS: read from memory where they are used, the pick of the
    // component costs a round trip for the weight biases and another for the chosen mean and std
    if (tid < 3 * P.K) mix_s[(tid / P.K) * kMaxMixture + tid % P.K] = regs.mix;  // published by the barriers below
    if (!FUSED) {
        stage_tile<T, D, NT, TR>(a0, LDD, static_cast<const T *>(P.x_last) + row0 * P.ld_row, P.ld_row, valid, tid);
        __syncthreads();
    }

    // ---- z = LayerNorm(x_last), one wavefront per row, in place
    {
        for (int r = wave; r < ROWS; r += NW) {
            T *row = a0 + r * LDD + lane * EPL;
            float x[EPL], sum = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                x[e] = to_f32(row[e]);
                sum += x[e];
            }
            const float mean = wave_sum(sum) / D;
            float q = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) q += (x[e] - mean) * (x[e] - mean);
            const float rstd = rsqrtf(wave_sum(q) / D + P.eps);
#pragma unroll
            for (int e = 0; e < EPL; ++e) row[e] = from_f32<T>((x[e] - mean) * rstd * gam[e] + bet[e]);
        }
    }
    __syncthreads();

    // ---- h = gelu(z W_h1^T + b_h1) -> a1
    if (ff_active) {
        typename TL::acc_t acc[NBF];
        w_1.run(acc, a0, LDD, c, hb);
#pragma unroll
        for (int b = 0; b < NBF; ++b)
#pragma unroll
            for (int g = 0; g < GB; ++g) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = acc[b][4 * g + e] + bias1[b][4 * g + e];
                    o[e] = 0.5f * v * (1.f + erff(v * 0.70710678118654752f));
                }
                store4f<T>(a1 + c * LDF + TL::col(nbf[b], g, hb), o[0], o[1], o[2], o[3]);
            }
    }
    before_draw();
    __syncthreads();

    // ---- raw = h W_h2^T + b_h2 (32 output columns, first wavefront), kept in float32
    if (wave == 0) {
        typename TL::acc_t acc[NB2];
        w_2.run(acc, a1, LDF, c, hb);
#pragma unroll
        for (int b = 0; b < NB2; ++b)
#pragma unroll
            for (int g = 0; g < GB; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    raw_s[c][TL::col(b, g, hb) + e] = acc[b][4 * g + e] + bias2[b][4 * g + e];
    }
    __syncthreads();

    // ---- one sample per trajectory: component by inverse CDF of the softmax weights, then a normal
    if (tid < TR) {
        float y = 0.f;
        if (tid < valid) {
            const long row = row0 + tid;
            const T *mb = mix_s, *sb = mix_s + kMaxMixture, *wb = mix_s + 2 * kMaxMixture;
            float logit[kMaxMixture], mx = -INFINITY;
#pragma unroll
            for (int k = 0; k < kMaxMixture; ++k)
                if (k < P.K) {
                    logit[k] = raw_s[tid][3 * k + 2] + to_f32(wb[k]);
                    mx = fmaxf(mx, logit[k]);
                }
            float z = 0.f;
#pragma unroll
            for (int k = 0; k < kMaxMixture; ++k)
                if (k < P.K) {
                    logit[k] = expf(logit[k] - mx);
                    z += logit[k];
                }
            const float target = my_u * z;
            int comp = P.K - 1;
            float cum = 0.f;
            bool found = false;
#pragma unroll
            for (int k = 0; k < kMaxMixture; ++k)
                if (k < P.K) {
                    cum += logit[k];
                    if (!found && cum > target) {
                        comp = k;
                        found = true;
                    }
                }
            const float mean = raw_s[tid][3 * comp] + to_f32(mb[comp]);
            const float sraw = raw_s[tid][3 * comp + 1] + to_f32(sb[comp]);
            const float sp = sraw > 20.f ? sraw : log1pf(expf(sraw));
            const float sd = fminf(sp, P.std_max) + P.std_min;
            const T yr = from_f32<T>(mean + sd * my_n);
            static_cast<T *>(P.preds)[row * P.Nt + t] = yr;
            y = to_f32(yr);
        }
        y_s[tid] = y;
    }
    __syncthreads();

    // ---- embedding of step t + 1: row 0 = buffer(x_t, y_t) + ar_token[(t + 1) % bs], row 1 = target(x_{t+1})
    {
        float fwx[8], fbx[8], fwy[8], fby[8], fmb[8], fmt[8], ftk[8];
        unpack8<T>(e_wx, fwx); unpack8<T>(e_bx, fbx); unpack8<T>(e_wy, fwy); unpack8<T>(e_by, fby);
        unpack8<T>(e_mb, fmb); unpack8<T>(e_mt, fmt); unpack8<T>(e_tok, ftk);
#pragma unroll
        for (int k = 0; k < E_ITEMS; ++k) {
            const int idx = tid + k * NT;
            const int which = (idx / CPR_E) & 1, r = idx / (2 * CPR_E);
            if (r >= valid) continue;
            const long row = row0 + r;
            const float xv = regs.xv[k];
            float o[8];
            if (which == 0) {
                const float yv = y_s[r];
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = xv * fwx[e] + fbx[e] + yv * fwy[e] + fby[e] + fmb[e] + ftk[e];
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = xv * fwx[e] + fbx[e] + fmt[e];
            }
            u32x4 val = {pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3]), pack2<T>(o[4], o[5]), pack2<T>(o[6], o[7])};
            *reinterpret_cast<u32x4 *>(static_cast<T *>(P.emb) + (row * 2 + which) * D + 8 * ch_e) = val;
            if (FUSED) *reinterpret_cast<u32x4 *>(x_next + (2 * r + which) * LDD + 8 * ch_e) = val;
        }
    }
}

// The caller's loop counters: every workgroup read the step index when it started, so the one
// that takes the last ticket may move them on.
__device__ __forceinline__ void take_ticket(const SampleEmbedParams &P) {  // one thread of the workgroup
    __threadfence();
    if (atomicAdd(P.ticket, 1u) == gridDim.x - 1) {
        for (int i = 0; i < P.n_advance; ++i) P.advance[i] += 1;
        *P.ticket = 0u;
    }
}
__device__ __forceinline__ void advance_loop_counters(const SampleEmbedParams &P) {
    if (P.advance) {
        __syncthreads();
        if (threadIdx.x == 0) take_ticket(P);
    }
}

template <typename T, int D, int F, int TR>
__global__ __launch_bounds__(fused_waves(D) * 64) void sample_embed_kernel(SampleEmbedParams P) {
    warm_kernel_arguments<sizeof(SampleEmbedParams)>();
    constexpr int NW = fused_waves(D);
    constexpr int LDD = D + 8, LDF = F + 8;
    __shared__ __attribute__((aligned(16))) T a0[TR * LDD];  // z = norm(x_last)
    __shared__ __attribute__((aligned(16))) T a1[TR * LDF];  // gelu(head layer 1)
    __shared__ float raw_s[TR][33];
    __shared__ float y_s[TR];
    __shared__ T mix_s[3 * kMaxMixture];
    const int t = *P.step;
    if (t < 0 || t >= P.Nt) return;  // uniform over the grid
    const long row0 = static_cast<long>(blockIdx.x) * TR;
    const int valid = static_cast<int>(min(static_cast<long>(TR), P.B - row0));
    WeightStream<T, D, fused_blocks<T, TR>(F, NW), TR> w_1;
    const auto regs = load_step_tail_regs<T, D, TR, false>(P, t, row0, valid);
    sample_embed_body<T, D, F, TR, false>(P, t, a0, a1, raw_s, y_s, mix_s, row0, valid, regs, w_1);
    advance_loop_counters(P);
}

// ---- the whole boundary between two decode steps in one launch: the post part of the last
// layer on the target rows, the step tail above, and the pre part of the first layer on the
// rows it has just embedded.  A workgroup owns TR / 2 trajectories: their target rows fill half
// a tile in the first two parts, their [buffer, target] rows of the next step the whole tile in
// the third.  Row for row the arithmetic (and, through the `tile` argument of the weight
// streams, its order) is that of fused_post_kernel, sample_embed_kernel and fused_pre_kernel
// launched one after the other; what disappears is two launches, the store and reload of the
// layer output and of the embedding, and two first round trips to memory.
// P: rows = trajectories (their target rows), `out` unused.  S: x_last unused.  N: x unused,
// rows = 2 * trajectories.  The head's hidden width equals the layers' feed-forward width F.
template <typename T, int D, int F, int TR>
__global__ __launch_bounds__(fused_waves(D) * 64) void decode_step_boundary_kernel(FusedPostParams P,
                                                                                    SampleEmbedParams S,
                                                                                    FusedPreParams N) {
    warm_kernel_arguments<sizeof(FusedPostParams) + sizeof(SampleEmbedParams) + sizeof(FusedPreParams)>();
    constexpr int TJ = TR / 2;
    constexpr int NW = fused_waves(D), LDD = D + 8, LDF = F + 8, LDM = LDD > LDF ? LDD : LDF;
    __shared__ __attribute__((aligned(16))) T a0[TR * LDM];
    __shared__ __attribute__((aligned(16))) T a1[TR * LDM];
    __shared__ float red_a[NW * TR], red_b[NW * TR];
    __shared__ float raw_s[TR][33];
    __shared__ float y_s[TR];
    constexpr int VW = D > F ? D : F;
    __shared__ __attribute__((aligned(16))) T vecs[kVecSlots * VW];
    const int t = *S.step;
    if (t < 0 || t >= S.Nt) return;  // uniform over the grid
    const long row0 = static_cast<long>(blockIdx.x) * TJ;
    const int valid = static_cast<int>(min(static_cast<long>(TJ), static_cast<long>(S.B) - row0));
    // tiles of the stand-alone launches that hold these rows
    const int tile_t = static_cast<int>(row0 / TR), tile_n = static_cast<int>(blockIdx.x);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int NB = fused_blocks<T, TR>(D, NW), NBF = fused_blocks<T, TR>(F, NW);
    int nblk[NB], nbf[NBF];
#pragma unroll
    for (int b = 0; b < NB; ++b) nblk[b] = wave + NW * b;
#pragma unroll
    for (int b = 0; b < NBF; ++b) nbf[b] = wave + NW * b;
    const bool head_active = wave < F / Tile<T, TR>::kBlock;
    WeightStream<T, D, NBF, TR> w_h1;
    WeightStream<T, D, NB, TR> next_fo, next_q;
    stage_pre_vectors<T, D, NW * 64>(N, vecs, VW, threadIdx.x);  // visible after the first barrier below
    // whole-matrix streams: the head's first matrix is requested during the feed-forward product
    constexpr bool kWhole = WeightStream<T, D, NB, TR>::kWhole && WeightStream<T, D, NBF, TR>::kWhole &&
                            WeightStream<T, F, NB, TR>::kWhole;
    // What the tail needs from memory is requested now, next to the post part's own prologue,
    // and lands in LDS (vectors) or in a few registers (per-thread scalars): requested where the
    // tail uses it, each item would cost a round trip between two phases that take far less.
    __shared__ __attribute__((aligned(16))) T hvec[8 * D + F + 32];  // norm g, b; x/y embedding w, b; markers target, buffer; token; head biases
    __shared__ T mix_s[3 * kMaxMixture];
    T *const h_g = hvec, *const h_b = hvec + D, *const h_wx = hvec + 2 * D, *const h_bx = hvec + 3 * D,
             *const h_wy = hvec + 4 * D, *const h_by = hvec + 5 * D, *const h_mk = hvec + 6 * D,
             *const h_tok = hvec + 7 * D, *const h_b1 = hvec + 8 * D, *const h_b2 = hvec + 8 * D + F;
    {
        constexpr int NT = NW * 64;
        const int tid = threadIdx.x;
        const T *mk = static_cast<const T *>(S.markers);
        dma_vector<T, D, NT>(h_g, S.norm_g, tid, 0);
        dma_vector<T, D, NT>(h_b, S.norm_b, tid, 1);
        dma_vector<T, D, NT>(h_wx, S.w_x, tid, 2);
        dma_vector<T, D, NT>(h_bx, S.b_x, tid, 3);
        dma_vector<T, D, NT>(h_wy, S.w_y, tid, 4);
        dma_vector<T, D, NT>(h_by, S.b_y, tid, 5);
        dma_vector<T, D, NT>(h_mk, mk, tid, 6);  // marker "target"
        dma_vector<T, D, NT>(h_tok, static_cast<const T *>(S.ar_tokens) + static_cast<long>((t + 1) % S.bs) * D, tid, 7);
        dma_vector<T, F, NT>(h_b1, S.b_h1, tid, 0);
        dma_vector<T, 32, NT>(h_b2, S.b_h2, tid, 1);
    }
    __shared__ __attribute__((aligned(16))) T h_mkb[D];
    dma_vector<T, D, NW * 64>(h_mkb, static_cast<const T *>(S.markers) + 2 * D, threadIdx.x, 2);
    const auto regs = load_step_tail_regs<T, D, TR, true>(S, t, row0, valid);
    const T *w_h1p = static_cast<const T *>(S.w_h1);
    fused_post_body<T, D, F, TR, false>(
        P, a0, a1, red_a, red_b, row0, valid,
        [&]() { if (kWhole && head_active) w_h1.begin(w_h1p, nbf, lane, tile_t); },
        [&](int ks) { if (kWhole && head_active) w_h1.request_share(ks, WeightStream<T, D, NBF, TR>::kPoints); },
        NoHook{}, NoHook{}, vecs, VW, tile_t);
    SampleEmbedParams S2 = S;  // the same tail, its small operands read from their LDS copies
    S2.norm_g = h_g; S2.norm_b = h_b; S2.w_x = h_wx; S2.b_x = h_bx; S2.w_y = h_wy; S2.b_y = h_by;
    S2.b_h1 = h_b1; S2.b_h2 = h_b2;
    sample_embed_body<T, D, F, TR, true, kWhole>(
        S2, t, a0, a1, raw_s, y_s, mix_s, row0, valid, regs, w_h1, a0, tile_t,
        [&]() {
            next_fo.start(static_cast<const T *>(N.w_fo), nblk, lane, tile_n);
            if (kWhole) next_q.start(static_cast<const T *>(N.w_qkv), nblk, lane, tile_n);
            // Every wavefront has read the step index (barriers of the post part lie behind it) and
            // the buffer passes of this step, which read the buffer length, were waited for inside
            // the post part: the loop counters may move on.  The last wavefront has nothing to do
            // until the embedding: it takes the workgroup's ticket.
            if (S.advance && threadIdx.x == NW * 64 - 1) take_ticket(S);
        },
        h_mk, h_mkb, h_tok);
    __syncthreads();  // the embedded rows are complete in a0
    fused_pre_body<T, D, TR, true, kWhole>(N, a0, a1, red_a, red_b, 2 * row0, 2 * valid, next_fo, next_q, vecs, VW,
                                           tile_n);
}

}  // namespace artab
