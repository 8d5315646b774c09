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
//     O^T[d,  q] = V^T[d, kv] . P^T[kv, q]   (A = V^T from LDS,    B = P in registers)
// With v_mfma_f32_32x32x16 a lane (c = lane % 32, hb = lane / 32) owns query
// column c and, in accumulator register v = 4g + r, row 8g + 4hb + r.  The 16
// scores a lane holds for one 32-key block are therefore keys {8g + 4hb + r};
// used directly as the B operand of the second product this enumerates the
// contraction index as e = 4(g mod 2) + r per 16-wide step t = g / 2.  V stays
// row-major in LDS; ds_read_b64_tr_b16 (the CDNA4 transposing LDS read) hands
// each lane the four keys {base + r} of one output dimension, so two such reads
// give the matching A operand for step t without any shuffling.
//
// Softmax.  Q is pre-multiplied by scale*log2(e) and rounded to the input type
// (the rounding model of the reference kernel, triton_kernels.py:120-121), so
// p = 2^s needs no multiply.  The fast path subtracts no running maximum at all:
// float32 holds 2^s for |s| < 126, bf16 keeps that exponent range, and the
// accumulators are float32.  A row whose probability mass leaves [2^-100, 2^100]
// (or any NaN/inf) makes the whole workgroup redo its tile range with the
// classical online-softmax (running maximum, rescaled accumulators); fp16, whose
// exponent range is too small for the fast path, always takes that robust path.
#pragma once

#include <type_traits>

#include "common.h"

namespace artab {

typedef short s16x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct MfmaOps;

template <>
struct MfmaOps<bf16_t> {
    typedef bf16x8 vec;
    static constexpr bool kWideExponent = true;
    static constexpr unsigned kOnes2 = 0x3f803f80u;  // (1, 1) packed
    static __device__ __forceinline__ f32x16 mma(vec a, vec b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mma16(vec a, vec b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
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
    static constexpr bool kWideExponent = false;
    static constexpr unsigned kOnes2 = 0x3c003c00u;  // (1, 1) packed
    static __device__ __forceinline__ f32x16 mma(vec a, vec b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mma16(vec a, vec b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(unsigned packed, float acc) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), __builtin_bit_cast(f16x2, 0x3c003c00u),
                                      acc, false);
    }
};

enum FlashMode : int { kFlashContext = 0, kFlashTeacher = 1, kFlashPrefill = 2, kFlashRowMask = 3 };

// The leading, scalar arguments of the kernel, which the command processor places in registers
// before the first instruction runs (the unit is compiled with -amdgpu-kernarg-preload-count=8):
// what a plain context launch over one shared context needs to request its first K/V tiles.
// sn == 0: no early requests (several context groups, K and V laid out differently, strides beyond
// 32 bits, any other mode); the kernel then works from FlashParams alone.
struct FlashEarly {
    const char *k, *v;   // kc.p, vc.p
    int sh, sn;          // head and row stride of both, in elements
    int kv_per_split, nc;
    int n_kvg;           // H (one group)
    int block0;          // = FlashParams::kvg_block0; bit 30 (kFlashStampedBit) set: FlashParams::stamps is set
};
constexpr int kFlashStampedBit = 1 << 30;

struct FlashParams {
    View q, kc, vc, kb, vb, out;
    View kcache, vcache;
    int cache_batches;
    float *lse;       // [B,H,Lq] final log-sum-exp (natural log) or nullptr
    void *part_o;     // split partials: [n_split][B*H*Lq][DH] normalised, in the input type (the
                      // reference merges partial outputs of the input type too, triton_kernels.py:478-524)
    float *part_lse;  // [n_split][B*H*Lq] natural log
    int B, H, Lq;
    int Nc, Nb, Nt;
    int G;                // query rows per group (B*Lq stacked, or Lq per batch entry)
    int tiles_per_group;  // ceil(G / BM)
    int n_groups;         // 1 (stacked) or B
    int n_split, kv_per_split;
    float qscale;  // softmax scale * log2(e), folded into Q
    int mode;
    int rm_nc, rm_attend;  // row-mask mode: context rows in front of the Nb buffer rows, attending chunks
    int force_robust;  // 1: skip the fast path (testing the online-softmax path)
    // A buffer pass runs beside this launch on the same compute units and streams `beside_rows`
    // rows per pair (read from device memory, or `beside_n` when the pointer is null).  From
    // `dense_below` rows on the context pass leaves the straight-line form of its tile loop alone
    // (0: no limit): measured at B=1024, H=8, N_ctx=16384 the straight-line form is 3 % faster alone
    // and worth 1.9 % of a decode step beside a short buffer pass; beside a long one the context
    // pass waits for its tiles behind the streaming loads either way and the denser issue only
    // takes slots from the buffer pass (256 steps: +0.3 % with the limit at 128 rows, 0 without).
    const int *beside_rows;
    int beside_n, dense_below;
    int yield_from;  // rows of the neighbouring buffer pass from which this pass lowers its wave priority (0: never)
    unsigned *started;  // optional counter that the first thread of the grid advances at once: "the
                        // launches ahead of this one on its queue are complete" for a watcher on
                        // another queue (queue_order.h); the kernel's own work does not depend on it
    // Benchmark builds only (null otherwise): time stamps of this launch from the 100 MHz wall
    // clock.  stamps[0] counts finished launches and names this launch's record, stamps[1] is the
    // ticket of the workgroups that have finished, stamps[2] collects the earliest start of the
    // launch under way, records start at stamps[4]: (earliest start, end of the last workgroup).
    // Launches that share the array must not overlap in time (they are launches of one queue).
    unsigned long long *stamps;
    int stamps_capacity;
    int kvg_block0;  // first block of eight (group, head) pairs of this launch (grid.z counts from here)
};

// Reading the wall clock is a request to one unit of the chip: a launch in which every wavefront
// reads it is several microseconds longer (measured: 4608 reads, +13 us on a 43 us launch).  So
// few do: the first wavefront of the first kStampStarters workgroups at the start (the earliest of
// them is the launch's start; workgroups are started in order), and the workgroup that takes the
// last ticket at the end (it is the last to finish by definition).
constexpr unsigned kStampStarters = 16;

// `t_entry`: the clock as the workgroup read it with its first instructions (a stamped launch says
// so in its leading arguments, see FlashEarly::block0), or 0.
__device__ __forceinline__ void flash_stamp_start(const FlashParams &P, unsigned long long t_entry) {  // first thread of a workgroup
    if (P.stamps && blockIdx.x < kStampStarters && blockIdx.y == 0 && blockIdx.z == 0)
        __hip_atomic_fetch_min(&P.stamps[2], t_entry ? t_entry : wall_clock64(), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
}

// First thread of a workgroup that is done.  Relaxed throughout: every access to the array is an
// atomic at agent scope (they execute in the L2 / memory side, in order per address), and the next
// reader is the next launch of the queue or the host after a synchronisation; an acquire/release
// here would write back and invalidate the L2 once per workgroup.
__device__ __forceinline__ void flash_stamp_end(const FlashParams &P) {
    const unsigned long long t =
        __hip_atomic_fetch_add(&P.stamps[1], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (t != static_cast<unsigned long long>(gridDim.x) * gridDim.y * gridDim.z - 1) return;
    const unsigned long long t1 = wall_clock64();
    const unsigned long long n = __hip_atomic_load(&P.stamps[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long t0 =
        __hip_atomic_exchange(&P.stamps[2], ~0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (n < static_cast<unsigned long long>(P.stamps_capacity)) {
        __hip_atomic_store(&P.stamps[4 + 2 * n], t0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&P.stamps[5 + 2 * n], t1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __hip_atomic_store(&P.stamps[1], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&P.stamps[0], n + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Probability mass (sum of 2^s over a row) the fast path accepts.
constexpr float kFastMassMax = 1.2676506e30f;  // 2^100
constexpr float kFastMassMin = 7.8886091e-31f; // 2^-100

// Largest / smallest teacher-forcing key limit over query rows [a, b] (inclusive).
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

template <bool V>
struct BoolTag {
    static constexpr bool value = V;
};

// LEAN selects the fast pass: false = the software-pipelined loop (two wavefronts per SIMD, 216
// registers), true = the plain loop built for four wavefronts per SIMD (see lean_pass).
// OCC: wavefronts per SIMD the register allocation is held to (1 = no constraint).
// PLAIN: the launch is a context pass (P.mode == kFlashContext): no buffer keys, no masks, no
// cache write — none of their state is computed or kept, which the 96-register form of the
// decode launch would otherwise park in scratch memory (60 bytes per lane, written by every
// wavefront whatever the mode).
template <typename T, int DH, int QB, int NW, int BN, bool LEAN = false, int OCC = 1, bool PLAIN = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
void flash_kernel(const char *early_k, const char *early_v, int early_sh, int early_sn, int early_kvps, int early_nc,
                  int early_nkvg, int early_block0, FlashParams P) {
    // The leading arguments arrive in registers (FlashEarly); the struct is on its way from memory.
    KernelArgumentLines<sizeof(FlashEarly) + sizeof(FlashParams)> arguments;
    arguments.request();
    typedef MfmaOps<T> Ops;
    typedef typename Ops::vec vec;
    constexpr int KS = DH / 16;
    constexpr int DB = DH / 32;
    constexpr int SB = BN / 32;
    constexpr int KPAD = DH + 8;   // K rows: 16-byte reads by 8 consecutive lanes hit 8 distinct bank groups
    constexpr int VPAD = DH + 16;  // V rows: row stride = 32 or 96 bytes mod 128 for the transposing reads
    constexpr int NT = NW * 64;
    constexpr int ROWS_W = 32 * QB;
    constexpr int BM = NW * ROWS_W;
    constexpr int CHUNKS = BN * DH / 8;  // 16-byte pieces of a K (or V) tile
    constexpr int NCH = (CHUNKS + NT - 1) / NT;
    constexpr int CPR = DH / 8;  // chunks per row

    // three stages; a stage is the K tile followed by the V tile, so that both have the same
    // stage stride and a stage index folds into the immediate offset of every LDS access
    constexpr int STAGE = BN * KPAD + BN * VPAD;
#ifndef ARTAB_LEAN_STAGES
#define ARTAB_LEAN_STAGES 4
#endif
    constexpr int NST = LEAN ? ARTAB_LEAN_STAGES : 3;  // stages: tiles are requested NST - 1 ahead at most
    // The lean pass keeps its tiles unpadded, as 1 KiB chunks in the order the operand reads want
    // them (see lean_pass): a stage is BN * DH elements of K and as many of V.  The robust pass,
    // which may follow it in the same launch, needs two stages of the padded layout.
    constexpr int LSTAGE = 2 * BN * DH;
    constexpr int LDS_ELEMS = LEAN ? (NST * LSTAGE > 2 * STAGE ? NST * LSTAGE : 2 * STAGE) : NST * STAGE;
    __shared__ __attribute__((aligned(1024))) T kv_lds[LDS_ELEMS];
    auto k_stage = [&](int st_) -> T * { return kv_lds + st_ * STAGE; };
    auto v_stage = [&](int st_) -> T * { return kv_lds + st_ * STAGE + BN * KPAD; };
    __shared__ int redo_flag;
    __shared__ int wg_lims[NW];

    // (release: whatever this queue's earlier launches wrote is visible to the watcher that sees
    // the new count)
    const int tid = threadIdx.x;
    // wavefront index as a scalar: everything derived from it (the wavefront's rows, its
    // teacher-forcing key limits) then steers scalar branches instead of exec-mask ones
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;

    // ---- direct loads of the lean pass.  In its steady state the tiles do not pass through
    // registers at all: a stage is NI chunks of one KiB, each filled by one direct global->LDS
    // load (lane l lands at base + 16 l; the lane's source address is whatever piece of the tile
    // belongs there), dealt over the wavefronts.  The loads are inline assembly: the compiler does
    // not know of them and therefore does not drain them in front of every LDS read; they are
    // waited for by hand (vmcnt) in front of the barrier that publishes their stage.
    constexpr int STAGE_BYTES = LSTAGE * static_cast<int>(sizeof(T));
    constexpr int NI = STAGE_BYTES / 1024, NKI = NI / 2;
    static_assert(STAGE_BYTES % 2048 == 0, "a stage is whole chunks of K and as many of V");
    constexpr int NR = (NI + NW - 1) / NW;
    static_assert(!LEAN || NR <= 2, "at most two direct loads per wavefront and tile");
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(kv_lds));
    unsigned d_off[NR];    // this lane's byte offset inside a tile
    const char *d_src[NR]; // the next tile to request (scalar)
    long d_step[NR];       // bytes from one tile to the next
    int n_dma = 0;         // direct loads this wavefront issues per tile
#pragma unroll
    for (int r = 0; r < NR; ++r)
        if (wave + NW * r < NI) ++n_dma;
    // chunk i of a stage (K chunks, then V chunks) of a source with row stride sn
    auto direct_load_lane = [&](int i, long sn, unsigned &off, long &step) {
        const bool is_v = i >= NKI;
        const int ch = i - (is_v ? NKI : 0);  // (sb, 16-column step) of the chunk
        const int sbk = ch / KS, cs = ch % KS;
        // lane l holds 16 bytes: K chunk [hb = l/32][key l%32], V chunk [key l/2][half l%2]
        const int row = 32 * sbk + (is_v ? lane / 2 : lane % 32);
        const int col = 16 * cs + 8 * (is_v ? lane % 2 : lane / 32);
        off = static_cast<unsigned>((row * sn + col) * static_cast<long>(sizeof(T)));
        step = static_cast<long>(BN) * sn * static_cast<long>(sizeof(T));
    };
    auto dma_tile = [&](auto stage_) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int i = wave + NW * r;
            if (i < NI) {
                const unsigned m0v = lds_base + stage_ * STAGE_BYTES + i * 1024;
                unsigned m0_saved;  // M0 (the LDS base of a direct load) is left as it was found
                asm volatile(
                    "s_mov_b32 %0, m0\n\t"
                    "s_mov_b32 m0, %1\n\t"
                    "global_load_lds_dwordx4 %2, %3\n\t"
                    "s_mov_b32 m0, %0"
                    : "=&s"(m0_saved)
                    : "s"(m0v), "v"(d_off[r]), "s"(d_src[r]));
            }
            d_src[r] += d_step[r];
        }
    };
    // The plain context launch requests its first NST - 1 tiles right here, from the arguments that
    // arrived in registers: the tiles travel while the argument struct is fetched and the rest of
    // the prologue (a chain of scalar loads and branches, about a microsecond) runs.
    bool early_tiles = false;
    unsigned long long t_entry = 0;  // a stamped launch starts its clock here, not behind the arguments' arrival
    if ((early_block0 & kFlashStampedBit) && blockIdx.x < kStampStarters && blockIdx.y == 0 && blockIdx.z == 0 &&
        wave == 0)
        t_entry = wall_clock64();
    if constexpr (LEAN && PLAIN) {
        if (early_sn > 0) {
            const int kvg_e = __builtin_amdgcn_readfirstlane(
                ((early_block0 & ~kFlashStampedBit) + static_cast<int>(blockIdx.z)) * 8 + (blockIdx.x & 7));
            const int begin_e = __builtin_amdgcn_readfirstlane(blockIdx.x >> 3) * early_kvps;
            const int end_e = min(early_nc, begin_e + early_kvps);
            if (kvg_e < early_nkvg && (end_e - begin_e) / BN >= NST - 1) {
                early_tiles = true;
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    const int i = wave + NW * r;
                    direct_load_lane(i, early_sn, d_off[r], d_step[r]);
                    d_src[r] = (i >= NKI ? early_v : early_k) +
                               (static_cast<long>(kvg_e) * early_sh + static_cast<long>(begin_e) * early_sn) *
                                   static_cast<long>(sizeof(T));
                }
                dma_tile(std::integral_constant<int, 0>{});
                dma_tile(std::integral_constant<int, 1>{});
#pragma unroll
                for (int t = 2; t < NST - 1; ++t) dma_tile(t);
            }
        }
    }
    arguments.await();

    if (LEAN && threadIdx.x == 0) redo_flag = 0;  // raised after the pass, at least one barrier later
    if (P.started && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
        __hip_atomic_fetch_add(P.started, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    if (threadIdx.x == 0) flash_stamp_start(P, t_entry);

    // ---- workgroup -> (kv-sharing group, q tile, context split).  The grid is three-dimensional
    // so that none of this takes an integer division (three of them were 0.4 us of every launch):
    // x = xcd + 8 * split, y = q tile, z = block of eight (group, head) pairs.  XCD-aware: the
    // hardware deals workgroups round-robin over the 8 XCDs in the order x, y, z, and grid.x is a
    // multiple of 8, so all workgroups that stream the same K/V (same pair, any tile and split)
    // run on the XCD `x mod 8` and share its L2.
    const int n_kvg = P.H * P.n_groups;
    const int xcd = blockIdx.x & 7;
    const int split = __builtin_amdgcn_readfirstlane(blockIdx.x >> 3);
    const int tile = __builtin_amdgcn_readfirstlane(blockIdx.y);
    const int kvg = __builtin_amdgcn_readfirstlane((P.kvg_block0 + static_cast<int>(blockIdx.z)) * 8 + xcd);
    if (kvg >= n_kvg) {
        if (P.stamps && threadIdx.x == 0) flash_stamp_end(P);
        return;
    }
    int h_ = kvg, g_ = 0;
    if (P.n_groups != 1) {  // (a branch, not a select: the shared-context launches skip the division)
        h_ = kvg % P.H;
        g_ = kvg / P.H;
    }
    // scalars by construction; said explicitly because base addresses built from them are scalar
    // operands of the direct-to-LDS loads
    const int h = __builtin_amdgcn_readfirstlane(h_), g = __builtin_amdgcn_readfirstlane(g_);
    const long kvb = P.n_groups == 1 ? 0 : g;  // batch entry whose K/V this group reads

    const int c = lane & 31, hb = lane >> 5;
    const int row0_wg = tile * BM;
    const int row0_w = row0_wg + wave * ROWS_W;

    // ---- Q fragments (B operand of S^T), pre-scaled by scale*log2e.
    // The loads are only requested here; they are scaled into qreg once the first K/V tiles have
    // been requested too, so that the kernel's first memory round trips overlap.
    vec qreg[QB][KS];
    int qi[QB];  // query index i within its batch entry, or -1
    // Batch entry b and index i of the query in column `col` (0..31) of block j of this wavefront;
    // false beyond the last row.  The epilogue asks again (with a column the compiler cannot
    // trace back to the lane index) instead of keeping addresses alive across the key loop.
    auto query_of = [&](int j, int col, long &b, int &i) {
        const int r = row0_w + 32 * j + col;
        const bool valid = r < P.G;
        const long flat = static_cast<long>(g) * P.G + (valid ? r : 0);
        if (P.Lq == 1) {  // decode: no 64-bit division on the way to the first load
            b = flat; i = 0;
        } else if (P.Lq == 2) {
            b = flat >> 1; i = static_cast<int>(flat & 1);
        } else {
            b = flat / P.Lq; i = static_cast<int>(flat % P.Lq);
        }
        return valid;
    };
#pragma unroll
    for (int j = 0; j < QB; ++j) {
        int i;
        long b;
        const bool valid = query_of(j, c, b, i);
        qi[j] = valid ? i : -1;
    }
    // Raw query fragments of this lane, and their scaled, rounded form in qreg.  `ln` is the lane
    // index: a pass that may run after the key loop (the robust one) hands it over as a value the
    // compiler cannot trace, so that rows and addresses are worked out afresh there instead of
    // staying live (parked in scratch memory at this register budget) across the loop.
    auto request_q = [&](u32x4(&qraw)[QB][KS], int ln) {
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            long b;
            int i;
            const bool valid = query_of(j, ln & 31, b, i);
            const T *qrow = view_row<T>(P.q, b, h, valid ? i : 0) + 8 * (ln >> 5);
#pragma unroll
            // unconditional: a column past the last row re-reads the group's first row (a valid
            // address) and is zeroed when it is scaled.  A load under a lane mask, merged with
            // zeros, made the compiler wait for the queries right here, a memory round trip in
            // front of the first tile requests.
            for (int ks = 0; ks < KS; ++ks) qraw[j][ks] = *reinterpret_cast<const u32x4 *>(qrow + 16 * ks);
        }
    };
    bool q_scaled = false;
    auto scale_q = [&](const u32x4(&qraw)[QB][KS], int ln) {
        q_scaled = true;
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            // columns past the last row carry zero queries
            const float qs = row0_w + 32 * j + (ln & 31) < P.G ? P.qscale : 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                u32x4 sc;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    sc[e] = pack2<T>(unpack_lo<T>(qraw[j][ks][e]) * qs, unpack_hi<T>(qraw[j][ks][e]) * qs);
                qreg[j][ks] = __builtin_bit_cast(vec, sc);
            }
        }
    };

    // ---- prefill: this tile's own K/V rows go to the cache.
    if (!PLAIN && P.mode == kFlashPrefill && P.kcache.p && g < P.cache_batches) {
        int nrows = min(BM, P.G - row0_wg);
        for (int idx = tid; idx < nrows * CPR; idx += NT) {
            int rr = row0_wg + idx / CPR, ch = idx % CPR;
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
    int lim[QB];  // per-lane visible buffer keys
    int wave_lim_min = 0, wave_lim_max = 0;
#pragma unroll
    for (int j = 0; j < QB; ++j) lim[j] = 0;
    if (!PLAIN && P.mode == kFlashTeacher) {
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
    } else if (!PLAIN && P.mode == kFlashRowMask) {
        // the limit is not monotone in the row here (targets count modulo Nb): the wavefront's and
        // the workgroup's bounds come from reductions over the rows' own limits
        int lo = P.Nb, hi = 0;
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            lim[j] = qi[j] >= 0 ? min(P.Nb, row_mask_limit(qi[j], P.rm_nc, P.Nb, P.rm_attend)) : 0;
            lo = min(lo, lim[j]);
            hi = max(hi, lim[j]);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            lo = min(lo, __shfl_xor(lo, o, 64));
            hi = max(hi, __shfl_xor(hi, o, 64));
        }
        wave_lim_min = __builtin_amdgcn_readfirstlane(lo);
        wave_lim_max = __builtin_amdgcn_readfirstlane(hi);
        if (lane == 0) wg_lims[wave] = wave_lim_max;
        __syncthreads();
        int wg_max = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) wg_max = max(wg_max, wg_lims[w]);
        buf_tiles = (wg_max + BN - 1) / BN;
    }
    const int n_tiles = ctx_tiles + buf_tiles;

    // ---- staging: global -> registers -> LDS.  Each thread owns NCH 16-byte chunks
    // (row st_row, column st_col) of the K tile and the same of V; their global
    // addresses are kept as running pointers that advance by one tile per fetch.
    // (In the lean form these tiles are the rare ones — a ragged last tile, buffer tiles under a
    // mask —, so the chunk's place is worked out where it is needed, from a thread index the
    // compiler cannot trace, instead of sitting in registers through the steady loop.)
    auto st_row = [&](int x) { return ((LEAN ? opaque(tid) : tid) + x * NT) / CPR; };
    auto st_col = [&](int x) { return (((LEAN ? opaque(tid) : tid) + x * NT) % CPR) * 8; };
    u32x4 kst[NCH], vst[NCH];
    const T *kp[NCH], *vp[NCH];
    long k_step = 0, v_step = 0;  // elements per tile
    int fetch_rows_left = 0;      // rows of the current segment from the next tile to fetch

    // Point the running pointers at tile `it` (first tile of the context slice or of
    // the buffer segment).
    auto seek = [&](int it) {
        const bool is_ctx = it < ctx_tiles;
        const View &ks_ = is_ctx ? P.kc : P.kb;
        const View &vs_ = is_ctx ? P.vc : P.vb;
        const long bb = is_ctx ? kvb : g;
        const int kv0 = is_ctx ? ctx_begin + it * BN : (it - ctx_tiles) * BN;
        fetch_rows_left = (is_ctx ? ctx_end : P.Nb) - kv0;
        const T *kbase = view_row<T>(ks_, bb, h, kv0);
        const T *vbase = view_row<T>(vs_, bb, h, kv0);
        k_step = static_cast<long>(BN) * ks_.sn;
        v_step = static_cast<long>(BN) * vs_.sn;
#pragma unroll
        for (int x = 0; x < NCH; ++x) {
            kp[x] = kbase + st_row(x) * ks_.sn + st_col(x);
            vp[x] = vbase + st_row(x) * vs_.sn + st_col(x);
        }
    };

    // Load tile `it` (the one the running pointers are at) into the given staging registers and
    // advance the pointers.
    auto fetch_into = [&](int it, u32x4(&kst)[NCH], u32x4(&vst)[NCH]) {
        if (it == 0 || it == ctx_tiles) seek(it);
        if (fetch_rows_left >= BN) {
#pragma unroll
            for (int x = 0; x < NCH; ++x) {
                if (NCH * NT == CHUNKS || tid + x * NT < CHUNKS) {
                    kst[x] = *reinterpret_cast<const u32x4 *>(kp[x]);
                    vst[x] = *reinterpret_cast<const u32x4 *>(vp[x]);
                }
            }
        } else {
#pragma unroll
            for (int x = 0; x < NCH; ++x) {
                kst[x] = u32x4{0u, 0u, 0u, 0u};
                vst[x] = u32x4{0u, 0u, 0u, 0u};
                if ((NCH * NT == CHUNKS || tid + x * NT < CHUNKS) && st_row(x) < fetch_rows_left) {
                    kst[x] = *reinterpret_cast<const u32x4 *>(kp[x]);
                    vst[x] = *reinterpret_cast<const u32x4 *>(vp[x]);
                }
            }
        }
        fetch_rows_left -= BN;
#pragma unroll
        for (int x = 0; x < NCH; ++x) {
            kp[x] += k_step;
            vp[x] += v_step;
        }
    };

    auto stash_from = [&](int buf, const u32x4(&kst)[NCH], const u32x4(&vst)[NCH]) {
#pragma unroll
        for (int x = 0; x < NCH; ++x) {
            if (NCH * NT == CHUNKS || tid + x * NT < CHUNKS) {
                *reinterpret_cast<u32x4 *>(k_stage(buf) + st_row(x) * KPAD + st_col(x)) = kst[x];
                *reinterpret_cast<u32x4 *>(v_stage(buf) + st_row(x) * VPAD + st_col(x)) = vst[x];
            }
        }
    };
    auto fetch = [&](int it) { fetch_into(it, kst, vst); };
    auto stash = [&](int buf) { stash_from(buf, kst, vst); };

    // ---- per-lane LDS read offsets (elements) of the padded layout (robust and pipelined pass).
    // Worked out inside those passes, from a lane index the compiler cannot trace: computed here
    // they would stay live across the lean pass, which has no register to spare for them.
    auto k_rd_of = [&]() { const int l = opaque(lane); return (l & 31) * KPAD + 8 * (l >> 5); };  // + 32*sb*KPAD + 16*ks
    auto v_rd_of = [&]() {
        const int l = opaque(lane);
        return (4 * (l >> 5) + ((l & 15) >> 2)) * VPAD + 16 * ((l >> 4) & 1) + 4 * (l & 3);
    };  //                                        + (32*sb + 16*t + 8*u)*VPAD + 32*db

    float m_run[QB], l_run[QB];
    f32x16 o_acc[QB][DB];

    // One pass over this workgroup's key tiles.  ROBUST selects the online softmax
    // with a running maximum; otherwise p = 2^s is accumulated as is.
    auto run_pass = [&](auto robust_tag) {
        constexpr bool ROBUST = decltype(robust_tag)::value;
        const int k_rd = k_rd_of(), v_rd = v_rd_of();
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            m_run[j] = ROBUST ? -INFINITY : 0.f;
            l_run[j] = 0.f;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o_acc[j][db][v] = 0.f;
        }

        if (!q_scaled) {  // else the fast pass has left qreg ready
            u32x4 qraw[QB][KS];
            const int ln = opaque(lane);
            request_q(qraw, ln);
            scale_q(qraw, ln);
        }
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
            const T *kt = k_stage(cur) + k_rd;
            const T *vt = v_stage(cur) + v_rd;

            auto block = [&](int sb, auto mask_tag) {
                constexpr bool MASK = decltype(mask_tag)::value;
                const int blk0 = kv0 + 32 * sb;
                vec ak[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    ak[ks] = *reinterpret_cast<const vec *>(kt + 32 * sb * KPAD + 16 * ks);

                f32x16 s[QB];
#pragma unroll
                for (int j = 0; j < QB; ++j) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[j][v] = 0.f;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) s[j] = Ops::mma(ak[ks], qreg[j][ks], s[j]);
                }

                if constexpr (MASK) {
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
                    if constexpr (ROBUST) {
                        float tmax = s[j][0];
#pragma unroll
                        for (int v = 1; v < 16; ++v) tmax = fmaxf(tmax, s[j][v]);
                        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
                        const float m_new = fmaxf(m_run[j], tmax);
                        // m_new = -inf only while every key so far was masked: keep state at zero
                        const float m_use = m_new == -INFINITY ? 0.f : m_new;
                        const float alpha = fast_exp2(m_run[j] - m_use);  // 2^(-inf) = 0 on the first block
                        if (__any(alpha != 1.f)) {
                            l_run[j] *= alpha;
#pragma unroll
                            for (int db = 0; db < DB; ++db)
#pragma unroll
                                for (int v = 0; v < 16; ++v) o_acc[j][db][v] *= alpha;
                        }
                        m_run[j] = m_new;
#pragma unroll
                        for (int v = 0; v < 16; ++v) s[j][v] -= m_use;
                    }
                    float lsum = l_run[j];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        pk[j][e] = pack2<T>(fast_exp2(s[j][2 * e]), fast_exp2(s[j][2 * e + 1]));
                        lsum = Ops::dot2(pk[j][e], lsum);
                    }
                    l_run[j] = lsum;
                }

#pragma unroll
                for (int db = 0; db < DB; ++db) {
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        const T *vp = vt + (32 * sb + 16 * t) * VPAD + 32 * db;
                        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) s16x4 *)(vp));
                        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) s16x4 *)(vp + 8 * VPAD));
                        typedef short s16x8 __attribute__((ext_vector_type(8)));
                        s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                        vec av = __builtin_bit_cast(vec, both);
#pragma unroll
                        for (int j = 0; j < QB; ++j) {
                            u32x4 pb = {pk[j][4 * t], pk[j][4 * t + 1], pk[j][4 * t + 2], pk[j][4 * t + 3]};
                            o_acc[j][db] = Ops::mma(av, __builtin_bit_cast(vec, pb), o_acc[j][db]);
                        }
                    }
                }
            };

#pragma unroll
            for (int sb = 0; sb < SB; ++sb) {
                const int blk0 = kv0 + 32 * sb;
                if (blk0 >= w_max) continue;  // wave-uniform: nothing visible to this wavefront
                if (blk0 + 32 > w_min)
                    block(sb, BoolTag<true>{});
                else
                    block(sb, BoolTag<false>{});
            }

            if (it + 1 < n_tiles) stash(cur ^ 1);
            __syncthreads();
        }
    };

    // Fast pass: p = 2^s without a running maximum, software-pipelined so that the
    // MFMAs of the next block's scores and of the previous block's PV product are
    // issued between the exp/convert/sum VALU work of the current block.  Three LDS
    // stages with one barrier per tile: tile it+2 is stored while tile it is
    // computed and block 0 of tile it+1 is already being multiplied.
    auto fast_pass = [&]() {
        const int k_rd = k_rd_of(), v_rd = v_rd_of();
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            m_run[j] = 0.f;
            l_run[j] = 0.f;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o_acc[j][db][v] = 0.f;
        }
        // the first two tiles and the queries are requested together: one memory round trip
        // before the loop instead of three
        u32x4 kst1[NCH], vst1[NCH], qraw[QB][KS];
        request_q(qraw, lane);
        if (n_tiles > 0) fetch(0);
        if (n_tiles > 1) fetch_into(1, kst1, vst1);
        scale_q(qraw, lane);
        if (n_tiles > 0) stash(0);
        if (n_tiles > 1) stash_from(1, kst1, vst1);
        __syncthreads();
        if (n_tiles == 0) return;

        // LDS operand fetches: K fragments of one 32-key block (A operand of S^T) and
        // the transposed V fragments of one block (A operand of O^T).
        auto load_k = [&](vec(&ak)[KS], const T *kblk) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) ak[ks] = *reinterpret_cast<const vec *>(kblk + 16 * ks);
        };
        auto load_v = [&](vec(&av)[DB][2], const T *vblk) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const T *vp_ = vblk + 16 * t * VPAD + 32 * db;
                    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp_));
                    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4 *)(vp_ + 8 * VPAD));
                    typedef short s16x8 __attribute__((ext_vector_type(8)));
                    s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    av[db][t] = __builtin_bit_cast(vec, both);
                }
        };
        auto scores = [&](f32x16(&dst)[QB], const vec(&ak)[KS]) {
#pragma unroll
            for (int j = 0; j < QB; ++j) {
#pragma unroll
                for (int v = 0; v < 16; ++v) dst[j][v] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) dst[j] = Ops::mma(ak[ks], qreg[j][ks], dst[j]);
            }
        };

        f32x16 s_cur[QB];
        {
            vec ak0[KS];
            load_k(ak0, k_stage(0) + k_rd);
            scores(s_cur, ak0);
        }

        int stage = 0;
        for (int it = 0; it < n_tiles; ++it) {
            if (it > 0) __syncthreads();
            if (it + 2 < n_tiles) fetch(it + 2);
            const int stage_next = stage == 2 ? 0 : stage + 1;
            const bool is_ctx = it < ctx_tiles;
            const int kv0 = is_ctx ? ctx_begin + it * BN : (it - ctx_tiles) * BN;
            const int seg_end = is_ctx ? ctx_end : P.Nb;
            const int w_min = is_ctx ? seg_end : wave_lim_min;
            const T *kt = k_stage(stage) + k_rd;
            const T *vt = v_stage(stage) + v_rd;
            // the block after this tile's last one is block 0 of the next tile (on the very
            // last tile any valid address will do: those scores are never used)
            const T *kt_next = (it + 1 < n_tiles) ? k_stage(stage_next) + k_rd : kt;

            auto tile_body = [&](auto mask_tag) {
                constexpr bool MASK = decltype(mask_tag)::value;
#pragma unroll
                for (int sb = 0; sb < SB; ++sb) {
                    if constexpr (MASK) {
                        const int blk0 = kv0 + 32 * sb;
#pragma unroll
                        for (int j = 0; j < QB; ++j) {
                            const int lj = is_ctx ? seg_end : lim[j];
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                int kv = blk0 + 8 * (v >> 2) + 4 * hb + (v & 3);
                                if (kv >= lj) s_cur[j][v] = -INFINITY;
                            }
                        }
                    }
                    vec ak_nx[KS], av_cu[DB][2];
                    load_v(av_cu, vt + 32 * sb * VPAD);
                    load_k(ak_nx, sb + 1 < SB ? kt + 32 * (sb + 1) * KPAD : kt_next);

                    f32x16 s_next[QB];
                    scores(s_next, ak_nx);

                    unsigned pk[QB][8];
#pragma unroll
                    for (int j = 0; j < QB; ++j) {
                        float lsum = l_run[j];
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            pk[j][e] = pack2<T>(fast_exp2(s_cur[j][2 * e]), fast_exp2(s_cur[j][2 * e + 1]));
                            lsum = Ops::dot2(pk[j][e], lsum);
                        }
                        l_run[j] = lsum;
                    }
#pragma unroll
                    for (int j = 0; j < QB; ++j)
#pragma unroll
                        for (int db = 0; db < DB; ++db)
#pragma unroll
                            for (int t = 0; t < 2; ++t) {
                                u32x4 pb = {pk[j][4 * t], pk[j][4 * t + 1], pk[j][4 * t + 2], pk[j][4 * t + 3]};
                                o_acc[j][db] = Ops::mma(av_cu[db][t], __builtin_bit_cast(vec, pb), o_acc[j][db]);
                            }
#pragma unroll
                    for (int j = 0; j < QB; ++j) s_cur[j] = s_next[j];

                    if constexpr (!MASK) {
                        // Issue order for this block: the score MFMAs of the next block ride
                        // under the first query block's exps, the PV MFMAs of query block j
                        // under the exps of block j+1.
                        __builtin_amdgcn_sched_group_barrier(0x100, KS + 4 * DB, 0);  // DS reads
#pragma unroll
                        for (int i = 0; i < QB * KS; ++i) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x400, 16 / (QB * KS) > 0 ? 16 / (QB * KS) : 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 16 / (QB * KS) > 0 ? 16 / (QB * KS) : 1, 0);
                        }
#pragma unroll
                        for (int j = 1; j < QB; ++j)
#pragma unroll
                            for (int i = 0; i < 2 * DB; ++i) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                                __builtin_amdgcn_sched_group_barrier(0x400, 16 / (2 * DB), 0);
                                __builtin_amdgcn_sched_group_barrier(0x002, 16 / (2 * DB), 0);
                            }
                    }
                }
            };

            if (kv0 + BN > w_min)
                tile_body(BoolTag<true>{});
            else
                tile_body(BoolTag<false>{});

            if (it + 2 < n_tiles) stash(stage == 0 ? 2 : stage - 1);
            stage = stage_next;
        }
        __syncthreads();
    };


    // Lean fast pass.  On this part a matrix instruction holds the SIMD's vector issue port for
    // its whole duration: MFMA and ordinary VALU work of the same SIMD do not overlap, whichever
    // wavefronts they come from (only the tail of a transcendental does).  The time of a 32x32
    // score block is therefore the SUM of its instructions' issue cycles, and software pipelining
    // inside a wavefront buys nothing that more resident wavefronts do not give as well.  So this
    // pass keeps the instruction count minimal and the register count low enough for four
    // wavefronts per SIMD:
    //  * a plain in-order block: K fragments, S = K Q^T, p = 2^s, P V; no second score buffer;
    //  * the row sum of the rounded probabilities comes from the matrix pipe: with
    //    v_mfma_f32_16x16x32 a lane's four packed registers are 8 contraction entries of column
    //    lane%16, contraction group lane/16.  A lane here is (query c = lane%32, half hb), i.e.
    //    column c%16 and group c/16 + 2 hb: an A operand that is all ones in row 0 for groups
    //    {0, 2} and in row 1 for groups {1, 3} sums queries 0..15 into row 0 and 16..31 into
    //    row 1 (lanes 0..15, registers 0 and 1).  Two such products per block replace eight
    //    v_dot2c (which, issued between MFMAs, cost five times their nominal four cycles).
    //  * K and V tiles of a stage are one list of 16-byte pieces dealt over the whole workgroup.
    // NST LDS stages (four), one barrier per tile, full tiles requested NST - 1 ahead.
    auto lean_pass = [&]() {
        f32x4 lsum[QB][2];
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            m_run[j] = 0.f;
            l_run[j] = 0.f;
            lsum[j][0] = f32x4{0.f, 0.f, 0.f, 0.f};
            lsum[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) o_acc[j][db][v] = 0.f;
        }
        const unsigned one2 = (lane == 0 || lane == 32 || lane == 17 || lane == 49) ? Ops::kOnes2 : 0u;
        const vec ones_sel = __builtin_bit_cast(vec, u32x4{one2, one2, one2, one2});

        // ---- staging.  A stage's 2*CHUNKS 16-byte pieces (K pieces, then V pieces) are dealt over
        // the workgroup, NP rounds of NT pieces.  CHUNKS is a multiple of 64, so whether a piece
        // is K or V is uniform over a wavefront: sources are a scalar base plus a 32-bit lane
        // offset, and the base moves on by one tile with scalar arithmetic.
        // ---- LDS layout of a lean stage.  No padding: every 1 KiB chunk is laid out so that the
        // operand reads of a wavefront sweep whole bank rows.
        //   K, chunk (sb, ks) [32 keys x 16 columns]: [hb][key][8 elements] — the A operand of S^T
        //      for lane (c, hb) is the 16 bytes at hb*512 + c*16: 32 consecutive lanes read 512
        //      consecutive bytes.
        //   V, chunk (sb, cb) [32 keys x 16 columns]: [key][16 elements] — a transposing read takes
        //      8 bytes per lane from rows 4*hb .. 4*hb+3 of one chunk: 16 consecutive lanes read 128
        //      consecutive bytes.
        // (With padded whole rows — 80-byte K rows, 96-byte V rows — a third of the LDS cycles of
        // this pass were bank conflicts, and a stage was 11 KiB instead of 8.)
        static_assert(DH % 16 == 0 && BN % 32 == 0, "chunks are 32 keys x 16 columns");
        constexpr int CH = 512;                       // elements per chunk
        constexpr int LK = BN * DH;                   // V region of a stage
        auto k_off = [](int row, int col) {          // element offset of K[row][col] inside a stage
            return ((row / 32) * KS + col / 16) * CH + ((col % 16) / 8) * 256 + (row % 32) * 8 + col % 8;
        };
        auto v_off = [](int row, int col) {
            return LK + ((row / 32) * KS + col / 16) * CH + (row % 32) * 16 + col % 16;
        };
        const int lk_rd = hb * 256 + c * 8;                                               // + (sb*KS + ks) * CH
        const int lv_rd = LK + (4 * hb + ((lane & 15) >> 2)) * 16 + ((lane >> 4) & 1) * CH + 4 * (lane & 3);
        //                                              + (sb*KS + 2*db) * CH + (16*t + 8*u) * 16

        constexpr int NP = (2 * CHUNKS + NT - 1) / NT;
        static_assert(CHUNKS % 64 == 0, "K/V choice must be wavefront-uniform");
        // Where piece x of this thread sits: worked out where a (rare) register-staged tile needs it,
        // from a lane index the compiler cannot trace — computed up front these values would sit in
        // registers through the steady loop, and at 96 registers that means scratch memory written
        // in the prologue of every launch.
        struct Piece {
            bool on, v;
            int row, col, dst;  // row and column in the tile; element offset inside a stage
        };
        auto piece = [&](int x) {
            Piece pc;
            const int idx0 = wave * 64 + x * NT;  // scalar: first piece of this wavefront in round x
            pc.on = idx0 < 2 * CHUNKS;
            pc.v = idx0 >= CHUNKS;
            const int cidx = idx0 + opaque(lane) - (pc.v ? CHUNKS : 0);
            pc.row = cidx / CPR;
            pc.col = (cidx % CPR) * 8;
            pc.dst = pc.v ? v_off(pc.row, pc.col) : k_off(pc.row, pc.col);
            return pc;
        };

        // Full context tiles (every row present, nothing masked): the steady state.
        const int n_main = (ctx_end - ctx_begin) / BN;
        bool yield_ = false;  // set once the neighbour's length is known (below)

        // (the direct-load machinery — d_off, d_src, d_step, dma_tile — sits at kernel scope: the
        // plain context launch starts it from its leading arguments before this pass is reached)
        if (!early_tiles) {
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                const int i = wave + NW * r;  // scalar: chunk of the stage
                const bool is_v = i >= NKI;
                const View &src = is_v ? P.vc : P.kc;
                direct_load_lane(i, src.sn, d_off[r], d_step[r]);
                d_src[r] = reinterpret_cast<const char *>(view_row<T>(src, kvb, h, ctx_begin));
            }
        }

        // Every other tile (the partial last context tile, buffer tiles of teacher forcing) goes
        // the general way: per-lane pointers, row guards, zero fill.
        const T *g_src[NP];
        long g_step[NP];
        int rows_left = 0;
        auto gseek = [&](int it) {
            const bool is_ctx = it < ctx_tiles;
            const View &ks_ = is_ctx ? P.kc : P.kb;
            const View &vs_ = is_ctx ? P.vc : P.vb;
            const long bb = is_ctx ? kvb : g;
            const int kv0 = is_ctx ? ctx_begin + it * BN : (it - ctx_tiles) * BN;
            rows_left = (is_ctx ? ctx_end : P.Nb) - kv0;
#pragma unroll
            for (int x = 0; x < NP; ++x) {
                const Piece pc = piece(x);
                const View &src = pc.v ? vs_ : ks_;
                g_src[x] = view_row<T>(src, bb, h, kv0) + pc.row * src.sn + pc.col;
                g_step[x] = static_cast<long>(BN) * src.sn;
            }
        };
        auto gfetch = [&](int it, u32x4(&st)[NP]) {
            if (it == n_main || it == ctx_tiles) gseek(it);
#pragma unroll
            for (int x = 0; x < NP; ++x) {
                st[x] = u32x4{0u, 0u, 0u, 0u};
                const Piece pc = piece(x);
                if (pc.on && (rows_left >= BN || pc.row < rows_left)) st[x] = *reinterpret_cast<const u32x4 *>(g_src[x]);
                g_src[x] += g_step[x];
            }
            rows_left -= BN;
        };
        auto stash_tile = [&](auto stage_, const u32x4(&st)[NP]) {
#pragma unroll
            for (int x = 0; x < NP; ++x)
            {
                const Piece pc = piece(x);
                if (pc.on) *reinterpret_cast<u32x4 *>(kv_lds + stage_ * LSTAGE + pc.dst) = st[x];
            }
        };

        // One 32-key block of the tile in `stage_` against this wavefront's queries.
        auto block = [&](auto stage_, int sb, auto mask_tag, int blk0, bool is_ctx, int seg_end) {
            constexpr bool MASK = decltype(mask_tag)::value;
            const T *kt = kv_lds + stage_ * LSTAGE + lk_rd;
            const T *vt = kv_lds + stage_ * LSTAGE + lv_rd;
            vec ak[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) ak[ks] = *reinterpret_cast<const vec *>(kt + (sb * KS + ks) * CH);
            vec av[DB][2];
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const T *vp_ = vt + (sb * KS + 2 * db) * CH + 16 * t * 16;
                    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp_));
                    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4 *)(vp_ + 8 * 16));
                    typedef short s16x8 __attribute__((ext_vector_type(8)));
                    s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    av[db][t] = __builtin_bit_cast(vec, both);
                }
#pragma unroll
            for (int j = 0; j < QB; ++j) {
                f32x16 s;
#pragma unroll
                for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) s = Ops::mma(ak[ks], qreg[j][ks], s);
                if constexpr (MASK) {
                    const int lj = is_ctx ? seg_end : lim[j];
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        int kv = blk0 + 8 * (v >> 2) + 4 * hb + (v & 3);
                        if (kv >= lj) s[v] = -INFINITY;
                    }
                }
                u32x4 pb[2];
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        pb[t][e] = pack2<T>(fast_exp2(s[8 * t + 2 * e]), fast_exp2(s[8 * t + 2 * e + 1]));
#pragma unroll
                for (int t = 0; t < 2; ++t) lsum[j][t] = Ops::mma16(ones_sel, __builtin_bit_cast(vec, pb[t]), lsum[j][t]);
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int t = 0; t < 2; ++t)
                        o_acc[j][db] = Ops::mma(av[db][t], __builtin_bit_cast(vec, pb[t]), o_acc[j][db]);
            }
        };

        // Tile `it` out of stage it % NST: barrier, request a later tile into a stage that is free,
        // compute.  STEADY: a full, unmasked context tile; it requests the full tile NST - 1 ahead (if
        // there is one) by direct global->LDS loads, into the stage that tile it - 1 has just left.
        // Otherwise: any tile; it requests the tile two ahead through registers and stores it after
        // the compute, unless that tile is a full one (then a direct load is or was under way).
        // So full tiles 2 .. n_main - 1 arrive by direct loads (tiles 2 .. NST - 2 from the prologue), all
        // others through registers, and the tile in front of the first non-full one is never STEADY.
        auto tile = [&](int it, auto stage_, auto steady_tag) {
            constexpr bool STEADY = decltype(steady_tag)::value;
            if constexpr (STEADY) {
                // Two workgroups share a compute unit and the hardware serves the older wavefront
                // first: left alone, one workgroup runs ahead and the other finishes the slice with
                // the SIMDs half empty.  The priority falls with progress, so whoever is behind is
                // served first (measured: the slower workgroup of a pair ends 2.5 us earlier).
                if (it == n_main / 4) {
                    if (yield_) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(2);
                } else if (it == n_main / 2) {
                    if (yield_) __builtin_amdgcn_s_setprio(0); else __builtin_amdgcn_s_setprio(1);
                } else if (it == 3 * n_main / 4) {
                    __builtin_amdgcn_s_setprio(0);
                }
                // this tile's direct loads must have landed; those of the next two full tiles may
                // still be on their way
                const int behind = n_main - 1 - it;
                switch ((behind >= NST - 2 ? NST - 2 : behind) * n_dma) {
                    case 0: __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); break;
                    case 1: __builtin_amdgcn_s_waitcnt(vmcnt_imm(1)); break;
                    case 2: __builtin_amdgcn_s_waitcnt(vmcnt_imm(2)); break;
                    case 3: __builtin_amdgcn_s_waitcnt(vmcnt_imm(3)); break;
                    case 4: __builtin_amdgcn_s_waitcnt(vmcnt_imm(4)); break;
                    case 5: __builtin_amdgcn_s_waitcnt(vmcnt_imm(5)); break;
                    case 6: __builtin_amdgcn_s_waitcnt(vmcnt_imm(6)); break;
                    default: __builtin_amdgcn_s_waitcnt(vmcnt_imm(8)); break;
                }
                static_assert(NST <= 6, "the wait counts above cover up to four tiles in flight, two loads each");
                __syncthreads();
                if (behind >= NST - 1) dma_tile((stage_ + NST - 1) % NST);
#pragma unroll
                for (int sb = 0; sb < SB; ++sb) block(stage_, sb, BoolTag<false>{}, 0, true, 0);
            } else {
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // direct loads of the steady state
                __syncthreads();
                const bool fetch = it + 2 < n_tiles && it + 2 >= n_main;
                u32x4 st_a[NP];  // (local: a staging register that lived across the steady loop would be parked in scratch)
                if (fetch) gfetch(it + 2, st_a);
                const bool is_ctx = it < ctx_tiles;
                const int kv0 = is_ctx ? ctx_begin + it * BN : (it - ctx_tiles) * BN;
                const int seg_end = is_ctx ? ctx_end : P.Nb;
                const int w_min = is_ctx ? seg_end : wave_lim_min;
                const int w_max = is_ctx ? seg_end : wave_lim_max;
#pragma unroll
                for (int sb = 0; sb < SB; ++sb) {
                    const int blk0 = kv0 + 32 * sb;
                    if (blk0 >= w_max) continue;  // wave-uniform: nothing visible to this wavefront
                    if (blk0 + 32 > w_min)
                        block(stage_, sb, BoolTag<true>{}, blk0, is_ctx, seg_end);
                    else
                        block(stage_, sb, BoolTag<false>{}, blk0, is_ctx, seg_end);
                }
                if (fetch) stash_tile((stage_ + 2) % NST, st_a);
            }
        };

        __builtin_amdgcn_s_setprio(3);
        // (read here, in front of the prologue's requests: where it is used the loop would wait for it)
        const int beside_now = (P.dense_below > 0 || P.yield_from > 0) && P.beside_rows ? *P.beside_rows : P.beside_n;
        {
            // the first NST - 1 tiles are requested together with the queries, full tiles by direct
            // loads into their stages.  A ragged or buffer tile among the first two goes through
            // registers and is stored at once (small problems only: nothing there is worth keeping
            // staging registers alive across the query scaling, which at 96 registers would park
            // them in scratch memory on every launch, the common one included).
            u32x4 qraw[QB][KS];
            request_q(qraw, lane);
            if (n_main >= NST - 1) {
                // The common case on a path of its own: where it shares basic blocks with the
                // register-staged tiles below, the compiler has to assume one of their loads
                // pending when the paths meet and drains the memory counter — the queries
                // included — in front of the first direct load: a whole round trip.
                if (!early_tiles) {
                    dma_tile(std::integral_constant<int, 0>{});
                    dma_tile(std::integral_constant<int, 1>{});
#pragma unroll
                    for (int t = 2; t < NST - 1; ++t) dma_tile(t);
                }
            } else {
                if (n_main > 0) {
                    dma_tile(std::integral_constant<int, 0>{});
                } else if (n_tiles > 0) {
                    u32x4 st[NP];
                    gfetch(0, st);
                    stash_tile(std::integral_constant<int, 0>{}, st);
                }
                if (n_main > 1) {
                    dma_tile(std::integral_constant<int, 1>{});
                } else if (n_tiles > 1) {
                    u32x4 st[NP];
                    gfetch(1, st);
                    stash_tile(std::integral_constant<int, 1>{}, st);
                }
#pragma unroll
                for (int t = 2; t < NST - 1; ++t)
                    if (n_main > t) dma_tile(t);
            }
            scale_q(qraw, lane);
        }

        int it = 0;
        // with nothing but full context tiles the whole slice is steady state; otherwise the last
        // two full tiles have to request tiles of the other kind and take the general route
        const int n_steady = n_tiles == n_main ? n_main : n_main - 2;
        // The bulk of a long slice: groups of NST full tiles that each have NST - 1 full tiles
        // behind them.  Nothing about such a tile depends on its index — the wait is for a constant
        // number of direct loads, the request NST - 1 ahead is unconditional — so the group is
        // straight-line code (the general steady tile below spends a dozen scalar branches on
        // these decisions); the priority steps sit between groups, at multiples of NST.
        const int n_ahead = n_steady < n_main - (NST - 1) ? n_steady : n_main - (NST - 1);
        const int n_fast = n_main >= 12 && n_ahead > 0 ? n_ahead / NST * NST : 0;
        bool dense = n_fast > 0;
        if (dense && P.dense_below > 0)  // (a scalar: the choice must stay a wavefront-uniform branch)
            dense = __builtin_amdgcn_readfirstlane(beside_now) < P.dense_below;
        // Beside a buffer pass that is the longer kernel of the two, this pass gives way: one
        // priority step lower throughout, so the neighbour's few instructions never queue behind it.
        yield_ = P.yield_from > 0 && __builtin_amdgcn_readfirstlane(beside_now) >= P.yield_from;
        if (yield_) __builtin_amdgcn_s_setprio(2);
        if (dense) {
            const bool two = n_dma == 2;  // direct loads of this wavefront per tile: one or two
            auto fast_tile = [&](auto stage_) {
                // this tile's loads have landed, those of the next NST - 2 tiles may be under way
                if (two)
                    __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * (NST - 2)));
                else
                    __builtin_amdgcn_s_waitcnt(vmcnt_imm(NST - 2));
                __syncthreads();
                constexpr int into = (decltype(stage_)::value + NST - 1) % NST;
#pragma unroll
                for (int r = 0; r < NR; ++r) {
                    if (r == 0 || two) {
                        const unsigned m0v = lds_base + into * STAGE_BYTES + (wave + NW * r) * 1024;
                        unsigned m0_saved;
                        asm volatile(
                            "s_mov_b32 %0, m0\n\t"
                            "s_mov_b32 m0, %1\n\t"
                            "global_load_lds_dwordx4 %2, %3\n\t"
                            "s_mov_b32 m0, %0"
                            : "=&s"(m0_saved)
                            : "s"(m0v), "v"(d_off[r]), "s"(d_src[r]));
                    }
                    d_src[r] += d_step[r];
                }
#pragma unroll
                for (int sb = 0; sb < SB; ++sb) block(stage_, sb, BoolTag<false>{}, 0, true, 0);
            };
            // the priority falls with progress (see the general steady tile): steps between groups
            const int q1 = (n_main / 4) / NST * NST, q2 = (n_main / 2) / NST * NST, q3 = (3 * n_main / 4) / NST * NST;
#pragma nounroll
            for (int part = 0; part < 4; ++part) {
                int end = part == 0 ? q1 : part == 1 ? q2 : part == 2 ? q3 : n_fast;
                end = end < n_fast ? end : n_fast;
#pragma nounroll
                for (; it < end; it += NST) {
                    fast_tile(std::integral_constant<int, 0>{});
                    fast_tile(std::integral_constant<int, 1>{});
                    fast_tile(std::integral_constant<int, 2>{});
                    fast_tile(std::integral_constant<int, 3>{});
                    if constexpr (NST > 4) fast_tile(std::integral_constant<int, 4>{});
                    if constexpr (NST > 5) fast_tile(std::integral_constant<int, 5>{});
                }
                if (part == 0 && it == q1)
                    __builtin_amdgcn_s_setprio(2);
                else if (part == 1 && it == q2)
                    __builtin_amdgcn_s_setprio(1);
                else if (part == 2 && it == q3)
                    __builtin_amdgcn_s_setprio(0);
            }
        }
        while (it < n_steady) {  // stages as compile-time constants: every LDS offset is an immediate
            tile(it, std::integral_constant<int, 0>{}, BoolTag<true>{});
            if (++it >= n_steady) break;
            tile(it, std::integral_constant<int, 1>{}, BoolTag<true>{});
            if (++it >= n_steady) break;
            tile(it, std::integral_constant<int, 2>{}, BoolTag<true>{});
            if (++it >= n_steady) break;
            tile(it, std::integral_constant<int, 3>{}, BoolTag<true>{});
            if constexpr (NST > 4) {
                if (++it >= n_steady) break;
                tile(it, std::integral_constant<int, 4>{}, BoolTag<true>{});
            }
            if constexpr (NST > 5) {
                if (++it >= n_steady) break;
                tile(it, std::integral_constant<int, 5>{}, BoolTag<true>{});
            }
            ++it;
        }
        for (int stage = it % NST; it < n_tiles; ++it) {
            tile(it, stage, BoolTag<false>{});
            stage = stage == NST - 1 ? 0 : stage + 1;
        }
        // row sums: query c of this lane's block sits in lane c % 16, register c / 16; the total
        // already covers both halves, so only the hb = 0 lane carries it into the epilogue
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            const float r0 = lsum[j][0][0] + lsum[j][1][0], r1 = lsum[j][0][1] + lsum[j][1][1];
            const float a0 = __shfl(r0, lane & 15, 64), a1 = __shfl(r1, lane & 15, 64);
            l_run[j] = hb == 0 ? ((lane & 16) ? a1 : a0) : 0.f;
        }
    };

    bool robust = !Ops::kWideExponent || P.force_robust;
    if (!robust) {
        if constexpr (LEAN)
            lean_pass();
        else
            fast_pass();
        bool bad = false;
#pragma unroll
        for (int j = 0; j < QB; ++j) {
            const float l_tot = l_run[j] + __shfl_xor(l_run[j], 32, 64);
            bad = bad || !(l_tot > kFastMassMin && l_tot < kFastMassMax);
        }
        if constexpr (LEAN) {
            // the pass ends without a barrier of its own: this one also separates its last LDS
            // reads from the stores of a second, robust pass
            if (bad) redo_flag = 1;
            __syncthreads();
        } else {
            if (tid == 0) redo_flag = 0;
            __syncthreads();
            if (bad) redo_flag = 1;
            __syncthreads();
        }
        robust = redo_flag != 0;
    }
    if (robust) run_pass(BoolTag<true>{});

    // ---- epilogue: normalise, write output (final or split partial) and log-sum-exp.
    const long total_rows = static_cast<long>(P.B) * P.H * P.Lq;
    // (the half of the wavefront again, from a lane index the compiler cannot trace: kept from the
    // prologue it would be parked in scratch memory across the key loop)
    const int hb_e = opaque(lane) >> 5;
#pragma unroll
    for (int j = 0; j < QB; ++j) {
        float l_tot = l_run[j] + __shfl_xor(l_run[j], 32, 64);
        long ob;
        int oi;
        if (!query_of(j, opaque(lane) & 31, ob, oi)) continue;
        const long orow_idx = (ob * P.H + h) * P.Lq + oi;  // row of the [B, H, Lq] order
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        const float m_fin = m_run[j] == -INFINITY ? 0.f : m_run[j];
        const float lse = l_tot > 0.f ? (m_fin + fast_log2(l_tot)) * kLn2 : -INFINITY;
        if (P.part_o) {
            T *po = static_cast<T *>(P.part_o) + (static_cast<long>(split) * total_rows + orow_idx) * DH;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    u32x2 val = {pack2<T>(o_acc[j][db][4 * gq] * inv, o_acc[j][db][4 * gq + 1] * inv),
                                 pack2<T>(o_acc[j][db][4 * gq + 2] * inv, o_acc[j][db][4 * gq + 3] * inv)};
                    *reinterpret_cast<u32x2 *>(po + 32 * db + 8 * gq + 4 * hb_e) = val;
                }
            if (hb_e == 0) P.part_lse[static_cast<long>(split) * total_rows + orow_idx] = lse;
        } else {
            T *orow = view_row<T>(P.out, ob, h, oi);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    u32x2 val = {pack2<T>(o_acc[j][db][4 * gq] * inv, o_acc[j][db][4 * gq + 1] * inv),
                                 pack2<T>(o_acc[j][db][4 * gq + 2] * inv, o_acc[j][db][4 * gq + 3] * inv)};
                    *reinterpret_cast<u32x2 *>(orow + 32 * db + 8 * gq + 4 * hb_e) = val;
                }
            if (P.lse && hb_e == 0) P.lse[orow_idx] = lse;
        }
    }
    if (P.stamps) {
        __syncthreads();  // every wavefront of the workgroup has issued its stores
        if (threadIdx.x == 0) flash_stamp_end(P);
    }
}

}  // namespace artab
