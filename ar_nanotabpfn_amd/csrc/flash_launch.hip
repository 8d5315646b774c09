// Launches of the matrix-core attention kernel (mfma_flash.h): template selection by element
// type, head_dim and query-tile size.
#include "launchers.h"

namespace artab {

constexpr int kFlashBN = 64;

// Keys per LDS tile: 64, or 128 for head_dim 32 when kTuneBN is 128.
static int flash_bn(int Dh) { return (Dh == 32 && tune(kTuneBN, 64) == 128) ? 128 : 64; }

// Grid of a launch: x = 8 * slices (the XCD in the low three bits), y = query tiles of a group,
// z = blocks of eight (group, head) pairs.  grid.z is limited to 65535: beyond that (more than
// half a million pairs) the blocks are spread over several launches.
constexpr int kMaxGridZ = 65535;

// The leading kernel arguments of a launch (FlashEarly): filled for a context-mode launch over one
// shared context whose K and V have the same head and row strides, all within 31 bits.
static FlashEarly flash_early(const FlashParams &P) {
    FlashEarly e = {nullptr, nullptr, 0, 0, 0, 0, 0, 0};
    constexpr long kIntMax = 0x7fffffffL;
    if (P.mode == kFlashContext && P.n_groups == 1 && P.kc.sh == P.vc.sh && P.kc.sn == P.vc.sn && P.kc.sn > 0 &&
        P.kc.sn <= kIntMax && P.kc.sh >= 0 && P.kc.sh <= kIntMax) {
        e.k = P.kc.p;
        e.v = P.vc.p;
        e.sh = static_cast<int>(P.kc.sh);
        e.sn = static_cast<int>(P.kc.sn);
        e.kv_per_split = P.kv_per_split;
        e.nc = P.Nc;
        e.n_kvg = P.H;
    }
    return e;
}

template <typename Kernel>
static void launch_one(Kernel kernel, dim3 grid, unsigned block, hipStream_t stream, const FlashParams &P0) {
    const int z_total = static_cast<int>(grid.z);
    FlashEarly e = flash_early(P0);
    for (int z0 = 0; z0 < z_total; z0 += kMaxGridZ) {
        FlashParams P = P0;
        P.kvg_block0 = z0;
        e.block0 = z0;
        grid.z = static_cast<unsigned>(z_total - z0 < kMaxGridZ ? z_total - z0 : kMaxGridZ);
        LaunchTiming t;
        const int how = observe_launch(kLaunchFlash, &t);
        if (how == kObserveEvents) {
            hipExtLaunchKernelGGL(kernel, grid, dim3(block), 0, stream, t.start, t.stop, 0, e.k, e.v, e.sh, e.sn,
                                  e.kv_per_split, e.nc, e.n_kvg, e.block0, P);
        } else if (how == kObserveStamps) {
            P.stamps = t.stamps;
            P.stamps_capacity = t.stamps_capacity;
            e.block0 |= kFlashStampedBit;
            hipLaunchKernelGGL(kernel, grid, dim3(block), 0, stream, e.k, e.v, e.sh, e.sn, e.kv_per_split, e.nc, e.n_kvg,
                               e.block0, P);
        } else {
            hipLaunchKernelGGL(kernel, grid, dim3(block), 0, stream, e.k, e.v, e.sh, e.sn, e.kv_per_split, e.nc, e.n_kvg,
                               e.block0, P);
        }
    }
}

template <typename T, int DH>
static hipError_t launch_flash_bm(const FlashParams &P, int BM, hipStream_t stream) {
    const long n_kvg = static_cast<long>(P.H) * P.n_groups;
    if (n_kvg == 0 || P.tiles_per_group <= 0 || P.n_split <= 0) return hipSuccess;
    if (P.tiles_per_group > 65535) return hipErrorInvalidConfiguration;  // 16 million query rows per group
    const dim3 grid(static_cast<unsigned>(8 * P.n_split), static_cast<unsigned>(P.tiles_per_group),
                    static_cast<unsigned>((n_kvg + 7) / 8));
    if constexpr (DH == 32) {
        if (flash_bn(DH) == 128) {
            if (BM == 256)
                launch_one(flash_kernel<T, DH, 2, 4, 128>, grid, 256, stream, P);
            else if (BM == 128)
                launch_one(flash_kernel<T, DH, 1, 4, 128>, grid, 256, stream, P);
            else
                launch_one(flash_kernel<T, DH, 1, 2, 128>, grid, 128, stream, P);
            return hipGetLastError();
        }
    }
    if constexpr (DH == 32) {
        // the lean pass: 256 query rows as eight wavefronts of one 32-row block each, four
        // wavefronts per SIMD (kTuneLean = 0 selects the software-pipelined form)
        if (BM == 256 && tune(kTuneLean, 1) != 0) {
            // 96 registers (five per SIMD by the register file) leave room for the streaming
            // buffer pass beside four of these wavefronts; kTuneLeanOcc = 4 takes 128
            if (tune(kTuneLeanOcc, 5) == 4)
                launch_one(flash_kernel<T, DH, 1, 8, kFlashBN, true, 4>, grid, 512, stream, P);
            else if (P.mode == kFlashContext)  // the decode launch: nothing but the context pass compiled in
                launch_one(flash_kernel<T, DH, 1, 8, kFlashBN, true, 5, true>, grid, 512, stream, P);
            else
                launch_one(flash_kernel<T, DH, 1, 8, kFlashBN, true, 5>, grid, 512, stream, P);
            return hipGetLastError();
        }
    }
    if constexpr (DH <= 64) {
        if (BM == 256) {
            launch_one(flash_kernel<T, DH, 2, 4, kFlashBN>, grid, 256, stream, P);
            return hipGetLastError();
        }
        if (BM == 128 && tune(kTuneNW, 4) == 2) {  // two wavefronts of two query blocks each
            launch_one(flash_kernel<T, DH, 2, 2, kFlashBN>, grid, 128, stream, P);
            return hipGetLastError();
        }
    }
    if (BM == 128) {
        launch_one(flash_kernel<T, DH, 1, 4, kFlashBN>, grid, 256, stream, P);
    } else {
        launch_one(flash_kernel<T, DH, 1, 2, kFlashBN>, grid, 128, stream, P);
    }
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_flash(const FlashParams &P, int Dh, int BM, hipStream_t stream) {
    switch (Dh) {
        case 32: return launch_flash_bm<T, 32>(P, BM, stream);
        case 64: return launch_flash_bm<T, 64>(P, BM, stream);
        default: return launch_flash_bm<T, 128>(P, BM, stream);
    }
}

hipError_t launch_flash_dtype(const FlashParams &P, bool is_bf16, int Dh, int BM, hipStream_t stream) {
    return is_bf16 ? launch_flash<bf16_t>(P, Dh, BM, stream) : launch_flash<f16_t>(P, Dh, BM, stream);
}


}  // namespace artab
