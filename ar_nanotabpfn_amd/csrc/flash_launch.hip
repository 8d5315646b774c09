// Launches of the matrix-core attention kernel (mfma_flash.h): template selection by element
// type, head_dim and query-tile size.
#include "launchers.h"

namespace artab {

constexpr int kFlashBN = 64;

// Keys per LDS tile: 64, or 128 for head_dim 32 when kTuneBN is 128.
static int flash_bn(int Dh) { return (Dh == 32 && tune(kTuneBN, 64) == 128) ? 128 : 64; }

template <typename Kernel>
static void launch_one(Kernel kernel, unsigned grid, unsigned block, hipStream_t stream, const FlashParams &P) {
    LaunchTiming t;
    const int how = observe_launch(kLaunchFlash, &t);
    if (how == kObserveEvents) {
        hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, stream, t.start, t.stop, 0, P);
    } else if (how == kObserveStamps) {
        FlashParams Q = P;
        Q.stamps = t.stamps;
        Q.stamps_capacity = t.stamps_capacity;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, stream, Q);
    } else {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, stream, P);
    }
}

template <typename T, int DH>
static hipError_t launch_flash_bm(const FlashParams &P, int BM, hipStream_t stream) {
    const int W = P.tiles_per_group * P.n_split;
    const int n_kvg = P.H * P.n_groups;
    const unsigned grid = static_cast<unsigned>(((n_kvg + 7) / 8) * W * 8);
    if (grid == 0) return hipSuccess;
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
