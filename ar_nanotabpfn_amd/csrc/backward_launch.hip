// Launches of the backward kernels of the training row attention (attention_backward.h):
// template selection by element type and head_dim.
#include "launchers.h"

namespace artab {

template <typename T>
static hipError_t launch_backward_portable(const BackwardParams &P, hipStream_t stream) {
    const long total = static_cast<long>(P.B) * P.H * P.R;
    const dim3 grid(static_cast<unsigned>((total + kPortableWaves - 1) / kPortableWaves)), block(kPortableWaves * 64);
    // the dK/dV kernel reads the delta workspace that the dQ kernel leaves: same stream, in this order
    if (P.Dh <= 64) {
        hipLaunchKernelGGL((backward_dq_portable_kernel<T, 1>), grid, block, 0, stream, P);
        hipLaunchKernelGGL((backward_dkv_portable_kernel<T, 1>), grid, block, 0, stream, P);
    } else if (P.Dh <= 128) {
        hipLaunchKernelGGL((backward_dq_portable_kernel<T, 2>), grid, block, 0, stream, P);
        hipLaunchKernelGGL((backward_dkv_portable_kernel<T, 2>), grid, block, 0, stream, P);
    } else {
        hipLaunchKernelGGL((backward_dq_portable_kernel<T, 4>), grid, block, 0, stream, P);
        hipLaunchKernelGGL((backward_dkv_portable_kernel<T, 4>), grid, block, 0, stream, P);
    }
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_backward_mfma(const BackwardParams &P, hipStream_t stream) {
    const long blocks = (P.R + kBackwardRows - 1) / kBackwardRows;
    const dim3 grid(static_cast<unsigned>(blocks * P.H * P.B)), block(kBackwardWaves * 64);
    if (P.Dh == 32) {
        hipLaunchKernelGGL((backward_dq_mfma_kernel<T, 32>), grid, block, 0, stream, P);
        hipLaunchKernelGGL((backward_dkv_mfma_kernel<T, 32>), grid, block, 0, stream, P);
    } else {
        hipLaunchKernelGGL((backward_dq_mfma_kernel<T, 64>), grid, block, 0, stream, P);
        hipLaunchKernelGGL((backward_dkv_mfma_kernel<T, 64>), grid, block, 0, stream, P);
    }
    return hipGetLastError();
}

hipError_t launch_row_mask_backward(const BackwardParams &P, int elem, bool use_mfma, hipStream_t stream) {
    if (static_cast<long>(P.B) * P.H * P.R == 0) return hipSuccess;
    if (use_mfma) return elem == kElemBf16 ? launch_backward_mfma<bf16_t>(P, stream) : launch_backward_mfma<f16_t>(P, stream);
    switch (elem) {
        case kElemBf16: return launch_backward_portable<bf16_t>(P, stream);
        case kElemF16: return launch_backward_portable<f16_t>(P, stream);
        default: return launch_backward_portable<float>(P, stream);
    }
}

}  // namespace artab
