// Launch functions of the kernel families that are compiled in translation units of their own
// (the matrix-core attention kernel and the fused layer kernels are by far the largest pieces of
// device code; built separately they compile in parallel).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdlib>

#include "attention_backward.h"
#include "fused_layer.h"
#include "mfma_flash.h"

namespace artab {

inline int env_int(const char *name, int fallback) {
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : fallback;
}

// Token rows per workgroup of the layer kernels: 16 while that still leaves the launch within a
// few workgroups per CU (everything a workgroup does per row is bound by its one CU), else 32
// (half the weight traffic per row).
inline int fused_tile_rows(long rows) {
    if (const char *e = getenv("ARTAB_TILE_ROWS")) {  // tuning / test hook
        const int v = atoi(e);
        if (v == kFusedRows || v == kFusedRowsSmall) return v;
    }
    return rows <= kFusedSmallMaxRows ? kFusedRowsSmall : kFusedRows;
}

// flash_launch.hip: BM = query rows per workgroup (256, 128 or 64), as planned by the caller
hipError_t launch_flash_dtype(const FlashParams &P, bool is_bf16, int Dh, int BM, hipStream_t stream);

// backward_launch.hip: dQ launch, then dK/dV launch, of the training row attention.  `elem` is
// the element type of every tensor; the matrix-core kernels take bf16 / f16 with head_dim 32 / 64.
enum BackwardElem : int { kElemF32 = 0, kElemBf16 = 1, kElemF16 = 2 };
hipError_t launch_row_mask_backward(const BackwardParams &P, int elem, bool use_mfma, hipStream_t stream);

// layer_launch.hip (one object per element type and kernel group)
hipError_t launch_layer_pre(const FusedPreParams &P, int D, bool is_bf16, hipStream_t st);
hipError_t launch_layer_post(const FusedPostParams &P, int D, int F, bool is_bf16, hipStream_t st);
hipError_t launch_layer_post_pre(const FusedPostParams &P, const FusedPreParams &N, int D, int F, bool is_bf16,
                                 hipStream_t st);
hipError_t launch_sample_embed(const SampleEmbedParams &P, int D, int F, bool is_bf16, hipStream_t st);
hipError_t launch_step_boundary(const FusedPostParams &P, const SampleEmbedParams &S, const FusedPreParams &N, int D,
                                int F, bool is_bf16, hipStream_t st);

}  // namespace artab
