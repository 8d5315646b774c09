// Launches of the fused layer kernels (fused_layer.h).  Compiled once per element type and kernel
// group: -DARTAB_LAYER_BF16=0|1 and -DARTAB_LAYER_GROUP=0 (pre, post) | 1 (post+pre) | 2 (step tail) | 3 (step boundary);
// the type-dispatching entry points live in the bf16 object of each group.
#include "launchers.h"

#ifndef ARTAB_LAYER_BF16
#error "define ARTAB_LAYER_BF16 (0 or 1) and ARTAB_LAYER_GROUP (0 .. 3)"
#endif

namespace artab {

#if ARTAB_LAYER_BF16
typedef bf16_t LayerT;
#else
typedef f16_t LayerT;
#endif

namespace {

template <typename T, int TR>
hipError_t launch_pre_r(const FusedPreParams &P, int D, hipStream_t st) {
    dim3 grid(static_cast<unsigned>((P.rows + TR - 1) / TR)), block(fused_waves(D) * 64);
    switch (D) {
        case 128: launch_observed(kLaunchLayer, fused_pre_kernel<T, 128, TR>, grid, block, 0, st, P); break;
        case 256: launch_observed(kLaunchLayer, fused_pre_kernel<T, 256, TR>, grid, block, 0, st, P); break;
        default: launch_observed(kLaunchLayer, fused_pre_kernel<T, 512, TR>, grid, block, 0, st, P); break;
    }
    return hipGetLastError();
}
template <typename T>
hipError_t launch_pre(const FusedPreParams &P, int D, hipStream_t st) {
    return fused_tile_rows(P.rows) == kFusedRowsSmall ? launch_pre_r<T, kFusedRowsSmall>(P, D, st)
                                                      : launch_pre_r<T, kFusedRows>(P, D, st);
}

template <typename T, int D, int TR>
hipError_t launch_post_d(const FusedPostParams &P, int F, hipStream_t st) {
    dim3 grid(static_cast<unsigned>((P.rows + TR - 1) / TR)), block(fused_waves(D) * 64);
    switch (F) {
        case 128: launch_observed(kLaunchLayer, fused_post_kernel<T, D, 128, TR>, grid, block, 0, st, P); break;
        case 256: launch_observed(kLaunchLayer, fused_post_kernel<T, D, 256, TR>, grid, block, 0, st, P); break;
        default: launch_observed(kLaunchLayer, fused_post_kernel<T, D, 512, TR>, grid, block, 0, st, P); break;
    }
    return hipGetLastError();
}

// Fetcher workgroups (fetch_weights_to_l2) of a layer-boundary launch of `tiles` row tiles: 8 per
// XCD (16 and 32 measured the same or worse) while the tiles leave a quarter of the compute units
// idle, none beyond.
int layer_fetchers(long tiles) {
    static int cus_of[16] = {0};  // per device, asked once (a launch of the eager paths should not pay for it)
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) dev = -1;
    if (dev >= 0) cus = cus_of[dev];
    if (cus <= 0) {
        if (dev < 0 || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        if (dev >= 0) cus_of[dev] = cus;
    }
    const int per_xcd = tune(kTuneLayerFetchers, 4 * tiles <= 3L * cus ? 8 : 0);
    return 8 * (per_xcd < 0 ? 0 : (per_xcd > 32 ? 32 : per_xcd));
}

template <typename T, int D, int TR>
hipError_t launch_post_pre_d(const FusedPostParams &P, const FusedPreParams &N, int F, hipStream_t st) {
    const long tiles = (P.rows + TR - 1) / TR;
    dim3 grid(static_cast<unsigned>(tiles + layer_fetchers(tiles))), block(fused_waves(D) * 64);
    switch (F) {
        case 128: launch_observed(kLaunchLayer, fused_post_pre_kernel<T, D, 128, TR>, grid, block, 0, st, P.w_o, P.rows, P, N); break;
        case 256: launch_observed(kLaunchLayer, fused_post_pre_kernel<T, D, 256, TR>, grid, block, 0, st, P.w_o, P.rows, P, N); break;
        default: launch_observed(kLaunchLayer, fused_post_pre_kernel<T, D, 512, TR>, grid, block, 0, st, P.w_o, P.rows, P, N); break;
    }
    return hipGetLastError();
}

template <typename T, int TR>
hipError_t launch_post_pre_r(const FusedPostParams &P, const FusedPreParams &N, int D, int F, hipStream_t st) {
    switch (D) {
        case 128: return launch_post_pre_d<T, 128, TR>(P, N, F, st);
        case 256: return launch_post_pre_d<T, 256, TR>(P, N, F, st);
        default: return launch_post_pre_d<T, 512, TR>(P, N, F, st);
    }
}
template <typename T>
hipError_t launch_post_pre(const FusedPostParams &P, const FusedPreParams &N, int D, int F, hipStream_t st) {
    return fused_tile_rows(P.rows) == kFusedRowsSmall ? launch_post_pre_r<T, kFusedRowsSmall>(P, N, D, F, st)
                                                      : launch_post_pre_r<T, kFusedRows>(P, N, D, F, st);
}

template <typename T, int TR>
hipError_t launch_post_r(const FusedPostParams &P, int D, int F, hipStream_t st) {
    switch (D) {
        case 128: return launch_post_d<T, 128, TR>(P, F, st);
        case 256: return launch_post_d<T, 256, TR>(P, F, st);
        default: return launch_post_d<T, 512, TR>(P, F, st);
    }
}
template <typename T>
hipError_t launch_post(const FusedPostParams &P, int D, int F, hipStream_t st) {
    return fused_tile_rows(P.rows) == kFusedRowsSmall ? launch_post_r<T, kFusedRowsSmall>(P, D, F, st)
                                                      : launch_post_r<T, kFusedRows>(P, D, F, st);
}

template <typename T, int D, int TR>
hipError_t launch_sample_d(const SampleEmbedParams &P, int F, hipStream_t st) {
    dim3 grid(static_cast<unsigned>((P.B + TR - 1) / TR)), block(fused_waves(D) * 64);
    switch (F) {
        case 128: launch_observed(kLaunchLayer, sample_embed_kernel<T, D, 128, TR>, grid, block, 0, st, P); break;
        case 256: launch_observed(kLaunchLayer, sample_embed_kernel<T, D, 256, TR>, grid, block, 0, st, P); break;
        default: launch_observed(kLaunchLayer, sample_embed_kernel<T, D, 512, TR>, grid, block, 0, st, P); break;
    }
    return hipGetLastError();
}

template <typename T, int TR>
hipError_t launch_sample_r(const SampleEmbedParams &P, int D, int F, hipStream_t st) {
    switch (D) {
        case 128: return launch_sample_d<T, 128, TR>(P, F, st);
        case 256: return launch_sample_d<T, 256, TR>(P, F, st);
        default: return launch_sample_d<T, 512, TR>(P, F, st);
    }
}
template <typename T>
hipError_t launch_sample(const SampleEmbedParams &P, int D, int F, hipStream_t st) {
    return fused_tile_rows(P.B) == kFusedRowsSmall ? launch_sample_r<T, kFusedRowsSmall>(P, D, F, st)
                                                   : launch_sample_r<T, kFusedRows>(P, D, F, st);
}

template <typename T, int D>
hipError_t launch_boundary_d(const FusedPostParams &P, const SampleEmbedParams &S, const FusedPreParams &N, int F,
                             hipStream_t st) {
    constexpr int TR = kFusedRowsSmall;
    dim3 grid(static_cast<unsigned>((S.B + TR / 2 - 1) / (TR / 2))), block(fused_waves(D) * 64);
    switch (F) {
        case 128: launch_observed(kLaunchLayer, decode_step_boundary_kernel<T, D, 128, TR>, grid, block, 0, st, P, S, N); break;
        case 256: launch_observed(kLaunchLayer, decode_step_boundary_kernel<T, D, 256, TR>, grid, block, 0, st, P, S, N); break;
        default: launch_observed(kLaunchLayer, decode_step_boundary_kernel<T, D, 512, TR>, grid, block, 0, st, P, S, N); break;
    }
    return hipGetLastError();
}
template <typename T>
hipError_t launch_boundary(const FusedPostParams &P, const SampleEmbedParams &S, const FusedPreParams &N, int D, int F,
                           hipStream_t st) {
    switch (D) {
        case 128: return launch_boundary_d<T, 128>(P, S, N, F, st);
        case 256: return launch_boundary_d<T, 256>(P, S, N, F, st);
        default: return launch_boundary_d<T, 512>(P, S, N, F, st);
    }
}

}  // namespace

// fp16 forms, defined in the fp16 objects
hipError_t launch_step_boundary_f16(const FusedPostParams &P, const SampleEmbedParams &S, const FusedPreParams &N,
                                    int D, int F, hipStream_t st);
hipError_t launch_layer_pre_f16(const FusedPreParams &P, int D, hipStream_t st);
hipError_t launch_layer_post_f16(const FusedPostParams &P, int D, int F, hipStream_t st);
hipError_t launch_layer_post_pre_f16(const FusedPostParams &P, const FusedPreParams &N, int D, int F, hipStream_t st);
hipError_t launch_sample_embed_f16(const SampleEmbedParams &P, int D, int F, hipStream_t st);

#if ARTAB_LAYER_GROUP == 0
#if ARTAB_LAYER_BF16
hipError_t launch_layer_pre(const FusedPreParams &P, int D, bool is_bf16, hipStream_t st) {
    return is_bf16 ? launch_pre<LayerT>(P, D, st) : launch_layer_pre_f16(P, D, st);
}
hipError_t launch_layer_post(const FusedPostParams &P, int D, int F, bool is_bf16, hipStream_t st) {
    return is_bf16 ? launch_post<LayerT>(P, D, F, st) : launch_layer_post_f16(P, D, F, st);
}
#else
hipError_t launch_layer_pre_f16(const FusedPreParams &P, int D, hipStream_t st) { return launch_pre<LayerT>(P, D, st); }
hipError_t launch_layer_post_f16(const FusedPostParams &P, int D, int F, hipStream_t st) {
    return launch_post<LayerT>(P, D, F, st);
}
#endif
#elif ARTAB_LAYER_GROUP == 1
#if ARTAB_LAYER_BF16
hipError_t launch_layer_post_pre(const FusedPostParams &P, const FusedPreParams &N, int D, int F, bool is_bf16,
                                 hipStream_t st) {
    return is_bf16 ? launch_post_pre<LayerT>(P, N, D, F, st) : launch_layer_post_pre_f16(P, N, D, F, st);
}
#else
hipError_t launch_layer_post_pre_f16(const FusedPostParams &P, const FusedPreParams &N, int D, int F, hipStream_t st) {
    return launch_post_pre<LayerT>(P, N, D, F, st);
}
#endif
#elif ARTAB_LAYER_GROUP == 3
#if ARTAB_LAYER_BF16
hipError_t launch_step_boundary(const FusedPostParams &P, const SampleEmbedParams &S, const FusedPreParams &N, int D,
                                int F, bool is_bf16, hipStream_t st) {
    return is_bf16 ? launch_boundary<LayerT>(P, S, N, D, F, st) : launch_step_boundary_f16(P, S, N, D, F, st);
}
#else
hipError_t launch_step_boundary_f16(const FusedPostParams &P, const SampleEmbedParams &S, const FusedPreParams &N,
                                    int D, int F, hipStream_t st) {
    return launch_boundary<LayerT>(P, S, N, D, F, st);
}
#endif
#else
#if ARTAB_LAYER_BF16
hipError_t launch_sample_embed(const SampleEmbedParams &P, int D, int F, bool is_bf16, hipStream_t st) {
    return is_bf16 ? launch_sample<LayerT>(P, D, F, st) : launch_sample_embed_f16(P, D, F, st);
}
#else
hipError_t launch_sample_embed_f16(const SampleEmbedParams &P, int D, int F, hipStream_t st) {
    return launch_sample<LayerT>(P, D, F, st);
}
#endif
#endif

}  // namespace artab
