// Launch functions of the kernel families that are compiled in translation units of their own
// (the matrix-core attention kernel and the fused layer kernels are by far the largest pieces of
// device code; built separately they compile in parallel).
#pragma once

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "attention_backward.h"
#include "fused_layer.h"
#include "mfma_flash.h"

namespace artab {

// Route and tile-size overrides (tests and tuning).  Each has an environment variable, read ONCE
// when the library is loaded; after that only artab_tuning_set() changes a value, so a host
// process's environment cannot change kernel routes between calls.
enum Tune : int {
    kTuneBM,              // ARTAB_BM: query rows per workgroup of the matrix-core attention kernel (64/128/256)
    kTuneSplit,           // ARTAB_SPLIT: number of context slices
    kTuneSmall,           // ARTAB_SMALL: 0 keeps small decode calls off the one-launch kernel
    kTuneStream,          // ARTAB_STREAM: 1 takes the streaming buffer pass without a second stream
    kTuneStreamPerCu,     // ARTAB_STREAM_PER_CU: workgroups of the streaming buffer pass per compute unit (1..32)
    kTuneStreamPrio,      // ARTAB_STREAM_PRIO: wave priority of the streaming buffer pass (0..3)
    kTuneStreamShort,     // ARTAB_STREAM_SHORT: buffer rows above which the streaming pass reads 16-row chunks
    kTuneStreamCalm,      // ARTAB_STREAM_CALM: buffer rows up to which the streaming pass keeps the base wave priority
    kTuneDenseBelow,      // ARTAB_DENSE_BELOW: buffer rows below which the context pass runs its straight-line tile groups
    kTuneCtxYield,        // ARTAB_CTX_YIELD: buffer rows from which the context pass lowers its wave priority (0: never)
    kTuneOrderGateLaunch, // ARTAB_ORDER_GATE_LAUNCH: 1 makes the layer kernel's wait for the side queue a launch of its own
    kTuneBN,              // ARTAB_BN: keys per LDS tile at head_dim 32 (64/128)
    kTuneLean,            // ARTAB_LEAN: 0 selects the software-pipelined pass at head_dim 32
    kTuneLeanOcc,         // ARTAB_LEAN_OCC: 4 gives the lean pass 128 registers
    kTuneNW,              // ARTAB_NW: 2 = two wavefronts of two query blocks for 128-row tiles
    kTuneTileRows,        // ARTAB_TILE_ROWS: token rows per workgroup of the layer kernels (16/32)
    kTuneLayerFetchers,   // ARTAB_LAYER_FETCHERS: weight-fetching workgroups per XCD of a layer-boundary launch (0..32)
    kTuneCount
};
// The override of `key` if one is set, else `fallback` (artab_api.hip).
int tune(Tune key, int fallback);

// Token rows per workgroup of the layer kernels: 16 while that still leaves the launch within a
// few workgroups per CU (everything a workgroup does per row is bound by its one CU), else 32
// (half the weight traffic per row).
inline int fused_tile_rows(long rows) {
    const int v = tune(kTuneTileRows, 0);
    if (v == kFusedRows || v == kFusedRowsSmall) return v;
    return rows <= kFusedSmallMaxRows ? kFusedRowsSmall : kFusedRows;
}

// What a benchmark build of the library hangs on a kernel launch: a pair of events that receive
// the launch's own start and end time stamps.  The product library's implementation
// (launch_observer_none.hip) never asks for any; the benchmark build's (bench_hooks.hip) does
// between artab_profile_begin and artab_profile_end.  `kind` says which kernel family it is.
enum LaunchKind : int {
    kLaunchFlash = 0,         // matrix-core attention kernel (context pass, teacher forcing, prefill, row mask)
    kLaunchStreamBuffer = 1,  // streaming buffer pass beside the context pass
    kLaunchBuffer = 2,        // register-staged buffer pass after the context pass
    kLaunchSmallDecode = 3,   // one-launch decode of small problems
    kLaunchLayer = 4,         // fused layer kernels (pre, post, boundary between two layers, step tail, step boundary)
};
struct LaunchTiming {
    hipEvent_t start, stop;          // kObserveEvents: the launch is made with these two events
    unsigned long long *stamps;      // kObserveStamps: the kernel writes its own time stamps here
    int stamps_capacity;             //   (kLaunchFlash only; legal inside a graph capture)
};
enum : int { kObserveEvents = 1, kObserveStamps = 2 };
int observe_launch(int kind, LaunchTiming *timing);  // 0 or one of the two

template <typename Kernel, typename... Args>
inline void launch_observed(int kind, Kernel kernel, dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                            Args... args) {
    LaunchTiming t;
    if (observe_launch(kind, &t) == kObserveEvents)
        hipExtLaunchKernelGGL(kernel, grid, block, static_cast<uint32_t>(lds_bytes), stream, t.start, t.stop, 0, args...);
    else
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args...);
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
