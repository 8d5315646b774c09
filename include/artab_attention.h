/*
 * artab_attention.h — C ABI of the MI355X (gfx950) attention library for the
 * AR-TabPFN inference hot path.
 *
 * The reference implementation (conorhassan/AR-nanoTabPFN) has no FFI layer: its
 * boundary is a set of Python callables in ar_tabpfn/model/triton_kernels.py and
 * the cache attributes handled by ar_tabpfn/model/inference.py.  Each entry point
 * below names the reference callable(s) it replaces.  A maintainer binds them
 * with ctypes (no torch types cross the boundary): device pointers, sizes,
 * element strides and a hipStream_t.
 *
 * Conventions
 *  - All tensors live in device memory of the current HIP device.  The library
 *    never allocates, frees or retains a pointer past the call, never
 *    synchronises, and launches only on `stream` (0 = the null stream).
 *  - A tensor is described by an artab_view: pointer to element [0,0,0,:] plus
 *    element strides for batch, head and row.  The head_dim axis is contiguous.
 *    A batch stride of 0 means "one copy shared by every batch entry"; that is
 *    how the shared context K/V `[H, Nc, Dh]` is passed.
 *  - dtype selects the element type of q/k/v/out (and caches); log-sum-exp
 *    outputs are always float32.  Softmax statistics and accumulation are
 *    float32 for every dtype.  A workspace is opaque scratch, 16-byte aligned
 *    (it holds the partial outputs of context slices in the input type, as the
 *    reference merges them, and their float32 log-sum-exps).
 *  - `scale` <= 0 selects the default head_dim^-0.5.
 *  - Every function returns ARTAB_OK (0) or a negative artab_status; on error
 *    nothing has been launched.  artab_last_error() gives a thread-local text.
 */
#ifndef ARTAB_ATTENTION_H
#define ARTAB_ATTENTION_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the library is built with hidden visibility; what is declared here is what it exports */
#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility push(default)
#endif

#define ARTAB_VERSION 7

typedef enum artab_dtype {
    ARTAB_BF16 = 0,
    ARTAB_F16 = 1,
    ARTAB_F32 = 2
} artab_dtype;

typedef enum artab_status {
    ARTAB_OK = 0,
    ARTAB_ERR_NULL_POINTER = -1,   /* a required pointer is NULL                       */
    ARTAB_ERR_BAD_SHAPE = -2,      /* a size is negative/zero where that is not allowed */
    ARTAB_ERR_BAD_STRIDE = -3,     /* misaligned pointer or stride for the chosen dtype */
    ARTAB_ERR_UNSUPPORTED = -4,    /* dtype / head_dim / flag combination not built     */
    ARTAB_ERR_WORKSPACE = -5,      /* workspace missing or too small                    */
    ARTAB_ERR_CAPACITY = -6,       /* buffer cache slot beyond its capacity             */
    ARTAB_ERR_LAUNCH = -7          /* hipLaunch reported an error                       */
} artab_status;

/* Selects the kernel family.  AUTO picks the MFMA kernels for 16-bit dtypes with
 * head_dim in {32, 64, 128} and the portable wave-per-row kernel otherwise. */
typedef enum artab_impl {
    ARTAB_IMPL_AUTO = 0,
    ARTAB_IMPL_PORTABLE = 1,
    ARTAB_IMPL_MFMA = 2
} artab_impl;

typedef struct artab_view {
    void *data;       /* device pointer to element [0,0,0,0]                  */
    int64_t stride_b; /* elements between batch entries (0 = shared)          */
    int64_t stride_h; /* elements between heads                                */
    int64_t stride_n; /* elements between rows; head_dim elements contiguous   */
} artab_view;

int artab_version(void);
const char *artab_status_string(int status);
const char *artab_last_error(void);

/*
 * Route and tile-size overrides, for tests and tuning; no counterpart in the reference, and a
 * drop-in caller never needs them.  Each key is also the name of an environment variable that is
 * read ONCE, when the library is loaded; afterwards only artab_tuning_set changes a value, so the
 * environment of the host process cannot change a kernel route between two calls.  Keys:
 * ARTAB_BM, ARTAB_SPLIT, ARTAB_SMALL, ARTAB_STREAM, ARTAB_STREAM_PER_CU, ARTAB_STREAM_PRIO,
 * ARTAB_STREAM_SHORT, ARTAB_STREAM_CALM, ARTAB_DENSE_BELOW, ARTAB_CTX_YIELD, ARTAB_ORDER_GATE_LAUNCH,
 * ARTAB_BN, ARTAB_LEAN, ARTAB_LEAN_OCC, ARTAB_NW, ARTAB_TILE_ROWS, ARTAB_LAYER_FETCHERS (what each
 * selects: csrc/launchers.h).
 *   artab_tuning_set: enable != 0 sets the override to `value`, enable == 0 removes it (the
 *                     library's own choice applies again).  Not thread-safe against running calls.
 *   artab_tuning_get: returns 1 if an override is set (its value in *value), 0 if not.
 * Both return ARTAB_ERR_UNSUPPORTED for an unknown key.
 */
int artab_tuning_set(const char *name, int value, int enable);
int artab_tuning_get(const char *name, int *value);

/* Bytes of workspace the split-context paths need for the given problem
 * (artab_context_attention, artab_decode_attention).  0 means no workspace is
 * needed.  Pure host arithmetic, no device access. */
size_t artab_workspace_bytes(int B, int H, int Lq, int Nc, int Dh, int dtype);

/*
 * Context attention with log-sum-exp.
 * Replaces triton_context_attention / triton_context_attention_multiq /
 * pytorch_context_attention (ar_tabpfn/model/triton_kernels.py:347-475, :532-567).
 *   q    [B,H,Lq,Dh]           out [B,H,Lq,Dh]
 *   k_ctx, v_ctx [*,H,Nc,Dh]   (stride_b 0 = shared context, else one per batch entry)
 *   lse  float32, contiguous [B,H,Lq]; may be NULL
 * Nc >= 1.
 */
int artab_context_attention(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                            const artab_view *out, float *lse,
                            int B, int H, int Lq, int Nc, int Dh, float scale, int dtype,
                            void *workspace, size_t workspace_bytes, int impl, void *stream);

/*
 * One decode step of row attention for Lq in {1,2} queries per trajectory.
 * Replaces the body of ARTabPFNPredictor._layer_decode_with_cache_shared between
 * the projections and out_proj (ar_tabpfn/model/inference.py:785-823): the two
 * hybrid_attention calls (triton_kernels.py:705-755: context pass, buffer pass,
 * merge_attention_outputs :478-524), the per-step torch.cat (:806-807) and the
 * slice-assign cache append (:816-821).
 *   q            [B,H,Lq,Dh]
 *   k_ctx,v_ctx  [*,H,Nc,Dh]   context K/V (stride_b 0 = shared)
 *   k_buf,v_buf  [B,H,cap,Dh]  preallocated buffer cache; rows [0,n_buf) are valid
 *   k_new,v_new  [B,H,1,Dh]    may be NULL (both).  When given, the row is written
 *                              in place to slot n_buf of the cache and every query
 *                              attends to rows [0,n_buf] (the new one included);
 *                              otherwise queries attend to rows [0,n_buf).
 *   out          [B,H,Lq,Dh]
 * An empty buffer (n_buf == 0 and no new row) gives context attention alone
 * (triton_kernels.py:735-741).  The caller advances n_buf (inference.py:256).
 *   n_buf_device may be NULL.  When given it points to one int32 in device memory
 *                that holds the committed length; the kernels read it when they run
 *                instead of using `n_buf`, so a launch recorded in a HIP graph can be
 *                replayed while the length advances.  `n_buf` must then be an upper
 *                bound of every value the cell will hold (it is what is validated
 *                against buf_capacity).
 * Route: a shared context with B*H small enough for every workgroup (8 trajectories of one
 * head) to be on the chip at once or twice, head_dim 32 or 64 and Nc*Dh <= 2048*64 runs as ONE
 * launch and touches no workspace; everything else as context pass (split over the workspace)
 * + buffer pass with the merge.  Both routes give the same result up to the rounding of the
 * partial results (16-bit in the workspace, float32 in the one-launch kernel).
 */
int artab_decode_attention(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                           const artab_view *k_buf, const artab_view *v_buf,
                           const artab_view *k_new, const artab_view *v_new,
                           const artab_view *out,
                           int B, int H, int Lq, int Nc, int n_buf, const int32_t *n_buf_device,
                           int buf_capacity, int Dh, float scale, int dtype,
                           void *workspace, size_t workspace_bytes, int impl, void *stream);

/*
 * artab_decode_attention for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the same kernels and results,
 * with the split-context workspace taken from a device array built into the library instead of
 * from the caller.  No counterpart in the reference.  It calls no hipMalloc, hipFree or other
 * allocating routine; inputs and outputs are still the caller's.
 *   - The array is ARTAB_STATIC_SCRATCH_BYTES per device and is held by every device the library
 *     is loaded on until the process ends.  A problem whose artab_workspace_bytes() exceeds it is
 *     rejected with ARTAB_ERR_WORKSPACE before anything is launched.
 *   - Every call on a device uses that device's one array, whose contents a call overwrites
 *     before it reads them (nothing has to be cleared): two calls that overlap in time on one
 *     device (different streams, no ordering between them) race on it.  Calls on one stream, or
 *     ordered by events, are fine.
 *   - The first call on a device looks up the array's device address (hipGetSymbolAddress, no
 *     allocation); make that first call outside a stream capture.
 */
#define ARTAB_STATIC_SCRATCH_BYTES (32u << 20)
int artab_decode_attention_static(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                                  const artab_view *k_buf, const artab_view *v_buf,
                                  const artab_view *k_new, const artab_view *v_new,
                                  const artab_view *out,
                                  int B, int H, int Lq, int Nc, int n_buf, const int32_t *n_buf_device,
                                  int buf_capacity, int Dh, float scale, int dtype, int impl, void *stream);

/*
 * artab_decode_attention with the two passes side by side.  The context pass (bound by the
 * matrix and vector units) is launched on `stream`; the buffer pass (bound by HBM) on
 * `side_stream`, forked from and joined back into `stream` with events, so the call is ordered
 * like the plain one from the caller's point of view and may be recorded into a graph.  For
 * head_dim 32 on the MFMA path the buffer pass is a streaming kernel built to share a SIMD with
 * the context pass (dot products on the matrix pipe, loads landing in LDS); it leaves its result
 * as one more partial and a combine launch on `stream` writes `out`.  The workspace of
 * artab_workspace_bytes covers the extra partial.  Same arguments, same results to rounding (the
 * merge order differs).  With a NULL side_stream, side_stream == stream, another head_dim or a
 * call the MFMA path does not cover it behaves exactly like artab_decode_attention.  Both streams
 * must belong to the current device and have the default priority.
 * The reference has no counterpart: it runs the two passes back to back
 * (ar_tabpfn/model/triton_kernels.py:705-755).
 */
int artab_decode_attention_overlapped(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                           const artab_view *k_buf, const artab_view *v_buf,
                           const artab_view *k_new, const artab_view *v_new,
                           const artab_view *out,
                           int B, int H, int Lq, int Nc, int n_buf, const int32_t *n_buf_device,
                           int buf_capacity, int Dh, float scale, int dtype,
                           void *workspace, size_t workspace_bytes, int impl, void *stream, void *side_stream);

/*
 * The attention result of a decode step left unmerged: the partial outputs of the context slices
 * and of the buffer pass with their log-sum-exps, as they lie in the caller's workspace.
 *   part_o    [n_slots][B*H*Lq][Dh]  normalised partial outputs, input type
 *   part_lse  [n_slots][B*H*Lq]      natural-log LSE of each partial (-inf = no key)
 * row (b*H + h)*Lq + i belongs to trajectory b, head h, query i.  The merged value is
 * sum_s w_s o_s / sum_s w_s with w_s = exp(lse_s - max_s lse_s) (triton_kernels.py:478-524).
 * The descriptor stays valid until the workspace is written again.
 */
typedef struct artab_attention_partials {
    const void *part_o;
    const float *part_lse;
    int n_slots;
    int B, H, Lq, Dh;
    /* Set by artab_decode_attention_partials_ordered, zero otherwise (see there): */
    uint32_t *order_state;      /* counters the consumer of these partials has to honour */
    uint64_t order_timeout_us;
    int order_flags;            /* ARTAB_ORDER_WAIT or 0 */
} artab_attention_partials;

/*
 * artab_decode_attention_overlapped without its last launch: the partials are not merged into
 * `out` but described in *partials for artab_layer_post_from_partials /
 * artab_layer_post_pre_from_partials, whose kernels merge them while they load their input — one
 * launch and one round trip of the attention output less per layer.  When the call does not
 * produce partials (another head_dim, no buffer rows and an unsplit context, the portable path)
 * it writes `out` as usual and sets partials->n_slots to 0; `out` is therefore always required.
 */
int artab_decode_attention_partials(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                           const artab_view *k_buf, const artab_view *v_buf,
                           const artab_view *k_new, const artab_view *v_new,
                           const artab_view *out,
                           int B, int H, int Lq, int Nc, int n_buf, const int32_t *n_buf_device,
                           int buf_capacity, int Dh, float scale, int dtype,
                           void *workspace, size_t workspace_bytes, int impl, void *stream, void *side_stream,
                           artab_attention_partials *partials);

/*
 * Ordering of the two streams of a decode step through device memory instead of events.  No
 * counterpart in the reference, whose decode step is a sequence of launches on one stream
 * (ar_tabpfn/model/inference.py:746-833); it exists because an event dependency between two
 * hardware queues costs 5-6 us on the waiting queue and a layer has two of them.
 *
 * `state` is ARTAB_ORDER_STATE_BYTES of device memory, 128-byte aligned, zero before the first
 * use: counter "main" (uint32 index 0), counter "side" (index 32), and `failed` (index 64).
 *   artab_order_signal(state, queue, stream)  one-thread launch on `stream`: counter[queue] += 1,
 *                                             after everything launched on `stream` before it.
 *   artab_order_wait(state, ARTAB_ORDER_SIDE, ...)  one-wavefront launch that holds `stream` until
 *                                             counter[main] >= counter[side] + 1;
 *   artab_order_wait(state, ARTAB_ORDER_MAIN, ...)  ... until counter[side] >= counter[main].
 * A wait gives up after timeout_us (0 = 2 s), adds 1 to `failed` and lets its stream continue;
 * while `failed` is non-zero every wait falls through.  The host must check `failed` before it
 * uses results ordered this way (a non-zero value means the two streams did not run
 * concurrently: they share a hardware queue, or a tool serialises launches) and fall back to
 * artab_decode_attention_partials.
 *
 * artab_decode_attention_partials_ordered is artab_decode_attention_partials with its two event
 * dependencies replaced by
 *   stream:       context pass (signals main as it starts)          wait(main)
 *   side_stream:  wait(side)    buffer pass     signal(side)
 * The caller makes side_stream wait for `stream` once before the first call of a sequence (so
 * that a graph capture covers both) and `stream` for side_stream once after the last; between
 * them no event is recorded.  Only the streaming schedule is supported (head_dim 32, bf16/fp16,
 * buffer rows or n_buf_device, side_stream != stream): anything else returns
 * ARTAB_ERR_UNSUPPORTED before a launch is made.
 *
 * On `stream` the signal costs no launch: the first thread of the context pass advances the main
 * counter (everything launched on `stream` before it is complete by then).  With
 * flags = ARTAB_ORDER_CONSUMER_WAITS the wait costs none either: the descriptor carries
 * order_state, order_timeout_us and order_flags = ARTAB_ORDER_WAIT, and whoever consumes the
 * partials (artab_layer_post_from_partials, artab_layer_post_pre_from_partials,
 * artab_merge_attention_partials) waits before reading them — inside its own workgroups when its
 * grid leaves half of the compute units free, else with a wait launch of its own.
 */
#define ARTAB_ORDER_STATE_BYTES 512
#define ARTAB_ORDER_MAIN 0
#define ARTAB_ORDER_SIDE 1
#define ARTAB_ORDER_WAIT 1            /* artab_attention_partials.order_flags */
#define ARTAB_ORDER_CONSUMER_WAITS 2  /* flags of artab_decode_attention_partials_ordered */
int artab_order_signal(uint32_t *state, int queue, void *stream);
int artab_order_wait(uint32_t *state, int queue, uint64_t timeout_us, void *stream);
int artab_decode_attention_partials_ordered(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                           const artab_view *k_buf, const artab_view *v_buf,
                           const artab_view *k_new, const artab_view *v_new,
                           const artab_view *out,
                           int B, int H, int Lq, int Nc, int n_buf, const int32_t *n_buf_device,
                           int buf_capacity, int Dh, float scale, int dtype,
                           void *workspace, size_t workspace_bytes, int impl, void *stream, void *side_stream,
                           artab_attention_partials *partials,
                                            uint32_t *order_state, uint64_t timeout_us, int flags);

/*
 * Teacher-forced attention over [Buffer_0..Nt-1, Target_0..Nt-1] queries.
 * Replaces hybrid_teacher_forcing_attention (triton_kernels.py:662-702: context
 * pass + masked buffer pass :620-659 + merge) and, with a per-batch context, the
 * flex_attention call under _create_teacher_forcing_mask
 * (inference.py:525-577, :735).  The mask is a tile schedule: buffer query i
 * sees buffer keys j <= i, target query i sees j < i, everyone sees the context,
 * target keys are never visited.
 *   q            [B,H,2*Nt,Dh]   out [B,H,2*Nt,Dh]
 *   k_ctx,v_ctx  [*,H,Nc,Dh]     (stride_b 0 = shared, else per dataset)
 *   k_buf,v_buf  [B,H,Nt,Dh]     K/V of the Nt buffer rows
 *   lse          float32 [B,H,2*Nt] contiguous, may be NULL (lse over context+buffer)
 */
int artab_teacher_forcing_attention(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                                    const artab_view *k_buf, const artab_view *v_buf,
                                    const artab_view *out, float *lse,
                                    int B, int H, int Nt, int Nc, int Dh, float scale, int dtype,
                                    int impl, void *stream);

/*
 * Context prefill: dense bidirectional self-attention plus the K/V cache write.
 * Replaces, in _layer_forward_with_cache(_shared), the cache slice-assign and the
 * flex_attention call under the dense mask (inference.py:618-622, :672-676;
 * mask from attention.py:72-83).
 *   q,k,v    [B,H,Nc,Dh]   (strided views of the [B,Nc,H*Dh] projections)
 *   out      [B,H,Nc,Dh]
 *   k_cache, v_cache  may be NULL (both).  When given, rows [0,Nc) of k and v are
 *            copied to k_cache[b,h,row,:] for b in [0, cache_batches) — use
 *            cache_batches = 1 with any stride_b for the shared `[H,Nc,Dh]` cache
 *            (only batch entry 0 is cached, inference.py:672-673) and
 *            cache_batches = B for the per-dataset cache (:618-619).
 */
int artab_prefill_attention(const artab_view *q, const artab_view *k, const artab_view *v,
                            const artab_view *out,
                            const artab_view *k_cache, const artab_view *v_cache, int cache_batches,
                            int B, int H, int Nc, int Dh, float scale, int dtype,
                            int impl, void *stream);

/*
 * Row attention of the training forward under the context / buffer / target mask.
 * Replaces flex_attention under create_row_mask (ar_tabpfn/model/attention.py:86-175), as called
 * by the training forward (ar_tabpfn/model/model.py:317-369 through :95-126).  Rows are
 * [context Nc | buffer Nb | target R - Nc - Nb]; q, k, v, out are [B,H,R,Dh].  The mask is a tile
 * schedule, not a tensor: every row sees the Nc context keys; buffer row j also sees buffer keys
 * [0, j]; target row with offset o sees buffer keys [0, o mod Nb] while o < attending_chunks * Nb
 * and no buffer key after that; target keys are never visited (no self-attention of targets).
 * lse: float32 [B,H,R] natural-log log-sum-exp of every row's scores (what the backward pass
 * needs), or NULL.  Nc >= 1.
 */
int artab_row_mask_attention(const artab_view *q, const artab_view *k, const artab_view *v, const artab_view *out,
                             float *lse, int B, int H, int R, int Nc, int Nb, int attending_chunks, int Dh,
                             float scale, int dtype, int impl, void *stream);

/*
 * Backward pass of artab_row_mask_attention: the gradients that autograd derives for
 * flex_attention under create_row_mask in the reference's training step
 * (ar_tabpfn/model/attention.py:52-61 under the mask of :86-175; ar_tabpfn/train.py:289-300).
 *   q, k, v, out, dout [B,H,R,Dh]: the forward's inputs, its output and the output's gradient;
 *   lse float32 [B,H,R]: the forward's log-sum-exp;
 *   delta float32 [B,H,R]: workspace (row sums of dout * out; written by the first launch, read by
 *                          the second);
 *   grad_q, grad_k, grad_v [B,H,R,Dh]: results, every element written (target keys get zeros).
 * With P the masked softmax: grad_v = P^T dout, dS = P o (dout v^T - delta),
 * grad_q = scale dS k, grad_k = scale dS^T q.  Two launches on `stream`, no atomics: the
 * result does not depend on the schedule.  The matrix-core kernels take bf16 / f16 with head_dim
 * 32 or 64; everything else runs the float32-arithmetic kernels.
 */
int artab_row_mask_attention_backward(const artab_view *q, const artab_view *k, const artab_view *v,
                                      const artab_view *out, const artab_view *dout, const float *lse, float *delta,
                                      const artab_view *grad_q, const artab_view *grad_k, const artab_view *grad_v,
                                      int B, int H, int R, int Nc, int Nb, int attending_chunks, int Dh, float scale,
                                      int dtype, int impl, void *stream);

/*
 * Buffer attention with log-sum-exp and an optional boolean mask.
 * Replaces pytorch_buffer_attention (triton_kernels.py:570-614).
 *   q [B,H,Lq,Dh], k_buf,v_buf [B,H,Nb,Dh], out [B,H,Lq,Dh], lse float32 [B,H,Lq] or NULL
 *   mask: uint8 (non-zero = attend), element strides (mask_sb, mask_sh, mask_sq) and
 *         contiguous along keys; NULL = no mask.  Strides of 0 broadcast.
 * Rows with no visible key give out = 0 and lse = -inf (:598-611).  Nb may be 0.
 */
int artab_buffer_attention(const artab_view *q, const artab_view *k_buf, const artab_view *v_buf,
                           const uint8_t *mask, int64_t mask_sb, int64_t mask_sh, int64_t mask_sq,
                           const artab_view *out, float *lse,
                           int B, int H, int Lq, int Nb, int Dh, float scale, int dtype, void *stream);

/*
 * Merge two partial attention results through their log-sum-exps.
 * Replaces merge_attention_outputs (triton_kernels.py:478-524).
 *   out_a, out_b, out [B,H,Lq,Dh]; lse_a, lse_b float32 contiguous [B,H,Lq].
 * A side whose lse is -inf contributes nothing; both -inf gives NaN, as the
 * reference formula does.
 */
int artab_merge_attention_outputs(const artab_view *out_a, const float *lse_a,
                                  const artab_view *out_b, const float *lse_b,
                                  const artab_view *out,
                                  int B, int H, int Lq, int Dh, int dtype, void *stream);

/*
 * Row-wise glue of the transformer layer around the attention call (the norm2 / feed-forward /
 * norm3 sequence of ar_tabpfn/model/inference.py:825-831 and the norm1 of :771-773), fused so a
 * decode step is not dominated by small launches.  Matrices are row-major with a row stride in
 * elements (ld*); `out` is contiguous [rows, D]; vectors are [D]; all of one dtype.
 *
 *   artab_add_layernorm:  out = LayerNorm(x + y + bias; gamma, beta, eps)   (y, bias may be NULL)
 *                         float32 statistics, biased variance — torch.nn.LayerNorm semantics.
 *                         D % 4 == 0, D <= 1024.
 *   artab_bias_gelu:      out = gelu(x + bias), erf form (torch.nn.GELU default); bias may be NULL.
 */
int artab_add_layernorm(const void *x, int64_t ldx, const void *y, int64_t ldy, const void *bias,
                        const void *gamma, const void *beta, void *out,
                        int64_t rows, int D, float eps, int dtype, void *stream);
int artab_bias_gelu(const void *x, int64_t ldx, const void *bias, void *out,
                    int64_t rows, int D, int dtype, void *stream);

/*
 * The whole non-attention part of one layer of the cached decode / teacher-forcing pass
 * (ar_tabpfn/model/inference.py:771-789 before the attention call, :825-831 after it) in two
 * launches.  bf16 / fp16 only; D and F (feed-forward width) in {128, 256, 512}; anything else
 * returns ARTAB_ERR_UNSUPPORTED and the caller composes the layer from GEMMs and the two
 * kernels above.  Projections carry no bias, as in ar_tabpfn/model/attention.py:23-26.
 *
 * Weights are constants of the model, so they are handed over pre-packed in the order the
 * matrix cores consume them: artab_pack_linear_weight turns a torch.nn.Linear weight W [N, K]
 * (row-major, contiguous, N % 32 == 0, K % 16 == 0) into [N/32][K/16][64][8] with
 *   packed[blk][ks][lane][e] = W[32*blk + lane%32][16*ks + 8*(lane/32) + e]
 * (same dtype, same number of elements; `packed` must not alias `w`).  Pack once per weight.
 *
 *   artab_layer_pre:   y   = LayerNorm1(x + x w_fo^T)        w_fo = pack(out_proj.weight @ v_proj.weight)
 *                      qkv = y w_qkv^T                       of the single-column feature attention,
 *                                                            w_qkv = pack([q_proj; k_proj; v_proj].weight)
 *                      x [rows, D] (row stride ldx), y [rows, D] and qkv [rows, 3D] contiguous.
 *   artab_layer_post:  x1  = LayerNorm2(y + attn w_o^T)
 *                      out = LayerNorm3(x1 + gelu(x1 w_1^T + b_1) w_2^T + b_2)
 *                      attn [rows, D] (row stride lda), y [rows, D] (row stride ldy),
 *                      out [rows, D] contiguous; w_o, w_1, w_2 packed; b_1, b_2 may be NULL.
 *   artab_layer_post_pre: artab_layer_post of one layer followed by artab_layer_pre of the next
 *                      on the same rows, in one launch: the layer output stays on chip (it is
 *                      rounded to the storage dtype exactly as if it had been stored), only the
 *                      next layer's y [rows, D] and qkv [rows, 3D] are written.
 * Accumulation, residual sums and LayerNorm statistics are float32; the intermediates x1 and
 * gelu(...) are rounded to the storage dtype once, as operands of the next product.
 */
int artab_pack_linear_weight(const void *w, void *packed, int N, int K, int dtype, void *stream);
int artab_layer_pre(const void *x, int64_t ldx, const void *w_fo, const void *ln1_gamma, const void *ln1_beta,
                    float eps1, const void *w_qkv, void *y, void *qkv,
                    int64_t rows, int D, int dtype, void *stream);
int artab_layer_post(const void *attn, int64_t lda, const void *y, int64_t ldy, const void *w_o,
                     const void *ln2_gamma, const void *ln2_beta, float eps2,
                     const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                     const void *ln3_gamma, const void *ln3_beta, float eps3, void *out,
                     int64_t rows, int D, int F, int dtype, void *stream);

/*
 * The tail of one autoregressive decode step in a single launch: final LayerNorm of the
 * target rows, the mixture-of-Gaussians head, one draw per trajectory, the write of the
 * prediction, and the embedding of the next step's [buffer, target] pair.  Replaces, for
 * dim_y = 1, ar_tabpfn/model/inference.py:278-320 (autoregressive_decode: embed -> decode ->
 * head.sample), ar_tabpfn/model/model.py:23-76 (embedder) and :150-272 (head parameters and
 * sampling) between two consecutive runs of the layer stack.
 *
 * Sampling follows the reference's law — component k with probability softmax(raw_w + weight_bias)_k,
 * then Normal(mean_k, std_k) with std_k = min(softplus(raw_s + std_bias), std_max) + std_min —
 * from caller-supplied variates: component = first k whose cumulative weight exceeds rand_u, and
 * y = mean_k + std_k * rand_n.  The step index t is read from device memory so the call can sit
 * in a recorded graph; a t outside [0, Nt) makes the launch a no-op.
 *
 * All model tensors are of `dtype` (bf16 / fp16); D and F (head hidden width) in {128, 256, 512};
 * K <= 10.  w_h1 is the packed [F, D] weight of head layer 1; w_h2 the packed [32, F] weight of
 * head layer 2 with rows >= 3K zero (output 3k + j: j = 0 mean, 1 std, 2 weight; model.py:195-196)
 * and b_h2 its bias padded to 32 entries.
 */
typedef struct artab_sample_embed_args {
    const void *x_last;      /* target row of trajectory b at x_last + b * ld_row elements, [D] */
    int64_t ld_row;
    const void *norm_gamma, *norm_beta; /* backbone.norm */
    float eps;
    const void *w_h1, *b_h1; /* head.head.0 (packed), bias [F] or NULL */
    const void *w_h2, *b_h2; /* head.head.2 padded to 32 outputs (packed), bias [32] or NULL */
    const void *mean_bias, *std_bias, *weight_bias; /* [K] */
    int K;
    float std_min, std_max;
    const float *rand_u;     /* [Nt, B] uniform in [0, 1) */
    const float *rand_n;     /* [Nt, B] standard normal */
    const void *x_mean;      /* [B, Nt] mean over features of every target row */
    const void *w_x, *b_x;   /* embedder.x_embed: weight [D, 1] as [D], bias [D] */
    const void *w_y, *b_y;   /* embedder.y_embed */
    const void *markers;     /* embedder.marker_embed.weight [3, D] */
    const void *ar_tokens;   /* [bs, D] */
    int bs;
    const int32_t *step;     /* device: index t of the target being sampled */
    int Nt;
    void *preds;             /* [B, Nt]; column t is written */
    void *emb_next;          /* [B, 2, D] contiguous: rows of step t + 1 */
    int B, D, F;
    /* Optional: the caller's device-side loop counters.  When `advance` is given, the last
     * workgroup to finish adds 1 to advance[0] .. advance[n_advance-1] (step index, buffer
     * length, ...), which saves the caller a launch per step.  `ticket` is one uint32 of device
     * memory that is zero before the first call; the kernel leaves it zero. */
    int32_t *advance;
    int n_advance;
    uint32_t *ticket;
} artab_sample_embed_args;

int artab_decode_sample_embed(const artab_sample_embed_args *args, int dtype, void *stream);

/*
 * The boundary between two decode steps in one launch: artab_layer_post (or
 * artab_layer_post_from_partials when `partials` is given and holds slots; `attn`, [B, D] with
 * row stride lda, is read otherwise) of the last layer on the B target rows y (row stride ldy),
 * artab_decode_sample_embed on its output (tail->x_last is not read), and artab_layer_pre of the
 * first layer on the 2 B rows just embedded (next_y [2B, D], next_qkv [2B, 3D]; tail->emb_next is
 * written as well).  Replaces inference.py:825-831 of the last layer, :318-320 and :355-362
 * (head, draw, next embedding) and :770-783 of the first layer of the next step.  Row for row
 * the results equal those of the three calls made one after the other, bit for bit.  The head's
 * hidden width tail->F must equal the layers' feed-forward width F; up to 4096 trajectories
 * (ARTAB_ERR_UNSUPPORTED otherwise: make the three calls).
 */
int artab_decode_step_boundary(const artab_attention_partials *partials, const void *attn, int64_t lda,
                               const void *y, int64_t ldy, const void *w_o,
                               const void *ln2_gamma, const void *ln2_beta, float eps2,
                               const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                               const void *ln3_gamma, const void *ln3_beta, float eps3,
                               const artab_sample_embed_args *tail,
                               const void *next_w_fo, const void *next_ln1_gamma, const void *next_ln1_beta,
                               float next_eps1, const void *next_w_qkv, void *next_y, void *next_qkv,
                               int F, int dtype, void *stream);

int artab_layer_post_pre(const void *attn, int64_t lda, const void *y, int64_t ldy, const void *w_o,
                         const void *ln2_gamma, const void *ln2_beta, float eps2,
                         const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                         const void *ln3_gamma, const void *ln3_beta, float eps3,
                         const void *next_w_fo, const void *next_ln1_gamma, const void *next_ln1_beta,
                         float next_eps1, const void *next_w_qkv, void *next_y, void *next_qkv,
                         int64_t rows, int D, int F, int dtype, void *stream);

/*
 * Merge of a partial descriptor into `out` [B,H,Lq,Dh] on its own: merge_attention_outputs
 * (triton_kernels.py:478-524) over n_slots operands instead of two — m = max lse, w = exp(lse - m),
 * out = sum(w * out_s) / sum(w) in float32, rounded once to the storage type.  For callers of
 * artab_decode_attention_partials whose next step is not one of the layer kernels.
 */
int artab_merge_attention_partials(const artab_attention_partials *partials, const artab_view *out, int dtype,
                                   void *stream);

/*
 * artab_layer_post / artab_layer_post_pre with the attention input given as unmerged partials
 * (artab_decode_attention_partials): token row r = b*Lq + i, columns [h*Dh, (h+1)*Dh) of the
 * attention matrix are merged from partial row (b*H + h)*Lq + i while the tile is loaded, rounded
 * once to the storage type exactly as the stand-alone merge would.  rows = B*Lq, D = H*Dh.
 */
int artab_layer_post_from_partials(const artab_attention_partials *partials, const void *y, int64_t ldy,
                                   const void *w_o, const void *ln2_gamma, const void *ln2_beta, float eps2,
                                   const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                                   const void *ln3_gamma, const void *ln3_beta, float eps3, void *out,
                                   int64_t rows, int D, int F, int dtype, void *stream);
int artab_layer_post_pre_from_partials(const artab_attention_partials *partials, const void *y, int64_t ldy,
                                       const void *w_o, const void *ln2_gamma, const void *ln2_beta, float eps2,
                                       const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                                       const void *ln3_gamma, const void *ln3_beta, float eps3,
                                       const void *next_w_fo, const void *next_ln1_gamma,
                                       const void *next_ln1_beta, float next_eps1, const void *next_w_qkv,
                                       void *next_y, void *next_qkv,
                                       int64_t rows, int D, int F, int dtype, void *stream);

#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* ARTAB_ATTENTION_H */
