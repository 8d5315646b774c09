/*
 * artab_bench.h — benchmark aids of the MI355X attention library.
 *
 * Nothing here has a counterpart in the reference (which times whole calls with perf_counter +
 * synchronize, ar_tabpfn/tests/test_triton_gpu.py:255-293), and nothing here is exported by the
 * drop-in library libartab_attention.so.  The functions below live in libartab_bench.so, a second
 * link of the same object files (same kernels, same entry points as include/artab_attention.h)
 * plus the two translation units csrc/bench_hooks.hip and csrc/mix_bench.hip.  Only bench.py
 * loads it.
 */
#ifndef ARTAB_BENCH_H
#define ARTAB_BENCH_H

#include "artab_attention.h"

#ifdef __cplusplus
extern "C" {
#endif
/* the library is built with hidden visibility; what is declared here is what it exports */
#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility push(default)
#endif

/*
 * Between artab_profile_begin and artab_profile_end every launch this library makes of
 *   kind 0  the matrix-core attention kernel (context pass of artab_context_attention /
 *           artab_decode_attention*, teacher forcing, prefill, the training row mask),
 *   kind 1  the streaming buffer pass (beside the context pass),
 *   kind 2  the register-staged buffer pass (after the context pass),
 *   kind 3  the one-launch decode kernel of small problems,
 *   kind 4  a fused layer kernel (artab_layer_*, artab_decode_sample_embed, artab_decode_step_boundary)
 * carries a pair of HIP events that receive the launch's own start and end time stamps
 * (hipExtLaunchKernelGGL), i.e. the duration a kernel trace reports for it; launches beyond
 * `max_records` are not timed.  _end waits for the events, writes the first `capacity` durations
 * (milliseconds) and kinds in launch order and returns the number of timed launches (or a
 * negative artab_status).  These two calls create events and synchronise; not thread-safe;
 * launches that are being captured into a HIP graph must not be observed.
 */
int artab_profile_begin(int max_records);
int artab_profile_end(float *each_ms, int *each_kind, int capacity);

/*
 * Time stamps taken by the matrix-core attention kernel itself (100 MHz wall clock: the earliest
 * start over the first workgroups of a launch, the end of its last workgroup), for launches that
 * cannot carry events: the ones inside a recorded HIP graph.  Between artab_stamps_begin and artab_stamps_end
 * every such launch this library makes -- or records -- points at one array in device memory that
 * the library allocates on the first call (hipMalloc; `capacity` launches; later calls may ask for
 * at most that many) and never frees, so a graph recorded in between stays valid.  _begin waits
 * for the device and clears the array; _end waits for the device, writes the durations of the
 * launches that completed since _begin, in order, in microseconds, and returns their number.
 * A stamped launch is one atomic operation per workgroup longer than an unstamped one; what a
 * kernel trace reports for the same launch is longer by the dispatch's start-up and its final
 * cache write-back, which a kernel cannot see.  Launches that share the array must be launches
 * of one queue (the context passes of a decode run are).
 */
int artab_stamps_begin(int capacity);
int artab_stamps_end(float *each_us, int capacity);

/*
 * The instruction mix of one 32x32 score block of the head_dim-32 attention kernel
 * (ar_tabpfn/model/triton_kernels.py:131-162 is the loop it stands for), issued from registers
 * with no memory traffic, to measure what the SIMD's issue port alone allows.  `workgroups`
 * workgroups of four wavefronts run `iters` (even) iterations; `lds_bytes` of dynamic LDS per
 * workgroup fixes how many share a compute unit.
 *   variant 0: 4 MFMA 32x32x16 + 16 exp2 + 8 cvt_pk + 8 dot2c    (software-pipelined pass)
 *   variant 1: 4 MFMA 32x32x16 + 2 MFMA 16x16x32 + 16 exp2 + 8 cvt_pk   (lean pass)
 *   variant 2: the matrix instructions of variant 1 alone; 3: its vector instructions alone
 * random_data != 0 fills the operands with pseudo-random bf16 values instead of constants.
 *   out     float32 [workgroups * 256] (written, contents meaningless)
 *   stamps  uint64 [workgroups * 4][2] or NULL: per wavefront, shader cycles and 100 MHz ticks spent
 * The call only launches on `stream`; the caller times it.
 */
int artab_bench_instruction_mix(int variant, int random_data, int workgroups, int iters, size_t lds_bytes,
                                float *out, unsigned long long *stamps, void *stream);

#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif

#endif /* ARTAB_BENCH_H */
