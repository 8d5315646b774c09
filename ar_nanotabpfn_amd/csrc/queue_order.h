// Ordering between two hardware queues through device memory (gfx950).
//
// A decode layer runs the context pass on one queue and the buffer pass on another.  Ordered with
// events, each dependency between the two queues costs 5-6 us on the waiting queue (a barrier
// packet, a signal, the command processor's round trip); a layer has two.  Here the two queues
// are ordered by two counters in device memory instead:
//
//   ready[main]  launches completed on the main queue whose results the side queue consumes
//                (the layer kernel that produces q and the new K/V row)
//   ready[side]  buffer passes completed on the side queue
//
// Each queue advances its own counter behind the producing kernel — with a one-thread "signal"
// launch, or by the first thread of the next kernel of that queue (the context pass does this for
// the main queue): on an in-order queue the producer has finished and released its writes before
// either starts, so a relaxed increment is enough and the producer itself pays nothing.
// (Signalling from inside the producer was tried and lost: every workgroup has to write back its
// XCD's L2 before it may count itself in, which cost more than the launch it saved.)  A queue
// waits for the other one with a one-wavefront "gate" launch placed in front of the consumer.
// The counters only ever grow and every step advances both by the same amount, so a gate needs no
// argument that changes from step to step and the launches can be recorded in a graph:
//
//   side gate:  wait until ready[main] >= ready[side] + 1   (queries of my next buffer pass exist)
//   main gate:  wait until ready[side] >= ready[main]       (every buffer pass asked for is done)
//
// A waiting workgroup must never hold registers or LDS that the kernel it waits for might still
// need to get onto the chip.  A gate launch is one wavefront with a handful of registers and is
// always safe.  A consumer may also wait inside its own workgroups (order_wait_device, one launch
// less on its queue) when its grid leaves at least half of the compute units free of them, so
// that the other queue's kernel can always be placed; the host decides.
//
// Every wait is bounded: after `limit_ticks` of the 100 MHz wall clock a gate gives up, records it
// in `failed`, and lets its queue continue (the results are then wrong and the host must discard
// them); once `failed` is set every later gate falls through at once, so a broken schedule (both
// "queues" mapped to one hardware queue, a tool that serialises launches) costs one time limit in
// all.
#pragma once

#include "common.h"

namespace artab {

constexpr int kOrderMain = 0, kOrderSide = 32, kOrderFailed = 64;  // uint32 indices: a 128-byte line each
constexpr size_t kOrderStateBytes = 512;

__device__ __forceinline__ unsigned order_load(const unsigned *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Wait of one queue for the other (see the file comment); called by one thread.
__device__ __forceinline__ void order_wait_device(unsigned *state, int side, unsigned long long limit_ticks) {
    // a queue's own counter is written by earlier launches of the same queue only: stable here
    const unsigned *other = state + (side ? kOrderMain : kOrderSide);
    unsigned *failed = state + kOrderFailed;
    const unsigned own = order_load(state + (side ? kOrderSide : kOrderMain));
    unsigned seen = order_load(other);  // both requests travel together: one round trip when nothing is pending
    const unsigned target = side ? own + 1u : own;
    if (static_cast<int>(seen - target) < 0) {
        // (the wall clock is read only when there is something to wait for: it is one unit of the
        // chip, and 128 workgroups asking it on their critical path is time the common case —
        // nothing pending — does not have to spend)
        const unsigned long long t0 = wall_clock64();
        do {
            if (order_load(failed) != 0u || wall_clock64() - t0 > limit_ticks) {
                atomicAdd(failed, 1u);
                break;
            }
            __builtin_amdgcn_s_sleep(8);
            seen = order_load(other);
        } while (static_cast<int>(seen - target) < 0);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

static __global__ __launch_bounds__(64) void order_signal_kernel(unsigned *counter) {
    if (threadIdx.x == 0) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

static __global__ __launch_bounds__(64) void order_gate_kernel(unsigned *state, int side, unsigned long long limit_ticks) {
    if (threadIdx.x == 0) order_wait_device(state, side, limit_ticks);
}

}  // namespace artab
