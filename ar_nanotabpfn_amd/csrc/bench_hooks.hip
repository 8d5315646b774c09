// The launch observer of the benchmark build (libartab_bench.so) and the two calls that switch it
// on and read it out (include/artab_bench.h).  While it is on, every observed kernel launch
// (launchers.h: LaunchKind) carries a pair of events that receive the launch's own start and end time
// stamps from its dispatch packet -- the figures a kernel trace reports, without the queueing
// time that events recorded in front of and behind a launch include.
#include <hip/hip_runtime.h>

#include "../../include/artab_bench.h"
#include "launchers.h"

namespace artab {

struct ObserverState {
    bool enabled = false;
    int capacity = 0, used = 0;
    hipEvent_t *start = nullptr, *stop = nullptr;
    int *kind = nullptr;
};
static ObserverState g_obs;

// In-kernel time stamps of the matrix-core attention launches: device memory that the launches
// (also recorded ones: a graph keeps the pointer) write into.  Never freed, so that a graph
// recorded while stamps were on stays valid for the life of the process.
struct StampState {
    bool enabled = false;
    unsigned long long *dev = nullptr;
    int capacity = 0;
};
static StampState g_stamps;

int observe_launch(int kind, LaunchTiming *timing) {
    if (g_stamps.enabled && kind == kLaunchFlash) {
        timing->stamps = g_stamps.dev;
        timing->stamps_capacity = g_stamps.capacity;
        return kObserveStamps;
    }
    if (!g_obs.enabled || g_obs.used >= g_obs.capacity) return 0;
    const int slot = g_obs.used++;
    g_obs.kind[slot] = kind;
    timing->start = g_obs.start[slot];
    timing->stop = g_obs.stop[slot];
    return kObserveEvents;
}

}  // namespace artab

using namespace artab;

extern "C" {

int artab_profile_begin(int max_records) {
    if (max_records <= 0) return ARTAB_ERR_BAD_SHAPE;
    if (g_obs.capacity < max_records) {
        for (int i = 0; i < g_obs.capacity; ++i) {
            (void)hipEventDestroy(g_obs.start[i]);
            (void)hipEventDestroy(g_obs.stop[i]);
        }
        delete[] g_obs.start;
        delete[] g_obs.stop;
        delete[] g_obs.kind;
        g_obs.start = new hipEvent_t[max_records];
        g_obs.stop = new hipEvent_t[max_records];
        g_obs.kind = new int[max_records];
        g_obs.capacity = 0;
        for (int i = 0; i < max_records; ++i) {
            if (hipEventCreate(&g_obs.start[i]) != hipSuccess || hipEventCreate(&g_obs.stop[i]) != hipSuccess)
                return ARTAB_ERR_LAUNCH;
            g_obs.capacity = i + 1;
        }
    }
    g_obs.used = 0;
    g_obs.enabled = true;
    return ARTAB_OK;
}

int artab_profile_end(float *each_ms, int *each_kind, int capacity) {
    g_obs.enabled = false;
    int n = 0;
    for (int i = 0; i < g_obs.used; ++i) {
        if (hipEventSynchronize(g_obs.stop[i]) != hipSuccess) continue;
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, g_obs.start[i], g_obs.stop[i]) != hipSuccess) continue;
        if (n < capacity) {
            if (each_ms) each_ms[n] = ms;
            if (each_kind) each_kind[n] = g_obs.kind[i];
        }
        ++n;
    }
    g_obs.used = 0;
    return n;
}

int artab_stamps_begin(int capacity) {
    if (capacity <= 0) return ARTAB_ERR_BAD_SHAPE;
    if (hipDeviceSynchronize() != hipSuccess) return ARTAB_ERR_LAUNCH;
    if (!g_stamps.dev) {
        if (hipMalloc(reinterpret_cast<void **>(&g_stamps.dev), (4 + 2 * static_cast<size_t>(capacity)) * 8) != hipSuccess)
            return ARTAB_ERR_WORKSPACE;
        g_stamps.capacity = capacity;
    } else if (capacity > g_stamps.capacity) {
        return ARTAB_ERR_WORKSPACE;  // recorded launches hold the first array: it cannot grow
    }
    // counters and records zero, the slot that collects the earliest start all ones
    const size_t words = 4 + 2 * static_cast<size_t>(g_stamps.capacity);
    unsigned long long *host = new unsigned long long[words];
    for (size_t i = 0; i < words; ++i) host[i] = i == 2 ? ~0ull : 0ull;  // [2]: earliest start so far
    const hipError_t e = hipMemcpy(g_stamps.dev, host, words * 8, hipMemcpyHostToDevice);
    delete[] host;
    if (e != hipSuccess) return ARTAB_ERR_LAUNCH;
    g_stamps.enabled = true;
    return ARTAB_OK;
}

int artab_stamps_end(float *each_us, int capacity) {
    g_stamps.enabled = false;
    if (!g_stamps.dev) return 0;
    if (hipDeviceSynchronize() != hipSuccess) return ARTAB_ERR_LAUNCH;
    const size_t words = 4 + 2 * static_cast<size_t>(g_stamps.capacity);
    unsigned long long *host = new unsigned long long[words];
    if (hipMemcpy(host, g_stamps.dev, words * 8, hipMemcpyDeviceToHost) != hipSuccess) {
        delete[] host;
        return ARTAB_ERR_LAUNCH;
    }
    const unsigned long long done = host[0];
    const int n = static_cast<int>(done < static_cast<unsigned long long>(g_stamps.capacity) ? done : g_stamps.capacity);
    for (int i = 0; i < n && i < capacity; ++i)
        if (each_us) each_us[i] = static_cast<float>(host[4 + 2 * i + 1] - host[4 + 2 * i]) * 0.01f;  // 100 MHz ticks
    delete[] host;
    return n;
}

}  // extern "C"
