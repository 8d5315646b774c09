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

bool observe_launch(int kind, LaunchTiming *timing) {
    if (!g_obs.enabled || g_obs.used >= g_obs.capacity) return false;
    const int slot = g_obs.used++;
    g_obs.kind[slot] = kind;
    timing->start = g_obs.start[slot];
    timing->stop = g_obs.stop[slot];
    return true;
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

}  // extern "C"
