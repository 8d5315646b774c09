// C ABI of the AR-TabPFN attention library for MI355X (gfx950): argument checks,
// kernel selection and launches.  See include/artab_attention.h for the contract.

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/artab_attention.h"
#include "common.h"
#include "decode_buffer.h"
#include "decode_small.h"
#include "decode_stream.h"
#include "fused_layer.h"
#include "glue_kernels.h"
#include "mfma_flash.h"
#include "portable_kernels.h"
#include "queue_order.h"
#include "launchers.h"

namespace artab {

static thread_local char g_err[512] = "";

// Route and tile-size overrides: one slot per key, filled from the environment once (the static
// initialiser below runs when the library is loaded) and afterwards only by artab_tuning_set().
struct TuneSlot {
    const char *name;
    bool set;
    int value;
};
static TuneSlot g_tune[kTuneCount] = {
    {"ARTAB_BM", false, 0},          {"ARTAB_SPLIT", false, 0},        {"ARTAB_SMALL", false, 0},
    {"ARTAB_STREAM", false, 0},      {"ARTAB_STREAM_PER_CU", false, 0}, {"ARTAB_STREAM_PRIO", false, 0},
    {"ARTAB_STREAM_SHORT", false, 0}, {"ARTAB_STREAM_CALM", false, 0},  {"ARTAB_DENSE_BELOW", false, 0},
    {"ARTAB_CTX_YIELD", false, 0},    {"ARTAB_ORDER_GATE_LAUNCH", false, 0},
    {"ARTAB_BN", false, 0},          {"ARTAB_LEAN", false, 0},         {"ARTAB_LEAN_OCC", false, 0},
    {"ARTAB_NW", false, 0},          {"ARTAB_TILE_ROWS", false, 0},    {"ARTAB_LAYER_FETCHERS", false, 0},
};
static const bool g_tune_loaded = [] {
    for (TuneSlot &t : g_tune) {
        const char *v = getenv(t.name);
        if (v && *v) {
            t.set = true;
            t.value = atoi(v);
        }
    }
    return true;
}();

int tune(Tune key, int fallback) { return g_tune[key].set ? g_tune[key].value : fallback; }

static int tune_index(const char *name) {
    if (!name) return -1;
    for (int i = 0; i < kTuneCount; ++i)
        if (strcmp(g_tune[i].name, name) == 0) return i;
    return -1;
}

static int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static inline int elem_size(int dtype) { return dtype == ARTAB_F32 ? 4 : 2; }

static inline View dv(const artab_view *v) {
    View r;
    if (v) {
        r.p = static_cast<char *>(v->data);
        r.sb = v->stride_b;
        r.sh = v->stride_h;
        r.sn = v->stride_n;
    } else {
        r.p = nullptr;
        r.sb = r.sh = r.sn = 0;
    }
    return r;
}

// Rows start on 16-byte boundaries and hold a whole number of 16-byte vectors.
static inline bool vec_aligned(const artab_view *v, int dtype, int Dh) {
    if (!v || !v->data) return true;
    const int64_t per = 16 / elem_size(dtype);
    return (reinterpret_cast<uintptr_t>(v->data) % 16 == 0) && (v->stride_b % per == 0) &&
           (v->stride_h % per == 0) && (v->stride_n % per == 0) && (Dh % per == 0);
}

static inline bool elem_aligned(const artab_view *v, int dtype) {
    return !v || !v->data || reinterpret_cast<uintptr_t>(v->data) % elem_size(dtype) == 0;
}

static int check_view(const artab_view *v, const char *name, int dtype, bool required) {
    if (!v || !v->data) {
        if (required) return fail(ARTAB_ERR_NULL_POINTER, "%s is NULL", name);
        return ARTAB_OK;
    }
    if (!elem_aligned(v, dtype)) return fail(ARTAB_ERR_BAD_STRIDE, "%s is not aligned to its element size", name);
    return ARTAB_OK;
}

static int check_common(int B, int H, int Lq, int Dh, int dtype) {
    if (dtype != ARTAB_BF16 && dtype != ARTAB_F16 && dtype != ARTAB_F32)
        return fail(ARTAB_ERR_UNSUPPORTED, "unknown dtype code %d", dtype);
    if (B < 0 || H <= 0 || Lq < 0) return fail(ARTAB_ERR_BAD_SHAPE, "bad sizes B=%d H=%d Lq=%d", B, H, Lq);
    if (Dh <= 0 || Dh > kPortableMaxDh)
        return fail(ARTAB_ERR_UNSUPPORTED, "head_dim %d outside [1,%d]", Dh, kPortableMaxDh);
    return ARTAB_OK;
}

static inline float resolve_scale(float scale, int Dh) {
    return scale > 0.f ? scale : 1.0f / std::sqrt(static_cast<float>(Dh));
}

static inline bool mfma_shape_ok(int dtype, int Dh) {
    return (dtype == ARTAB_BF16 || dtype == ARTAB_F16) && (Dh == 32 || Dh == 64 || Dh == 128);
}

// ---------------------------------------------------------------------------------------------
// Flash (MFMA) launch planning
// ---------------------------------------------------------------------------------------------

constexpr int kFlashBN = 64;
constexpr int kTargetWorkgroups = 512;  // 2 per CU on a 256-CU part

struct FlashPlan {
    int BM;        // query rows per workgroup: 256, 128 or 64
    int n_split;   // context slices
    int kv_per_split;
    int tiles_per_group;
    int n_groups;
    int G;
};

// Tile planning.  Query tiles of 256 rows (two 32-row blocks per wavefront) give the
// best MFMA-per-LDS-byte ratio; smaller tiles are used only when a group has fewer
// rows (no wavefronts of pure padding) or, for the unsplittable phases, when the
// grid would not cover the chip.  Missing parallelism on long contexts comes from
// slicing the context (each slice returns a normalised partial + log-sum-exp).
// kTuneBM / kTuneSplit override the choice.
static FlashPlan plan_flash(int B, int H, int Lq, int Nc, int Dh, bool stacked, bool allow_split) {
    FlashPlan pl;
    pl.n_groups = stacked ? 1 : B;
    pl.G = stacked ? B * Lq : Lq;
    auto wgs = [&](int bm) { return static_cast<long>((pl.G + bm - 1) / bm) * pl.n_groups * H; };
    int bm = Dh == 128 ? 128 : 256;  // head_dim 128: one 32-row block per wavefront (register budget)
    while (bm > 64 && pl.G <= bm / 2) bm /= 2;
    if (!allow_split)
        while (bm > 64 && wgs(bm) < 512) bm /= 2;
    const int bm_env = tune(kTuneBM, 0);
    if ((bm_env == 64 || bm_env == 128 || (bm_env == 256 && Dh != 128))) bm = bm_env;
    pl.BM = bm;
    pl.tiles_per_group = (pl.G + bm - 1) / bm;
    const long base = wgs(bm);
    int n_split = 1;
    if (allow_split && base < kTargetWorkgroups) {
        const int max_split = Nc / 512 > 0 ? Nc / 512 : 1;  // at least 512 keys per slice
        const int want = static_cast<int>((kTargetWorkgroups + base - 1) / base);
        n_split = want < max_split ? want : max_split;
        if (n_split > 32) n_split = 32;
        // Eight slices and the buffer pass are what the merge fetches in one round (kMergeBatch);
        // beyond one workgroup per compute unit more slices buy the context pass nothing
        // (measured at 1024 stacked rows: 31 us with 16 slices, 30 us with 8) and cost the merge a
        // second round.
        if (n_split > 8 && base * 8 >= kTargetWorkgroups / 2) n_split = 8;
        const int sp_env = tune(kTuneSplit, 0);
        if (sp_env > 0) n_split = sp_env < max_split ? sp_env : max_split;
    }
    int per = (Nc + n_split - 1) / n_split;
    per = (per + 127) / 128 * 128;  // whole LDS tiles for either tile length
    if (per <= 0) per = 128;
    pl.kv_per_split = per;
    pl.n_split = (Nc + per - 1) / per;
    if (pl.n_split < 1) pl.n_split = 1;
    return pl;
}

template <typename T, int LQ>
static hipError_t launch_decode_lq(const DecodeParams &P, int Dh, hipStream_t stream) {
    const long pairs = static_cast<long>(P.B) * P.H;
    if (pairs == 0) return hipSuccess;
    dim3 grid(static_cast<unsigned>((pairs + kDecodeWaves - 1) / kDecodeWaves)), block(kDecodeWaves * 64);
    switch (Dh) {
        case 32: launch_observed(kLaunchBuffer, decode_buffer_kernel<T, 32, LQ>, grid, block, 0, stream, P); break;
        case 64: launch_observed(kLaunchBuffer, decode_buffer_kernel<T, 64, LQ>, grid, block, 0, stream, P); break;
        default: launch_observed(kLaunchBuffer, decode_buffer_kernel<T, 128, LQ>, grid, block, 0, stream, P); break;
    }
    return hipGetLastError();
}

static hipError_t launch_decode(const DecodeParams &P, int dtype, int Dh, int Lq, hipStream_t stream) {
    if (dtype == ARTAB_BF16)
        return Lq == 1 ? launch_decode_lq<bf16_t, 1>(P, Dh, stream) : launch_decode_lq<bf16_t, 2>(P, Dh, stream);
    return Lq == 1 ? launch_decode_lq<f16_t, 1>(P, Dh, stream) : launch_decode_lq<f16_t, 2>(P, Dh, stream);
}

// The whole decode call in one launch (decode_small.h).  Worth it while the three launches of the
// general route are mostly launch latency: few enough workgroups to be on the chip at once or
// twice, and a context that a CU streams from L2 in a few microseconds (every workgroup reads its
// head's whole context: 2.6 us for 1024 rows of 64 at the ~100 GB/s a CU draws from L2).
static bool small_decode_applies(int B, int H, int Lq, int Nc, int Dh) {
    if (tune(kTuneSmall, 1) == 0 || (Dh != 32 && Dh != 64) || Lq < 1 || Lq > 2) return false;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    const long groups = static_cast<long>((B + kSmallTraj - 1) / kSmallTraj) * H;
    return groups <= 2L * cus && static_cast<long>(Nc) * Dh <= 2048L * 64;
}

template <typename T>
static hipError_t launch_small_t(const DecodeParams &P, const View &kc, const View &vc, int Nc, int Dh, int Lq,
                                 hipStream_t stream) {
    dim3 grid(static_cast<unsigned>((P.B + kSmallTraj - 1) / kSmallTraj) * P.H), block(kSmallWaves * 64);
    // the context as leading scalar arguments (the caller has checked that the strides fit)
    const char *kp = kc.p, *vp = vc.p;
    const int ksh = static_cast<int>(kc.sh), ksn = static_cast<int>(kc.sn), vsh = static_cast<int>(vc.sh),
              vsn = static_cast<int>(vc.sn);
    if (Dh == 32) {
        if (Lq == 1)
            launch_observed(kLaunchSmallDecode, decode_small_kernel<T, 32, 1>, grid, block, 0, stream, kp, vp, ksh, ksn, vsh,
                            vsn, P.H, Nc, P);
        else
            launch_observed(kLaunchSmallDecode, decode_small_kernel<T, 32, 2>, grid, block, 0, stream, kp, vp, ksh, ksn, vsh,
                            vsn, P.H, Nc, P);
    } else {
        if (Lq == 1)
            launch_observed(kLaunchSmallDecode, decode_small_kernel<T, 64, 1>, grid, block, 0, stream, kp, vp, ksh, ksn, vsh,
                            vsn, P.H, Nc, P);
        else
            launch_observed(kLaunchSmallDecode, decode_small_kernel<T, 64, 2>, grid, block, 0, stream, kp, vp, ksh, ksn, vsh,
                            vsn, P.H, Nc, P);
    }
    return hipGetLastError();
}

// The streaming buffer pass: one wavefront per workgroup.  Two of them fit on a CU beside the context
// pass, four or five once it has left (LDS).  The grid holds one workgroup per task up to 32 per CU:
// which wavefront takes which task is then the dispatcher's decision, made when a slot frees up,
// not a static deal that leaves the late starters with a full share (measured at B*H = 32768, 256
// steps: 500 target-steps/s with 4 per CU, 506 with 6, 508 with 16, 512 with 32; at B*H = 8192,
// where 8 per CU already is one per task, no difference).
template <typename T>
static hipError_t launch_stream_t(const DecodeParams &P, int Lq, hipStream_t stream) {
    const long pairs = static_cast<long>(P.B) * P.H;
    if (pairs == 0) return hipSuccess;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    const long tasks = (pairs + 3) / 4;  // of the 4-pair chunk shape; the 16-pair shape leaves the surplus idle
    long per_cu = 32;
    if (const int v = tune(kTuneStreamPerCu, 0); v >= 1 && v <= 32) per_cu = v;
    dim3 grid(static_cast<unsigned>(tasks < per_cu * cus ? tasks : per_cu * cus)), block(64);
    const int prio = tune(kTuneStreamPrio, 3);
    if (Lq == 1)
        launch_observed(kLaunchStreamBuffer, decode_stream_kernel<T, 1>, grid, block, kStreamLdsBytes, stream, P);
    else if (prio == 0)
        launch_observed(kLaunchStreamBuffer, decode_stream_kernel<T, 2, 0>, grid, block, kStreamLdsBytes, stream, P);
    else if (prio == 1)
        launch_observed(kLaunchStreamBuffer, decode_stream_kernel<T, 2, 1>, grid, block, kStreamLdsBytes, stream, P);
    else if (prio == 2)
        launch_observed(kLaunchStreamBuffer, decode_stream_kernel<T, 2, 2>, grid, block, kStreamLdsBytes, stream, P);
    else
        launch_observed(kLaunchStreamBuffer, decode_stream_kernel<T, 2>, grid, block, kStreamLdsBytes, stream, P);
    return hipGetLastError();
}

static hipError_t launch_stream(const DecodeParams &P, int dtype, int Lq, hipStream_t stream) {
    return dtype == ARTAB_BF16 ? launch_stream_t<bf16_t>(P, Lq, stream) : launch_stream_t<f16_t>(P, Lq, stream);
}

static hipError_t launch_portable_dtype(const PortableParams &P, int dtype, hipStream_t stream) {
    switch (dtype) {
        case ARTAB_BF16: return launch_portable<bf16_t>(P, stream);
        case ARTAB_F16: return launch_portable<f16_t>(P, stream);
        default: return launch_portable<float>(P, stream);
    }
}

// Combine split-context partials of arbitrary Lq into the final output: one thread
// per (row, 4 output elements).
struct CombineParams {
    View out;
    const void *part_o;  // input type
    const float *part_lse;
    float *lse;
    long rows;
    int H, Lq, Dh, n_split;
};

template <typename T>
__global__ __launch_bounds__(256) void combine_kernel(CombineParams P) {
    const int per_row = P.Dh / 4;
    long idx = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= P.rows * per_row) return;
    long row = idx / per_row;
    int d0 = static_cast<int>(idx % per_row) * 4;
    float mx = -INFINITY;
    for (int s = 0; s < P.n_split; ++s) mx = fmaxf(mx, P.part_lse[s * P.rows + row]);
    float wsum = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < P.n_split; ++s) {
        float w = merge_weight(P.part_lse[s * P.rows + row], mx);
        const T *o = static_cast<const T *>(P.part_o) + (s * P.rows + row) * P.Dh + d0;
        wsum += w;
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(w, to_f32(o[e]), acc[e]);
    }
    int i = static_cast<int>(row % P.Lq);
    int h = static_cast<int>((row / P.Lq) % P.H);
    long b = row / (static_cast<long>(P.Lq) * P.H);
    T *orow = view_row<T>(P.out, b, h, i) + d0;
    float inv = 1.f / wsum;
#pragma unroll
    for (int e = 0; e < 4; ++e) orow[e] = from_f32<T>(acc[e] * inv);
    if (P.lse && d0 == 0) P.lse[row] = mx + logf(wsum);
}

// Partial outputs in the input type (16-bit on this path) followed by float32 log-sum-exps.
static size_t split_workspace_bytes(long rows, int Dh, int n_split) {
    return static_cast<size_t>(n_split) * static_cast<size_t>(rows) * (Dh * 2 + sizeof(float));
}

static float *split_lse_base(void *workspace, long rows, int Dh, int n_split) {
    return reinterpret_cast<float *>(static_cast<char *>(workspace) + static_cast<size_t>(n_split) * rows * Dh * 2);
}

}  // namespace artab

using namespace artab;

#define ARTAB_TRY(expr)                 \
    do {                                \
        int rc__ = (expr);              \
        if (rc__ != ARTAB_OK) return rc__; \
    } while (0)

static int launch_status(hipError_t e, const char *what) {
    if (e == hipSuccess) return ARTAB_OK;
    return fail(ARTAB_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

// Event pairs for forking work onto a side stream and joining it back; a small ring per
// device, created on first use (timing disabled).  A wait binds to the record that precedes it,
// so re-recording an event of the ring later does not disturb earlier waits.
static int fork_join_events(hipEvent_t *fork, hipEvent_t *join) {
    constexpr int kDevices = 16, kRing = 8;
    struct Ring {
        hipEvent_t ev[2 * kRing];
        int next = 0;
        bool ready = false;
    };
    static Ring rings[kDevices];
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kDevices)
        return fail(ARTAB_ERR_UNSUPPORTED, "no current HIP device (or index above %d)", kDevices - 1);
    std::lock_guard<std::mutex> lock(mu);
    Ring &r = rings[dev];
    if (!r.ready) {
        for (int i = 0; i < 2 * kRing; ++i)
            if (hipEventCreateWithFlags(&r.ev[i], hipEventDisableTiming) != hipSuccess)
                return fail(ARTAB_ERR_LAUNCH, "hipEventCreateWithFlags failed");
        r.ready = true;
    }
    *fork = r.ev[2 * r.next];
    *join = r.ev[2 * r.next + 1];
    r.next = (r.next + 1) % kRing;
    return ARTAB_OK;
}

namespace {

bool fused_width_ok(int n) { return n == 128 || n == 256 || n == 512; }
bool misaligned16(const void *p) { return p && reinterpret_cast<uintptr_t>(p) % 16 != 0; }

}  // namespace

extern "C" {

int artab_version(void) { return ARTAB_VERSION; }

const char *artab_status_string(int status) {
    switch (status) {
        case ARTAB_OK: return "ok";
        case ARTAB_ERR_NULL_POINTER: return "null pointer";
        case ARTAB_ERR_BAD_SHAPE: return "bad shape";
        case ARTAB_ERR_BAD_STRIDE: return "bad stride or alignment";
        case ARTAB_ERR_UNSUPPORTED: return "unsupported dtype/head_dim/implementation";
        case ARTAB_ERR_WORKSPACE: return "workspace missing or too small";
        case ARTAB_ERR_CAPACITY: return "buffer cache capacity exceeded";
        case ARTAB_ERR_LAUNCH: return "kernel launch failed";
        default: return "unknown status";
    }
}

const char *artab_last_error(void) { return g_err; }

int artab_tuning_set(const char *name, int value, int enable) {
    const int i = tune_index(name);
    if (i < 0) return fail(ARTAB_ERR_UNSUPPORTED, "unknown tuning key %s", name ? name : "(null)");
    g_tune[i].set = enable != 0;
    g_tune[i].value = value;
    return ARTAB_OK;
}

int artab_tuning_get(const char *name, int *value) {
    const int i = tune_index(name);
    if (i < 0) return fail(ARTAB_ERR_UNSUPPORTED, "unknown tuning key %s", name ? name : "(null)");
    if (value) *value = g_tune[i].value;
    return g_tune[i].set ? 1 : 0;
}

size_t artab_workspace_bytes(int B, int H, int Lq, int Nc, int Dh, int dtype) {
    if (B <= 0 || H <= 0 || Lq <= 0 || Nc <= 0 || !mfma_shape_ok(dtype, Dh)) return 0;
    // Upper bound over the two schedules (queries stacked over a shared context, or
    // grouped per batch entry over per-dataset contexts).
    FlashPlan a = plan_flash(B, H, Lq, Nc, Dh, /*stacked=*/true, /*allow_split=*/true);
    FlashPlan b = plan_flash(B, H, Lq, Nc, Dh, /*stacked=*/false, /*allow_split=*/true);
    const int n_split = a.n_split > b.n_split ? a.n_split : b.n_split;
    // one slot more than the context slices: the streaming buffer pass leaves a partial of its own
    return split_workspace_bytes(static_cast<long>(B) * H * Lq, Dh, n_split + 1);
}

int artab_context_attention(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                            const artab_view *out, float *lse, int B, int H, int Lq, int Nc, int Dh,
                            float scale, int dtype, void *workspace, size_t workspace_bytes, int impl,
                            void *stream) {
    ARTAB_TRY(check_common(B, H, Lq, Dh, dtype));
    if (Nc < 1) return fail(ARTAB_ERR_BAD_SHAPE, "context attention needs Nc >= 1 (got %d)", Nc);
    if (B == 0 || Lq == 0) return ARTAB_OK;
    ARTAB_TRY(check_view(q, "q", dtype, true));
    ARTAB_TRY(check_view(k_ctx, "k_ctx", dtype, true));
    ARTAB_TRY(check_view(v_ctx, "v_ctx", dtype, true));
    ARTAB_TRY(check_view(out, "out", dtype, true));
    hipStream_t st = static_cast<hipStream_t>(stream);
    scale = resolve_scale(scale, Dh);
    const bool aligned = vec_aligned(q, dtype, Dh) && vec_aligned(k_ctx, dtype, Dh) &&
                         vec_aligned(v_ctx, dtype, Dh) && vec_aligned(out, dtype, Dh);
    bool use_mfma = impl != ARTAB_IMPL_PORTABLE && mfma_shape_ok(dtype, Dh) && aligned;
    if (impl == ARTAB_IMPL_MFMA && !use_mfma)
        return fail(ARTAB_ERR_UNSUPPORTED, "MFMA path needs bf16/f16, head_dim in {32,64,128}, 16-byte aligned rows");

    if (!use_mfma) {
        PortableParams P;
        memset(&P, 0, sizeof(P));
        P.q = dv(q); P.kc = dv(k_ctx); P.vc = dv(v_ctx); P.out = dv(out);
        P.lse = lse;
        P.B = B; P.H = H; P.Lq = Lq; P.Nc = Nc; P.Nb = 0;
        P.new_row = -1; P.mode = kModePlain; P.Dh = Dh; P.scale = scale;
        P.vec_ok = aligned ? 1 : 0;
        return launch_status(launch_portable_dtype(P, dtype, st), "context attention (portable)");
    }

    const bool stacked = (k_ctx->stride_b == 0 && v_ctx->stride_b == 0) || B == 1;
    const long rows = static_cast<long>(B) * H * Lq;
    FlashPlan pl = plan_flash(B, H, Lq, Nc, Dh, stacked, /*allow_split=*/true);
    if (pl.n_split > 1) {
        size_t need = split_workspace_bytes(rows, Dh, pl.n_split);
        if (!workspace || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16) {
            // Without a (usable) workspace the unsplit schedule is still correct, only less parallel.
            pl.n_split = 1;
            pl.kv_per_split = (Nc + 127) / 128 * 128;
        }
    }
    FlashParams F;
    memset(&F, 0, sizeof(F));
    F.q = dv(q); F.kc = dv(k_ctx); F.vc = dv(v_ctx); F.out = dv(out);
    F.lse = lse;
    F.B = B; F.H = H; F.Lq = Lq; F.Nc = Nc;
    F.G = pl.G; F.tiles_per_group = pl.tiles_per_group; F.n_groups = pl.n_groups;
    F.n_split = pl.n_split; F.kv_per_split = pl.kv_per_split;
    F.qscale = scale * kLog2e;
    F.mode = kFlashContext;
    if (pl.n_split > 1) {
        F.part_o = workspace;
        F.part_lse = split_lse_base(workspace, rows, Dh, pl.n_split);
    }
    {
        ARTAB_TRY(launch_status(launch_flash_dtype(F, dtype == ARTAB_BF16, Dh, pl.BM, st), "context attention (mfma)"));
    }
    if (pl.n_split > 1) {
        CombineParams C;
        C.out = dv(out); C.part_o = F.part_o; C.part_lse = F.part_lse; C.lse = lse;
        C.rows = rows; C.H = H; C.Lq = Lq; C.Dh = Dh; C.n_split = pl.n_split;
        unsigned grid = static_cast<unsigned>((rows * (Dh / 4) + 255) / 256);
        if (dtype == ARTAB_BF16)
            hipLaunchKernelGGL((combine_kernel<bf16_t>), dim3(grid), dim3(256), 0, st, C);
        else
            hipLaunchKernelGGL((combine_kernel<f16_t>), dim3(grid), dim3(256), 0, st, C);
        return launch_status(hipGetLastError(), "split combine");
    }
    return ARTAB_OK;
}

static int order_signal(uint32_t *state, int queue, hipStream_t st) {
    hipLaunchKernelGGL(order_signal_kernel, dim3(1), dim3(64), 0, st,
                       state + (queue == ARTAB_ORDER_SIDE ? kOrderSide : kOrderMain));
    return launch_status(hipGetLastError(), "queue-order signal");
}

static int order_wait(uint32_t *state, int queue, uint64_t timeout_us, hipStream_t st) {
    if (timeout_us == 0) timeout_us = 2000000;  // 2 s
    hipLaunchKernelGGL(order_gate_kernel, dim3(1), dim3(64), 0, st, state, queue == ARTAB_ORDER_SIDE ? 1 : 0,
                       static_cast<unsigned long long>(timeout_us) * 100ull);  // 100 MHz wall clock
    return launch_status(hipGetLastError(), "queue-order wait");
}

static int check_order_args(const uint32_t *state, int queue) {
    if (!state) return fail(ARTAB_ERR_NULL_POINTER, "queue-order state is NULL");
    if (reinterpret_cast<uintptr_t>(state) % 128) return fail(ARTAB_ERR_BAD_STRIDE, "queue-order state must be 128-byte aligned");
    if (queue != ARTAB_ORDER_MAIN && queue != ARTAB_ORDER_SIDE)
        return fail(ARTAB_ERR_BAD_SHAPE, "queue must be ARTAB_ORDER_MAIN or ARTAB_ORDER_SIDE, got %d", queue);
    return ARTAB_OK;
}

int artab_order_signal(uint32_t *state, int queue, void *stream) {
    ARTAB_TRY(check_order_args(state, queue));
    return order_signal(state, queue, static_cast<hipStream_t>(stream));
}

int artab_order_wait(uint32_t *state, int queue, uint64_t timeout_us, void *stream) {
    ARTAB_TRY(check_order_args(state, queue));
    return order_wait(state, queue, timeout_us, static_cast<hipStream_t>(stream));
}

constexpr long kLastLevelCacheBytes = 256L << 20;  // MI355X: 256 MiB memory-side cache in front of HBM

static int decode_impl(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                       const artab_view *k_buf, const artab_view *v_buf, const artab_view *k_new,
                       const artab_view *v_new, const artab_view *out, int B, int H, int Lq, int Nc,
                       int n_buf, const int32_t *n_buf_device, int buf_capacity, int Dh, float scale,
                       int dtype, void *workspace, size_t workspace_bytes, int impl, void *stream,
                       void *side_stream, artab_attention_partials *leave_partials = nullptr,
                       uint32_t *order_state = nullptr, uint64_t order_timeout_us = 0, int order_flags = 0) {
    if (leave_partials) memset(leave_partials, 0, sizeof(*leave_partials));
    ARTAB_TRY(check_common(B, H, Lq, Dh, dtype));
    if (Lq != 1 && Lq != 2)
        return fail(ARTAB_ERR_BAD_SHAPE, "decode supports Lq=1 (target) or Lq=2 (buffer, target); got %d", Lq);
    if (Nc < 1) return fail(ARTAB_ERR_BAD_SHAPE, "decode needs a prefilled context (Nc=%d)", Nc);
    if (n_buf < 0 || buf_capacity < 0) return fail(ARTAB_ERR_BAD_SHAPE, "negative buffer length");
    const bool k_new_given = k_new && k_new->data, v_new_given = v_new && v_new->data;
    if (k_new_given != v_new_given) return fail(ARTAB_ERR_NULL_POINTER, "k_new and v_new must be given together");
    const int has_new = k_new_given ? 1 : 0;
    if (n_buf + has_new > buf_capacity)
        return fail(ARTAB_ERR_CAPACITY, "buffer cache exceeded: %d rows + %d new > capacity %d", n_buf, has_new,
                    buf_capacity);
    if (B == 0) return ARTAB_OK;
    ARTAB_TRY(check_view(q, "q", dtype, true));
    ARTAB_TRY(check_view(k_ctx, "k_ctx", dtype, true));
    ARTAB_TRY(check_view(v_ctx, "v_ctx", dtype, true));
    ARTAB_TRY(check_view(out, "out", dtype, true));
    const bool need_buf = n_buf + has_new > 0 || n_buf_device != nullptr;
    ARTAB_TRY(check_view(k_buf, "k_buf", dtype, need_buf));
    ARTAB_TRY(check_view(v_buf, "v_buf", dtype, need_buf));
    ARTAB_TRY(check_view(k_new, "k_new", dtype, false));
    ARTAB_TRY(check_view(v_new, "v_new", dtype, false));
    hipStream_t st = static_cast<hipStream_t>(stream);
    scale = resolve_scale(scale, Dh);

    const bool aligned = vec_aligned(q, dtype, Dh) && vec_aligned(k_ctx, dtype, Dh) &&
                         vec_aligned(v_ctx, dtype, Dh) && vec_aligned(out, dtype, Dh) &&
                         vec_aligned(k_buf, dtype, Dh) && vec_aligned(v_buf, dtype, Dh) &&
                         vec_aligned(k_new, dtype, Dh) && vec_aligned(v_new, dtype, Dh);
    const bool shared_ctx = (k_ctx->stride_b == 0 && v_ctx->stride_b == 0) || B == 1;
    bool use_mfma = impl != ARTAB_IMPL_PORTABLE && mfma_shape_ok(dtype, Dh) && aligned && shared_ctx;
    const long rows = static_cast<long>(B) * H * Lq;
    // (the one-launch kernel takes the context's strides as 32-bit arguments)
    const auto fits_int = [](int64_t v) { return v >= 0 && v <= 0x7fffffffLL; };
    const bool ctx_strides_small = fits_int(k_ctx->stride_h) && fits_int(k_ctx->stride_n) &&
                                   fits_int(v_ctx->stride_h) && fits_int(v_ctx->stride_n);
    if (use_mfma && !leave_partials && !order_state && tune(kTuneStream, 0) == 0 && ctx_strides_small &&
        small_decode_applies(B, H, Lq, Nc, Dh)) {
        DecodeParams D;
        memset(&D, 0, sizeof(D));
        D.q = dv(q); D.kb = dv(k_buf); D.vb = dv(v_buf); D.knew = dv(k_new); D.vnew = dv(v_new); D.out = dv(out);
        D.B = B; D.H = H; D.n_buf = n_buf; D.n_buf_dev = n_buf_device; D.has_new = has_new;
        D.capacity = buf_capacity;
        D.qscale = scale * kLog2e;
        const View kc = dv(k_ctx), vc = dv(v_ctx);
        const hipError_t e = dtype == ARTAB_BF16 ? launch_small_t<bf16_t>(D, kc, vc, Nc, Dh, Lq, st)
                                                 : launch_small_t<f16_t>(D, kc, vc, Nc, Dh, Lq, st);
        return launch_status(e, "decode attention (one launch)");
    }
    FlashPlan pl;
    size_t need_ws = 0;
    bool stream_buf = false;
    if (use_mfma) {
        pl = plan_flash(B, H, Lq, Nc, Dh, /*stacked=*/true, /*allow_split=*/true);
        const bool direct = !need_buf && pl.n_split == 1;  // context pass writes the final output
        // the streaming buffer pass exists for head_dim 32 (the shape whose context pass leaves room
        // for it on a SIMD); it is used when the caller offers a second stream to run it on
        stream_buf = need_buf && Dh == 32 &&
                     ((side_stream && side_stream != stream) || tune(kTuneStream, 0) != 0);
        if (order_state && !(stream_buf && side_stream && side_stream != stream))
            return fail(ARTAB_ERR_UNSUPPORTED,
                        "counter-ordered decode needs the streaming buffer pass (head_dim 32, buffer rows) and a second stream");
        need_ws = direct ? 0 : split_workspace_bytes(rows, Dh, pl.n_split + (stream_buf ? 1 : 0));
        if (need_ws && (!workspace || workspace_bytes < need_ws || reinterpret_cast<uintptr_t>(workspace) % 16)) {
            if (impl == ARTAB_IMPL_MFMA)
                return fail(ARTAB_ERR_WORKSPACE, "decode needs %zu workspace bytes, got %zu", need_ws,
                            workspace_bytes);
            use_mfma = false;
        }
    } else if (impl == ARTAB_IMPL_MFMA) {
        return fail(ARTAB_ERR_UNSUPPORTED,
                    "MFMA decode needs bf16/f16, head_dim in {32,64,128}, aligned rows and a shared context");
    }
    if (order_state && !use_mfma)
        return fail(ARTAB_ERR_UNSUPPORTED, "counter-ordered decode needs the matrix-core path with its workspace");

    // Per-trajectory context stored in front of the buffer rows of the same cache (the
    // per-dataset layout, inference.py:687-744): context and buffer are one run of rows per
    // (trajectory, head), which the buffer kernel streams as it is (HBM-bound, no context pass).
    if (!use_mfma && impl != ARTAB_IMPL_PORTABLE && !shared_ctx && mfma_shape_ok(dtype, Dh) && aligned &&
        k_buf && v_buf && k_buf->data && v_buf->data) {
        const size_t esz = static_cast<size_t>(elem_size(dtype));
        auto follows = [&](const artab_view *ctx, const artab_view *buf) {
            return ctx->stride_b == buf->stride_b && ctx->stride_h == buf->stride_h && ctx->stride_n == buf->stride_n &&
                   static_cast<const char *>(buf->data) ==
                       static_cast<const char *>(ctx->data) + static_cast<size_t>(Nc) * ctx->stride_n * esz;
        };
        if (follows(k_ctx, k_buf) && follows(v_ctx, v_buf)) {
            DecodeParams D;
            memset(&D, 0, sizeof(D));
            D.q = dv(q); D.kb = dv(k_ctx); D.vb = dv(v_ctx); D.knew = dv(k_new); D.vnew = dv(v_new); D.out = dv(out);
            D.B = B; D.H = H; D.n_split = 0; D.n_buf = n_buf; D.n_buf_dev = n_buf_device; D.n_base = Nc;
            D.has_new = has_new; D.capacity = buf_capacity;
            D.qscale = scale * kLog2e;
            return launch_status(launch_decode(D, dtype, Dh, Lq, st), "decode over a per-trajectory cache");
        }
    }

    if (!use_mfma) {
        PortableParams P;
        memset(&P, 0, sizeof(P));
        P.q = dv(q); P.kc = dv(k_ctx); P.vc = dv(v_ctx); P.kb = dv(k_buf); P.vb = dv(v_buf);
        P.knew = dv(k_new); P.vnew = dv(v_new); P.out = dv(out);
        P.B = B; P.H = H; P.Lq = Lq; P.Nc = Nc; P.Nb = n_buf + has_new;
        P.new_row = has_new ? n_buf : -1;
        P.append = has_new;
        P.nbuf_dev = n_buf_device;
        P.capacity = buf_capacity;
        P.mode = kModePlain; P.Dh = Dh; P.scale = scale;
        P.vec_ok = aligned ? 1 : 0;
        return launch_status(launch_portable_dtype(P, dtype, st), "decode attention (portable)");
    }

    FlashParams F;
    memset(&F, 0, sizeof(F));
    F.q = dv(q); F.kc = dv(k_ctx); F.vc = dv(v_ctx); F.out = dv(out);
    F.B = B; F.H = H; F.Lq = Lq; F.Nc = Nc;
    F.G = pl.G; F.tiles_per_group = pl.tiles_per_group; F.n_groups = pl.n_groups;
    F.n_split = pl.n_split; F.kv_per_split = pl.kv_per_split;
    F.qscale = scale * kLog2e;
    F.mode = kFlashContext;
    const int slots = pl.n_split + (stream_buf ? 1 : 0);
    if (need_ws) {
        F.part_o = workspace;
        F.part_lse = split_lse_base(workspace, rows, Dh, slots);
    }
    DecodeParams D;
    memset(&D, 0, sizeof(D));
    D.q = dv(q); D.kb = dv(k_buf); D.vb = dv(v_buf); D.knew = dv(k_new); D.vnew = dv(v_new); D.out = dv(out);
    D.part_o = F.part_o; D.part_lse = F.part_lse; D.lse = nullptr;
    D.B = B; D.H = H; D.n_split = pl.n_split; D.n_buf = n_buf; D.n_buf_dev = n_buf_device; D.has_new = has_new;
    D.capacity = buf_capacity;
    D.qscale = scale * kLog2e;

    if (!stream_buf) {
        {
            ARTAB_TRY(launch_status(launch_flash_dtype(F, dtype == ARTAB_BF16, Dh, pl.BM, st), "decode context pass"));
        }
        if (!need_ws) return ARTAB_OK;
        if (!need_buf) {
            // A split context and nothing else: no buffer row, no new row, and k_buf / v_buf may be
            // NULL or hold no row at all.  The partials are merged by the elementwise kernel; the
            // buffer kernel (which reads the cache) is not launched.
            CombineParams C;
            C.out = dv(out); C.part_o = F.part_o; C.part_lse = F.part_lse; C.lse = nullptr;
            C.rows = rows; C.H = H; C.Lq = Lq; C.Dh = Dh; C.n_split = pl.n_split;
            const unsigned cgrid = static_cast<unsigned>((rows * (Dh / 4) + 255) / 256);
            if (dtype == ARTAB_BF16)
                hipLaunchKernelGGL((combine_kernel<bf16_t>), dim3(cgrid), dim3(256), 0, st, C);
            else
                hipLaunchKernelGGL((combine_kernel<f16_t>), dim3(cgrid), dim3(256), 0, st, C);
            return launch_status(hipGetLastError(), "decode combine (context only)");
        }
        return launch_status(launch_decode(D, dtype, Dh, Lq, st), "decode buffer pass");
    }

    // Streaming schedule: the buffer pass (HBM-bound, on the matrix pipe) leaves its result as one
    // more partial; with a side stream it runs next to the context pass (forked and joined with
    // events, so the call stays ordered on `stream` and can be recorded into a graph).
    // Chunk shape of the streaming pass: 16 rows of 4 pairs per request once the rows in use outgrow
    // the 256 MiB last-level cache (measured: B=2048, H=16, 256 steps: +5.7 % target-steps/s with
    // the switch at 64 rows, +4.6 % at 32; B=1024, H=8, whose whole cache fits: -1 % at 32 or 64
    // against never switching), 4 rows of 16 pairs below.
    {
        const long per_row = static_cast<long>(B) * H * 2 * Dh * 2;  // K and V bytes of one buffer row of every pair
        const long fit = per_row > 0 ? kLastLevelCacheBytes / per_row : 0;
        const long rows = fit > kStreamShortRows ? fit : kStreamShortRows;
        D.stream_short_rows = tune(kTuneStreamShort, static_cast<int>(rows < 1 << 20 ? rows : 1 << 20));
        // Wave priority of the streaming pass: raised only once the pass is long enough to be what the
        // layer waits for.  A short buffer pass ends long before the context pass beside it, and at
        // the raised priority it only takes issue slots from that one (measured at B=1024, H=8:
        // base priority +1.0 % target-steps/s over steps 0..63, -3 % over steps 64..95; the buffers
        // hold 64 MiB at the switch).  Only while one round of tasks covers all pairs (16 pairs per
        // task, two wavefronts per compute unit beside the context pass): with more rounds than
        // that the pass is nearly as long as its neighbour from the first row on (B=2048, H=16:
        // -0.3 % with a switch at 16 rows, so none there).
        const long one_round = 16L * 2 * 256;
        const long calm = per_row > 0 && static_cast<long>(B) * H <= one_round ? (64L << 20) / per_row : 0;
        D.stream_calm_rows = tune(kTuneStreamCalm, static_cast<int>(calm < 1 << 20 ? calm : 1 << 20));
    }
    if (side_stream && side_stream != stream) {  // the two passes share the compute units
        F.beside_rows = n_buf_device;
        F.beside_n = n_buf;
        F.dense_below = tune(kTuneDenseBelow, 128);
        // From the buffer length at which the buffer pass is about to become the longer kernel of
        // the two, the context pass runs one priority step lower: it is no longer what the layer
        // waits for.  Estimated from the work: buffer bytes at 5 TB/s against context flops at
        // 900 TFLOP/s, switch at 0.8 of the context pass's time (146 rows at B=1024, H=8,
        // N_ctx=16384; 36 at B=2048, H=16, N_ctx=4096).  Measured: +0.9 % target-steps/s over 256
        // steps at the first shape (switch anywhere in 128..192), +1.0 % at the second.
        const double ctx_flops = 4.0 * B * H * Lq * static_cast<double>(Nc) * Dh;
        const double per_row = static_cast<double>(B) * H * 2 * Dh * 2;
        const double yield_rows = per_row > 0 ? ctx_flops * 4.4e-3 / per_row : 0;
        F.yield_from = tune(kTuneCtxYield, static_cast<int>(yield_rows < 1 ? 1 : (yield_rows < 1 << 20 ? yield_rows : 1 << 20)));
    }
    D.buf_part_o = static_cast<char *>(workspace) + static_cast<size_t>(pl.n_split) * rows * Dh * 2;
    D.buf_part_lse = F.part_lse + static_cast<size_t>(pl.n_split) * rows;
    hipStream_t side = (side_stream && side_stream != stream) ? static_cast<hipStream_t>(side_stream) : st;
    if (order_state) {
        // Ordered by the two counters: the caller has forked `side` from `stream` once (and joins
        // it once, after its last call); no event per layer.
        hipStreamCaptureStatus cap_main = hipStreamCaptureStatusNone, cap_side = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cap_main) != hipSuccess || hipStreamIsCapturing(side, &cap_side) != hipSuccess)
            return fail(ARTAB_ERR_LAUNCH, "hipStreamIsCapturing failed");
        if (cap_main != cap_side)
            return fail(ARTAB_ERR_UNSUPPORTED,
                        "counter-ordered decode: one stream is being captured and the other is not; make the side "
                        "stream wait for the main one before the first call");
        F.started = order_state + kOrderMain;  // q and the new K/V row are ready once the context pass starts
        ARTAB_TRY(order_wait(order_state, ARTAB_ORDER_SIDE, order_timeout_us, side));
        hipError_t e_ctx, e_buf;
        {
            e_ctx = launch_flash_dtype(F, dtype == ARTAB_BF16, Dh, pl.BM, st);
        }
        e_buf = launch_stream(D, dtype, Lq, side);
        ARTAB_TRY(launch_status(e_ctx, "decode context pass"));
        ARTAB_TRY(launch_status(e_buf, "decode buffer pass (stream)"));
        ARTAB_TRY(order_signal(order_state, ARTAB_ORDER_SIDE, side));    // the buffer pass's partial is ready
        if (order_flags & ARTAB_ORDER_CONSUMER_WAITS) {
            leave_partials->order_state = order_state;
            leave_partials->order_timeout_us = order_timeout_us;
            leave_partials->order_flags = ARTAB_ORDER_WAIT;
        } else {
            ARTAB_TRY(order_wait(order_state, ARTAB_ORDER_MAIN, order_timeout_us, st));
        }
        leave_partials->part_o = F.part_o; leave_partials->part_lse = F.part_lse; leave_partials->n_slots = slots;
        leave_partials->B = B; leave_partials->H = H; leave_partials->Lq = Lq; leave_partials->Dh = Dh;
        return ARTAB_OK;
    }
    hipEvent_t fork = nullptr, join = nullptr;
    if (side != st) {
        ARTAB_TRY(fork_join_events(&fork, &join));
        hipError_t e = hipEventRecord(fork, st);
        if (e == hipSuccess) e = hipStreamWaitEvent(side, fork, 0);
        if (e != hipSuccess) return launch_status(e, "decode fork");
    }
    hipError_t e_ctx, e_buf, e_join = hipSuccess;
    {
        e_ctx = launch_flash_dtype(F, dtype == ARTAB_BF16, Dh, pl.BM, st);
    }
    e_buf = launch_stream(D, dtype, Lq, side);
    if (side != st) {
        // always rejoin, so that a failed launch does not leave the side stream forked (e.g. inside a capture)
        e_join = hipEventRecord(join, side);
        if (e_join == hipSuccess) e_join = hipStreamWaitEvent(st, join, 0);
    }
    ARTAB_TRY(launch_status(e_ctx, "decode context pass"));
    ARTAB_TRY(launch_status(e_buf, "decode buffer pass (stream)"));
    ARTAB_TRY(launch_status(e_join, "decode join"));
    if (leave_partials) {  // the caller's next kernel merges them (artab_layer_post*_from_partials)
        leave_partials->part_o = F.part_o; leave_partials->part_lse = F.part_lse; leave_partials->n_slots = slots;
        leave_partials->B = B; leave_partials->H = H; leave_partials->Lq = Lq; leave_partials->Dh = Dh;
        return ARTAB_OK;
    }
    CombineParams C;
    C.out = dv(out); C.part_o = F.part_o; C.part_lse = F.part_lse; C.lse = nullptr;
    C.rows = rows; C.H = H; C.Lq = Lq; C.Dh = Dh; C.n_split = slots;
    unsigned cgrid = static_cast<unsigned>((rows * (Dh / 4) + 255) / 256);
    if (dtype == ARTAB_BF16)
        hipLaunchKernelGGL((combine_kernel<bf16_t>), dim3(cgrid), dim3(256), 0, st, C);
    else
        hipLaunchKernelGGL((combine_kernel<f16_t>), dim3(cgrid), dim3(256), 0, st, C);
    return launch_status(hipGetLastError(), "decode combine");
}

int artab_merge_attention_partials(const artab_attention_partials *partials, const artab_view *out, int dtype,
                                   void *stream) {
    if (!partials || !out || !out->data) return fail(ARTAB_ERR_NULL_POINTER, "merge partials: null argument");
    if (dtype != ARTAB_BF16 && dtype != ARTAB_F16)
        return fail(ARTAB_ERR_UNSUPPORTED, "merge partials: partial outputs exist in bf16/fp16 only");
    if (partials->n_slots < 1 || !partials->part_o || !partials->part_lse || partials->B < 1 || partials->H < 1 ||
        partials->Lq < 1 || partials->Dh < 4 || partials->Dh % 4)
        return fail(ARTAB_ERR_BAD_SHAPE, "merge partials: empty or malformed descriptor");
    CombineParams C;
    C.out = dv(out); C.part_o = partials->part_o; C.part_lse = partials->part_lse; C.lse = nullptr;
    C.rows = static_cast<long>(partials->B) * partials->H * partials->Lq;
    C.H = partials->H; C.Lq = partials->Lq; C.Dh = partials->Dh; C.n_split = partials->n_slots;
    unsigned grid = static_cast<unsigned>((C.rows * (C.Dh / 4) + 255) / 256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (partials->order_flags & ARTAB_ORDER_WAIT) {
        ARTAB_TRY(check_order_args(partials->order_state, ARTAB_ORDER_MAIN));
        ARTAB_TRY(order_wait(partials->order_state, ARTAB_ORDER_MAIN, partials->order_timeout_us, st));
    }
    if (dtype == ARTAB_BF16)
        hipLaunchKernelGGL((combine_kernel<bf16_t>), dim3(grid), dim3(256), 0, st, C);
    else
        hipLaunchKernelGGL((combine_kernel<f16_t>), dim3(grid), dim3(256), 0, st, C);
    return launch_status(hipGetLastError(), "merge partials");
}

int artab_decode_attention(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                           const artab_view *k_buf, const artab_view *v_buf, const artab_view *k_new,
                           const artab_view *v_new, const artab_view *out, int B, int H, int Lq, int Nc,
                           int n_buf, const int32_t *n_buf_device, int buf_capacity, int Dh, float scale,
                           int dtype, void *workspace, size_t workspace_bytes, int impl, void *stream) {
    return decode_impl(q, k_ctx, v_ctx, k_buf, v_buf, k_new, v_new, out, B, H, Lq, Nc, n_buf, n_buf_device,
                       buf_capacity, Dh, scale, dtype, workspace, workspace_bytes, impl, stream, nullptr);
}

// ---------------------------------------------------------------------------------------------
// The entry point that allocates nothing: the split-context workspace of artab_decode_attention
// in a file-scope device array instead of caller memory.
// ---------------------------------------------------------------------------------------------

static __device__ __align__(256) unsigned char scratch[ARTAB_STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current device.  In host code the array's name is only a
// stand-in for the symbol, and every device holds its own copy at its own address: the address
// is looked up once per device, with that device current, and kept.
static int static_scratch(void **ptr) {
    constexpr int kDevices = 16;
    static void *addr[kDevices];
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kDevices)
        return fail(ARTAB_ERR_UNSUPPORTED, "no current HIP device (or index above %d)", kDevices - 1);
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(ARTAB_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        addr[dev] = p;
    }
    *ptr = addr[dev];
    return ARTAB_OK;
}

int artab_decode_attention_static(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                                  const artab_view *k_buf, const artab_view *v_buf, const artab_view *k_new,
                                  const artab_view *v_new, const artab_view *out, int B, int H, int Lq, int Nc,
                                  int n_buf, const int32_t *n_buf_device, int buf_capacity, int Dh, float scale,
                                  int dtype, int impl, void *stream) {
    // the bound that artab_workspace_bytes gives callers of artab_decode_attention
    const size_t need = artab_workspace_bytes(B, H, Lq, Nc, Dh, dtype);
    if (need > static_cast<size_t>(ARTAB_STATIC_SCRATCH_BYTES))
        return fail(ARTAB_ERR_WORKSPACE,
                    "artab_decode_attention_static: this problem needs %zu bytes of scratch, the built-in array holds "
                    "%zu; use artab_decode_attention with a workspace of your own",
                    need, static_cast<size_t>(ARTAB_STATIC_SCRATCH_BYTES));
    void *ws = nullptr;
    ARTAB_TRY(static_scratch(&ws));
    return decode_impl(q, k_ctx, v_ctx, k_buf, v_buf, k_new, v_new, out, B, H, Lq, Nc, n_buf, n_buf_device,
                       buf_capacity, Dh, scale, dtype, ws, static_cast<size_t>(ARTAB_STATIC_SCRATCH_BYTES), impl, stream,
                       nullptr);
}

int artab_decode_attention_partials(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                                    const artab_view *k_buf, const artab_view *v_buf, const artab_view *k_new,
                                    const artab_view *v_new, const artab_view *out, int B, int H, int Lq, int Nc,
                                    int n_buf, const int32_t *n_buf_device, int buf_capacity, int Dh, float scale,
                                    int dtype, void *workspace, size_t workspace_bytes, int impl, void *stream,
                                    void *side_stream, artab_attention_partials *partials) {
    if (!partials) return fail(ARTAB_ERR_NULL_POINTER, "partials descriptor is NULL");
    return decode_impl(q, k_ctx, v_ctx, k_buf, v_buf, k_new, v_new, out, B, H, Lq, Nc, n_buf, n_buf_device,
                       buf_capacity, Dh, scale, dtype, workspace, workspace_bytes, impl, stream, side_stream, partials);
}

int artab_decode_attention_partials_ordered(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                                            const artab_view *k_buf, const artab_view *v_buf, const artab_view *k_new,
                                            const artab_view *v_new, const artab_view *out, int B, int H, int Lq,
                                            int Nc, int n_buf, const int32_t *n_buf_device, int buf_capacity, int Dh,
                                            float scale, int dtype, void *workspace, size_t workspace_bytes, int impl,
                                            void *stream, void *side_stream, artab_attention_partials *partials,
                                            uint32_t *order_state, uint64_t timeout_us, int flags) {
    if (!partials) return fail(ARTAB_ERR_NULL_POINTER, "partials descriptor is NULL");
    ARTAB_TRY(check_order_args(order_state, ARTAB_ORDER_MAIN));
    if (flags & ~ARTAB_ORDER_CONSUMER_WAITS)
        return fail(ARTAB_ERR_BAD_SHAPE, "unknown ordering flags 0x%x", flags);
    return decode_impl(q, k_ctx, v_ctx, k_buf, v_buf, k_new, v_new, out, B, H, Lq, Nc, n_buf, n_buf_device,
                       buf_capacity, Dh, scale, dtype, workspace, workspace_bytes, impl, stream, side_stream, partials,
                       order_state, timeout_us, flags);
}

int artab_decode_attention_overlapped(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                                      const artab_view *k_buf, const artab_view *v_buf, const artab_view *k_new,
                                      const artab_view *v_new, const artab_view *out, int B, int H, int Lq, int Nc,
                                      int n_buf, const int32_t *n_buf_device, int buf_capacity, int Dh, float scale,
                                      int dtype, void *workspace, size_t workspace_bytes, int impl, void *stream,
                                      void *side_stream) {
    return decode_impl(q, k_ctx, v_ctx, k_buf, v_buf, k_new, v_new, out, B, H, Lq, Nc, n_buf, n_buf_device,
                       buf_capacity, Dh, scale, dtype, workspace, workspace_bytes, impl, stream, side_stream);
}

int artab_teacher_forcing_attention(const artab_view *q, const artab_view *k_ctx, const artab_view *v_ctx,
                                    const artab_view *k_buf, const artab_view *v_buf, const artab_view *out,
                                    float *lse, int B, int H, int Nt, int Nc, int Dh, float scale, int dtype,
                                    int impl, void *stream) {
    ARTAB_TRY(check_common(B, H, 2 * Nt, Dh, dtype));
    if (Nt < 0) return fail(ARTAB_ERR_BAD_SHAPE, "negative num_targets");
    if (Nc < 1) return fail(ARTAB_ERR_BAD_SHAPE, "teacher forcing needs a context (Nc=%d)", Nc);
    if (B == 0 || Nt == 0) return ARTAB_OK;
    ARTAB_TRY(check_view(q, "q", dtype, true));
    ARTAB_TRY(check_view(k_ctx, "k_ctx", dtype, true));
    ARTAB_TRY(check_view(v_ctx, "v_ctx", dtype, true));
    ARTAB_TRY(check_view(k_buf, "k_buf", dtype, true));
    ARTAB_TRY(check_view(v_buf, "v_buf", dtype, true));
    ARTAB_TRY(check_view(out, "out", dtype, true));
    hipStream_t st = static_cast<hipStream_t>(stream);
    scale = resolve_scale(scale, Dh);
    const bool aligned = vec_aligned(q, dtype, Dh) && vec_aligned(k_ctx, dtype, Dh) &&
                         vec_aligned(v_ctx, dtype, Dh) && vec_aligned(out, dtype, Dh) &&
                         vec_aligned(k_buf, dtype, Dh) && vec_aligned(v_buf, dtype, Dh);
    const bool use_mfma = impl != ARTAB_IMPL_PORTABLE && mfma_shape_ok(dtype, Dh) && aligned;
    if (impl == ARTAB_IMPL_MFMA && !use_mfma)
        return fail(ARTAB_ERR_UNSUPPORTED, "MFMA path needs bf16/f16, head_dim in {32,64,128}, 16-byte aligned rows");
    const int Lq = 2 * Nt;
    if (!use_mfma) {
        PortableParams P;
        memset(&P, 0, sizeof(P));
        P.q = dv(q); P.kc = dv(k_ctx); P.vc = dv(v_ctx); P.kb = dv(k_buf); P.vb = dv(v_buf); P.out = dv(out);
        P.lse = lse;
        P.B = B; P.H = H; P.Lq = Lq; P.Nc = Nc; P.Nb = Nt; P.Nt = Nt;
        P.new_row = -1; P.mode = kModeTeacher; P.Dh = Dh; P.scale = scale;
        P.vec_ok = aligned ? 1 : 0;
        return launch_status(launch_portable_dtype(P, dtype, st), "teacher forcing (portable)");
    }
    FlashPlan pl = plan_flash(B, H, Lq, Nc, Dh, /*stacked=*/false, /*allow_split=*/false);
    FlashParams F;
    memset(&F, 0, sizeof(F));
    F.q = dv(q); F.kc = dv(k_ctx); F.vc = dv(v_ctx); F.kb = dv(k_buf); F.vb = dv(v_buf); F.out = dv(out);
    F.lse = lse;
    F.B = B; F.H = H; F.Lq = Lq; F.Nc = Nc; F.Nb = Nt; F.Nt = Nt;
    F.G = pl.G; F.tiles_per_group = pl.tiles_per_group; F.n_groups = pl.n_groups;
    F.n_split = 1; F.kv_per_split = pl.kv_per_split;
    F.qscale = scale * kLog2e;
    F.mode = kFlashTeacher;
    return launch_status(launch_flash_dtype(F, dtype == ARTAB_BF16, Dh, pl.BM, st), "teacher forcing (mfma)");
}

// More attending chunks than the target rows can fill change nothing; clamped so that
// attending_chunks * Nb (the kernels' comparison) stays far from the integer range.
static int clamp_attending_chunks(int attending_chunks, int R, int Nb) {
    const int most = R / (Nb > 0 ? Nb : 1) + 1;
    return attending_chunks < most ? attending_chunks : most;
}

int artab_row_mask_attention(const artab_view *q, const artab_view *k, const artab_view *v, const artab_view *out,
                             float *lse, int B, int H, int R, int Nc, int Nb, int attending_chunks, int Dh, float scale,
                             int dtype, int impl, void *stream) {
    ARTAB_TRY(check_common(B, H, R, Dh, dtype));
    if (Nc < 1 || Nb < 0 || Nc + Nb > R || attending_chunks < 0)
        return fail(ARTAB_ERR_BAD_SHAPE, "row mask needs 1 <= Nc, 0 <= Nb, Nc + Nb <= R, attending_chunks >= 0 (got Nc=%d Nb=%d R=%d A=%d)",
                    Nc, Nb, R, attending_chunks);
    if (B == 0 || R == 0) return ARTAB_OK;
    attending_chunks = clamp_attending_chunks(attending_chunks, R, Nb);
    ARTAB_TRY(check_view(q, "q", dtype, true));
    ARTAB_TRY(check_view(k, "k", dtype, true));
    ARTAB_TRY(check_view(v, "v", dtype, true));
    ARTAB_TRY(check_view(out, "out", dtype, true));
    hipStream_t st = static_cast<hipStream_t>(stream);
    scale = resolve_scale(scale, Dh);
    const bool aligned = vec_aligned(q, dtype, Dh) && vec_aligned(k, dtype, Dh) && vec_aligned(v, dtype, Dh) &&
                         vec_aligned(out, dtype, Dh);
    const bool use_mfma = impl != ARTAB_IMPL_PORTABLE && mfma_shape_ok(dtype, Dh) && aligned;
    if (impl == ARTAB_IMPL_MFMA && !use_mfma)
        return fail(ARTAB_ERR_UNSUPPORTED, "MFMA path needs bf16/f16, head_dim in {32,64,128}, 16-byte aligned rows");
    // buffer keys: rows [Nc, Nc + Nb) of the same tensors
    View kb = dv(k), vb = dv(v);
    kb.p += static_cast<size_t>(Nc) * k->stride_n * elem_size(dtype);
    vb.p += static_cast<size_t>(Nc) * v->stride_n * elem_size(dtype);
    if (!use_mfma) {
        PortableParams P;
        memset(&P, 0, sizeof(P));
        P.q = dv(q); P.kc = dv(k); P.vc = dv(v); P.kb = kb; P.vb = vb; P.out = dv(out);
        P.B = B; P.H = H; P.Lq = R; P.Nc = Nc; P.Nb = Nb;
        P.rm_nc = Nc; P.rm_attend = attending_chunks; P.lse = lse;
        P.new_row = -1; P.mode = kModeRowMask; P.Dh = Dh; P.scale = scale;
        P.vec_ok = aligned ? 1 : 0;
        return launch_status(launch_portable_dtype(P, dtype, st), "row-mask attention (portable)");
    }
    FlashPlan pl = plan_flash(B, H, R, Nc, Dh, /*stacked=*/false, /*allow_split=*/false);
    FlashParams F;
    memset(&F, 0, sizeof(F));
    F.q = dv(q); F.kc = dv(k); F.vc = dv(v); F.kb = kb; F.vb = vb; F.out = dv(out);
    F.B = B; F.H = H; F.Lq = R; F.Nc = Nc; F.Nb = Nb;
    F.rm_nc = Nc; F.rm_attend = attending_chunks; F.lse = lse;
    F.G = pl.G; F.tiles_per_group = pl.tiles_per_group; F.n_groups = pl.n_groups;
    F.n_split = 1; F.kv_per_split = pl.kv_per_split;
    F.qscale = scale * kLog2e;
    F.mode = kFlashRowMask;
    return launch_status(launch_flash_dtype(F, dtype == ARTAB_BF16, Dh, pl.BM, st), "row-mask attention (mfma)");
}

int artab_row_mask_attention_backward(const artab_view *q, const artab_view *k, const artab_view *v,
                                      const artab_view *out, const artab_view *dout, const float *lse, float *delta,
                                      const artab_view *grad_q, const artab_view *grad_k, const artab_view *grad_v,
                                      int B, int H, int R, int Nc, int Nb, int attending_chunks, int Dh, float scale,
                                      int dtype, int impl, void *stream) {
    ARTAB_TRY(check_common(B, H, R, Dh, dtype));
    if (Nc < 1 || Nb < 0 || Nc + Nb > R || attending_chunks < 0)
        return fail(ARTAB_ERR_BAD_SHAPE, "row mask needs 1 <= Nc, 0 <= Nb, Nc + Nb <= R, attending_chunks >= 0 (got Nc=%d Nb=%d R=%d A=%d)",
                    Nc, Nb, R, attending_chunks);
    if (B == 0 || R == 0) return ARTAB_OK;
    const artab_view *views[8] = {q, k, v, out, dout, grad_q, grad_k, grad_v};
    const char *names[8] = {"q", "k", "v", "out", "dout", "grad_q", "grad_k", "grad_v"};
    bool aligned = true;
    for (int i = 0; i < 8; ++i) {
        ARTAB_TRY(check_view(views[i], names[i], dtype, true));
        aligned = aligned && vec_aligned(views[i], dtype, Dh);
    }
    if (!lse || !delta) return fail(ARTAB_ERR_NULL_POINTER, "lse and delta must be given");
    attending_chunks = clamp_attending_chunks(attending_chunks, R, Nb);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool use_mfma = impl != ARTAB_IMPL_PORTABLE && (dtype == ARTAB_BF16 || dtype == ARTAB_F16) &&
                          (Dh == 32 || Dh == 64) && aligned;
    if (impl == ARTAB_IMPL_MFMA && !use_mfma)
        return fail(ARTAB_ERR_UNSUPPORTED, "MFMA backward needs bf16/f16, head_dim in {32,64}, 16-byte aligned rows");
    BackwardParams P;
    memset(&P, 0, sizeof(P));
    P.q = dv(q); P.k = dv(k); P.v = dv(v); P.out = dv(out); P.dout = dv(dout);
    P.dq = dv(grad_q); P.dk = dv(grad_k); P.dv = dv(grad_v);
    P.lse = lse; P.delta = delta;
    P.B = B; P.H = H; P.R = R; P.Nc = Nc; P.Nb = Nb; P.attend = attending_chunks;
    P.Dh = Dh; P.scale = resolve_scale(scale, Dh); P.vec_ok = aligned ? 1 : 0;
    const int elem = dtype == ARTAB_BF16 ? kElemBf16 : dtype == ARTAB_F16 ? kElemF16 : kElemF32;
    return launch_status(launch_row_mask_backward(P, elem, use_mfma, st),
                         use_mfma ? "row-mask attention backward (mfma)" : "row-mask attention backward (portable)");
}

int artab_prefill_attention(const artab_view *q, const artab_view *k, const artab_view *v, const artab_view *out,
                            const artab_view *k_cache, const artab_view *v_cache, int cache_batches, int B, int H,
                            int Nc, int Dh, float scale, int dtype, int impl, void *stream) {
    ARTAB_TRY(check_common(B, H, Nc, Dh, dtype));
    if (B == 0 || Nc == 0) return ARTAB_OK;
    ARTAB_TRY(check_view(q, "q", dtype, true));
    ARTAB_TRY(check_view(k, "k", dtype, true));
    ARTAB_TRY(check_view(v, "v", dtype, true));
    ARTAB_TRY(check_view(out, "out", dtype, true));
    const bool kc_given = k_cache && k_cache->data, vc_given = v_cache && v_cache->data;
    if (kc_given != vc_given) return fail(ARTAB_ERR_NULL_POINTER, "k_cache and v_cache must be given together");
    if (kc_given && (cache_batches < 1 || cache_batches > B))
        return fail(ARTAB_ERR_BAD_SHAPE, "cache_batches=%d outside [1,%d]", cache_batches, B);
    ARTAB_TRY(check_view(k_cache, "k_cache", dtype, false));
    ARTAB_TRY(check_view(v_cache, "v_cache", dtype, false));
    hipStream_t st = static_cast<hipStream_t>(stream);
    scale = resolve_scale(scale, Dh);
    const bool aligned = vec_aligned(q, dtype, Dh) && vec_aligned(k, dtype, Dh) && vec_aligned(v, dtype, Dh) &&
                         vec_aligned(out, dtype, Dh) && vec_aligned(k_cache, dtype, Dh) &&
                         vec_aligned(v_cache, dtype, Dh);
    const bool use_mfma = impl != ARTAB_IMPL_PORTABLE && mfma_shape_ok(dtype, Dh) && aligned;
    if (impl == ARTAB_IMPL_MFMA && !use_mfma)
        return fail(ARTAB_ERR_UNSUPPORTED, "MFMA path needs bf16/f16, head_dim in {32,64,128}, 16-byte aligned rows");
    if (!use_mfma) {
        PortableParams P;
        memset(&P, 0, sizeof(P));
        P.q = dv(q); P.kc = dv(k); P.vc = dv(v); P.out = dv(out);
        P.kcache = dv(kc_given ? k_cache : nullptr); P.vcache = dv(kc_given ? v_cache : nullptr);
        P.cache_batches = kc_given ? cache_batches : 0;
        P.B = B; P.H = H; P.Lq = Nc; P.Nc = Nc; P.Nb = 0;
        P.new_row = -1; P.mode = kModePlain; P.Dh = Dh; P.scale = scale;
        P.vec_ok = aligned ? 1 : 0;
        return launch_status(launch_portable_dtype(P, dtype, st), "prefill (portable)");
    }
    FlashPlan pl = plan_flash(B, H, Nc, Nc, Dh, /*stacked=*/false, /*allow_split=*/false);
    FlashParams F;
    memset(&F, 0, sizeof(F));
    F.q = dv(q); F.kc = dv(k); F.vc = dv(v); F.out = dv(out);
    F.kcache = dv(kc_given ? k_cache : nullptr); F.vcache = dv(kc_given ? v_cache : nullptr);
    F.cache_batches = kc_given ? cache_batches : 0;
    F.B = B; F.H = H; F.Lq = Nc; F.Nc = Nc;
    F.G = pl.G; F.tiles_per_group = pl.tiles_per_group; F.n_groups = pl.n_groups;
    F.n_split = 1; F.kv_per_split = pl.kv_per_split;
    F.qscale = scale * kLog2e;
    F.mode = kFlashPrefill;
    return launch_status(launch_flash_dtype(F, dtype == ARTAB_BF16, Dh, pl.BM, st), "prefill (mfma)");
}

int artab_buffer_attention(const artab_view *q, const artab_view *k_buf, const artab_view *v_buf,
                           const uint8_t *mask, int64_t mask_sb, int64_t mask_sh, int64_t mask_sq,
                           const artab_view *out, float *lse, int B, int H, int Lq, int Nb, int Dh, float scale,
                           int dtype, void *stream) {
    ARTAB_TRY(check_common(B, H, Lq, Dh, dtype));
    if (Nb < 0) return fail(ARTAB_ERR_BAD_SHAPE, "negative buffer length");
    if (B == 0 || Lq == 0) return ARTAB_OK;
    ARTAB_TRY(check_view(q, "q", dtype, true));
    ARTAB_TRY(check_view(out, "out", dtype, true));
    ARTAB_TRY(check_view(k_buf, "k_buf", dtype, Nb > 0));
    ARTAB_TRY(check_view(v_buf, "v_buf", dtype, Nb > 0));
    PortableParams P;
    memset(&P, 0, sizeof(P));
    P.q = dv(q); P.kb = dv(k_buf); P.vb = dv(v_buf); P.out = dv(out);
    P.lse = lse;
    P.mask = mask; P.m_sb = mask_sb; P.m_sh = mask_sh; P.m_sq = mask_sq;
    P.B = B; P.H = H; P.Lq = Lq; P.Nc = 0; P.Nb = Nb;
    P.new_row = -1; P.mode = mask ? kModeMasked : kModePlain; P.Dh = Dh;
    P.scale = resolve_scale(scale, Dh);
    P.vec_ok = (vec_aligned(q, dtype, Dh) && vec_aligned(k_buf, dtype, Dh) && vec_aligned(v_buf, dtype, Dh)) ? 1 : 0;
    return launch_status(launch_portable_dtype(P, dtype, static_cast<hipStream_t>(stream)), "buffer attention");
}

int artab_merge_attention_outputs(const artab_view *out_a, const float *lse_a, const artab_view *out_b,
                                  const float *lse_b, const artab_view *out, int B, int H, int Lq, int Dh,
                                  int dtype, void *stream) {
    ARTAB_TRY(check_common(B, H, Lq, Dh, dtype));
    if (B == 0 || Lq == 0) return ARTAB_OK;
    ARTAB_TRY(check_view(out_a, "out_a", dtype, true));
    ARTAB_TRY(check_view(out_b, "out_b", dtype, true));
    ARTAB_TRY(check_view(out, "out", dtype, true));
    if (!lse_a || !lse_b) return fail(ARTAB_ERR_NULL_POINTER, "lse_a / lse_b is NULL");
    MergeParams P;
    P.a = dv(out_a); P.b = dv(out_b); P.out = dv(out);
    P.lse_a = lse_a; P.lse_b = lse_b;
    P.rows = static_cast<long>(B) * H * Lq; P.H = H; P.Lq = Lq; P.Dh = Dh;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e;
    switch (dtype) {
        case ARTAB_BF16: e = launch_merge<bf16_t>(P, st); break;
        case ARTAB_F16: e = launch_merge<f16_t>(P, st); break;
        default: e = launch_merge<float>(P, st); break;
    }
    return launch_status(e, "merge");
}

int artab_add_layernorm(const void *x, int64_t ldx, const void *y, int64_t ldy, const void *bias, const void *gamma,
                        const void *beta, void *out, int64_t rows, int D, float eps, int dtype, void *stream) {
    if (dtype != ARTAB_BF16 && dtype != ARTAB_F16 && dtype != ARTAB_F32)
        return fail(ARTAB_ERR_UNSUPPORTED, "unknown dtype code %d", dtype);
    if (rows < 0 || D <= 0) return fail(ARTAB_ERR_BAD_SHAPE, "bad sizes rows=%lld D=%d", (long long)rows, D);
    if (D % 4 || D > 256 * kGlueMaxPerLane)
        return fail(ARTAB_ERR_UNSUPPORTED, "add_layernorm needs D %% 4 == 0 and D <= %d (got %d)", 256 * kGlueMaxPerLane, D);
    if (rows == 0) return ARTAB_OK;
    if (!x || !gamma || !beta || !out) return fail(ARTAB_ERR_NULL_POINTER, "x, gamma, beta and out are required");
    const int64_t per = 16 / elem_size(dtype) / 2;  // 4-element vectors: 8 bytes (16-bit) or 16 bytes (float32)
    const uintptr_t align = dtype == ARTAB_F32 ? 16 : 8;
    auto bad = [&](const void *p) { return p && reinterpret_cast<uintptr_t>(p) % align != 0; };
    if (bad(x) || bad(y) || bad(bias) || bad(gamma) || bad(beta) || bad(out) || ldx % 4 || (y && ldy % 4))
        return fail(ARTAB_ERR_BAD_STRIDE, "add_layernorm operands must be aligned to 4 elements");
    (void)per;
    AddLayerNormParams P;
    P.x = x; P.y = y; P.bias = bias; P.gamma = gamma; P.beta = beta; P.out = out;
    P.rows = rows; P.ldx = ldx; P.ldy = ldy; P.D = D; P.eps = eps;
    dim3 grid(static_cast<unsigned>((rows + kGlueWaves - 1) / kGlueWaves)), block(kGlueWaves * 64);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case ARTAB_BF16: hipLaunchKernelGGL((add_layernorm_kernel<bf16_t>), grid, block, 0, st, P); break;
        case ARTAB_F16: hipLaunchKernelGGL((add_layernorm_kernel<f16_t>), grid, block, 0, st, P); break;
        default: hipLaunchKernelGGL((add_layernorm_kernel<float>), grid, block, 0, st, P); break;
    }
    return launch_status(hipGetLastError(), "add_layernorm");
}

int artab_bias_gelu(const void *x, int64_t ldx, const void *bias, void *out, int64_t rows, int D, int dtype,
                    void *stream) {
    if (dtype != ARTAB_BF16 && dtype != ARTAB_F16 && dtype != ARTAB_F32)
        return fail(ARTAB_ERR_UNSUPPORTED, "unknown dtype code %d", dtype);
    if (rows < 0 || D <= 0) return fail(ARTAB_ERR_BAD_SHAPE, "bad sizes rows=%lld D=%d", (long long)rows, D);
    if (D % 4) return fail(ARTAB_ERR_UNSUPPORTED, "bias_gelu needs D %% 4 == 0 (got %d)", D);
    if (rows == 0) return ARTAB_OK;
    if (!x || !out) return fail(ARTAB_ERR_NULL_POINTER, "x and out are required");
    const uintptr_t align = dtype == ARTAB_F32 ? 16 : 8;
    auto bad = [&](const void *p) { return p && reinterpret_cast<uintptr_t>(p) % align != 0; };
    if (bad(x) || bad(bias) || bad(out) || ldx % 4)
        return fail(ARTAB_ERR_BAD_STRIDE, "bias_gelu operands must be aligned to 4 elements");
    BiasGeluParams P;
    P.x = x; P.bias = bias; P.out = out; P.rows = rows; P.ldx = ldx; P.D = D;
    const long total = rows * (D / 4);
    dim3 grid(static_cast<unsigned>((total + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case ARTAB_BF16: hipLaunchKernelGGL((bias_gelu_kernel<bf16_t>), grid, dim3(256), 0, st, P); break;
        case ARTAB_F16: hipLaunchKernelGGL((bias_gelu_kernel<f16_t>), grid, dim3(256), 0, st, P); break;
        default: hipLaunchKernelGGL((bias_gelu_kernel<float>), grid, dim3(256), 0, st, P); break;
    }
    return launch_status(hipGetLastError(), "bias_gelu");
}

int artab_pack_linear_weight(const void *w, void *packed, int N, int K, int dtype, void *stream) {
    if (dtype != ARTAB_BF16 && dtype != ARTAB_F16)
        return fail(ARTAB_ERR_UNSUPPORTED, "pack_linear_weight supports bf16 and fp16 only (dtype code %d)", dtype);
    if (N <= 0 || K <= 0 || N % 32 || K % 16)
        return fail(ARTAB_ERR_BAD_SHAPE, "pack_linear_weight needs N %% 32 == 0 and K %% 16 == 0 (got %d, %d)", N, K);
    if (!w || !packed) return fail(ARTAB_ERR_NULL_POINTER, "w and packed are required");
    if (misaligned16(w) || misaligned16(packed)) return fail(ARTAB_ERR_BAD_STRIDE, "w and packed must be 16-byte aligned");
    const char *a = static_cast<const char *>(w), *b = static_cast<const char *>(packed);
    const size_t bytes = static_cast<size_t>(N) * K * 2;
    if (a < b + bytes && b < a + bytes) return fail(ARTAB_ERR_BAD_STRIDE, "packed must not overlap w");
    const long chunks = static_cast<long>(N) * K / 8;
    dim3 grid(static_cast<unsigned>((chunks + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == ARTAB_BF16)
        hipLaunchKernelGGL((pack_weight_kernel<bf16_t>), grid, dim3(256), 0, st, static_cast<const bf16_t *>(w),
                           static_cast<bf16_t *>(packed), N, K);
    else
        hipLaunchKernelGGL((pack_weight_kernel<f16_t>), grid, dim3(256), 0, st, static_cast<const f16_t *>(w),
                           static_cast<f16_t *>(packed), N, K);
    return launch_status(hipGetLastError(), "pack_linear_weight");
}

static int fill_pre(FusedPreParams &P, const void *x, int64_t ldx, const void *w_fo, const void *ln1_gamma,
                    const void *ln1_beta, float eps1, const void *w_qkv, void *y, void *qkv, int64_t rows, int D,
                    bool x_required) {
    if (!fused_width_ok(D)) return fail(ARTAB_ERR_UNSUPPORTED, "layer_pre needs D in {128, 256, 512} (got %d)", D);
    if ((x_required && !x) || !w_fo || !ln1_gamma || !ln1_beta || !w_qkv || !y || !qkv)
        return fail(ARTAB_ERR_NULL_POINTER, "layer_pre: every pointer is required");
    if (misaligned16(x) || misaligned16(w_fo) || misaligned16(w_qkv) || misaligned16(y) || misaligned16(qkv) ||
        misaligned16(ln1_gamma) || misaligned16(ln1_beta) || (x_required && (ldx % 8 || ldx < D)))
        return fail(ARTAB_ERR_BAD_STRIDE, "layer_pre operands must be 16-byte aligned with ldx %% 8 == 0, ldx >= D");
    P.x = x; P.ldx = ldx; P.w_fo = w_fo; P.g1 = ln1_gamma; P.b1 = ln1_beta; P.w_qkv = w_qkv;
    P.y = y; P.qkv = qkv; P.rows = rows; P.eps = eps1;
    return ARTAB_OK;
}

static int fill_post(FusedPostParams &P, const void *attn, int64_t lda, const void *y, int64_t ldy, const void *w_o,
                     const void *ln2_gamma, const void *ln2_beta, float eps2, const void *w_1, const void *b_1,
                     const void *w_2, const void *b_2, const void *ln3_gamma, const void *ln3_beta, float eps3,
                     void *out, int64_t rows, int D, int F, bool out_required,
                     const artab_attention_partials *parts = nullptr) {
    if (!fused_width_ok(D) || !fused_width_ok(F))
        return fail(ARTAB_ERR_UNSUPPORTED, "layer_post needs D and F in {128, 256, 512} (got %d, %d)", D, F);
    if (parts) {
        if (!parts->part_o || !parts->part_lse) return fail(ARTAB_ERR_NULL_POINTER, "partials are NULL");
        if (parts->n_slots < 1 || parts->H < 1 || parts->Lq < 1 || parts->B < 0 || parts->Dh < 8 || parts->Dh % 8 ||
            parts->H * parts->Dh != D || static_cast<int64_t>(parts->B) * parts->Lq != rows)
            return fail(ARTAB_ERR_BAD_SHAPE,
                        "partials (B=%d H=%d Lq=%d Dh=%d, %d slots) do not describe %lld rows of width %d", parts->B,
                        parts->H, parts->Lq, parts->Dh, parts->n_slots, (long long)rows, D);
        if (misaligned16(parts->part_o)) return fail(ARTAB_ERR_BAD_STRIDE, "partials must be 16-byte aligned");
        if (static_cast<int64_t>(parts->B) * parts->H * parts->Lq >= (int64_t{1} << 31))
            return fail(ARTAB_ERR_BAD_SHAPE, "partials: B*H*Lq must stay below 2^31");  // the kernel indexes rows in 32 bits
        P.part_o = parts->part_o; P.part_lse = parts->part_lse; P.n_slots = parts->n_slots;
        P.part_rows = static_cast<long>(parts->B) * parts->H * parts->Lq; P.H = parts->H; P.Lq = parts->Lq;
        attn = parts->part_o;  // placeholder for the checks below
        lda = D;
    }
    if (!attn || !y || !w_o || !ln2_gamma || !ln2_beta || !w_1 || !w_2 || !ln3_gamma || !ln3_beta ||
        (out_required && !out))
        return fail(ARTAB_ERR_NULL_POINTER, "layer_post: only b_1 and b_2 may be NULL");
    if (misaligned16(attn) || misaligned16(y) || misaligned16(w_o) || misaligned16(w_1) || misaligned16(w_2) ||
        misaligned16(b_1) || misaligned16(b_2) || misaligned16(ln2_gamma) || misaligned16(ln2_beta) ||
        misaligned16(ln3_gamma) || misaligned16(ln3_beta) || misaligned16(out) || lda % 8 || ldy % 8 || lda < D ||
        ldy < D)
        return fail(ARTAB_ERR_BAD_STRIDE, "layer_post operands must be 16-byte aligned with row strides %% 8 == 0");
    P.attn = attn; P.lda = lda; P.y = y; P.ldy = ldy; P.w_o = w_o; P.g2 = ln2_gamma; P.b2 = ln2_beta;
    P.w_1 = w_1; P.bias_1 = b_1; P.w_2 = w_2; P.bias_2 = b_2; P.g3 = ln3_gamma; P.b3 = ln3_beta;
    P.out = out; P.rows = rows; P.eps2 = eps2; P.eps3 = eps3;
    return ARTAB_OK;
}

// Ordering that a partial descriptor asks of its consumer.  The wait goes into the kernel when its grid leaves half of the compute units
// free — a waiting workgroup must not keep the buffer pass it waits for off the chip — and into a
// launch of its own otherwise.
static int apply_partials_order(const artab_attention_partials *parts, FusedPostParams &P, int64_t rows,
                                hipStream_t st, int64_t grid_of_launch = -1) {
    if (!parts || !(parts->order_flags & ARTAB_ORDER_WAIT)) return ARTAB_OK;
    ARTAB_TRY(check_order_args(parts->order_state, ARTAB_ORDER_MAIN));
    if (rows == 0) return fail(ARTAB_ERR_BAD_SHAPE, "ordered partials with no rows");
    {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            cus = 0;
        const int64_t grid =
            grid_of_launch >= 0 ? grid_of_launch : (rows + fused_tile_rows(rows) - 1) / fused_tile_rows(rows);
        const uint64_t us = parts->order_timeout_us ? parts->order_timeout_us : 2000000;
        if (grid * 2 <= cus && tune(kTuneOrderGateLaunch, 0) == 0) {
            P.order_wait = parts->order_state;
            P.order_limit = us * 100ull;  // 100 MHz wall clock
        } else {
            ARTAB_TRY(order_wait(parts->order_state, ARTAB_ORDER_MAIN, us, st));
        }
    }
    return ARTAB_OK;
}

static int check_layer_dtype_rows(const char *what, int dtype, int64_t rows) {
    if (dtype != ARTAB_BF16 && dtype != ARTAB_F16)
        return fail(ARTAB_ERR_UNSUPPORTED, "%s supports bf16 and fp16 only (dtype code %d)", what, dtype);
    if (rows < 0) return fail(ARTAB_ERR_BAD_SHAPE, "%s: negative row count %lld", what, (long long)rows);
    return ARTAB_OK;
}

int artab_layer_pre(const void *x, int64_t ldx, const void *w_fo, const void *ln1_gamma, const void *ln1_beta,
                    float eps1, const void *w_qkv, void *y, void *qkv, int64_t rows, int D, int dtype,
                    void *stream) {
    ARTAB_TRY(check_layer_dtype_rows("layer_pre", dtype, rows));
    FusedPreParams P{};
    ARTAB_TRY(fill_pre(P, x, ldx, w_fo, ln1_gamma, ln1_beta, eps1, w_qkv, y, qkv, rows, D, true));
    if (rows == 0) return ARTAB_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e = launch_layer_pre(P, D, dtype == ARTAB_BF16, st);
    return launch_status(e, "layer_pre");
}

int artab_layer_post(const void *attn, int64_t lda, const void *y, int64_t ldy, const void *w_o,
                     const void *ln2_gamma, const void *ln2_beta, float eps2, const void *w_1, const void *b_1,
                     const void *w_2, const void *b_2, const void *ln3_gamma, const void *ln3_beta, float eps3,
                     void *out, int64_t rows, int D, int F, int dtype, void *stream) {
    ARTAB_TRY(check_layer_dtype_rows("layer_post", dtype, rows));
    FusedPostParams P{};
    ARTAB_TRY(fill_post(P, attn, lda, y, ldy, w_o, ln2_gamma, ln2_beta, eps2, w_1, b_1, w_2, b_2, ln3_gamma,
                        ln3_beta, eps3, out, rows, D, F, true));
    if (rows == 0) return ARTAB_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e = launch_layer_post(P, D, F, dtype == ARTAB_BF16, st);
    return launch_status(e, "layer_post");
}

static int layer_post_pre_impl(const artab_attention_partials *parts, const void *attn, int64_t lda, const void *y,
                               int64_t ldy, const void *w_o, const void *ln2_gamma, const void *ln2_beta, float eps2,
                               const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                               const void *ln3_gamma, const void *ln3_beta, float eps3, const void *next_w_fo,
                               const void *next_ln1_gamma, const void *next_ln1_beta, float next_eps1,
                               const void *next_w_qkv, void *next_y, void *next_qkv, int64_t rows, int D, int F,
                               int dtype, void *stream) {
    ARTAB_TRY(check_layer_dtype_rows("layer_post_pre", dtype, rows));
    FusedPostParams P{};
    FusedPreParams N{};
    ARTAB_TRY(fill_post(P, attn, lda, y, ldy, w_o, ln2_gamma, ln2_beta, eps2, w_1, b_1, w_2, b_2, ln3_gamma,
                        ln3_beta, eps3, nullptr, rows, D, F, false, parts));
    ARTAB_TRY(fill_pre(N, nullptr, 0, next_w_fo, next_ln1_gamma, next_ln1_beta, next_eps1, next_w_qkv, next_y,
                       next_qkv, rows, D, false));
    hipStream_t st = static_cast<hipStream_t>(stream);
    ARTAB_TRY(apply_partials_order(parts, P, rows, st));
    if (rows == 0) return ARTAB_OK;
    hipError_t e = launch_layer_post_pre(P, N, D, F, dtype == ARTAB_BF16, st);
    return launch_status(e, "layer_post_pre");
}

int artab_layer_post_pre(const void *attn, int64_t lda, const void *y, int64_t ldy, const void *w_o,
                         const void *ln2_gamma, const void *ln2_beta, float eps2, const void *w_1, const void *b_1,
                         const void *w_2, const void *b_2, const void *ln3_gamma, const void *ln3_beta, float eps3,
                         const void *next_w_fo, const void *next_ln1_gamma, const void *next_ln1_beta,
                         float next_eps1, const void *next_w_qkv, void *next_y, void *next_qkv, int64_t rows, int D,
                         int F, int dtype, void *stream) {
    return layer_post_pre_impl(nullptr, attn, lda, y, ldy, w_o, ln2_gamma, ln2_beta, eps2, w_1, b_1, w_2, b_2,
                               ln3_gamma, ln3_beta, eps3, next_w_fo, next_ln1_gamma, next_ln1_beta, next_eps1,
                               next_w_qkv, next_y, next_qkv, rows, D, F, dtype, stream);
}

int artab_layer_post_pre_from_partials(const artab_attention_partials *parts, const void *y, int64_t ldy,
                                       const void *w_o, const void *ln2_gamma, const void *ln2_beta, float eps2,
                                       const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                                       const void *ln3_gamma, const void *ln3_beta, float eps3,
                                       const void *next_w_fo, const void *next_ln1_gamma,
                                       const void *next_ln1_beta, float next_eps1, const void *next_w_qkv,
                                       void *next_y, void *next_qkv, int64_t rows, int D, int F, int dtype,
                                       void *stream) {
    if (!parts) return fail(ARTAB_ERR_NULL_POINTER, "partials descriptor is NULL");
    return layer_post_pre_impl(parts, nullptr, 0, y, ldy, w_o, ln2_gamma, ln2_beta, eps2, w_1, b_1, w_2, b_2,
                               ln3_gamma, ln3_beta, eps3, next_w_fo, next_ln1_gamma, next_ln1_beta, next_eps1,
                               next_w_qkv, next_y, next_qkv, rows, D, F, dtype, stream);
}

int artab_layer_post_from_partials(const artab_attention_partials *parts, const void *y, int64_t ldy,
                                   const void *w_o, const void *ln2_gamma, const void *ln2_beta, float eps2,
                                   const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                                   const void *ln3_gamma, const void *ln3_beta, float eps3, void *out, int64_t rows,
                                   int D, int F, int dtype, void *stream) {
    if (!parts) return fail(ARTAB_ERR_NULL_POINTER, "partials descriptor is NULL");
    ARTAB_TRY(check_layer_dtype_rows("layer_post", dtype, rows));
    FusedPostParams P{};
    ARTAB_TRY(fill_post(P, nullptr, 0, y, ldy, w_o, ln2_gamma, ln2_beta, eps2, w_1, b_1, w_2, b_2, ln3_gamma,
                        ln3_beta, eps3, out, rows, D, F, true, parts));
    hipStream_t st = static_cast<hipStream_t>(stream);
    ARTAB_TRY(apply_partials_order(parts, P, rows, st));
    if (rows == 0) return ARTAB_OK;
    hipError_t e = launch_layer_post(P, D, F, dtype == ARTAB_BF16, st);
    return launch_status(e, "layer_post");
}

static int fill_sample(SampleEmbedParams &P, const artab_sample_embed_args *a, int dtype, bool x_required) {
    if (!a) return fail(ARTAB_ERR_NULL_POINTER, "args is NULL");
    if (dtype != ARTAB_BF16 && dtype != ARTAB_F16)
        return fail(ARTAB_ERR_UNSUPPORTED, "decode_sample_embed supports bf16 and fp16 only (dtype code %d)", dtype);
    if (a->B < 0 || a->Nt <= 0 || a->K <= 0 || a->bs <= 0)
        return fail(ARTAB_ERR_BAD_SHAPE, "bad sizes B=%d Nt=%d K=%d bs=%d", a->B, a->Nt, a->K, a->bs);
    if (!fused_width_ok(a->D) || !fused_width_ok(a->F) || a->K > kMaxMixture)
        return fail(ARTAB_ERR_UNSUPPORTED, "decode_sample_embed needs D, F in {128, 256, 512} and K <= %d (got %d, %d, %d)",
                    kMaxMixture, a->D, a->F, a->K);
    if (a->B == 0) return ARTAB_OK;
    if ((x_required && !a->x_last) || !a->norm_gamma || !a->norm_beta || !a->w_h1 || !a->w_h2 || !a->mean_bias ||
        !a->std_bias || !a->weight_bias || !a->rand_u || !a->rand_n || !a->x_mean || !a->w_x || !a->b_x || !a->w_y ||
        !a->b_y || !a->markers || !a->ar_tokens || !a->step || !a->preds || !a->emb_next)
        return fail(ARTAB_ERR_NULL_POINTER, "decode_sample_embed: only b_h1 and b_h2 may be NULL");
    if ((x_required && (misaligned16(a->x_last) || a->ld_row % 8 || a->ld_row < a->D)) || misaligned16(a->w_h1) ||
        misaligned16(a->w_h2) || misaligned16(a->b_h1) || misaligned16(a->b_h2) || misaligned16(a->norm_gamma) ||
        misaligned16(a->norm_beta) || misaligned16(a->w_x) || misaligned16(a->b_x) || misaligned16(a->w_y) ||
        misaligned16(a->b_y) || misaligned16(a->markers) || misaligned16(a->ar_tokens) || misaligned16(a->emb_next))
        return fail(ARTAB_ERR_BAD_STRIDE, "decode_sample_embed: model vectors and rows must be 16-byte aligned");
    P.x_last = a->x_last; P.ld_row = a->ld_row; P.norm_g = a->norm_gamma; P.norm_b = a->norm_beta; P.eps = a->eps;
    P.w_h1 = a->w_h1; P.b_h1 = a->b_h1; P.w_h2 = a->w_h2; P.b_h2 = a->b_h2;
    P.mean_bias = a->mean_bias; P.std_bias = a->std_bias; P.weight_bias = a->weight_bias;
    P.K = a->K; P.std_min = a->std_min; P.std_max = a->std_max;
    P.rand_u = a->rand_u; P.rand_n = a->rand_n; P.x_mean = a->x_mean;
    P.w_x = a->w_x; P.b_x = a->b_x; P.w_y = a->w_y; P.b_y = a->b_y; P.markers = a->markers;
    P.ar_tokens = a->ar_tokens; P.bs = a->bs; P.step = a->step; P.Nt = a->Nt;
    P.preds = a->preds; P.emb = a->emb_next; P.B = a->B;
    if (a->advance && (a->n_advance < 1 || a->n_advance > 8 || !a->ticket))
        return fail(ARTAB_ERR_BAD_SHAPE, "advance needs 1..8 counters and a ticket word");
    P.advance = a->advance; P.n_advance = a->advance ? a->n_advance : 0; P.ticket = a->ticket;
    return ARTAB_OK;
}

int artab_decode_sample_embed(const artab_sample_embed_args *a, int dtype, void *stream) {
    SampleEmbedParams P{};
    ARTAB_TRY(fill_sample(P, a, dtype, true));
    if (a->B == 0) return ARTAB_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e = launch_sample_embed(P, a->D, a->F, dtype == ARTAB_BF16, st);
    return launch_status(e, "decode_sample_embed");
}

int artab_decode_step_boundary(const artab_attention_partials *parts, const void *attn, int64_t lda, const void *y,
                               int64_t ldy, const void *w_o, const void *ln2_gamma, const void *ln2_beta, float eps2,
                               const void *w_1, const void *b_1, const void *w_2, const void *b_2,
                               const void *ln3_gamma, const void *ln3_beta, float eps3,
                               const artab_sample_embed_args *tail, const void *next_w_fo,
                               const void *next_ln1_gamma, const void *next_ln1_beta, float next_eps1,
                               const void *next_w_qkv, void *next_y, void *next_qkv, int F, int dtype, void *stream) {
    SampleEmbedParams S{};
    ARTAB_TRY(fill_sample(S, tail, dtype, false));
    const int64_t B = tail->B;
    const int D = tail->D;
    if (F != tail->F)
        return fail(ARTAB_ERR_UNSUPPORTED, "decode_step_boundary: head width %d differs from the layers' feed-forward width %d",
                    tail->F, F);
    if (fused_tile_rows(2 * B) != kFusedRowsSmall || fused_tile_rows(B) != kFusedRowsSmall)
        return fail(ARTAB_ERR_UNSUPPORTED, "decode_step_boundary covers up to %ld trajectories on %d-row tiles",
                    kFusedSmallMaxRows / 2, kFusedRowsSmall);
    if (parts && parts->n_slots == 0) parts = nullptr;  // the call that made them wrote `attn` instead
    FusedPostParams P{};
    FusedPreParams N{};
    ARTAB_TRY(fill_post(P, attn, lda, y, ldy, w_o, ln2_gamma, ln2_beta, eps2, w_1, b_1, w_2, b_2, ln3_gamma, ln3_beta,
                        eps3, nullptr, B, D, F, false, parts));
    ARTAB_TRY(fill_pre(N, nullptr, 0, next_w_fo, next_ln1_gamma, next_ln1_beta, next_eps1, next_w_qkv, next_y, next_qkv,
                       2 * B, D, false));
    hipStream_t st = static_cast<hipStream_t>(stream);
    ARTAB_TRY(apply_partials_order(parts, P, B, st, (B + kFusedRowsSmall / 2 - 1) / (kFusedRowsSmall / 2)));
    if (B == 0) return ARTAB_OK;
    hipError_t e = launch_step_boundary(P, S, N, D, F, dtype == ARTAB_BF16, st);
    return launch_status(e, "decode_step_boundary");
}

}  // extern "C"
