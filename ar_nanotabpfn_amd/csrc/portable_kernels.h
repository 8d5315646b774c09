// Portable attention kernels: one wavefront per query row, float32 arithmetic,
// any dtype, any head_dim <= 256.  They implement every entry point of the C ABI
// (context / decode / teacher forcing / prefill / masked buffer attention / merge)
// and serve the float32 path and the shapes the MFMA kernels do not cover.
#pragma once

#include "common.h"

namespace artab {

enum PortableMode : int {
    kModePlain = 0,    // every query row sees buffer keys [0, Nb)
    kModeTeacher = 1,  // per-row limit tf_limit(i, Nt)
    kModeRowMask = 3,  // per-row limit row_mask_limit(i, rm_nc, Nb, rm_attend)
    kModeMasked = 2    // explicit uint8 mask over the buffer keys
};

struct PortableParams {
    View q, kc, vc, kb, vb, knew, vnew, out;
    View kcache, vcache;  // prefill: copy of kc/vc rows (p == nullptr: none)
    int cache_batches;
    float *lse;
    const uint8_t *mask;
    long m_sb, m_sh, m_sq;
    int B, H, Lq, Nc, Nb;
    int new_row;  // buffer row index served from knew/vnew, or -1
    const int *nbuf_dev;  // decode: committed buffer length read at run time (overrides Nb / new_row)
    int capacity;         // rows the buffer cache holds (bound for a length read from nbuf_dev)
    int rm_nc, rm_attend; // kModeRowMask: context rows in front of the buffer rows, attending chunks
    int append;   // copy knew/vnew to kb/vb[new_row]
    int mode;
    int Nt;
    int Dh;
    float scale;
    int vec_ok;  // rows 16-byte aligned and Dh a multiple of the vector width
};

constexpr int kPortableWaves = 4;
constexpr int kPortableMaxDh = 256;

template <typename T>
__device__ __forceinline__ float dot_row(const float *q_lds, const T *row, int Dh, int vec_ok) {
    float s = 0.f;
    constexpr int VEC = 16 / sizeof(T);
    if (vec_ok) {
        for (int d = 0; d < Dh; d += VEC) {
            if constexpr (sizeof(T) == 4) {
                const f32x4 raw = *reinterpret_cast<const f32x4 *>(row + d);
#pragma unroll
                for (int e = 0; e < 4; ++e) s = fmaf(q_lds[d + e], raw[e], s);
            } else {
                const u32x4 raw = *reinterpret_cast<const u32x4 *>(row + d);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s = fmaf(q_lds[d + 2 * e], unpack_lo<T>(raw[e]), s);
                    s = fmaf(q_lds[d + 2 * e + 1], unpack_hi<T>(raw[e]), s);
                }
            }
        }
    } else {
        for (int d = 0; d < Dh; ++d) s = fmaf(q_lds[d], to_f32<T>(row[d]), s);
    }
    return s;
}

// Online-softmax state of one query row, spread over a wavefront: lane l owns
// output elements d = l, l+64, ...
template <int DPL>
struct RowState {
    float m, l;
    float acc[DPL];
};

// Fold `cnt` (<= 64) keys starting at kv0 of one K/V segment into the row state.
// `visible` tells whether this lane's key (kv0 + lane) takes part.
template <typename T, int DPL>
__device__ __forceinline__ void fold_chunk(RowState<DPL> &st, const float *q_lds, float *p_lds,
                                           const T *krow, bool visible, float scale, int Dh, int vec_ok,
                                           int lane, int cnt, const View &vseg, long b, long h, int kv0,
                                           const T *vnew_row, int new_row) {
    float s = -INFINITY;
    if (visible) s = dot_row<T>(q_lds, krow, Dh, vec_ok) * scale;
    float cm = wave_max(s);
    if (cm == -INFINITY) return;  // nothing visible in this chunk (wave-uniform)
    float m_new = fmaxf(st.m, cm);
    float alpha = expf(st.m - m_new);  // st.m = -inf -> 0
    float p = visible ? expf(s - m_new) : 0.f;
    st.l = st.l * alpha + wave_sum(p);
    st.m = m_new;
    p_lds[lane] = p;
#pragma unroll
    for (int x = 0; x < DPL; ++x) st.acc[x] *= alpha;
    __builtin_amdgcn_wave_barrier();
    for (int kk = 0; kk < cnt; ++kk) {
        float pk = p_lds[kk];
        int kv = kv0 + kk;
        const T *vrow = (kv == new_row) ? vnew_row : view_row<T>(vseg, b, h, kv);
#pragma unroll
        for (int x = 0; x < DPL; ++x) {
            int d = lane + 64 * x;
            if (d < Dh) st.acc[x] = fmaf(pk, to_f32<T>(vrow[d]), st.acc[x]);
        }
    }
    __builtin_amdgcn_wave_barrier();
}

template <typename T, int DPL>
__global__ __launch_bounds__(kPortableWaves * 64) void portable_attention_kernel(PortableParams P) {
    __shared__ float q_s[kPortableWaves][kPortableMaxDh];
    __shared__ float p_s[kPortableWaves][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long row = static_cast<long>(blockIdx.x) * kPortableWaves + wave;
    const long total = static_cast<long>(P.B) * P.H * P.Lq;
    if (row >= total) return;  // whole wavefront leaves together; no block-wide barrier below
    const int i = static_cast<int>(row % P.Lq);
    const int h = static_cast<int>((row / P.Lq) % P.H);
    const long b = row / (static_cast<long>(P.Lq) * P.H);
    float *q_lds = q_s[wave];
    float *p_lds = p_s[wave];
    const int Dh = P.Dh;

    const T *qrow = view_row<T>(P.q, b, h, i);
    for (int d = lane; d < Dh; d += 64) q_lds[d] = to_f32<T>(qrow[d]);
    __builtin_amdgcn_wave_barrier();

    RowState<DPL> st;
    st.m = -INFINITY;
    st.l = 0.f;
#pragma unroll
    for (int x = 0; x < DPL; ++x) st.acc[x] = 0.f;

    // Context segment: every key visible.
    for (int kv0 = 0; kv0 < P.Nc; kv0 += 64) {
        int kv = kv0 + lane;
        bool vis = kv < P.Nc;
        const T *krow = view_row<T>(P.kc, b, h, vis ? kv : 0);
        int cnt = min(64, P.Nc - kv0);
        fold_chunk<T, DPL>(st, q_lds, p_lds, krow, vis, P.scale, Dh, P.vec_ok, lane, cnt, P.vc, b, h, kv0,
                           nullptr, -1);
    }

    // Buffer segment: keys [0, limit) with the mode's visibility rule.
    if (P.nbuf_dev) {
        // a length read from device memory is clamped to the cache; a new row that would land
        // behind the last slot is attended but not stored
        const int hi = P.capacity - (P.new_row >= 0 ? 1 : 0);
        const int raw = *P.nbuf_dev;
        const int n = raw < 0 ? 0 : (raw > hi ? (hi > 0 ? hi : 0) : raw);
        if (raw != n) P.append = 0;
        P.Nb = n + (P.new_row >= 0 ? 1 : 0);
        if (P.new_row >= 0) P.new_row = n;
    }
    int limit = P.Nb;
    if (P.mode == kModeTeacher) limit = min(P.Nb, tf_limit(i, P.Nt));
    if (P.mode == kModeRowMask) limit = min(P.Nb, row_mask_limit(i, P.rm_nc, P.Nb, P.rm_attend));
    const T *knew_row = P.new_row >= 0 ? view_row<T>(P.knew, b, h, 0) : nullptr;
    const T *vnew_row = P.new_row >= 0 ? view_row<T>(P.vnew, b, h, 0) : nullptr;
    const uint8_t *mrow = P.mask ? P.mask + b * P.m_sb + h * P.m_sh + static_cast<long>(i) * P.m_sq : nullptr;
    for (int kv0 = 0; kv0 < limit; kv0 += 64) {
        int kv = kv0 + lane;
        bool vis = kv < limit;
        if (vis && mrow) vis = mrow[kv] != 0;
        const T *krow = (kv == P.new_row) ? knew_row : view_row<T>(P.kb, b, h, kv < limit ? kv : 0);
        if (kv >= limit) krow = qrow;  // never dereferenced for invisible keys; keep a valid pointer
        int cnt = min(64, limit - kv0);
        fold_chunk<T, DPL>(st, q_lds, p_lds, krow, vis, P.scale, Dh, P.vec_ok, lane, cnt, P.vb, b, h, kv0,
                           vnew_row, P.new_row);
    }

    T *orow = view_row<T>(P.out, b, h, i);
    const float inv = st.l > 0.f ? 1.f / st.l : 0.f;  // no visible key: out = 0, lse = -inf
#pragma unroll
    for (int x = 0; x < DPL; ++x) {
        int d = lane + 64 * x;
        if (d < Dh) orow[d] = from_f32<T>(st.acc[x] * inv);
    }
    if (P.lse && lane == 0) P.lse[row] = st.l > 0.f ? st.m + logf(st.l) : -INFINITY;

    // In-place append of the new buffer row (done by the wavefront of query 0).
    if (P.append && i == 0) {
        T *kdst = view_row<T>(P.kb, b, h, P.new_row);
        T *vdst = view_row<T>(P.vb, b, h, P.new_row);
        for (int d = lane; d < Dh; d += 64) {
            kdst[d] = knew_row[d];
            vdst[d] = vnew_row[d];
        }
    }
    // Prefill cache write: row i of K/V goes to the cache in [.., row, :] layout.
    if (P.kcache.p && b < P.cache_batches) {
        const T *ksrc = view_row<T>(P.kc, b, h, i);
        const T *vsrc = view_row<T>(P.vc, b, h, i);
        T *kdst = view_row<T>(P.kcache, b, h, i);
        T *vdst = view_row<T>(P.vcache, b, h, i);
        for (int d = lane; d < Dh; d += 64) {
            kdst[d] = ksrc[d];
            vdst[d] = vsrc[d];
        }
    }
}

struct MergeParams {
    View a, b, out;
    const float *lse_a, *lse_b;
    long rows;  // B*H*Lq
    int H, Lq, Dh;
};

// out = (w_a a + w_b b) / (w_a + w_b), w = exp(lse - max(lse_a, lse_b)); float32 weights.
template <typename T>
__global__ __launch_bounds__(256) void merge_kernel(MergeParams P) {
    long idx = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    long total = P.rows * P.Dh;
    if (idx >= total) return;
    long row = idx / P.Dh;
    int d = static_cast<int>(idx % P.Dh);
    int i = static_cast<int>(row % P.Lq);
    int h = static_cast<int>((row / P.Lq) % P.H);
    long b = row / (static_cast<long>(P.Lq) * P.H);
    float la = P.lse_a[row], lb = P.lse_b[row];
    float mx = fmaxf(la, lb);
    float wa = expf(la - mx), wb = expf(lb - mx);  // both -inf: exp(nan) -> NaN, as the reference formula
    float wt = wa + wb;
    wa /= wt;
    wb /= wt;
    float va = to_f32<T>(view_row<T>(P.a, b, h, i)[d]);
    float vb = to_f32<T>(view_row<T>(P.b, b, h, i)[d]);
    view_row<T>(P.out, b, h, i)[d] = from_f32<T>(wa * va + wb * vb);
}

template <typename T>
inline hipError_t launch_portable(const PortableParams &P, hipStream_t stream) {
    long total = static_cast<long>(P.B) * P.H * P.Lq;
    if (total == 0) return hipSuccess;
    dim3 grid(static_cast<unsigned>((total + kPortableWaves - 1) / kPortableWaves));
    dim3 block(kPortableWaves * 64);
    if (P.Dh <= 64)
        hipLaunchKernelGGL((portable_attention_kernel<T, 1>), grid, block, 0, stream, P);
    else if (P.Dh <= 128)
        hipLaunchKernelGGL((portable_attention_kernel<T, 2>), grid, block, 0, stream, P);
    else
        hipLaunchKernelGGL((portable_attention_kernel<T, 4>), grid, block, 0, stream, P);
    return hipGetLastError();
}

template <typename T>
inline hipError_t launch_merge(const MergeParams &P, hipStream_t stream) {
    long total = P.rows * P.Dh;
    if (total == 0) return hipSuccess;
    dim3 grid(static_cast<unsigned>((total + 255) / 256));
    hipLaunchKernelGGL((merge_kernel<T>), grid, dim3(256), 0, stream, P);
    return hipGetLastError();
}

}  // namespace artab
