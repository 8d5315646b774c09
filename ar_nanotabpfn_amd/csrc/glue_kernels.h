// Row-wise glue kernels of the transformer layer around attention (gfx950):
// residual + bias + LayerNorm in one pass, and bias + exact GELU.  One wavefront per
// row, 16-byte loads, float32 statistics; HBM-bound (each element read and written once).
#pragma once

#include "common.h"

namespace artab {

struct AddLayerNormParams {
    const void *x;      // [rows, D] residual stream (row stride ldx)
    const void *y;      // [rows, D] branch output to add, or nullptr (row stride ldy)
    const void *bias;   // [D] added to y, or nullptr
    const void *gamma;  // [D]
    const void *beta;   // [D]
    void *out;          // [rows, D] contiguous
    long rows, ldx, ldy;
    int D;
    float eps;
};

constexpr int kGlueWaves = 4;
constexpr int kGlueMaxPerLane = 4;  // D <= 64 lanes * 4 elems * kGlueMaxPerLane

template <typename T>
__device__ __forceinline__ void load4(const T *p, float (&f)[4]) {
    if constexpr (sizeof(T) == 4) {
        f32x4 v = *reinterpret_cast<const f32x4 *>(p);
#pragma unroll
        for (int e = 0; e < 4; ++e) f[e] = v[e];
    } else {
        u32x2 v = *reinterpret_cast<const u32x2 *>(p);
        f[0] = unpack_lo<T>(v[0]);
        f[1] = unpack_hi<T>(v[0]);
        f[2] = unpack_lo<T>(v[1]);
        f[3] = unpack_hi<T>(v[1]);
    }
}

template <typename T>
__device__ __forceinline__ void store4(T *p, const float (&f)[4]) {
    if constexpr (sizeof(T) == 4) {
        f32x4 v = {f[0], f[1], f[2], f[3]};
        *reinterpret_cast<f32x4 *>(p) = v;
    } else {
        u32x2 v = {pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3])};
        *reinterpret_cast<u32x2 *>(p) = v;
    }
}

// out = LayerNorm(x + y + bias) * gamma + beta, biased variance, eps inside the root.
template <typename T>
__global__ __launch_bounds__(kGlueWaves * 64) void add_layernorm_kernel(AddLayerNormParams P) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long row = static_cast<long>(blockIdx.x) * kGlueWaves + wave;
    if (row >= P.rows) return;
    const T *x = static_cast<const T *>(P.x) + row * P.ldx;
    const T *y = P.y ? static_cast<const T *>(P.y) + row * P.ldy : nullptr;
    const T *bias = static_cast<const T *>(P.bias);
    float v[kGlueMaxPerLane][4];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < kGlueMaxPerLane; ++i) {
        const int d = 4 * lane + 256 * i;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[i][e] = 0.f;
        if (d < P.D) {
            load4<T>(x + d, v[i]);
            if (y) {
                float t[4];
                load4<T>(y + d, t);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[i][e] += t[e];
            }
            if (bias) {
                float t[4];
                load4<T>(bias + d, t);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[i][e] += t[e];
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) sum += v[i][e];
        }
    }
    const float mean = wave_sum(sum) / P.D;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < kGlueMaxPerLane; ++i) {
        const int d = 4 * lane + 256 * i;
        if (d < P.D) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float c = v[i][e] - mean;
                sq += c * c;
            }
        }
    }
    const float rstd = rsqrtf(wave_sum(sq) / P.D + P.eps);
    T *out = static_cast<T *>(P.out) + row * P.D;
    const T *gamma = static_cast<const T *>(P.gamma), *beta = static_cast<const T *>(P.beta);
#pragma unroll
    for (int i = 0; i < kGlueMaxPerLane; ++i) {
        const int d = 4 * lane + 256 * i;
        if (d < P.D) {
            float g[4], b[4], o[4];
            load4<T>(gamma + d, g);
            load4<T>(beta + d, b);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (v[i][e] - mean) * rstd * g[e] + b[e];
            store4<T>(out + d, o);
        }
    }
}

struct BiasGeluParams {
    const void *x;     // [rows, D], row stride ldx
    const void *bias;  // [D] or nullptr
    void *out;         // [rows, D] contiguous
    long rows, ldx;
    int D;
};

// out = gelu(x + bias), erf form.
template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_kernel(BiasGeluParams P) {
    const long per_row = P.D / 4;
    const long idx = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= P.rows * per_row) return;
    const long row = idx / per_row;
    const int d = static_cast<int>(idx % per_row) * 4;
    float v[4];
    load4<T>(static_cast<const T *>(P.x) + row * P.ldx + d, v);
    if (P.bias) {
        float t[4];
        load4<T>(static_cast<const T *>(P.bias) + d, t);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += t[e];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = 0.5f * v[e] * (1.f + erff(v[e] * 0.70710678118654752f));
    store4<T>(static_cast<T *>(P.out) + row * P.D + d, v);
}

}  // namespace artab
