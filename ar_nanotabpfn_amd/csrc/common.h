// Shared device/host helpers for the AR-TabPFN attention kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace artab {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Device-side tensor view: strides in elements, head_dim contiguous.
struct View {
    char *p;
    long sb, sh, sn;
};

template <typename T>
__device__ __forceinline__ T *view_row(const View &v, long b, long h, long n) {
    return reinterpret_cast<T *>(v.p) + b * v.sb + h * v.sh + n * v.sn;
}

template <typename T>
__device__ __forceinline__ float to_f32(T x) {
    return static_cast<float>(x);
}

template <typename T>
__device__ __forceinline__ T from_f32(float x) {
    return static_cast<T>(x);
}

// Two floats -> two packed 16-bit values (round to nearest even), low half = a.
template <typename T>
__device__ __forceinline__ unsigned pack2(float a, float b);

template <>
__device__ __forceinline__ unsigned pack2<bf16_t>(float a, float b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v;
    v[0] = static_cast<__bf16>(a);
    v[1] = static_cast<__bf16>(b);
    return __builtin_bit_cast(unsigned, v);
}

template <>
__device__ __forceinline__ unsigned pack2<f16_t>(float a, float b) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f16x2 v;
    v[0] = static_cast<_Float16>(a);
    v[1] = static_cast<_Float16>(b);
    return __builtin_bit_cast(unsigned, v);
}

template <typename T>
__device__ __forceinline__ float unpack_lo(unsigned u);
template <typename T>
__device__ __forceinline__ float unpack_hi(unsigned u);

template <>
__device__ __forceinline__ float unpack_lo<bf16_t>(unsigned u) {
    return __builtin_bit_cast(float, u << 16);
}
template <>
__device__ __forceinline__ float unpack_hi<bf16_t>(unsigned u) {
    return __builtin_bit_cast(float, u & 0xffff0000u);
}
template <>
__device__ __forceinline__ float unpack_lo<f16_t>(unsigned u) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(u & 0xffffu)));
}
template <>
__device__ __forceinline__ float unpack_hi<f16_t>(unsigned u) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(u >> 16)));
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Sum / max across the 64 lanes of a wavefront.
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// Visible-key limit of teacher-forcing query row i among Nt buffer keys: buffer
// query i (< Nt) sees keys [0, i]; target query i (>= Nt) sees keys [0, i - Nt).
__host__ __device__ __forceinline__ int tf_limit(int i, int Nt) { return i < Nt ? i + 1 : i - Nt; }

}  // namespace artab
