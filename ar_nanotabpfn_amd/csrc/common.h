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

// Eight packed 16-bit values -> float32.
template <typename T>
__device__ __forceinline__ void unpack8(const u32x4 &raw, float (&f)[8]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        f[2 * e] = unpack_lo<T>(raw[e]);
        f[2 * e + 1] = unpack_hi<T>(raw[e]);
    }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// Weight of a partial attention result in a log-sum-exp merge, exp(lse - max): one hardware exp2.
// Every merge of partials (the stand-alone launch and the one inside the layer kernels) uses this
// one expression, so that they agree bit for bit.
__device__ __forceinline__ float merge_weight(float lse, float mx) { return fast_exp2((lse - mx) * kLog2e); }
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

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding).
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

// 16 bytes per lane from global memory straight into LDS: lane l lands at lds + 16 l (lds is
// wavefront-uniform; lanes switched off write nothing and leave their 16 bytes untouched).
// Kept in a plain function: called directly from a kernel template the builtin makes the host
// pass drop the kernel's launch stub.
__device__ __forceinline__ void load_to_lds_16(const void *global_src, void *lds_dst) {
    __builtin_amdgcn_global_load_lds(global_src, lds_dst, 16, 0, 0);
}

// A 64-byte row per lane in four 16-byte pieces, piece t of lane l landing at lds + 1024 t + 16 l.
// The instruction's immediate offset moves the global AND the LDS address, hence the 1008 = 1024 - 16
// per piece on the LDS side: no per-piece address arithmetic in vector registers.
__device__ __forceinline__ void load_row64_to_lds(const void *global_src, unsigned char *lds_dst) {
    __builtin_amdgcn_global_load_lds(global_src, lds_dst, 16, 0, 0);
    __builtin_amdgcn_global_load_lds(global_src, lds_dst + 1008, 16, 16, 0);
    __builtin_amdgcn_global_load_lds(global_src, lds_dst + 2016, 16, 32, 0);
    __builtin_amdgcn_global_load_lds(global_src, lds_dst + 3024, 16, 48, 0);
}

// Kernel arguments are read with scalar loads through a cache that a launch finds cold, and the
// compiler places each load where its field is first used: a prologue that steers by a dozen
// fields of a 400-byte argument block pays one miss (200-300 ns) per 64-byte line, one after the
// other.  Called first thing in a kernel, this touches every line of the first `BYTES` bytes of
// the argument segment with one batch of loads and one wait; the loads that follow hit the cache.
template <int BYTES>
__device__ __forceinline__ void warm_kernel_arguments() {
    typedef const unsigned __attribute__((address_space(4))) *ConstPtr;
    ConstPtr ka = (ConstPtr)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int LINES = (BYTES + 63) / 64;
    static_assert(LINES >= 1 && LINES <= 16, "argument blocks of up to 1 KiB");
    unsigned w[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) w[i] = ka[16 * (i < LINES ? i : LINES - 1)];
    asm volatile("" ::"s"(w[0]), "s"(w[1]), "s"(w[2]), "s"(w[3]), "s"(w[4]), "s"(w[5]), "s"(w[6]), "s"(w[7]), "s"(w[8]),
                 "s"(w[9]), "s"(w[10]), "s"(w[11]), "s"(w[12]), "s"(w[13]), "s"(w[14]), "s"(w[15]));
}

// The same in two halves, for a kernel whose first memory requests need nothing but arguments that
// arrive in registers (the leading scalar arguments of a kernel are preloaded into SGPRs by the
// command processor when the unit is compiled with -amdgpu-kernarg-preload-count): request()
// starts the loads, the kernel issues those first requests, await() is the one wait.
template <int BYTES>
struct KernelArgumentLines {
    unsigned w[16];
    // (Inline assembly: as ordinary loads the compiler moves them down to await(), behind the
    // requests they are meant to travel beside.  The compiler does not know that the registers of
    // w are written late: EVERY path of the kernel must pass await() before it ends or branches
    // far, or a register it has reused in the meantime is overwritten when the load lands.)
    __device__ __forceinline__ void request() {
        typedef const unsigned __attribute__((address_space(4))) *ConstPtr;
        ConstPtr ka = (ConstPtr)__builtin_amdgcn_kernarg_segment_ptr();
        constexpr int LINES = (BYTES + 63) / 64;
        static_assert(LINES >= 1 && LINES <= 16, "argument blocks of up to 1 KiB");
#pragma unroll
        for (int i = 0; i < LINES; ++i) asm volatile("s_load_dword %0, %1, %2" : "=s"(w[i]) : "s"(ka), "n"(64 * i));
    }
    __device__ __forceinline__ void await() const {
        constexpr int LINES = (BYTES + 63) / 64;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < LINES; ++i) asm volatile("" ::"s"(w[i]));
    }
};

// A value again, as one the compiler cannot trace (typically the lane index): what rarely
// executed code derives from it (rows, base addresses) is then computed where it is used instead
// of being kept in registers across a hot loop that does not need it.
__device__ __forceinline__ int opaque(int v) {
    asm volatile("" : "+v"(v));
    return v;
}

// acc + a.lo * b.lo + a.hi * b.hi of two packed 16-bit pairs, accumulated in float32
template <typename T>
__device__ __forceinline__ float dot2_acc(unsigned a, unsigned b, float acc);
template <>
__device__ __forceinline__ float dot2_acc<bf16_t>(unsigned a, unsigned b, float acc) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc, false);
}
template <>
__device__ __forceinline__ float dot2_acc<f16_t>(unsigned a, unsigned b, float acc) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), acc, false);
}

__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Visible-key limit of teacher-forcing query row i among Nt buffer keys: buffer
// query i (< Nt) sees keys [0, i]; target query i (>= Nt) sees keys [0, i - Nt).
__host__ __device__ __forceinline__ int tf_limit(int i, int Nt) { return i < Nt ? i + 1 : i - Nt; }

// Visible-key limit among the Nb buffer keys of row i under the training row mask (rows are
// [context Nc | buffer Nb | target ...], ar_tabpfn/model/attention.py:86-175): a context row sees
// no buffer key, buffer row j sees keys [0, j], target row with offset o sees keys [0, o mod Nb]
// while o < attend * Nb and none after that.  Every row sees the whole context; nobody sees a
// target key.
__host__ __device__ __forceinline__ int row_mask_limit(int i, int Nc, int Nb, int attend) {
    if (i < Nc || Nb <= 0) return 0;
    if (i < Nc + Nb) return i - Nc + 1;
    const int o = i - Nc - Nb;
    return o < attend * Nb ? o % Nb + 1 : 0;
}

}  // namespace artab
