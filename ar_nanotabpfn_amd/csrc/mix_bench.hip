// Instruction-mix benchmark of one 32x32 score block of the head_dim-32 attention kernel, with no
// memory traffic at all: what the SIMD's issue port alone allows.  A workgroup is four wavefronts
// (one per SIMD); the caller fixes how many workgroups share a compute unit through the dynamic
// LDS size it asks for.  Per iteration and wavefront:
//   variant 0  the software-pipelined pass:  4 MFMA 32x32x16, 16 exp2, 8 cvt_pk, 8 dot2c (row sum)
//   variant 1  the lean pass:                4 MFMA 32x32x16, 2 MFMA 16x16x32 (row sum), 16 exp2, 8 cvt_pk
//   variant 2  the matrix instructions of variant 1 alone
//   variant 3  the vector instructions of variant 1 alone
// Operands are constant or pseudo-random bit patterns (random data raises the power the matrix
// pipe draws, and with it lowers the clock the part sustains).
#include <hip/hip_runtime.h>

#include "../../include/artab_bench.h"
#include "common.h"

namespace artab {

__device__ __forceinline__ unsigned mix_hash(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}
// two bf16 values in [1, 2) with random sign and mantissa
__device__ __forceinline__ unsigned mix_pair(unsigned seed) {
    const unsigned h = mix_hash(seed);
    return (0x3f80u | (h & 0x807fu)) | ((0x3f80u | ((h >> 16) & 0x807fu)) << 16);
}

template <int VARIANT>
__global__ __launch_bounds__(256) void mix_kernel(float *out, unsigned long long *stamps, int iters, int random_data) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    u32x4 a[2], b[2], vf[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const unsigned seed = (blockIdx.x * 256 + threadIdx.x) * 64 + i * 8 + e;
            a[i][e] = random_data ? mix_pair(seed) : 0x3c003c00u;
            b[i][e] = random_data ? mix_pair(seed + 17) : 0x3c013c00u;
            vf[i][e] = random_data ? mix_pair(seed + 33) : 0x3c003c00u;
        }
    const int lane = threadIdx.x & 63;
    const unsigned one2 = (lane == 0 || lane == 32 || lane == 17 || lane == 49) ? 0x3f803f80u : 0u;
    const u32x4 ones = {one2, one2, one2, one2};
    f32x16 s = {0.f}, s2 = {0.f}, o = {0.f};
    f32x4 l0 = {0.f, 0.f, 0.f, 0.f}, l1 = {0.f, 0.f, 0.f, 0.f};
    float lsum = 0.f;
    unsigned pk[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) pk[i] = 0x3f803f80u + i;
    // scores of a few units either way, as the kernel sees them: random operands give sums of
    // sixteen products of magnitude 1..4; they are used as exponents as they are
    const unsigned long long t0 = __builtin_readcyclecounter(), w0 = __builtin_amdgcn_s_memrealtime();
    auto step = [&](f32x16 &s_out, const f32x16 &s_in) {
        if (VARIANT != 3) {
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(s_out) : "v"(a[0]), "v"(b[0]));
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s_out) : "v"(a[1]), "v"(b[1]));
        }
        if (VARIANT != 2) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                bf16x2 p;
                p[0] = static_cast<__bf16>(fast_exp2(s_in[2 * i]));
                p[1] = static_cast<__bf16>(fast_exp2(s_in[2 * i + 1]));
                pk[i] = __builtin_bit_cast(unsigned, p);
                if (VARIANT == 0)
                    lsum = __builtin_amdgcn_fdot2_f32_bf16(p, __builtin_bit_cast(bf16x2, 0x3f803f80u), lsum, false);
            }
        }
        const u32x4 p0 = {pk[0], pk[1], pk[2], pk[3]}, p1 = {pk[4], pk[5], pk[6], pk[7]};
        if (VARIANT == 1 || VARIANT == 2) {
            l0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones), __builtin_bit_cast(bf16x8, p0), l0, 0, 0, 0);
            l1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones), __builtin_bit_cast(bf16x8, p1), l1, 0, 0, 0);
        }
        if (VARIANT != 3) {
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(o) : "v"(vf[0]), "v"(p0));
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(o) : "v"(vf[1]), "v"(p1));
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(pk[i]));
        if (VARIANT == 3) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(s_out[i]));
        }
    };
    for (int it = 0; it < iters; it += 2) {  // the exponentials of a block run while the next block's scores are formed
        step(s2, s);
        step(s, s2);
    }
    const unsigned long long t1 = __builtin_readcyclecounter(), w1 = __builtin_amdgcn_s_memrealtime();
    float r = lsum + l0[0] + l1[1];
#pragma unroll
    for (int i = 0; i < 16; ++i) r += s[i] + s2[i] + o[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) r += static_cast<float>(pk[i]);
    out[blockIdx.x * 256 + threadIdx.x] = r;
    if (lane == 0 && stamps) {
        stamps[2 * (blockIdx.x * 4 + (threadIdx.x >> 6))] = t1 - t0;      // shader cycles
        stamps[2 * (blockIdx.x * 4 + (threadIdx.x >> 6)) + 1] = w1 - w0;  // 100 MHz ticks
    }
}

}  // namespace artab

extern "C" int artab_bench_instruction_mix(int variant, int random_data, int workgroups, int iters, size_t lds_bytes,
                                           float *out, unsigned long long *stamps, void *stream) {
    using namespace artab;
    if (variant < 0 || variant > 3 || workgroups <= 0 || iters <= 0 || (iters & 1) || !out || lds_bytes > 160 * 1024)
        return ARTAB_ERR_BAD_SHAPE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const void *fn = variant == 0 ? reinterpret_cast<const void *>(mix_kernel<0>)
                     : variant == 1 ? reinterpret_cast<const void *>(mix_kernel<1>)
                     : variant == 2 ? reinterpret_cast<const void *>(mix_kernel<2>)
                                    : reinterpret_cast<const void *>(mix_kernel<3>);
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)) != hipSuccess)
        return ARTAB_ERR_LAUNCH;
    switch (variant) {
        case 0: hipLaunchKernelGGL(mix_kernel<0>, dim3(workgroups), dim3(256), lds_bytes, st, out, stamps, iters, random_data); break;
        case 1: hipLaunchKernelGGL(mix_kernel<1>, dim3(workgroups), dim3(256), lds_bytes, st, out, stamps, iters, random_data); break;
        case 2: hipLaunchKernelGGL(mix_kernel<2>, dim3(workgroups), dim3(256), lds_bytes, st, out, stamps, iters, random_data); break;
        default: hipLaunchKernelGGL(mix_kernel<3>, dim3(workgroups), dim3(256), lds_bytes, st, out, stamps, iters, random_data); break;
    }
    return hipGetLastError() == hipSuccess ? ARTAB_OK : ARTAB_ERR_LAUNCH;
}
