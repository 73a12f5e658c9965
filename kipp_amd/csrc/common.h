// Shared device helpers for the gfx950 kernels: bfloat16 bits, wave (64 lanes)
// and workgroup reductions with a fixed order, launch error plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define KIPP_WAVE 64

typedef uint16_t bf16_t;  // raw bfloat16 bits

enum { KIPP_F32 = 0, KIPP_BF16 = 1 };

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// Round to nearest even, as /root/reference/src/kipp.c:2181-2186; NaN stays NaN.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t bits = __float_as_uint(f);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((bits >> 16) | 0x40u);
    uint32_t rounding = 0x7fffu + ((bits >> 16) & 1u);
    return (bf16_t)((bits + rounding) >> 16);
}

__device__ __forceinline__ float load_f(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float load_f(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
__device__ __forceinline__ void store_f(float* p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void store_f(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// The per-head norm and the rotation with every rounding spelt out: nothing is left for the
// compiler to contract one way in one kernel and another way in the next, so whichever kernel
// prepares a head (the rotary kernels, the fused decode attention) gives the same bits
// (/root/reference/src/kipp.c:2480-2500, 2368-2382).
__device__ __forceinline__ float square_add(float ss, float v) { return fmaf(v, v, ss); }
__device__ __forceinline__ float head_norm_scale(float ss, float width, float eps) {
    return 1.0f / sqrtf(__fadd_rn(ss / width, eps));
}
__device__ __forceinline__ float rotate_lo(float a, float b, float cs, float sn) { return fmaf(a, cs, -__fmul_rn(b, sn)); }
__device__ __forceinline__ float rotate_hi(float a, float b, float cs, float sn) { return fmaf(b, cs, __fmul_rn(a, sn)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, KIPP_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, KIPP_WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of LDS.  The order of the additions is
// fixed by the thread layout, so equal inputs give equal bits.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int wave = threadIdx.x / KIPP_WAVE;
    const int waves = (blockDim.x + KIPP_WAVE - 1) / KIPP_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < waves; ++w) total += scratch[w];
    return total;
}

#define KIPP_LAUNCH_CHECK() ((int)hipGetLastError())
