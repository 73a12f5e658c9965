// What this GPU's memory gives a kernel that does nothing but read: the yardstick for the
// decode kernels, which are bound by reading weights and cache once.  Every wave keeps DEPTH
// 16-byte loads a lane in flight (a ring, as the product kernels do) and walks its own
// contiguous stretch of the buffer; the values are folded into one word so that no load is dropped.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

template <int DEPTH>
__global__ void __launch_bounds__(256) stream_read_kernel(const u32x4* __restrict__ src, size_t units_per_wave,
                                                          uint32_t* __restrict__ sink) {
    const int lane = threadIdx.x & 63;
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const u32x4* p = src + wave * units_per_wave + lane;          // a unit: 16 bytes; a step: 64 units (1 KB)
    const size_t steps = units_per_wave / 64;
    u32x4 ring[DEPTH], acc = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) ring[u] = p[(size_t)u * 64];
    size_t s = 0;
    for (; s + 2 * DEPTH <= steps; s += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            acc ^= ring[u];
            ring[u] = p[(s + DEPTH + u) * 64];
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) acc ^= ring[u];
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = 1;   // never true for the buffers used; keeps the loads
}

// What the matrix cores sustain when nothing else happens: every wave multiplies operands that never leave its
// registers into ACC independent 32x32 accumulators (the instruction of the prompt products), no memory, no LDS.
// The rate depends on the operands' bits (a chip at its power limit clocks down, and zeros cost less than random
// values), on how many compute units work and on how long the kernel runs: the yardstick for the prompt products.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <int ACC>
__global__ void __launch_bounds__(256) mfma_rate_kernel(const u32x4* __restrict__ data, int iters, uint32_t* __restrict__ sink) {
    union {
        u32x4 u;
        bf16x8 v;
    } a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i].u = data[(threadIdx.x + 64 * i) & 1023];
        b[i].u = data[(threadIdx.x * 3 + 17 * i + 512) & 1023];
    }
    f32x16 acc[ACC];
#pragma unroll
    for (int i = 0; i < ACC; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < ACC; ++i)
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i & 3].v, b[(i >> 2) & 3].v, acc[i], 0, 0, 0);
    }
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < ACC; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) total += acc[i][j];
    if (total == 123.456f) sink[0] = 1;          // keeps the products
}

extern "C" {

// `workgroups` of 4 waves, each wave `iters` rounds over `accumulators` (8 or 16) products of 32x32x16 from
// `data` (16 KiB of bfloat16 bits).  Returns the floating-point operations launched, or -1.
long long kipp_probe_mfma_rate(const void* data, int workgroups, int accumulators, int iters, void* sink, hipStream_t stream) {
    if (workgroups <= 0 || iters <= 0) return -1;
    if (accumulators == 16)
        hipLaunchKernelGGL(mfma_rate_kernel<16>, dim3(workgroups), dim3(256), 0, stream, (const u32x4*)data, iters, (uint32_t*)sink);
    else if (accumulators == 8)
        hipLaunchKernelGGL(mfma_rate_kernel<8>, dim3(workgroups), dim3(256), 0, stream, (const u32x4*)data, iters, (uint32_t*)sink);
    else
        return -1;
    if (KIPP_LAUNCH_CHECK() != 0) return -1;
    return (long long)workgroups * 4 * accumulators * iters * 32768LL;
}

// Reads `bytes` (rounded down to what `workgroups` x 4 waves x whole rings cover) once.  Returns the bytes read, or -1.
long long kipp_probe_stream_read(const void* src, long long bytes, int workgroups, int depth, void* sink, hipStream_t stream) {
    if (bytes <= 0 || workgroups <= 0) return -1;
    const size_t waves = (size_t)workgroups * 4;
    const size_t ring_units = (size_t)depth * 64;
    const size_t units_per_wave = ((size_t)bytes / 16 / waves) / ring_units * ring_units;
    if (units_per_wave < 2 * ring_units) return -1;
    switch (depth) {
        case 4: hipLaunchKernelGGL(stream_read_kernel<4>, dim3(workgroups), dim3(256), 0, stream, (const u32x4*)src, units_per_wave, (uint32_t*)sink); break;
        case 8: hipLaunchKernelGGL(stream_read_kernel<8>, dim3(workgroups), dim3(256), 0, stream, (const u32x4*)src, units_per_wave, (uint32_t*)sink); break;
        case 16: hipLaunchKernelGGL(stream_read_kernel<16>, dim3(workgroups), dim3(256), 0, stream, (const u32x4*)src, units_per_wave, (uint32_t*)sink); break;
        default: return -1;
    }
    if (KIPP_LAUNCH_CHECK() != 0) return -1;
    return (long long)(units_per_wave * waves * 16);
}

}  // extern "C"
