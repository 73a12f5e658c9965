// Token choice on the device, one workgroup per row of float32 logits.
#include "common.h"
#include <math.h>

// Greedy: the largest logit, the lowest index among equals
// (/root/reference/src/kipp.c:3459-3464: strict '>' in index order).
__global__ void __launch_bounds__(1024) argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out,
                                                      int vocab) {
    __shared__ float best_v[16];
    __shared__ int best_i[16];
    const float* row = logits + (size_t)blockIdx.x * vocab;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        const float v = row[i];
        if (v > bv || (bi == 0x7fffffff && !(v != v))) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, KIPP_WAVE);
        const int oi = __shfl_xor(bi, off, KIPP_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    const int lane = threadIdx.x & (KIPP_WAVE - 1), wave = threadIdx.x / KIPP_WAVE;
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int waves = blockDim.x / KIPP_WAVE;
        for (int w = 1; w < waves; ++w) {
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        }
        out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

extern "C" int kipp_argmax(const float* logits, int32_t* out, int rows, int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return -1;
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, stream, logits, out, vocab);
    return KIPP_LAUNCH_CHECK();
}
