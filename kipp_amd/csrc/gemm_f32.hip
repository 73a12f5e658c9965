// True 32-bit matrix product for the float32 path: Y[M,N] = X[M,K] . W[N,K]^T
// with W stored [out][in] row-major like every projection of the model
// (/root/reference/src/kipp.c:2233-2244).  Plain FMA in float32, no matrix
// cores, no reduced-precision mode.  Each output element is one accumulator
// that runs over k = 0..K-1 in order, so its bits do not depend on M, on the
// tile it falls in or on what else is in the batch.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

template <typename TW>
__global__ void __launch_bounds__(256) gemm_f32_kernel(const float* __restrict__ X, const TW* __restrict__ W,
                                                       float* __restrict__ Y, int M, int N, int K) {
    __shared__ float Xs[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + i * 256;
            const int r = idx / BK, kk = idx % BK;
            const int gk = k0 + kk;
            const int gm = m0 + r, gn = n0 + r;
            Xs[kk][r] = (gm < M && gk < K) ? X[(size_t)gm * K + gk] : 0.0f;
            Ws[kk][r] = (gn < N && gk < K) ? load_f(W, (size_t)gn * K + gk) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = Xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn < N) Y[(size_t)gm * N + gn] = acc[i][j];
        }
    }
}

extern "C" int kipp_gemm_f32(const float* X, const void* W, int w_dtype, float* Y, int M, int N, int K,
                             hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return -1;
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM), block(256);
    if (w_dtype == KIPP_BF16)
        hipLaunchKernelGGL(gemm_f32_kernel<bf16_t>, grid, block, 0, stream, X, (const bf16_t*)W, Y, M, N, K);
    else
        hipLaunchKernelGGL(gemm_f32_kernel<float>, grid, block, 0, stream, X, (const float*)W, Y, M, N, K);
    return KIPP_LAUNCH_CHECK();
}
