// Embedding gather, RMSNorm (with the residual add fused in), SwiGLU, casts.
// Activations of the residual stream are float32; norms and sums are computed
// in float32 whatever the storage type of inputs and outputs.
#include "common.h"

// x[t, :] = table[token[t], :] widened to float32
// (/root/reference/src/kipp.c:2579-2585: a plain row gather, no scaling).
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int32_t* __restrict__ tokens,
                             float* __restrict__ out, int hidden) {
    const size_t t = blockIdx.x;
    const size_t row = (size_t)tokens[t] * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[t * hidden + i] = load_f(table, row + i);
}

// One workgroup per row.  If `delta` is given, x += delta first and the sum is
// written back (the residual add of the block before); `delta` may come in
// `parts` slabs [parts, rows, width] that are added in order (a product whose
// contraction was split over workgroups), then
// y = x * rsqrt(mean(x^2) + eps) * w   (/root/reference/src/kipp.c:2221-2231:
// eps inside the root, (x * scale) * w).
template <typename TD, typename TO>
__global__ void rmsnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                               const float* __restrict__ weight, TO* __restrict__ out,
                               int width, float eps, int parts, size_t part_stride) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * width;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = x[base + i];
        if (delta != nullptr) {
            for (int p = 0; p < parts; ++p) v += load_f(delta, p * part_stride + base + i);
            x[base + i] = v;
        }
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        store_f(out, base + i, x[base + i] * scale * weight[i]);
    }
}

// x += delta (the last residual add when no norm follows in the same kernel).
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ x, const TD* __restrict__ delta, size_t n, int parts) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        float v = x[i];
        for (int p = 0; p < parts; ++p) v += load_f(delta, p * n + i);
        x[i] = v;
    }
}

// out[t, i] = silu(gu[t, i]) * gu[t, inner + i], silu(z) = z / (1 + exp(-z))
// (/root/reference/src/kipp.c:2402, 2644-2648).
template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inner, size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    size_t t = idx / inner;
    int i = (int)(idx - t * inner);
    float g = load_f(gu, t * 2 * (size_t)inner + i);
    float u = load_f(gu, t * 2 * (size_t)inner + inner + i);
    store_f(out, idx, g / (1.0f + expf(-g)) * u);
}

template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) store_f(out, i, load_f(in, i));
}

// rows[i, :] = x[index[i], :]  (float32 rows; used to pick the positions whose
// logits are wanted before the final norm and the output head).
__global__ void gather_rows_kernel(const float* __restrict__ x, const int32_t* __restrict__ index,
                                   float* __restrict__ out, int width) {
    const size_t src = (size_t)index[blockIdx.x] * width;
    const size_t dst = (size_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[dst + i] = x[src + i];
}

extern "C" {

int kipp_embed(const void* table, int table_dtype, const int32_t* tokens, float* out,
               int n_tokens, int hidden, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens), block(256);
    if (table_dtype == KIPP_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, tokens, out, hidden);
    else
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, (const float*)table, tokens, out, hidden);
    return KIPP_LAUNCH_CHECK();
}

int kipp_rmsnorm(float* x, const void* delta, int delta_dtype, int parts, const float* weight, void* out, int out_dtype,
                 int rows, int width, float eps, hipStream_t stream) {
    if (rows <= 0) return 0;
    dim3 grid(rows), block(width >= 2048 ? 512 : 256);
#define KIPP_RN(TD, TO) hipLaunchKernelGGL((rmsnorm_kernel<TD, TO>), grid, block, 0, stream, x, (const TD*)delta, weight, (TO*)out, width, eps, parts, (size_t)rows * width)
    if (delta_dtype == KIPP_BF16) {
        if (out_dtype == KIPP_BF16) KIPP_RN(bf16_t, bf16_t); else KIPP_RN(bf16_t, float);
    } else {
        if (out_dtype == KIPP_BF16) KIPP_RN(float, bf16_t); else KIPP_RN(float, float);
    }
#undef KIPP_RN
    return KIPP_LAUNCH_CHECK();
}

int kipp_residual_add(float* x, const void* delta, int delta_dtype, int parts, size_t n, hipStream_t stream) {
    if (n == 0) return 0;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (delta_dtype == KIPP_BF16)
        hipLaunchKernelGGL(residual_add_kernel<bf16_t>, grid, block, 0, stream, x, (const bf16_t*)delta, n, parts);
    else
        hipLaunchKernelGGL(residual_add_kernel<float>, grid, block, 0, stream, x, (const float*)delta, n, parts);
    return KIPP_LAUNCH_CHECK();
}

int kipp_swiglu(const void* gu, int in_dtype, void* out, int out_dtype, int rows, int inner, hipStream_t stream) {
    size_t total = (size_t)rows * inner;
    if (total == 0) return 0;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
#define KIPP_SW(TI, TO) hipLaunchKernelGGL((swiglu_kernel<TI, TO>), grid, block, 0, stream, (const TI*)gu, (TO*)out, inner, total)
    if (in_dtype == KIPP_BF16) {
        if (out_dtype == KIPP_BF16) KIPP_SW(bf16_t, bf16_t); else KIPP_SW(bf16_t, float);
    } else {
        if (out_dtype == KIPP_BF16) KIPP_SW(float, bf16_t); else KIPP_SW(float, float);
    }
#undef KIPP_SW
    return KIPP_LAUNCH_CHECK();
}

int kipp_cast(const void* in, int in_dtype, void* out, int out_dtype, size_t n, hipStream_t stream) {
    if (n == 0) return 0;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
#define KIPP_CA(TI, TO) hipLaunchKernelGGL((cast_kernel<TI, TO>), grid, block, 0, stream, (const TI*)in, (TO*)out, n)
    if (in_dtype == KIPP_BF16) {
        if (out_dtype == KIPP_BF16) KIPP_CA(bf16_t, bf16_t); else KIPP_CA(bf16_t, float);
    } else {
        if (out_dtype == KIPP_BF16) KIPP_CA(float, bf16_t); else KIPP_CA(float, float);
    }
#undef KIPP_CA
    return KIPP_LAUNCH_CHECK();
}

int kipp_gather_rows(const float* x, const int32_t* index, float* out, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(rows), dim3(256), 0, stream, x, index, out, width);
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
