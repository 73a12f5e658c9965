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

// The same for widths that are a multiple of 4 and at most 1024 * CH: the row stays in
// registers between the sum of squares and the scaling (one read of x, 16-byte accesses).
__device__ __forceinline__ float4 load4(const float* p, size_t i4) { return ((const float4*)p)[i4]; }
__device__ __forceinline__ float4 load4(const bf16_t* p, size_t i4) {
    const uint2 r = ((const uint2*)p)[i4];
    return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                       __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u));
}
__device__ __forceinline__ void store4(float* p, size_t i4, float4 v) { ((float4*)p)[i4] = v; }
__device__ __forceinline__ void store4(bf16_t* p, size_t i4, float4 v) {
    uint2 r;
    r.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    r.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    ((uint2*)p)[i4] = r;
}

template <typename TD, typename TO, int CH, int THREADS = 256>
__global__ void __launch_bounds__(THREADS) rmsnorm_rows_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                                           const float* __restrict__ weight, TO* __restrict__ out,
                                                           int width, float eps, int parts, size_t part_stride) {
    __shared__ float scratch[16];
    const int n4 = width / 4;
    const size_t base4 = (size_t)blockIdx.x * n4;
    float4 v[CH], w[CH];
    float ss = 0.0f;
    // every load is issued before anything is added: the kernel is a few round trips to memory long
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int i = threadIdx.x + c * THREADS;
        v[c] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        w[c] = v[c];
        if (i < n4) {
            v[c] = load4(x, base4 + i);
            w[c] = load4(weight, (size_t)i);
        }
    }
    if (delta != nullptr) {
        for (int p0 = 0; p0 < parts; p0 += 4) {
            float4 d[CH][4];
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int i = threadIdx.x + c * THREADS;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    d[c][q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    if (i < n4 && p0 + q < parts) d[c][q] = load4(delta, (p0 + q) * (part_stride / 4) + base4 + i);
                }
            }
#pragma unroll
            for (int c = 0; c < CH; ++c)
#pragma unroll
                for (int q = 0; q < 4; ++q) {   // slabs in order
                    v[c].x += d[c][q].x;
                    v[c].y += d[c][q].y;
                    v[c].z += d[c][q].z;
                    v[c].w += d[c][q].w;
                }
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int i = threadIdx.x + c * THREADS;
            if (i < n4) store4(x, base4 + i, v[c]);
        }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) ss += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int i = threadIdx.x + c * THREADS;
        if (i < n4)
            store4(out, base4 + i, make_float4(v[c].x * scale * w[c].x, v[c].y * scale * w[c].y, v[c].z * scale * w[c].z,
                                               v[c].w * scale * w[c].w));
    }
}

// out[t, :] = rows[t, :] * rsqrt(sum_p sumsq[t, p] / width + eps), sumsq in rows of `stride`: the normalized rows, for a consumer that
// does not apply the scale itself (rows = bfloat16(x * norm weight), sumsq = partial sums of x^2).
// `steps_major`: `rows` come as [width / 32][rows][32] (what the few-rows products write for each other); out is [rows][width].
__global__ void __launch_bounds__(256) scale_rows_kernel(const bf16_t* __restrict__ rows, const float* __restrict__ sumsq,
                                                         bf16_t* __restrict__ out, int width, int parts, int stride, float eps,
                                                         int steps_major) {
    __shared__ float scratch[16];
    float a = 0.0f;
    for (int p = threadIdx.x; p < parts; p += 256) a += sumsq[(size_t)blockIdx.x * stride + p];
    a = block_sum(a, scratch);
    const float scale = 1.0f / sqrtf(a / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += 256) {
        const size_t at = (size_t)blockIdx.x * width + i;
        const size_t from = steps_major ? ((size_t)(i >> 5) * gridDim.x + blockIdx.x) * 32 + (i & 31) : at;
        out[at] = f32_to_bf16(bf16_to_f32(rows[from]) * scale);
    }
}

// The streaming layout of a bfloat16 matrix [n, k] (k a multiple of 32) that the few-rows products read:
// [tile of 16 rows][step of 32 columns][lane][8 values], lane l holding row l % 16 and columns 8 (l / 16) .. + 7
// of the step, rows padded to whole tiles with zeros.  `inner` > 0: the matrix is [gate; up] of `inner` rows
// each and tile t holds gate rows 8 t .. 8 t + 7 over up rows 8 t .. 8 t + 7.  A thread moves 16 bytes.
__global__ void __launch_bounds__(256) tile_weight_kernel(const uint4* __restrict__ rows, uint4* __restrict__ tiles, int n, int k,
                                                          int inner, size_t units) {
    const size_t u = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (u >= units) return;
    const int steps = k / 32, lane = (int)(u & 63), r = lane & 15, h = lane >> 4;
    const size_t tile = u / ((size_t)steps * 64);
    const int step = (int)((u >> 6) % (size_t)steps);
    long long row;
    if (inner > 0) {
        const long long i = (long long)tile * 8 + (r & 7);
        row = i < inner ? (r < 8 ? i : inner + i) : -1;
    } else {
        row = (long long)tile * 16 + r;
        if (row >= n) row = -1;
    }
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (row >= 0) v = rows[((size_t)row * k + 32 * step + 8 * h) / 8];
    tiles[u] = v;
}

// x += delta (the last residual add when no norm follows in the same kernel).
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ x, const TD* __restrict__ delta, size_t n, int parts) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        float v = x[i];
        for (int p0 = 0; p0 < parts; p0 += 4) {   // slabs in order; four at a time, all asked for before the first is added
            float d[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) d[q] = p0 + q < parts ? load_f(delta, (p0 + q) * n + i) : 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) v += d[q];
        }
        x[i] = v;
    }
}

// out[t, i] = silu(gu[t, i]) * gu[t, inner + i], silu(z) = z / (1 + exp(-z))
// (/root/reference/src/kipp.c:2402, 2644-2648).  `pairs`: the columns of gu come in tiles of 16,
// 8 gates over the 8 matching ups (the product of a weight in the paired streaming layout):
// gate i at 16 (i / 8) + i % 8, its up 8 further, rows of 16 ceil(inner / 8) columns.
template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inner, size_t total, int parts, int pairs) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    size_t t = idx / inner;
    int i = (int)(idx - t * inner);
    const size_t width = pairs ? 16 * (size_t)((inner + 7) / 8) : 2 * (size_t)inner;
    const size_t slab = (total / inner) * width;
    const size_t at_g = t * width + (pairs ? 16 * (i >> 3) + (i & 7) : i), at_u = at_g + (pairs ? 8 : inner);
    float g = 0.0f, u = 0.0f;
    for (int p0 = 0; p0 < parts; p0 += 4) {   // slabs of a split product, in order; four at a time, all asked for before the first is added
        float gs[4], us[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            gs[q] = p0 + q < parts ? load_f(gu, (p0 + q) * slab + at_g) : 0.0f;
            us[q] = p0 + q < parts ? load_f(gu, (p0 + q) * slab + at_u) : 0.0f;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            g += gs[q];
            u += us[q];
        }
    }
    store_f(out, idx, g / (1.0f + expf(-g)) * u);
}

// The same, eight columns a thread with 16-byte accesses (inner a multiple of 8); the slabs of a split product are added
// in order, four at a time with all their loads asked for before the first is added.
__device__ __forceinline__ float4 add4(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }

template <typename TI, typename TO>
__global__ void swiglu_vec_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inner, size_t total8, int pairs, int parts,
                                  size_t slab4) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total8) return;
    const int per_row = inner / 8;
    const size_t t = idx / per_row;
    const int i4 = (int)(idx - t * per_row) * 2;              // in units of 4 columns
    const size_t row4 = t * 2 * (size_t)inner / 4;
    const size_t g4 = row4 + (pairs ? 2 * i4 : i4), u4 = g4 + (pairs ? 2 : inner / 4);
    float4 g0 = load4(gu, g4), g1 = load4(gu, g4 + 1);
    float4 u0 = load4(gu, u4), u1 = load4(gu, u4 + 1);
    for (int p0 = 1; p0 < parts; p0 += 4) {
        float4 more[4][4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const size_t at = (size_t)min(p0 + q, parts - 1) * slab4;
            more[q][0] = load4(gu, at + g4);
            more[q][1] = load4(gu, at + g4 + 1);
            more[q][2] = load4(gu, at + u4);
            more[q][3] = load4(gu, at + u4 + 1);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (p0 + q < parts) {
                g0 = add4(g0, more[q][0]);
                g1 = add4(g1, more[q][1]);
                u0 = add4(u0, more[q][2]);
                u1 = add4(u1, more[q][3]);
            }
        }
    }
    const size_t o4 = t * (size_t)inner / 4 + i4;
    store4(out, o4, make_float4(g0.x / (1.0f + expf(-g0.x)) * u0.x, g0.y / (1.0f + expf(-g0.y)) * u0.y,
                                g0.z / (1.0f + expf(-g0.z)) * u0.z, g0.w / (1.0f + expf(-g0.w)) * u0.w));
    store4(out, o4 + 1, make_float4(g1.x / (1.0f + expf(-g1.x)) * u1.x, g1.y / (1.0f + expf(-g1.y)) * u1.y,
                                    g1.z / (1.0f + expf(-g1.z)) * u1.z, g1.w / (1.0f + expf(-g1.w)) * u1.w));
}

template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) store_f(out, i, load_f(in, i));
}

// out = in, 16 bytes a lane and step where both are aligned so, else 4 (whole 4-byte words, copied bit for bit).
__global__ void __launch_bounds__(256) copy_words_kernel(const uint32_t* __restrict__ in, uint32_t* __restrict__ out,
                                                         size_t words, int wide) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (wide) {
        const uint4* in4 = (const uint4*)in;
        uint4* out4 = (uint4*)out;
        const size_t quads = words / 4;
        for (size_t q = i; q < quads; q += stride) out4[q] = in4[q];
        for (size_t w = quads * 4 + i; w < words; w += stride) out[w] = in[w];
    } else {
        for (; i < words; i += stride) out[i] = in[i];
    }
}

// words[0 .. n) = 0
__global__ void __launch_bounds__(256) fill_zero_kernel(uint32_t* __restrict__ out, size_t words) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += stride) out[i] = 0u;
}

// rows[i, :] = x[index[i], :]  (rows of 4-byte words, copied bit for bit; used to pick the positions whose
// logits are wanted before the final norm and the output head, and the tokens of the requests that go on).
__global__ void gather_rows_kernel(const uint32_t* __restrict__ x, const int32_t* __restrict__ index,
                                   uint32_t* __restrict__ out, int width) {
    const size_t src = (size_t)index[blockIdx.x] * width;
    const size_t dst = (size_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[dst + i] = x[src + i];
}

template <typename TD, typename TO>
static void launch_rmsnorm(float* x, const void* delta, const float* weight, void* out, int rows, int width, float eps,
                           int parts, hipStream_t stream) {
    const size_t stride = (size_t)rows * width;
    const int n4 = width / 4;
    // Few rows are few workgroups, each a few round trips to memory long: a workgroup of up to 1,024 threads then takes its
    // row in one pass (measured at 2,560 columns with 6 to 8 slabs: 3.8 instead of 5.1 us at 16 rows, 4.8 instead of 5.8
    // at 64).  Under bfloat16 only: the order of the sum of squares follows the workgroup's size, and the float32 path
    // promises a row the same bits in every batch.
    constexpr bool rounds = sizeof(TO) == 2;
    if (rounds && (width & 3) == 0 && rows <= 256 && n4 > 256 && n4 <= 2048) {
#define KIPP_RW(CH, THREADS) hipLaunchKernelGGL((rmsnorm_rows_kernel<TD, TO, CH, THREADS>), dim3(rows), dim3(THREADS), 0, stream, x, (const TD*)delta, weight, (TO*)out, width, eps, parts, stride)
        if (n4 <= 512) KIPP_RW(1, 512);
        else if (n4 <= 1024) KIPP_RW(1, 1024);
        else KIPP_RW(2, 1024);
#undef KIPP_RW
    } else if ((width & 3) == 0 && n4 <= 256 * 8) {
#define KIPP_RV(CH) hipLaunchKernelGGL((rmsnorm_rows_kernel<TD, TO, CH>), dim3(rows), dim3(256), 0, stream, x, (const TD*)delta, weight, (TO*)out, width, eps, parts, stride)
        if (n4 <= 256) KIPP_RV(1);
        else if (n4 <= 512) KIPP_RV(2);
        else if (n4 <= 1024) KIPP_RV(4);
        else KIPP_RV(8);
#undef KIPP_RV
    } else {
        hipLaunchKernelGGL((rmsnorm_kernel<TD, TO>), dim3(rows), dim3(width >= 2048 ? 512 : 256), 0, stream, x,
                           (const TD*)delta, weight, (TO*)out, width, eps, parts, stride);
    }
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
    if (delta_dtype == KIPP_BF16) {
        if (out_dtype == KIPP_BF16) launch_rmsnorm<bf16_t, bf16_t>(x, delta, weight, out, rows, width, eps, parts, stream);
        else launch_rmsnorm<bf16_t, float>(x, delta, weight, out, rows, width, eps, parts, stream);
    } else {
        if (out_dtype == KIPP_BF16) launch_rmsnorm<float, bf16_t>(x, delta, weight, out, rows, width, eps, parts, stream);
        else launch_rmsnorm<float, float>(x, delta, weight, out, rows, width, eps, parts, stream);
    }
    return KIPP_LAUNCH_CHECK();
}

int kipp_scale_rows(const void* rows, const float* sumsq, void* out, int n_rows, int width, int parts, int stride, float eps,
                    int steps_major, hipStream_t stream) {
    if (n_rows <= 0 || width <= 0) return 0;
    if (parts <= 0 || stride < parts || (steps_major && (width & 31))) return -1;
    hipLaunchKernelGGL(scale_rows_kernel, dim3(n_rows), dim3(256), 0, stream, (const bf16_t*)rows, sumsq, (bf16_t*)out, width,
                       parts, stride, eps, steps_major);
    return KIPP_LAUNCH_CHECK();
}

// tiles: bfloat16 [ceil(n / 16) 16, k] (`inner` 0) or [ceil(inner / 8) 16, k] (`inner` > 0, n = 2 inner), as above.
int kipp_tile_weight(const void* rows, void* tiles, int n, int k, int inner, hipStream_t stream) {
    if (n <= 0 || k <= 0 || (k & 31) || inner < 0 || (inner > 0 && n != 2 * inner)) return -1;
    const size_t tile_count = inner > 0 ? ((size_t)inner + 7) / 8 : ((size_t)n + 15) / 16;
    const size_t units = tile_count * (size_t)(k / 32) * 64;
    if ((units + 255) / 256 > 0x7fffffffu) return -2;
    hipLaunchKernelGGL(tile_weight_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, stream, (const uint4*)rows, (uint4*)tiles,
                       n, k, inner, units);
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

int kipp_swiglu(const void* gu, int in_dtype, int parts, void* out, int out_dtype, int rows, int inner, int pairs,
                hipStream_t stream) {
    size_t total = (size_t)rows * inner;
    if (total == 0) return 0;
    if (parts >= 1 && (inner & 7) == 0) {
        const size_t total8 = total / 8;
        const size_t slab4 = (size_t)rows * 2 * inner / 4;       // a slab in units of four values (paired tiles are as wide: 16 columns for 8 outputs)
        dim3 grid8((unsigned)((total8 + 255) / 256)), block8(256);
#define KIPP_SV(TI, TO) hipLaunchKernelGGL((swiglu_vec_kernel<TI, TO>), grid8, block8, 0, stream, (const TI*)gu, (TO*)out, inner, total8, pairs, parts, slab4)
        if (in_dtype == KIPP_BF16) {
            if (out_dtype == KIPP_BF16) KIPP_SV(bf16_t, bf16_t); else KIPP_SV(bf16_t, float);
        } else {
            if (out_dtype == KIPP_BF16) KIPP_SV(float, bf16_t); else KIPP_SV(float, float);
        }
#undef KIPP_SV
        return KIPP_LAUNCH_CHECK();
    }
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
#define KIPP_SW(TI, TO) hipLaunchKernelGGL((swiglu_kernel<TI, TO>), grid, block, 0, stream, (const TI*)gu, (TO*)out, inner, total, parts, pairs)
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

int kipp_gather_rows(const void* x, const int32_t* index, void* out, int rows, int width, hipStream_t stream) {
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(rows), dim3(width >= 256 ? 256 : 64), 0, stream, (const uint32_t*)x, index,
                       (uint32_t*)out, width);
    return KIPP_LAUNCH_CHECK();
}

// out[0 .. words) = in[0 .. words), 4-byte words
int kipp_copy_words(const void* in, void* out, size_t words, hipStream_t stream) {
    if (words == 0) return 0;
    const int wide = (((uintptr_t)in | (uintptr_t)out) & 15) == 0;
    const size_t units = wide ? (words + 3) / 4 : words;
    const unsigned blocks = (unsigned)((units + 255) / 256 < 4096 ? (units + 255) / 256 : 4096);
    hipLaunchKernelGGL(copy_words_kernel, dim3(blocks), dim3(256), 0, stream, (const uint32_t*)in, (uint32_t*)out, words, wide);
    return KIPP_LAUNCH_CHECK();
}

// out[0 .. words) = 0, 4-byte words (a kernel, not a memset: it may be recorded into a graph)
int kipp_fill_zero(void* out, size_t words, hipStream_t stream) {
    if (words == 0) return 0;
    const unsigned blocks = (unsigned)((words + 255) / 256 < 2048 ? (words + 255) / 256 : 2048);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, stream, (uint32_t*)out, words);
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
