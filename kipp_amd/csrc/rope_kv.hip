// Per-head q/k RMSNorm, rotary position encoding and the write of keys and
// values into the paged cache, in one pass over the projection output.
//
// Input row layout of `qkv`: [n_q heads | n_kv key heads | n_kv value heads],
// each head `d` wide; `qkv` may come in `parts` slabs [parts, tokens, width] that are added
// in order (a product whose contraction was split over workgroups).  One wave handles one head of one token.
//   norm   u_j *= rsqrt(mean(u^2) + eps) * w_j, the same w for every head
//          (/root/reference/src/kipp.c:2480-2500), before the rotation;
//   rotary (u_i, u_{i+r/2}) <- (u_i c - u_{i+r/2} s, u_{i+r/2} c + u_i s),
//          angle = float(pos) * inv_freq[i]  (kipp.c:2368-2382); dims >= r pass;
//   write  key/value row of position pos goes to page table[pos / page], slot
//          pos % page; cache layout [page][kv head][slot][d].
#include "common.h"

#define HEADS_PER_BLOCK 4
#define MAX_D 256

template <typename TI, typename TO, typename TC>
__global__ void qk_norm_rope_kv_kernel(
    const TI* __restrict__ qkv, TO* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ inv_freq, int rotary_dim,
    int n_q, int n_kv, int d, int page, int n_slots, int parts, size_t part_stride) {
    __shared__ float buf[HEADS_PER_BLOCK][MAX_D];
    const int wave = threadIdx.x / KIPP_WAVE;
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y;
    int slot = blockIdx.x * HEADS_PER_BLOCK + wave;
    const bool active = slot < n_slots;
    if (!active) slot = n_slots - 1;  // stay in step with the barriers below
    const int kind = slot < n_q ? 0 : (slot < n_q + n_kv ? 1 : 2);  // q, k, v
    const int row_width = (n_q + 2 * n_kv) * d;
    const TI* src = qkv + (size_t)t * row_width + (size_t)slot * d;
    const int pos = positions[t];

    float vals[MAX_D / KIPP_WAVE];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
        const int e = lane + c * KIPP_WAVE;
        float v = 0.0f;
        if (e < d)
            for (int p = 0; p < parts; ++p) v += load_f(src, p * part_stride + e);   // slabs of a split product, in order
        vals[c] = v;
        ss += v * v;
    }
    const float* norm_w = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
    if (norm_w != nullptr) {
        ss = wave_sum(ss);
        const float scale = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            if (e < d) vals[c] *= scale * norm_w[e];
        }
    }
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
        const int e = lane + c * KIPP_WAVE;
        if (e < d) buf[wave][e] = vals[c];
    }
    __syncthreads();
    // Barriers stay outside the conditions: waves of one workgroup hold heads
    // of different kinds.
    const bool rotate = kind != 2 && inv_freq != nullptr;
    const int half = rotary_dim / 2;
    float lo[MAX_D / 2 / KIPP_WAVE], hi[MAX_D / 2 / KIPP_WAVE];
#pragma unroll
    for (int c = 0; c < MAX_D / 2 / KIPP_WAVE; ++c) {
        const int i = lane + c * KIPP_WAVE;
        lo[c] = hi[c] = 0.0f;
        if (rotate && i < half) {
            const float angle = (float)pos * inv_freq[i];
            const float cs = cosf(angle), sn = sinf(angle);
            const float a = buf[wave][i], b = buf[wave][i + half];
            lo[c] = a * cs - b * sn;
            hi[c] = b * cs + a * sn;
        }
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < MAX_D / 2 / KIPP_WAVE; ++c) {
        const int i = lane + c * KIPP_WAVE;
        if (rotate && i < half) {
            buf[wave][i] = lo[c];
            buf[wave][i + half] = hi[c];
        }
    }
    __syncthreads();
    if (!active) return;
    if (kind == 0) {
        TO* dst = q_out + ((size_t)t * n_q + slot) * d;
        for (int e = lane; e < d; e += KIPP_WAVE) store_f(dst, e, buf[wave][e]);
    } else {
        const int head = kind == 1 ? slot - n_q : slot - n_q - n_kv;
        const int seq = seq_of_token[t];
        const int page_id = block_table[(size_t)seq * max_blocks + pos / page];
        TC* dst = (kind == 1 ? k_cache : v_cache) +
                  (((size_t)page_id * n_kv + head) * page + pos % page) * d;
        for (int e = lane; e < d; e += KIPP_WAVE) store_f(dst, e, buf[wave][e]);
    }
}

extern "C" int kipp_qk_norm_rope_kv(
    const void* qkv, int in_dtype, void* q_out, int q_dtype, void* k_cache, void* v_cache, int cache_dtype,
    const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    const float* q_norm_w, const float* k_norm_w, float eps, const float* inv_freq, int rotary_dim,
    int n_tokens, int n_q, int n_kv, int d, int page, int write_kv, int parts, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d > MAX_D || d <= 0 || rotary_dim > d || (rotary_dim & 1)) return -1;
    const int n_slots = write_kv ? n_q + 2 * n_kv : n_q;
    dim3 grid((n_slots + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK, n_tokens), block(HEADS_PER_BLOCK * KIPP_WAVE);
#define KIPP_RK(TI, TO, TC)                                                                                  \
    hipLaunchKernelGGL((qk_norm_rope_kv_kernel<TI, TO, TC>), grid, block, 0, stream, (const TI*)qkv,         \
                       (TO*)q_out, (TC*)k_cache, (TC*)v_cache, positions, seq_of_token, block_table,         \
                       max_blocks, q_norm_w, k_norm_w, eps, inv_freq, rotary_dim, n_q, n_kv, d, page, n_slots, parts,      \
                       (size_t)n_tokens * (n_q + 2 * n_kv) * d)
    if (in_dtype == KIPP_F32 && q_dtype == KIPP_F32 && cache_dtype == KIPP_F32) KIPP_RK(float, float, float);
    else if (in_dtype == KIPP_F32 && q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_RK(float, bf16_t, bf16_t);
    else if (in_dtype == KIPP_BF16 && q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_RK(bf16_t, bf16_t, bf16_t);
    else return -2;
#undef KIPP_RK
    return KIPP_LAUNCH_CHECK();
}
