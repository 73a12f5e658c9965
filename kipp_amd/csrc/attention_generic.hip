// Causal grouped-query attention over the paged cache for any mix of query
// tokens (prompt portions and single decoded tokens alike), any head size up
// to 256 and any storage type.  One wave per (token, query head); this is the
// float32 path's kernel and the fallback of sizes the MFMA kernels refuse.
//
// For query position p of a sequence the keys are s in [max(0, p-window+1), p]
// (window 0: from 0), score = (q . k_s) * scale, softmax with the maximum
// subtracted, out = sum p_s v_s  (/root/reference/src/kipp.c:2882-2922).  Keys are
// taken in tiles of 64 aligned to absolute key index, so the sequence of
// operations for one query depends on its own position only, never on what
// else is in the batch.
#include "common.h"
#include <math.h>

#define HEADS_PER_BLOCK 4
#define MAX_D 256

template <typename TQ, typename TC, typename TO>
__global__ void paged_attention_generic_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache, TO* __restrict__ out,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks,
    int n_q, int n_kv, int d, int page, float scale, int window) {
    __shared__ float q_s[HEADS_PER_BLOCK][MAX_D];
    __shared__ float p_s[HEADS_PER_BLOCK][KIPP_WAVE];
    __shared__ unsigned long long off_s[HEADS_PER_BLOCK][KIPP_WAVE];
    const int wave = threadIdx.x / KIPP_WAVE;
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y;
    int head = blockIdx.x * HEADS_PER_BLOCK + wave;
    const bool active = head < n_q;
    if (!active) head = n_q - 1;
    const int g = head / (n_q / n_kv);
    const int pos = positions[t];
    const int seq = seq_of_token[t];
    const int32_t* table = block_table + (size_t)seq * max_blocks;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;

    const TQ* q_row = q + ((size_t)t * n_q + head) * d;
    for (int e = lane; e < d; e += KIPP_WAVE) q_s[wave][e] = load_f(q_row, e);
    __syncthreads();

    float m = -INFINITY, l = 0.0f;
    float acc[MAX_D / KIPP_WAVE];
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) acc[c] = 0.0f;

    for (int s0 = (lo / KIPP_WAVE) * KIPP_WAVE; s0 <= pos; s0 += KIPP_WAVE) {
        const int s = s0 + lane;
        const bool valid = s >= lo && s <= pos;
        float score = -INFINITY;
        unsigned long long off = 0;
        if (valid) {
            const int page_id = table[s / page];
            off = (((unsigned long long)page_id * n_kv + g) * page + s % page) * d;
            const TC* k_row = k_cache + off;
            float dot = 0.0f;
            for (int e = 0; e < d; ++e) dot += q_s[wave][e] * load_f(k_row, e);
            score = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(score));
        const float alpha = expf(m - m_new);
        const float p = valid ? expf(score - m_new) : 0.0f;
        l = l * alpha + wave_sum(p);
        m = m_new;
        __syncthreads();
        p_s[wave][lane] = p;
        off_s[wave][lane] = off;
        __syncthreads();
        const int j_lo = max(0, lo - s0);
        const int j_hi = min(KIPP_WAVE, pos - s0 + 1);
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            if (e < d) {
                float a = acc[c] * alpha;
                for (int j = j_lo; j < j_hi; ++j) a += p_s[wave][j] * load_f(v_cache + off_s[wave][j], e);
                acc[c] = a;
            }
        }
    }
    if (!active) return;
    TO* o_row = out + ((size_t)t * n_q + head) * d;
    const float inv = 1.0f / l;
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
        const int e = lane + c * KIPP_WAVE;
        if (e < d) store_f(o_row, e, acc[c] * inv);
    }
}

extern "C" int kipp_paged_attention_generic(
    const void* q, int q_dtype, const void* k_cache, const void* v_cache, int cache_dtype, void* out, int out_dtype,
    const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int n_tokens, int n_q, int n_kv, int d, int page, float scale, int window, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d > MAX_D || d <= 0 || n_kv <= 0 || n_q % n_kv) return -1;
    dim3 grid((n_q + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK, n_tokens), block(HEADS_PER_BLOCK * KIPP_WAVE);
#define KIPP_PA(TQ, TC, TO)                                                                                    \
    hipLaunchKernelGGL((paged_attention_generic_kernel<TQ, TC, TO>), grid, block, 0, stream, (const TQ*)q,     \
                       (const TC*)k_cache, (const TC*)v_cache, (TO*)out, positions, seq_of_token, block_table, \
                       max_blocks, n_q, n_kv, d, page, scale, window)
    if (q_dtype == KIPP_F32 && cache_dtype == KIPP_F32 && out_dtype == KIPP_F32) KIPP_PA(float, float, float);
    else if (q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16 && out_dtype == KIPP_BF16) KIPP_PA(bf16_t, bf16_t, bf16_t);
    else return -2;
#undef KIPP_PA
    return KIPP_LAUNCH_CHECK();
}
