/*
 * Scalar C references of the kernels: one plain loop per operation, float32
 * values, every sum running in index order in one float, as the reference's own
 * host path computes (/root/reference/src/kipp.c:2174-2186, 2221-2244, 2368-2404,
 * 2480-2562, 2882-2922).  Compiled for the host; the kernel tests compare each
 * kernel with its function here, and the host's scalar path is made of them.
 *
 * Matrices are [rows][columns] row-major; `dtype` says how a weight or a cache
 * is stored: 0 float32, 1 bfloat16 (widened element by element).
 */
#ifndef KIPP_REF_OPS_H
#define KIPP_REF_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define REF_F32 0
#define REF_BF16 1

float ref_bf16_to_float(uint16_t bits);
uint16_t ref_float_to_bf16(float value); /* round to nearest, ties to even; NaN stays NaN */
float ref_load(const void *base, int dtype, size_t index);
void ref_store(void *base, int dtype, size_t index, float value);

/* out[t] = table[token_t] widened */
void ref_embed(const void *table, int dtype, const int32_t *tokens, float *out, size_t n, size_t hidden);
/* out_i = (x_i * s) * w_i with s = 1 / sqrtf(sum(x^2) / n + eps) */
void ref_rms_norm(const float *x, const float *weight, float *out, size_t n, float eps);
/* out[r] = sum_c w[r][c] x[c] */
void ref_matvec(const void *weight, int dtype, const float *x, float *out, size_t rows, size_t columns);
/* every head vector of `values` [heads][d]: v_j *= (1 / sqrtf(sum(v^2) / d + eps)) * w_j; weight NULL: nothing */
void ref_head_norm(float *values, size_t heads, size_t d, const float *weight, float eps);
/* rotation of the first `rotary_dim` dims of one head at `position`; pair i is (i, i + rotary_dim / 2) or, interleaved, (2i, 2i + 1) */
void ref_rope(float *head, size_t rotary_dim, int32_t position, const float *inv_freq, int interleaved);
void ref_softmax(float *values, size_t count);
float ref_silu(float value);
/* out_i = silu(gate_up_i) * gate_up_{inner + i} */
void ref_swiglu(const float *gate_up, float *out, size_t inner);

/* slot of position `pos` of a sequence in a cache laid out [page][kv head][slot][d]: element offset of (kv head, pos, dim 0) */
size_t ref_cache_offset(const int32_t *table, size_t page_tokens, size_t n_kv, size_t d, size_t kv_head, size_t pos);
/* k, v [n_kv][d] of one token at `pos` into their page */
void ref_kv_write(void *k_cache, void *v_cache, int dtype, const int32_t *table, size_t page_tokens, size_t n_kv, size_t d, size_t pos,
                  const float *k, const float *v);
/* one query token at `pos` over the keys of its sequence (from max(0, pos - window + 1) when window > 0): out [n_q][d];
 * `scores` is room for pos + 1 floats */
void ref_paged_gqa(const float *q, const void *k_cache, const void *v_cache, int dtype, const int32_t *table, size_t page_tokens,
                   size_t n_q, size_t n_kv, size_t d, size_t pos, size_t window, float scale, float *scores, float *out);
/* the same over keys and values that lie one after the other, [tokens][n_kv][d] float32: every token of a whole sequence */
void ref_causal_gqa(const float *q, const float *k, const float *v, size_t tokens, size_t n_q, size_t n_kv, size_t d, size_t window,
                    float scale, float *scores, float *out);
/* index of the largest value, the lowest index among equals */
uint32_t ref_argmax(const float *values, size_t count);

#ifdef __cplusplus
}
#endif
#endif
