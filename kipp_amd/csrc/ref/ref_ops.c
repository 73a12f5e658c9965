/* Scalar references of the kernels; see ref_ops.h. */
#include "ref_ops.h"

#include <math.h>
#include <string.h>

float ref_bf16_to_float(uint16_t bits) {
    uint32_t wide = (uint32_t)bits << 16;
    float value;
    memcpy(&value, &wide, sizeof(value));
    return value;
}

uint16_t ref_float_to_bf16(float value) {
    uint32_t bits;
    memcpy(&bits, &value, sizeof(bits));
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((bits >> 16) | 0x0040u); /* NaN stays NaN */
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}

float ref_load(const void *base, int dtype, size_t index) {
    return dtype == REF_BF16 ? ref_bf16_to_float(((const uint16_t *)base)[index]) : ((const float *)base)[index];
}

void ref_store(void *base, int dtype, size_t index, float value) {
    if (dtype == REF_BF16) ((uint16_t *)base)[index] = ref_float_to_bf16(value);
    else ((float *)base)[index] = value;
}

void ref_embed(const void *table, int dtype, const int32_t *tokens, float *out, size_t n, size_t hidden) {
    for (size_t t = 0; t < n; ++t) {
        for (size_t i = 0; i < hidden; ++i) out[t * hidden + i] = ref_load(table, dtype, (size_t)tokens[t] * hidden + i);
    }
}

void ref_rms_norm(const float *x, const float *weight, float *out, size_t n, float eps) {
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) sum += x[i] * x[i];
    float scale = 1.0f / sqrtf(sum / (float)n + eps);
    for (size_t i = 0; i < n; ++i) out[i] = (x[i] * scale) * weight[i];
}

void ref_matvec(const void *weight, int dtype, const float *x, float *out, size_t rows, size_t columns) {
    for (size_t r = 0; r < rows; ++r) {
        float sum = 0.0f;
        if (dtype == REF_BF16) {
            const uint16_t *row = (const uint16_t *)weight + r * columns;
            for (size_t c = 0; c < columns; ++c) sum += ref_bf16_to_float(row[c]) * x[c];
        } else {
            const float *row = (const float *)weight + r * columns;
            for (size_t c = 0; c < columns; ++c) sum += row[c] * x[c];
        }
        out[r] = sum;
    }
}

void ref_head_norm(float *values, size_t heads, size_t d, const float *weight, float eps) {
    if (weight == NULL) return;
    for (size_t h = 0; h < heads; ++h) {
        float *v = values + h * d;
        float sum = 0.0f;
        for (size_t j = 0; j < d; ++j) sum += v[j] * v[j];
        float scale = 1.0f / sqrtf(sum / (float)d + eps);
        for (size_t j = 0; j < d; ++j) v[j] *= scale * weight[j];
    }
}

void ref_rope(float *head, size_t rotary_dim, int32_t position, const float *inv_freq, int interleaved) {
    size_t half = rotary_dim / 2;
    for (size_t i = 0; i < half; ++i) {
        float angle = (float)position * inv_freq[i];
        float c = cosf(angle), s = sinf(angle);
        size_t a = interleaved ? 2 * i : i, b = interleaved ? 2 * i + 1 : i + half;
        float x = head[a], y = head[b];
        head[a] = x * c - y * s;
        head[b] = y * c + x * s;
    }
}

void ref_softmax(float *values, size_t count) {
    if (count == 0) return;
    float largest = values[0];
    for (size_t i = 1; i < count; ++i) {
        if (values[i] > largest) largest = values[i];
    }
    float sum = 0.0f;
    for (size_t i = 0; i < count; ++i) {
        values[i] = expf(values[i] - largest);
        sum += values[i];
    }
    float inverse = 1.0f / sum;
    for (size_t i = 0; i < count; ++i) values[i] *= inverse;
}

float ref_silu(float value) { return value / (1.0f + expf(-value)); }

void ref_swiglu(const float *gate_up, float *out, size_t inner) {
    for (size_t i = 0; i < inner; ++i) out[i] = ref_silu(gate_up[i]) * gate_up[inner + i];
}

size_t ref_cache_offset(const int32_t *table, size_t page_tokens, size_t n_kv, size_t d, size_t kv_head, size_t pos) {
    size_t page = (size_t)table[pos / page_tokens];
    return ((page * n_kv + kv_head) * page_tokens + pos % page_tokens) * d;
}

void ref_kv_write(void *k_cache, void *v_cache, int dtype, const int32_t *table, size_t page_tokens, size_t n_kv, size_t d, size_t pos,
                  const float *k, const float *v) {
    for (size_t g = 0; g < n_kv; ++g) {
        size_t at = ref_cache_offset(table, page_tokens, n_kv, d, g, pos);
        for (size_t j = 0; j < d; ++j) {
            ref_store(k_cache, dtype, at + j, k[g * d + j]);
            ref_store(v_cache, dtype, at + j, v[g * d + j]);
        }
    }
}

void ref_paged_gqa(const float *q, const void *k_cache, const void *v_cache, int dtype, const int32_t *table, size_t page_tokens,
                   size_t n_q, size_t n_kv, size_t d, size_t pos, size_t window, float scale, float *scores, float *out) {
    size_t group = n_q / n_kv;
    size_t first = window > 0 && pos + 1 > window ? pos + 1 - window : 0;
    for (size_t h = 0; h < n_q; ++h) {
        size_t g = h / group;
        const float *query = q + h * d;
        for (size_t s = first; s <= pos; ++s) {
            size_t at = ref_cache_offset(table, page_tokens, n_kv, d, g, s);
            float dot = 0.0f;
            for (size_t j = 0; j < d; ++j) dot += query[j] * ref_load(k_cache, dtype, at + j);
            scores[s - first] = dot * scale;
        }
        ref_softmax(scores, pos - first + 1);
        float *o = out + h * d;
        for (size_t j = 0; j < d; ++j) o[j] = 0.0f;
        for (size_t s = first; s <= pos; ++s) {
            size_t at = ref_cache_offset(table, page_tokens, n_kv, d, g, s);
            float p = scores[s - first];
            for (size_t j = 0; j < d; ++j) o[j] += p * ref_load(v_cache, dtype, at + j);
        }
    }
}

void ref_causal_gqa(const float *q, const float *k, const float *v, size_t tokens, size_t n_q, size_t n_kv, size_t d, size_t window,
                    float scale, float *scores, float *out) {
    size_t group = n_q / n_kv;
    for (size_t t = 0; t < tokens; ++t) {
        size_t first = window > 0 && t + 1 > window ? t + 1 - window : 0;
        for (size_t h = 0; h < n_q; ++h) {
            size_t g = h / group;
            const float *query = q + (t * n_q + h) * d;
            for (size_t s = first; s <= t; ++s) {
                const float *key = k + (s * n_kv + g) * d;
                float dot = 0.0f;
                for (size_t j = 0; j < d; ++j) dot += query[j] * key[j];
                scores[s - first] = dot * scale;
            }
            ref_softmax(scores, t - first + 1);
            float *o = out + (t * n_q + h) * d;
            for (size_t j = 0; j < d; ++j) o[j] = 0.0f;
            for (size_t s = first; s <= t; ++s) {
                const float *value = v + (s * n_kv + g) * d;
                float p = scores[s - first];
                for (size_t j = 0; j < d; ++j) o[j] += p * value[j];
            }
        }
    }
}

uint32_t ref_argmax(const float *values, size_t count) {
    size_t best = 0;
    for (size_t i = 1; i < count; ++i) {
        if (values[i] > values[best]) best = i;
    }
    return (uint32_t)best;
}
