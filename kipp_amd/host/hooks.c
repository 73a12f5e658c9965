/* Each scalar operation of the host path alone, for tests (the reference exposes its own the same way,
 * /root/reference/src/kipp.h:299-340). */
#include <math.h>
#include <stdlib.h>

#include "../csrc/ref/ref_ops.h"
#include "kipp_amd.h"

float kipp_test_bf16_to_float(uint16_t value) { return ref_bf16_to_float(value); }
uint16_t kipp_test_float_to_bf16(float value) { return ref_float_to_bf16(value); }

void kipp_test_rms_norm(const float *input, const float *weight, float *output, size_t length, float epsilon) {
    ref_rms_norm(input, weight, output, length, epsilon);
}

void kipp_test_matvec(const float *weight, const float *input, float *output, size_t rows, size_t columns) {
    ref_matvec(weight, REF_F32, input, output, rows, columns);
}

void kipp_test_matvec_bf16(const uint16_t *weight, const float *input, float *output, size_t rows, size_t columns) {
    ref_matvec(weight, REF_BF16, input, output, rows, columns);
}

/* pairs (i, i + head_dim / 2), frequency theta^(-2i / head_dim) in float as the reference computes it
 * (/root/reference/src/kipp.c:2368-2382) */
void kipp_test_rope(float *head, size_t head_dim, uint32_t position, float theta) {
    size_t half = head_dim / 2;
    float *inv_freq = malloc((half ? half : 1) * sizeof(float));
    if (inv_freq == NULL) return;
    for (size_t i = 0; i < half; ++i) inv_freq[i] = powf(theta, -(float)(2 * i) / (float)head_dim);
    ref_rope(head, head_dim, (int32_t)position, inv_freq, 0);
    free(inv_freq);
}

void kipp_test_softmax(float *values, size_t count) { ref_softmax(values, count); }
float kipp_test_silu(float value) { return ref_silu(value); }

void kipp_test_causal_gqa(const float *query, const float *key, const float *value, float *output, size_t token_count,
                          size_t query_head_count, size_t kv_head_count, size_t head_dim) {
    float *scores = malloc((token_count ? token_count : 1) * sizeof(float));
    if (scores == NULL) return;
    ref_causal_gqa(query, key, value, token_count, query_head_count, kv_head_count, head_dim, 0, 1.0f / sqrtf((float)head_dim), scores, output);
    free(scores);
}
