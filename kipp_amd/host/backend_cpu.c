/*
 * The scalar float32 path on the host: every operation of a forward pass as
 * plain loops over the references in csrc/ref/ref_ops.c, block tables and pages
 * included.  It is the oracle of the GPU paths (the role of the reference's own
 * host path, /root/reference/src/kipp.c:2588-2661 and :2882-3020) and needs no GPU.
 * Weights are widened to float32 when placed; the cache is float32.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "../csrc/ref/ref_ops.h"
#include "backend.h"

static void cpu_destroy(kipp_runtime *rt) { free(rt); }

static void *cpu_alloc(kipp_runtime *rt, size_t bytes, kipp_error *error) {
    (void)rt;
    void *memory = calloc(1, bytes ? bytes : 1);
    if (memory == NULL) kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for %zu bytes", bytes);
    return memory;
}

static void cpu_free(kipp_runtime *rt, void *memory) {
    (void)rt;
    free(memory);
}

static int cpu_zero(kipp_runtime *rt, void *memory, size_t bytes, kipp_error *error) {
    (void)rt;
    (void)error;
    memset(memory, 0, bytes);
    return 0;
}

static int cpu_move(kipp_runtime *rt, void *to, const void *from, size_t bytes, kipp_error *error) {
    (void)rt;
    (void)error;
    if (bytes != 0) memmove(to, from, bytes);
    return 0;
}

static float widen(const kipp_tensor *tensor, size_t index) {
    if (tensor->dtype == KIPP_F32) return ((const float *)tensor->data)[index];
    uint16_t bits = ((const uint16_t *)tensor->data)[index];
    if (tensor->dtype == KIPP_BF16) return ref_bf16_to_float(bits);
    /* float16, widened exactly */
    uint32_t sign = (uint32_t)(bits & 0x8000u) << 16, exponent = (bits >> 10) & 0x1f, fraction = bits & 0x3ffu, wide;
    if (exponent == 0) {
        if (fraction == 0) wide = sign;
        else {
            int shift = 0;
            while (!(fraction & 0x400u)) {
                fraction <<= 1;
                ++shift;
            }
            wide = sign | ((uint32_t)(127 - 15 + 1 - shift) << 23) | ((fraction & 0x3ffu) << 13);
        }
    } else if (exponent == 31) wide = sign | 0x7f800000u | (fraction << 13);
    else wide = sign | ((exponent + 127 - 15) << 23) | (fraction << 13);
    float value;
    memcpy(&value, &wide, sizeof(value));
    return value;
}

static int cpu_place_matrix(kipp_runtime *rt, const kipp_tensor *const *pieces, size_t piece_count, kipp_weight_layout layout, kipp_weight *out,
                            kipp_error *error) {
    (void)rt;
    (void)layout;
    uint64_t rows = 0, columns = pieces[0]->shape[1];
    for (size_t p = 0; p < piece_count; ++p) rows += pieces[p]->shape[0];
    size_t count;
    if (rows > UINT32_MAX || columns > UINT32_MAX || kipp_mul_size((size_t)rows, (size_t)columns, &count) != 0 || count > SIZE_MAX / 4)
        return kipp_fail(error, KIPP_ERROR_RANGE, "a matrix of %llu x %llu is too large", (unsigned long long)rows, (unsigned long long)columns);
    float *data = malloc(count ? count * sizeof(float) : 4);
    if (data == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a matrix of %zu values", count);
    size_t at = 0;
    for (size_t p = 0; p < piece_count; ++p) {
        size_t n = (size_t)(pieces[p]->shape[0] * pieces[p]->shape[1]);
        for (size_t i = 0; i < n; ++i) data[at++] = widen(pieces[p], i);
    }
    *out = (kipp_weight){data, KIPP_F32, (uint32_t)rows, (uint32_t)columns, NULL, false};
    return 0;
}

static int cpu_place_vector(kipp_runtime *rt, const kipp_tensor *tensor, float **out, kipp_error *error) {
    (void)rt;
    size_t n = (size_t)tensor->shape[0];
    float *data = malloc(n ? n * sizeof(float) : 4);
    if (data == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a vector of %zu values", n);
    for (size_t i = 0; i < n; ++i) data[i] = widen(tensor, i);
    *out = data;
    return 0;
}

static void cpu_free_weight(kipp_runtime *rt, kipp_weight *weight) {
    (void)rt;
    free(weight->data);
    weight->data = NULL;
}

static int cpu_embed(kipp_runtime *rt, const kipp_weight *table, const int32_t *tokens, float *out, uint32_t n, kipp_error *error) {
    (void)rt;
    (void)error;
    ref_embed(table->data, REF_F32, tokens, out, n, table->k);
    return 0;
}

static void add_delta(float *x, const kipp_delta *delta, size_t count) {
    for (int p = 0; p < delta->parts; ++p) {
        const float *slab = delta->data + (size_t)p * count;
        for (size_t i = 0; i < count; ++i) x[i] += slab[i];
    }
}

static int cpu_rmsnorm(kipp_runtime *rt, float *x, kipp_delta *delta, const float *weight, kipp_rows *out, uint32_t rows, uint32_t width,
                       float eps, bool may_leave_scale, kipp_error *error) {
    (void)may_leave_scale; /* this path finishes every row */
    if (delta != NULL && kipp_settle(rt, delta, error) != 0) return -1;
    if (delta != NULL && delta->parts > 0) add_delta(x, delta, (size_t)rows * width);
    for (uint32_t r = 0; r < rows; ++r) ref_rms_norm(x + (size_t)r * width, weight, (float *)out->data + (size_t)r * width, width, eps);
    out->sumsq = NULL;
    return 0;
}

static int cpu_residual_add(kipp_runtime *rt, float *x, kipp_delta *delta, uint32_t rows, uint32_t width, kipp_error *error) {
    if (kipp_settle(rt, delta, error) != 0) return -1;
    add_delta(x, delta, (size_t)rows * width);
    return 0;
}

static int cpu_argmax(kipp_runtime *rt, const float *logits, int32_t *out, uint32_t rows, uint32_t vocab, kipp_error *error) {
    (void)rt;
    (void)error;
    for (uint32_t r = 0; r < rows; ++r) out[r] = (int32_t)ref_argmax(logits + (size_t)r * vocab, vocab);
    return 0;
}

static int cpu_row_nll(kipp_runtime *rt, const float *logits, const uint32_t *targets, double *out, uint32_t rows, uint32_t vocab, kipp_error *error) {
    (void)rt;
    (void)error;
    for (uint32_t r = 0; r < rows; ++r) {
        const float *row = logits + (size_t)r * vocab;
        float top = row[0];
        for (uint32_t t = 1; t < vocab; ++t) top = row[t] > top ? row[t] : top;
        double sum = 0.0;
        for (uint32_t t = 0; t < vocab; ++t) sum += exp((double)row[t] - (double)top);
        out[r] = (double)top + log(sum) - (double)row[targets[r]];
    }
    return 0;
}

static int cpu_linear(kipp_runtime *rt, const kipp_rows *rows_in, const kipp_weight *w, uint32_t m, int max_parts, kipp_delta *out, kipp_error *error) {
    (void)max_parts;
    if (rows_in->sumsq != NULL || rows_in->steps_major) return kipp_fail(error, KIPP_ERROR_INTERNAL, "rows without their scale on the host path");
    const void *x = rows_in->data;
    size_t count;
    if (kipp_mul_size(m, w->n, &count) != 0 || count > SIZE_MAX / 4) return kipp_fail(error, KIPP_ERROR_RANGE, "a product's size overflows");
    float *y = kipp_scratch(rt, count * sizeof(float), error);
    if (y == NULL) return -1;
    for (uint32_t r = 0; r < m; ++r) ref_matvec(w->data, REF_F32, (const float *)x + (size_t)r * w->k, y + (size_t)r * w->n, w->n, w->k);
    *out = (kipp_delta){y, 1, NULL, NULL, 0, 0, false};
    return 0;
}

static int cpu_swiglu(kipp_runtime *rt, const kipp_delta *gate_up, void *out, uint32_t rows, uint32_t inner, kipp_error *error) {
    (void)rt;
    if (gate_up->parts != 1) return kipp_fail(error, KIPP_ERROR_INTERNAL, "the host path computes products in one part");
    for (uint32_t r = 0; r < rows; ++r) ref_swiglu(gate_up->data + (size_t)r * 2 * inner, (float *)out + (size_t)r * inner, inner);
    return 0;
}

static int cpu_rotary_angles(kipp_runtime *rt, const int32_t *positions, const float *inv_freq, uint32_t n, uint32_t half,
                             const float **out_rotation, kipp_error *error) {
    (void)rt;
    (void)positions;
    (void)n;
    (void)half;
    (void)error;
    *out_rotation = inv_freq; /* the host path computes every angle where it is used, as the reference does */
    return 0;
}

static int cpu_qk_norm_rope_kv(kipp_runtime *rt, const kipp_delta *qkv, void *q_out, const kipp_cache_view *cache, const kipp_batch *batch,
                               const kipp_attention_geometry *geometry, const float *q_norm_w, const float *k_norm_w, float eps,
                               const float *rotation, uint32_t rotary_dim, int interleaved, kipp_error *error) {
    (void)rt;
    if (qkv->parts != 1) return kipp_fail(error, KIPP_ERROR_INTERNAL, "the host path computes products in one part");
    const size_t d = geometry->head_dim, n_q = geometry->n_q, n_kv = geometry->n_kv, width = (n_q + 2 * n_kv) * d;
    const float *inv_freq = rotation; /* see cpu_rotary_angles */
    for (uint32_t t = 0; t < batch->n_tokens; ++t) {
        float *row = qkv->data + (size_t)t * width; /* the product's own buffer: normed and rotated in place */
        float *q = row, *k = row + n_q * d, *v = k + n_kv * d;
        ref_head_norm(q, n_q, d, q_norm_w, eps);
        ref_head_norm(k, n_kv, d, k_norm_w, eps);
        if (inv_freq != NULL) {
            for (size_t h = 0; h < n_q; ++h) ref_rope(q + h * d, rotary_dim, batch->positions[t], inv_freq, interleaved);
            for (size_t h = 0; h < n_kv; ++h) ref_rope(k + h * d, rotary_dim, batch->positions[t], inv_freq, interleaved);
        }
        memcpy((float *)q_out + (size_t)t * n_q * d, q, n_q * d * sizeof(float));
        if (cache->writable) {
            const int32_t *table = batch->tables[cache->group] + (size_t)batch->seq_of_token[t] * batch->max_blocks;
            ref_kv_write(cache->k, cache->v, REF_F32, table, cache->page_tokens, n_kv, d, (size_t)batch->positions[t], k, v);
        }
    }
    return 0;
}

static int cpu_attention(kipp_runtime *rt, const void *q, const kipp_cache_view *cache, void *out, kipp_batch *batch,
                         const kipp_attention_geometry *geometry, kipp_error *error) {
    const size_t d = geometry->head_dim, n_q = geometry->n_q;
    size_t longest = 0;
    for (uint32_t t = 0; t < batch->n_tokens; ++t) {
        if ((size_t)batch->positions[t] + 1 > longest) longest = (size_t)batch->positions[t] + 1;
    }
    float *scores = kipp_scratch(rt, longest * sizeof(float), error);
    if (scores == NULL) return -1;
    for (uint32_t t = 0; t < batch->n_tokens; ++t) {
        const int32_t *table = batch->tables[cache->group] + (size_t)batch->seq_of_token[t] * batch->max_blocks;
        ref_paged_gqa((const float *)q + (size_t)t * n_q * d, cache->k, cache->v, REF_F32, table, cache->page_tokens, n_q, geometry->n_kv, d,
                      (size_t)batch->positions[t], geometry->window, geometry->scale, scores, (float *)out + (size_t)t * n_q * d);
    }
    return 0;
}

static int cpu_gather_rows(kipp_runtime *rt, const float *x, const int32_t *index, float *out, uint32_t n, uint32_t width, kipp_error *error) {
    (void)rt;
    (void)error;
    for (uint32_t r = 0; r < n; ++r) memcpy(out + (size_t)r * width, x + (size_t)index[r] * width, (size_t)width * sizeof(float));
    return 0;
}

kipp_runtime *kipp_runtime_cpu(kipp_error *error) {
    kipp_runtime *rt = calloc(1, sizeof(*rt));
    if (rt == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    rt->name = "cpu-fp32";
    rt->path = KIPP_PATH_CPU_FP32;
    rt->act_dtype = KIPP_F32;
    rt->on_host = true;
    rt->destroy = cpu_destroy;
    rt->mem_alloc = cpu_alloc;
    rt->mem_free = cpu_free;
    rt->mem_zero = cpu_zero;
    rt->upload = cpu_move;
    rt->download = cpu_move;
    rt->copy = cpu_move;
    rt->place_matrix = cpu_place_matrix;
    rt->place_vector = cpu_place_vector;
    rt->free_weight = cpu_free_weight;
    rt->embed = cpu_embed;
    rt->rmsnorm = cpu_rmsnorm;
    rt->residual_add = cpu_residual_add;
    rt->linear = cpu_linear;
    rt->swiglu = cpu_swiglu;
    rt->rotary_angles = cpu_rotary_angles;
    rt->qk_norm_rope_kv = cpu_qk_norm_rope_kv;
    rt->attention = cpu_attention;
    rt->gather_rows = cpu_gather_rows;
    rt->argmax = cpu_argmax;
    rt->row_nll = cpu_row_nll;
    return rt;
}
