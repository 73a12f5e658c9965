/*
 * The device side that parts share: where memory lives, how a tensor is placed,
 * and the operations of a forward pass, as a table of functions.  Two tables
 * exist: the GPU's (backend_hip.c: the kernel libraries' launchers on buffers
 * from hipMalloc, in bfloat16 or in float32) and the host's (backend_cpu.c: the
 * scalar references, float32).  A part calls only this table and never asks
 * which one it is.
 *
 * Types: activations between operations have `act_dtype` (the cache too); the
 * residual stream, deltas, norm weights and logits are float32 everywhere.
 */
#ifndef KIPP_AMD_BACKEND_H
#define KIPP_AMD_BACKEND_H

#include "internal.h"

typedef struct kipp_runtime kipp_runtime;

/* Geometry of one attention launch. */
typedef struct {
    uint32_t n_q, n_kv, head_dim, window; /* window 0: every key */
    float scale;
} kipp_attention_geometry;

struct kipp_runtime {
    const char *name;
    kipp_path path;
    int act_dtype;
    bool on_host;
    void *state; /* the table's own */

    void (*destroy)(kipp_runtime *rt);
    void *(*mem_alloc)(kipp_runtime *rt, size_t bytes, kipp_error *error); /* zeroed */
    void (*mem_free)(kipp_runtime *rt, void *memory);
    int (*mem_zero)(kipp_runtime *rt, void *memory, size_t bytes, kipp_error *error);
    int (*upload)(kipp_runtime *rt, void *to, const void *from_host, size_t bytes, kipp_error *error);
    int (*download)(kipp_runtime *rt, void *to_host, const void *from, size_t bytes, kipp_error *error); /* waits for the work before it */
    int (*copy)(kipp_runtime *rt, void *to, const void *from, size_t bytes, kipp_error *error);

    /* Placement: rows of several tensors one under the other as one matrix ([Wq; Wk; Wv], [gate; up]); a tensor stored in
     * bfloat16 stays so on the bfloat16 path, 32-bit stays 32-bit, pieces of different types and everything on the
     * 32-bit paths are widened.  A vector is always widened to float32. */
    int (*place_matrix)(kipp_runtime *rt, const kipp_tensor *const *pieces, size_t piece_count, kipp_weight *out, kipp_error *error);
    int (*place_vector)(kipp_runtime *rt, const kipp_tensor *tensor, float **out, kipp_error *error);
    void (*free_weight)(kipp_runtime *rt, kipp_weight *weight);

    /* x[t] = table[token_t], float32 */
    int (*embed)(kipp_runtime *rt, const kipp_weight *table, const int32_t *tokens, float *out, uint32_t n, kipp_error *error);
    /* out = norm(x [+ delta]) * weight in the activation type; with a delta, x += delta (its slabs in order) in place first */
    int (*rmsnorm)(kipp_runtime *rt, float *x, const kipp_delta *delta, const float *weight, void *out, uint32_t rows, uint32_t width,
                   float eps, kipp_error *error);
    int (*residual_add)(kipp_runtime *rt, float *x, const kipp_delta *delta, uint32_t rows, uint32_t width, kipp_error *error);
    /* out (workspace of the step) = x [m, k] . w^T as float32 slabs; `max_parts` 1 asks for the finished sum */
    int (*linear)(kipp_runtime *rt, const void *x, const kipp_weight *w, uint32_t m, int max_parts, kipp_delta *out, kipp_error *error);
    /* out[t, i] = silu(gate_up[t, i]) * gate_up[t, inner + i] in the activation type */
    int (*swiglu)(kipp_runtime *rt, const kipp_delta *gate_up, void *out, uint32_t rows, uint32_t inner, kipp_error *error);
    /* The rotation of a step's positions in the form this table's `qk_norm_rope_kv` rotates from, made once for every layer
     * that turns with these frequencies: on the GPU cos(float(pos_t) f_i) for every i, then the sines, float32 [n, 2 half] in
     * the step's workspace; on the host the frequencies themselves. */
    int (*rotary_angles)(kipp_runtime *rt, const int32_t *positions, const float *inv_freq, uint32_t n, uint32_t half,
                         const float **out_rotation, kipp_error *error);
    /* per-head norm of q and k (weights may be NULL), rotation at every token's position, q to q_out, k and v into their pages */
    int (*qk_norm_rope_kv)(kipp_runtime *rt, const kipp_delta *qkv, void *q_out, const kipp_cache_view *cache, const kipp_batch *batch,
                           const kipp_attention_geometry *geometry, const float *q_norm_w, const float *k_norm_w, float eps,
                           const float *rotation, uint32_t rotary_dim, int interleaved, kipp_error *error);
    /* causal grouped-query attention of every token of the batch over its sequence's pages */
    int (*attention)(kipp_runtime *rt, const void *q, const kipp_cache_view *cache, void *out, kipp_batch *batch,
                     const kipp_attention_geometry *geometry, kipp_error *error);
    int (*gather_rows)(kipp_runtime *rt, const float *x, const int32_t *index, float *out, uint32_t n, uint32_t width, kipp_error *error);

    /* the step's workspace: chunks that are kept from step to step and handed out from the start again (runtime.c) */
    struct {
        void **chunks;
        size_t *sizes;
        size_t count, current, used;
    } workspace;
};

kipp_runtime *kipp_runtime_cpu(kipp_error *error);
kipp_runtime *kipp_runtime_hip(kipp_path path, int device, const char *kernel_dir, kipp_error *error);
void kipp_runtime_destroy(kipp_runtime *rt);
/* Memory for the rest of the step, aligned to 256 bytes. */
void *kipp_scratch(kipp_runtime *rt, size_t bytes, kipp_error *error);
void kipp_scratch_reset(kipp_runtime *rt);
size_t kipp_dtype_bytes(int dtype);

#endif
