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
     * 32-bit paths are widened.  `layout`: whether the few-rows products read this matrix (a table may then keep it a second
     * time in the layout they stream fastest).  A vector is always widened to float32. */
    int (*place_matrix)(kipp_runtime *rt, const kipp_tensor *const *pieces, size_t piece_count, kipp_weight_layout layout, kipp_weight *out,
                        kipp_error *error);
    int (*place_vector)(kipp_runtime *rt, const kipp_tensor *tensor, float **out, kipp_error *error);
    void (*free_weight)(kipp_runtime *rt, kipp_weight *weight);

    /* x[t] = table[token_t], float32 */
    int (*embed)(kipp_runtime *rt, const kipp_weight *table, const int32_t *tokens, float *out, uint32_t n, kipp_error *error);
    /* out->data = norm(x [+ delta]) * weight in the activation type; with a delta, x += delta (its slabs in order, or its
     * product, launched here) in place first.  With `may_leave_scale` a table may leave the rows without their scale
     * (out->sumsq says so): a product that was not launched yet then adds itself to x, and prepares the norm, in one kernel. */
    int (*rmsnorm)(kipp_runtime *rt, float *x, kipp_delta *delta, const float *weight, kipp_rows *out, uint32_t rows, uint32_t width,
                   float eps, bool may_leave_scale, kipp_error *error);
    int (*residual_add)(kipp_runtime *rt, float *x, kipp_delta *delta, uint32_t rows, uint32_t width, kipp_error *error);
    /* out (workspace of the step) = x [m, k] . w^T as float32 slabs; `max_parts` 1 asks for the finished sum.  Rows that
     * lack their scale are taken as they are where the product's kernel applies it, and finished first elsewhere. */
    int (*linear)(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w, uint32_t m, int max_parts, kipp_delta *out, kipp_error *error);
    /* May this product wait for the norm that follows it (kipp_linear_defer)?  NULL: never. */
    bool (*defers)(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w, uint32_t m);
    /* out = in's rows with their scale applied (only a table that leaves scales has it) */
    int (*scale_rows)(kipp_runtime *rt, const kipp_rows *in, void *out, uint32_t rows, uint32_t width, kipp_error *error);
    /* Optional (NULL: none).  act[t, i] = silu(x . gate_i) * (x . up_i) for w = [gate; up], in one kernel where the table has
     * one for this shape: *done says whether it ran (else the caller takes linear and swiglu).  act->data is given; `reader` is
     * the matrix that act is multiplied with next (the table may write act in the order that product reads fastest, and says so
     * in act->steps_major). */
    int (*gated)(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w_gate_up, const kipp_weight *reader, kipp_rows *act, uint32_t m,
                 bool *done, kipp_error *error);
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
    /* Optional (NULL: none).  A step of single tokens: the QKV product, the per-head norms, the rotation, the write of the new
     * keys and values and the attention over the pages, with as few kernels as the table has for this shape; *done says
     * whether it ran (else the caller takes linear, qk_norm_rope_kv and attention).  out->data is given; `reader` is the matrix
     * that the mixed heads are multiplied with next (as for `gated`). */
    int (*decode_attention)(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w_qkv, const kipp_cache_view *cache,
                            const kipp_weight *reader, kipp_rows *out, kipp_batch *batch, const kipp_attention_geometry *geometry,
                            const float *q_norm_w, const float *k_norm_w, float eps, const float *rotation, uint32_t rotary_dim,
                            int interleaved, bool *done, kipp_error *error);
    int (*gather_rows)(kipp_runtime *rt, const float *x, const int32_t *index, float *out, uint32_t n, uint32_t width, kipp_error *error);
    /* out[r] = the index of the largest of logits[r, :vocab], the lowest among equals (/root/reference/src/kipp.c:3459-3464) */
    int (*argmax)(kipp_runtime *rt, const float *logits, int32_t *out, uint32_t rows, uint32_t vocab, kipp_error *error);
    /* out[r] (host memory, float64) = -log softmax(logits[r, :vocab])[targets[r]] (`targets`: host memory, inside the
     * vocabulary): the row's maximum in float32, exponentials and their sum in float64 (/root/reference/src/kipp_cli.c:759-778).
     * It waits for the result, and takes nothing from the step's workspace. */
    int (*row_nll)(kipp_runtime *rt, const float *logits, const uint32_t *targets, double *out, uint32_t rows, uint32_t vocab, kipp_error *error);
    /* Optional (NULL: the caller samples on the host).  *out = memory of the path's own with one token a row, each chosen as
     * kipp_sample_ex would choose it with `params[r]` (host memory; bias and penalties change the row of logits where it
     * lies) and the draw `uniform[r]`; it takes nothing from the step's workspace, so it may follow a recorded step. */
    int (*sample)(kipp_runtime *rt, float *logits, const kipp_sample_params *params, const double *uniform, int32_t **out, uint32_t rows,
                  uint32_t vocab, kipp_error *error);

    /* Optional (NULL: none).  Recording: between graph_begin and graph_end the operations above are recorded instead of run
     * (no memory may be made meanwhile: the step's workspace says so, and the recording is dropped); graph_end with `keep`
     * gives what graph_launch runs again, with the addresses and sizes of the recording. */
    int (*graph_begin)(kipp_runtime *rt, kipp_error *error);
    int (*graph_end)(kipp_runtime *rt, bool keep, void **out_graph, kipp_error *error);
    int (*graph_launch)(kipp_runtime *rt, void *graph, kipp_error *error);
    void (*graph_free)(kipp_runtime *rt, void *graph);
    bool recording;
    uint64_t generation; /* counts moves of buffers that recordings hold addresses of */
    uint64_t cut_attention_steps; /* work lists of portions whose keys were cut over more workgroups (for tests) */

    /* Optional (NULL: none): what a table has to put right after a step that failed. */
    void (*after_failed_step)(kipp_runtime *rt);

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
/* A delta whose product was not launched yet becomes its slabs. */
int kipp_settle(kipp_runtime *rt, kipp_delta *delta, kipp_error *error);
/* Rows that lack their scale become finished rows (in workspace of the step). */
int kipp_finish_rows(kipp_runtime *rt, kipp_rows *rows, uint32_t m, uint32_t width, kipp_error *error);
/* x . w^T as a delta of the residual stream: left to the norm that follows where the table can add and norm in the product's kernel. */
int kipp_linear_defer(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w, uint32_t m, int max_parts, kipp_delta *out, kipp_error *error);

#endif
