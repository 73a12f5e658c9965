/* Types the files of the host share.  Nothing here is part of the interface. */
#ifndef KIPP_AMD_INTERNAL_H
#define KIPP_AMD_INTERNAL_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "kipp_amd.h"

#define KIPP_F32 0 /* the codes the kernel launchers take */
#define KIPP_BF16 1
#define KIPP_F16 2 /* in files only: widened when placed */

/* ------------------------------------------------------------------ errors (error.c) */
int kipp_fail(kipp_error *error, kipp_error_code code, const char *format, ...) __attribute__((format(printf, 3, 4)));
void kipp_error_clear(kipp_error *error);
int kipp_add_size(size_t left, size_t right, size_t *result);
int kipp_mul_size(size_t left, size_t right, size_t *result);

/* A growing text, for the one error that lists many tensors. */
typedef struct {
    char *data;
    size_t length, capacity;
    bool failed;
} kipp_text;
void kipp_text_add(kipp_text *text, const char *format, ...) __attribute__((format(printf, 2, 3)));
void kipp_text_free(kipp_text *text);

/* ------------------------------------------------------------------ JSON (json.c) */
typedef enum { KJ_NULL, KJ_BOOL, KJ_NUMBER, KJ_STRING, KJ_ARRAY, KJ_OBJECT } kj_type;

/* A document is one array of nodes; children of an array or object are linked through `next`. */
typedef struct {
    kj_type type;
    bool boolean;
    bool is_integer;    /* a number written without fraction or exponent that fits int64 */
    int64_t integer;
    double number;
    const char *string; /* decoded, nul-terminated (strings and nothing else) */
    size_t string_length;
    const char *key;    /* of a member of an object, else NULL */
    uint32_t first, next, count; /* index of the first child / next sibling (0: none), number of children */
} kj_node;

typedef struct {
    kj_node *nodes;
    size_t count, capacity;
    char *strings; /* every decoded string and key, one after the other */
    size_t strings_length, strings_capacity;
} kj_doc;

int kj_parse(const char *text, size_t length, kj_doc *doc, kipp_error *error);
void kj_free(kj_doc *doc);
const kj_node *kj_root(const kj_doc *doc);
const kj_node *kj_get(const kj_doc *doc, const kj_node *object, const char *key); /* NULL if absent */
const kj_node *kj_first(const kj_doc *doc, const kj_node *parent);
const kj_node *kj_next(const kj_doc *doc, const kj_node *child);
int kipp_read_file(const char *path, char **out_text, size_t *out_length, kipp_error *error);

/* ------------------------------------------------------------------ the decoder as data (config.c) */
#define KIPP_NAME 128

typedef struct {
    uint32_t width;
    float eps;
    char prefix[KIPP_NAME];
} kipp_rms_norm_spec;

typedef struct {
    uint32_t head_dim;
    double theta;
    uint32_t rotary_dim;
    int interleaved; /* 0: dim i turns with dim i + rotary_dim / 2; 1: dim 2i with dim 2i + 1 */
} kipp_rope_spec;

typedef struct {
    uint32_t hidden, n_heads, n_kv_heads, head_dim;
    bool qk_norm;
    float qk_norm_eps;
    uint32_t window;      /* 0: every key */
    float scale;          /* 0: 1 / sqrt(head_dim) */
    uint32_t page_tokens; /* 0: the engine's */
    char position_kind[24]; /* "rope" or "none" */
    kipp_rope_spec rope;
    char prefix[KIPP_NAME];
} kipp_attention_spec;

typedef struct {
    uint32_t hidden, inner;
    char prefix[KIPP_NAME];
} kipp_gated_mlp_spec;

typedef struct {
    uint32_t vocab, hidden;
    char prefix[KIPP_NAME];
} kipp_embedding_spec;

typedef struct {
    uint32_t vocab, hidden;
    bool tied;
    char prefix[KIPP_NAME];
} kipp_head_spec;

/* One part of a layer by the role it plays in the block arrangement. */
typedef struct {
    char role[16];
    char category[16];
    char kind[24];
    void *spec; /* the kind's own struct, owned by the model spec */
} kipp_role_spec;

#define KIPP_MAX_ROLES 6
typedef struct {
    char block[24];
    uint32_t hidden; /* width of the residual stream */
    kipp_role_spec roles[KIPP_MAX_ROLES];
    uint32_t role_count;
} kipp_layer_spec;

/* One entry of the run order: a layer, and optionally an earlier entry whose cache it reads. */
typedef struct {
    uint32_t layer;
    int32_t cache_of; /* -1: its own */
} kipp_layer_run;

typedef struct {
    char architecture[64];
    uint32_t hidden, vocab, max_position;
    kipp_embedding_spec embedding;
    kipp_layer_spec *layers;
    uint32_t layer_count;
    kipp_layer_run *order;
    uint32_t run_count;
    char final_norm_kind[24];
    void *final_norm;
    kipp_head_spec head;
    uint32_t stop_tokens[KIPP_MAX_STOP_TOKENS];
    uint32_t stop_token_count;
    kipp_model_info info; /* what get_info reports of the architecture's own numbers */
} kipp_model_spec;

typedef int (*kipp_parse_config)(const kj_doc *doc, kipp_model_spec *spec, kipp_error *error);
int kipp_register_architecture(const char *name, kipp_parse_config parse);
int kipp_spec_from_folder(const char *model_dir, kipp_model_spec *spec, kipp_error *error);
int kipp_spec_from_json(const char *text, size_t length, kipp_model_spec *spec, kipp_error *error);
void kipp_spec_free(kipp_model_spec *spec);
int kipp_spec_add_role(kipp_layer_spec *layer, const char *role, const char *category, const char *kind, const void *spec,
                       size_t spec_size, kipp_error *error);

/* ------------------------------------------------------------------ safetensors (safetensors.c) */
typedef struct {
    char name[KIPP_NAME];
    int dtype; /* KIPP_F32, KIPP_BF16, KIPP_F16 or -1 (a type this engine does not read; named in `dtype_name`) */
    char dtype_name[12];
    uint32_t ndim;
    uint64_t shape[4];
    const void *data; /* inside the mapping */
    uint64_t bytes;
    bool bound;
} kipp_tensor;

typedef struct {
    void **mappings;
    size_t *mapping_sizes;
    size_t mapping_count;
    kipp_tensor *tensors;
    size_t tensor_count, tensor_capacity;
    uint64_t mapped_bytes;
} kipp_tensor_file;

int kipp_tensors_open(const char *model_dir, kipp_tensor_file *out, kipp_error *error);
void kipp_tensors_close(kipp_tensor_file *file);
kipp_tensor *kipp_tensors_find(const kipp_tensor_file *file, const char *name);

/* ------------------------------------------------------------------ pages (pool.c) */
#define KIPP_NO_PAGE 0xffffffffu

typedef struct {
    uint32_t ref_count;
    uint64_t hash;
    bool indexed;
    uint32_t hash_next;            /* next page of the same bucket */
    uint32_t prev_free, next_free; /* the free list, least recently released first */
    bool on_free_list;
} kipp_page;

typedef struct {
    uint32_t page_count, page_tokens;
    kipp_page *pages;
    uint32_t *tokens; /* page_count x page_tokens: what an indexed page holds */
    uint32_t *buckets;
    uint32_t bucket_count; /* a power of two, at least twice the pages */
    uint32_t free_head, free_tail, free_count;
    uint64_t reused_total, evicted_total;
    bool force_hash; /* tests: every hash collides */
    uint64_t forced_hash;
} kipp_pool;

int kipp_pool_init(kipp_pool *pool, uint32_t page_count, uint32_t page_tokens, const uint32_t *order, kipp_error *error);
void kipp_pool_free(kipp_pool *pool);
uint64_t kipp_pool_chain_hash(uint64_t parent, const uint32_t *tokens, size_t count);
uint32_t kipp_pool_alloc(kipp_pool *pool);  /* KIPP_NO_PAGE when every page is held */
void kipp_pool_retain(kipp_pool *pool, uint32_t page);
int kipp_pool_release(kipp_pool *pool, uint32_t page); /* -1: the page was not held */
/* Publishes a full held page; returns its hash.  A page whose content is already indexed stays private. */
uint64_t kipp_pool_seal(kipp_pool *pool, uint32_t page, uint64_t parent, const uint32_t *tokens);
bool kipp_pool_is_indexed(const kipp_pool *pool, uint32_t page);
/* Retains the pages of the longest known beginning, at most (count - 1) / page_tokens; returns how many. */
uint32_t kipp_pool_prefix_match(kipp_pool *pool, const uint32_t *tokens, size_t count, uint32_t *out_pages, uint32_t capacity,
                                uint64_t *out_chain);
int kipp_pool_check(const kipp_pool *pool, kipp_error *error);

/* ------------------------------------------------------------------ the device side (backend.h has the table) */
struct kipp_backend;
struct kipp_runtime;

/* A matrix [n, k] where the path computes: its rows as stored, and (bfloat16 on the GPU, k a multiple of 32) the same
 * values once more in the layout that the few-rows products stream fastest, [tile of 16 rows][step of 32 columns][lane][8].
 * `pairs`: the matrix is [gate; up] and a tile holds 8 gate rows over the 8 matching up rows. */
typedef struct {
    void *data;
    int dtype;
    uint32_t n, k;
    void *tiles;
    bool pairs;
} kipp_weight;

typedef enum { KIPP_LAYOUT_ROWS = 0, KIPP_LAYOUT_STREAM, KIPP_LAYOUT_STREAM_PAIRS } kipp_weight_layout;

/* Rows in the activation type.  With `sumsq` they still lack the scale of their RMS norm: data = rows * norm weight, and
 * row t's scale is rsqrt(sum(sumsq[t, :sumsq_parts]) / width + eps), sumsq in rows of sumsq_parts rounded up to 4.  A row's
 * scale commutes with a product over the row, so a product may apply it to its own rows; kipp_finish_rows gives any other
 * consumer the finished rows.  Rows that one few-rows product writes for the next may be in steps-major order (below):
 * only those products read it, and whoever makes such rows knows that their reader is one. */
typedef struct {
    void *data;
    const float *sumsq;
    int sumsq_parts;
    float eps;
    bool steps_major; /* data is [width / 32][rows][32], the order the few-rows products read fastest, not [rows][width] */
} kipp_rows;

/* A delta of the residual stream: float32 [parts, rows, width] whose sum over parts is the value; or (parts 0, w given) the
 * product x [m, k] . w^T that has not been launched yet, which the norm that follows may launch together with the residual
 * add and kipp_settle launches as it is. */
typedef struct {
    float *data;
    int parts;
    const void *x;
    const kipp_weight *w;
    uint32_t m;
    int max_parts;
    bool x_steps_major;
} kipp_delta;

static inline bool kipp_delta_any(const kipp_delta *delta) { return delta != NULL && (delta->parts > 0 || delta->w != NULL); }

/* What a mixer keeps per token (in pages) and per session (of fixed size). */
typedef struct {
    bool any;
    uint32_t n_kv_heads, head_dim, window, page_tokens;
} kipp_kv_need;

typedef struct {
    bool any;
    uint64_t bytes;
} kipp_state_need;

/* ------------------------------------------------------------------ the cache manager (cache.c) */
typedef struct {
    uint32_t index;
    kipp_kv_need need;
    uint32_t page_tokens;
    uint32_t *runs;
    uint32_t run_count;
    kipp_pool pool;
    void **k, **v; /* per run of the group: [pages + 1][kv heads][page][head_dim] */
    uint64_t slab_bytes;
} kipp_cache_group;

struct kipp_session {
    kipp_model *model;
    uint32_t slot;
    uint32_t capacity, length;
    uint32_t *tokens; /* capacity */
    int32_t **tables; /* per group: page of every block, -1 once given back */
    uint32_t *table_lengths;
    uint32_t *adopted; /* per group: leading pages taken from the index */
    uint32_t adopted_tokens;
    bool in_step; /* set while a step holds it: a session may appear once in a step */
    /* a session that will never be truncated below them may publish its full pages as soon as they are written, so that
     * sessions running beside it can adopt them (a scheduler's requests do) */
    bool publish_early;
    uint32_t published; /* leading blocks that are adopted or published */
    uint64_t chain;     /* chained hash after them */
};

typedef struct {
    struct kipp_runtime *rt;
    kipp_cache_group *groups;
    uint32_t group_count;
    int32_t *run_group;   /* per run: its group, or -1 */
    int32_t *run_in_group; /* per run: its index among the group's runs */
    kipp_state_need *state_needs;
    void **states; /* per run: [slots + 1] x bytes, or NULL */
    uint32_t run_count;
    uint32_t page_tokens, max_sessions, max_position;
    bool share;
    uint32_t *free_slots;
    uint32_t free_slot_count;
    uint32_t live_sessions;
} kipp_cache;

int kipp_cache_init(kipp_cache *cache, struct kipp_runtime *rt, const kipp_kv_need *kv_needs, const kipp_state_need *state_needs,
                    const kipp_layer_run *order, uint32_t run_count, uint32_t page_tokens, uint32_t pool_pages, uint32_t max_sessions,
                    uint32_t max_position, bool share, const uint32_t *page_order, kipp_error *error);
void kipp_cache_free(kipp_cache *cache);
int kipp_cache_open(kipp_cache *cache, kipp_session *session, uint32_t capacity, kipp_error *error);
int kipp_cache_adopt(kipp_cache *cache, kipp_session *session, const uint32_t *tokens, size_t count, uint32_t *matched,
                     kipp_error *error);
/* Claim the pages that `count` more tokens need, in every group; on failure nothing is claimed. */
int kipp_cache_reserve_one(kipp_cache *cache, kipp_session *session, size_t count, kipp_error *error);
void kipp_cache_trim(kipp_cache *cache, kipp_session *session);
void kipp_cache_commit(kipp_cache *cache, kipp_session *session, const uint32_t *tokens, size_t count);
int kipp_cache_truncate(kipp_cache *cache, kipp_session *session, uint32_t length, kipp_error *error);
/* Publish full pages (where sharing is on), give every page back; the slot stays with the session. */
void kipp_cache_clear(kipp_cache *cache, kipp_session *session);
void kipp_cache_close(kipp_cache *cache, kipp_session *session);
int kipp_cache_check(const kipp_cache *cache, kipp_session *const *sessions, size_t session_count, kipp_error *error);

/* What a mixer sees of the cache in one run. */
typedef struct {
    uint32_t group;
    void *k, *v;
    uint32_t page_tokens;
    uint32_t page_count;
    bool writable;
} kipp_cache_view;

bool kipp_cache_view_of(const kipp_cache *cache, uint32_t run, int32_t cache_of, kipp_cache_view *out);

/* ------------------------------------------------------------------ one step's batch, flattened (step.c) */
typedef struct {
    uint32_t n_tokens, n_seqs, n_want, n_decode, n_portions;
    bool want_every_row; /* the wanted rows are all rows, in order */
    uint32_t max_decode_ctx, max_blocks;
    /* on the host */
    int32_t *h_all;
    int32_t *h_q_start, *h_q_len, *h_ctx_len;
    /* where the path computes: one buffer, the lists one after the other */
    int32_t *d_all;
    int32_t *tokens, *positions, *seq_of_token, *q_start, *q_len, *ctx_len, *slots, *want_rows, *decode_rows;
    int32_t **tables; /* per group: [n_seqs][max_blocks] */
    int32_t *item_seq, *item_tile; /* work list of the kernel for portions: (entry, tile of query rows), longest key range first */
    uint32_t n_items;
    uint64_t items_of; /* the attention geometry the list was made for (0: none yet) */
    /* where the list alone would leave compute units idle its keys are cut as well: an item is then (entry, tile, cut) */
    int32_t *item_cut, *merge_rows, *merge_cuts; /* the cut of every item; the rows to merge afterwards and how many cuts each has */
    uint32_t cut_keys, n_merge, most_cuts;       /* keys of a cut (0: not cut) */
    float *cut_acc, *cut_ml;                     /* the cuts' sums, and their maxima and denominators */
    size_t capacity; /* ints the two buffers hold */
    /* values of this forward pass that parts share */
    const float *rotation;    /* what the table's rotary_angles made */
    uint64_t rotation_of;     /* the `same_as` of the frequencies it was made from (0: none yet) */
    void *decode_workspace[3];
    size_t decode_workspace_key;
} kipp_batch;

/* ------------------------------------------------------------------ parts (parts.c) */
typedef struct {
    char name[KIPP_NAME + 32];
    uint32_t ndim;
    uint64_t shape[2];
} kipp_param;

typedef struct {
    kipp_param *items;
    size_t count, capacity;
} kipp_param_list;

int kipp_params_add(kipp_param_list *list, const char *prefix, const char *local, uint32_t ndim, uint64_t d0, uint64_t d1,
                    kipp_error *error);

/* What every part kind brings, whatever its category. */
typedef struct kipp_part_kind {
    const char *category, *kind;
    size_t spec_size;
    int (*params)(const void *spec, kipp_param_list *out, kipp_error *error);
    void *(*create)(const void *spec, struct kipp_runtime *rt, kipp_error *error);
    int (*load)(void *part, const kipp_tensor_file *tensors, void *context, kipp_error *error);
    void (*destroy)(void *part);
    const void *fn; /* the functions of its category, below */
} kipp_part_kind;

typedef struct {
    /* out->data (given by the caller) = norm(x [+ delta]) in the activation type; with a delta, x += delta in place first.
     * `may_leave_scale`: the consumer takes rows that lack their scale (out->sumsq then says so). */
    int (*forward)(void *part, float *x, kipp_delta *delta, kipp_rows *out, uint32_t rows, bool may_leave_scale, kipp_error *error);
} kipp_norm_fn;

typedef struct {
    /* frequencies where the path computes (NULL: no rotation), the dims they turn, the pairing, and a number that two parts
     * share exactly if they turn alike (0: no rotation) */
    int (*table)(void *part, const float **inv_freq, uint32_t *rotary_dim, int *interleaved, uint64_t *same_as);
} kipp_position_fn;

typedef struct {
    void (*cache_need)(const void *spec, kipp_kv_need *out);
    void (*state_need)(const void *spec, kipp_state_need *out);
    /* x: [tokens, hidden] in the activation type; out: the delta, in workspace of the step (or a product not yet launched) */
    int (*forward)(void *part, const kipp_rows *x, kipp_batch *batch, const kipp_cache_view *cache, void *state, kipp_delta *out,
                   kipp_error *error);
    bool takes_scaled_rows; /* false: the block finishes rows that lack their scale before it calls */
} kipp_mixer_fn;

typedef struct {
    int (*forward)(void *part, const kipp_rows *x, kipp_batch *batch, kipp_delta *out, kipp_error *error);
    bool takes_scaled_rows;
} kipp_ffn_fn;

typedef struct {
    /* roles the arrangement needs, NULL-terminated pairs (role, category) */
    const char *const *roles;
    /* x: the residual stream, updated in place; pending: a delta not yet added (parts 0: none), replaced by the block's last */
    int (*forward)(void *block, float *x, kipp_delta *pending, kipp_batch *batch, const kipp_cache_view *cache, void *state,
                   kipp_error *error);
    void *(*mixer_of)(void *block, const kipp_part_kind **kind, const void **spec);
} kipp_block_fn;

int kipp_register_part(const kipp_part_kind *kind);
const kipp_part_kind *kipp_part_kind_of(const char *category, const char *kind, kipp_error *error);
void kipp_register_builtin_parts(void);
void kipp_register_builtin_architectures(void);

/* A block instance is built by its kind from the layer spec. */
typedef struct {
    const kipp_part_kind *kind;
    void *part;
} kipp_built_part;

/* ------------------------------------------------------------------ the model (model.c) */
struct kipp_model {
    kipp_model_spec spec;
    kipp_model_open_config config;
    struct kipp_runtime *rt;
    kipp_tensor_file tensors;
    kipp_built_part embedding, final_norm, head;
    kipp_built_part *blocks;
    kipp_cache cache;
    kipp_batch batch;
    kipp_session **sessions;
    size_t session_count, session_capacity;
    uint64_t weight_bytes;
    int fail_forward_after; /* tests: < 0 never; else the forward pass after that many fails */
    /* steps of single tokens, recorded once a shape has come twice and run again as a graph (step.c) */
    struct kipp_step_graph *graphs;
    size_t graph_count, graph_capacity;
    uint64_t graph_replays, graph_clock;
};

/* One recorded shape: rows, the width of the block tables, the longest context (both rounded up), logits or their largest. */
typedef struct kipp_step_graph {
    uint64_t key;
    uint32_t seen;
    bool refused;          /* recording it failed once: it runs as it is */
    void *graph;
    const void *batch_base; /* what the recording read its integers from: valid while the batch's buffer has not moved */
    uint64_t generation;    /* ... and while the table of operations has not moved its own buffers */
    float *logits;
    int32_t *chosen;
    uint64_t used; /* the model's graph_clock when it last ran */
} kipp_step_graph;

int kipp_model_params(const kipp_model_spec *spec, kipp_param_list *out, kipp_error *error);
int kipp_model_forward(kipp_model *model, kipp_batch *batch, float **out_logits, kipp_error *error);
int kipp_embedding_forward(void *part, const int32_t *tokens, float *out, uint32_t n, kipp_error *error);
int kipp_head_forward(void *part, const kipp_rows *x, uint32_t rows, kipp_delta *out, kipp_error *error);
uint64_t kipp_weight_bytes(const kipp_weight *w);
int kipp_check_tensors(const char *where, kipp_tensor_file *found, const kipp_param_list *expected, kipp_error *error);

#endif
