/*
 * Layers put together from parts: mixer, feed-forward, norm, position encoding
 * and their arrangement in a block.  A part kind is a record of functions
 * registered under (category, kind); the model looks kinds up by the names in
 * its spec and never by architecture, and no part knows which model it is in:
 * every size and constant comes from the part's own spec.
 *
 * Built in: norm "rms_norm", position "rope" and "none", mixer "attention",
 * feed_forward "gated_mlp", block "pre_norm", embedding "embedding", head
 * "lm_head".  Another kind is one more record and a call of kipp_register_part.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "backend.h"
#include "internal.h"

/* ------------------------------------------------------------------ the registry */
#define KIPP_MAX_KINDS 64
static const kipp_part_kind *kinds[KIPP_MAX_KINDS];
static size_t kind_count;

int kipp_register_part(const kipp_part_kind *kind) {
    for (size_t i = 0; i < kind_count; ++i) {
        if (strcmp(kinds[i]->category, kind->category) == 0 && strcmp(kinds[i]->kind, kind->kind) == 0) {
            kinds[i] = kind;
            return 0;
        }
    }
    if (kind_count == KIPP_MAX_KINDS) return -1;
    kinds[kind_count++] = kind;
    return 0;
}

const kipp_part_kind *kipp_part_kind_of(const char *category, const char *kind, kipp_error *error) {
    kipp_register_builtin_parts();
    for (size_t i = 0; i < kind_count; ++i) {
        if (strcmp(kinds[i]->category, category) == 0 && strcmp(kinds[i]->kind, kind) == 0) return kinds[i];
    }
    kipp_text known = {0};
    for (size_t i = 0; i < kind_count; ++i) {
        if (strcmp(kinds[i]->category, category) == 0) kipp_text_add(&known, "%s%s", known.length ? ", " : "", kinds[i]->kind);
    }
    kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "no %s part registered for kind '%s'; known: %s", category, kind,
              known.data != NULL ? known.data : "(none)");
    kipp_text_free(&known);
    return NULL;
}

int kipp_params_add(kipp_param_list *list, const char *prefix, const char *local, uint32_t ndim, uint64_t d0, uint64_t d1,
                    kipp_error *error) {
    if (list->count == list->capacity) {
        size_t capacity = list->capacity == 0 ? 64 : list->capacity * 2;
        kipp_param *grown = realloc(list->items, capacity * sizeof(kipp_param));
        if (grown == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for the list of tensors");
        list->items = grown;
        list->capacity = capacity;
    }
    kipp_param *p = &list->items[list->count];
    if (snprintf(p->name, sizeof(p->name), "%s%s", prefix, local) >= (int)sizeof(p->name))
        return kipp_fail(error, KIPP_ERROR_RANGE, "a tensor name is too long: %s%s", prefix, local);
    for (size_t i = 0; i < list->count; ++i) {
        if (strcmp(list->items[i].name, p->name) == 0) return kipp_fail(error, KIPP_ERROR_INTERNAL, "two parts declare the tensor '%s'", p->name);
    }
    p->ndim = ndim;
    p->shape[0] = d0;
    p->shape[1] = d1;
    ++list->count;
    return 0;
}

static const kipp_tensor *tensor_of(const kipp_tensor_file *tensors, const char *prefix, const char *local, kipp_error *error) {
    char name[KIPP_NAME + 32];
    snprintf(name, sizeof(name), "%s%s", prefix, local);
    const kipp_tensor *tensor = kipp_tensors_find(tensors, name);
    if (tensor == NULL) kipp_fail(error, KIPP_ERROR_FORMAT, "missing tensor '%s'", name);
    return tensor;
}

/* ------------------------------------------------------------------ norm: rms_norm */
typedef struct {
    kipp_rms_norm_spec spec;
    kipp_runtime *rt;
    float *weight;
} rms_norm_part;

static int rms_norm_params(const void *spec_, kipp_param_list *out, kipp_error *error) {
    const kipp_rms_norm_spec *spec = spec_;
    return kipp_params_add(out, spec->prefix, "weight", 1, spec->width, 0, error);
}

static void *rms_norm_create(const void *spec, kipp_runtime *rt, kipp_error *error) {
    rms_norm_part *part = calloc(1, sizeof(*part));
    if (part == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    part->spec = *(const kipp_rms_norm_spec *)spec;
    part->rt = rt;
    return part;
}

static int rms_norm_load(void *part_, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    rms_norm_part *part = part_;
    (void)context;
    const kipp_tensor *w = tensor_of(tensors, part->spec.prefix, "weight", error);
    return w == NULL ? -1 : part->rt->place_vector(part->rt, w, &part->weight, error);
}

static void rms_norm_destroy(void *part_) {
    rms_norm_part *part = part_;
    if (part->weight != NULL) part->rt->mem_free(part->rt, part->weight);
    free(part);
}

/* y = x * rsqrt(mean(x^2) + eps) * w  (/root/reference/src/kipp.c:2221-2231) */
static int rms_norm_forward(void *part_, float *x, kipp_delta *delta, kipp_rows *out, uint32_t rows, bool may_leave_scale, kipp_error *error) {
    rms_norm_part *part = part_;
    return part->rt->rmsnorm(part->rt, x, delta, part->weight, out, rows, part->spec.width, part->spec.eps, may_leave_scale, error);
}

static const kipp_norm_fn rms_norm_fn = {rms_norm_forward};
static const kipp_part_kind rms_norm_kind = {"norm",        "rms_norm",    sizeof(kipp_rms_norm_spec), rms_norm_params, rms_norm_create,
                                             rms_norm_load, rms_norm_destroy, &rms_norm_fn};

/* ------------------------------------------------------------------ position: rope, none */
typedef struct {
    kipp_rope_spec spec;
    kipp_runtime *rt;
    float *inv_freq; /* where the path computes */
    uint64_t same_as; /* a hash of the frequencies' bits: layers that turn alike share one step's angles */
} rope_part;

static int no_params(const void *spec, kipp_param_list *out, kipp_error *error) {
    (void)spec;
    (void)out;
    (void)error;
    return 0;
}

/* inv_freq[i] = theta^(-2i / rotary_dim), made in double and rounded once; the angle is float32(pos) * inv_freq[i]
 * (/root/reference/src/kipp.c:2368-2382) */
static void *rope_create(const void *spec_, kipp_runtime *rt, kipp_error *error) {
    const kipp_rope_spec *spec = spec_;
    if (spec->rotary_dim == 0 || spec->rotary_dim % 2 != 0 || spec->rotary_dim > spec->head_dim || !(spec->theta > 0.0)) {
        kipp_fail(error, KIPP_ERROR_ARGUMENT, "rope: rotary_dim %u must be even and in (0, head_dim = %u], theta positive", spec->rotary_dim,
                  spec->head_dim);
        return NULL;
    }
    rope_part *part = calloc(1, sizeof(*part));
    uint32_t half = spec->rotary_dim / 2;
    float *host = malloc(half * sizeof(float));
    if (part == NULL || host == NULL) {
        free(part);
        free(host);
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    part->spec = *spec;
    part->rt = rt;
    for (uint32_t i = 0; i < half; ++i) host[i] = (float)pow(spec->theta, -(2.0 * (double)i) / (double)spec->rotary_dim);
    part->same_as = 1469598103934665603ull ^ spec->rotary_dim;
    for (uint32_t i = 0; i < half; ++i) {
        uint32_t bits;
        memcpy(&bits, &host[i], sizeof(bits));
        part->same_as = (part->same_as ^ bits) * 1099511628211ull;
    }
    if (part->same_as == 0) part->same_as = 1;
    part->inv_freq = rt->mem_alloc(rt, half * sizeof(float), error);
    if (part->inv_freq == NULL || rt->upload(rt, part->inv_freq, host, half * sizeof(float), error) != 0) {
        if (part->inv_freq != NULL) rt->mem_free(rt, part->inv_freq);
        free(part);
        free(host);
        return NULL;
    }
    free(host);
    return part;
}

static int nothing_to_load(void *part, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    (void)part;
    (void)tensors;
    (void)context;
    (void)error;
    return 0;
}

static void rope_destroy(void *part_) {
    rope_part *part = part_;
    part->rt->mem_free(part->rt, part->inv_freq);
    free(part);
}

static int rope_table(void *part_, const float **inv_freq, uint32_t *rotary_dim, int *interleaved, uint64_t *same_as) {
    rope_part *part = part_;
    *inv_freq = part->inv_freq;
    *rotary_dim = part->spec.rotary_dim;
    *interleaved = part->spec.interleaved;
    *same_as = part->same_as;
    return 0;
}

static const kipp_position_fn rope_fn = {rope_table};
static const kipp_part_kind rope_kind = {"position", "rope", sizeof(kipp_rope_spec), no_params, rope_create, nothing_to_load, rope_destroy,
                                         &rope_fn};

static void *none_create(const void *spec, kipp_runtime *rt, kipp_error *error) {
    (void)spec;
    (void)rt;
    void *part = calloc(1, 8);
    if (part == NULL) kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    return part;
}

static int none_table(void *part, const float **inv_freq, uint32_t *rotary_dim, int *interleaved, uint64_t *same_as) {
    (void)part;
    *inv_freq = NULL;
    *rotary_dim = 0;
    *interleaved = 0;
    *same_as = 0;
    return 0;
}

static const kipp_position_fn none_fn = {none_table};
static const kipp_part_kind none_kind = {"position", "none", 0, no_params, none_create, nothing_to_load, free, &none_fn};

/* ------------------------------------------------------------------ mixer: attention */
typedef struct {
    kipp_attention_spec spec;
    kipp_runtime *rt;
    kipp_built_part position;
    kipp_weight w_qkv, w_o;
    float *q_norm, *k_norm;
    float scale;
} attention_part;

static int attention_params(const void *spec_, kipp_param_list *out, kipp_error *error) {
    const kipp_attention_spec *s = spec_;
    uint64_t q_dim = (uint64_t)s->n_heads * s->head_dim, kv_dim = (uint64_t)s->n_kv_heads * s->head_dim;
    if (kipp_params_add(out, s->prefix, "q_proj.weight", 2, q_dim, s->hidden, error) != 0 ||
        kipp_params_add(out, s->prefix, "k_proj.weight", 2, kv_dim, s->hidden, error) != 0 ||
        kipp_params_add(out, s->prefix, "v_proj.weight", 2, kv_dim, s->hidden, error) != 0 ||
        kipp_params_add(out, s->prefix, "o_proj.weight", 2, s->hidden, q_dim, error) != 0)
        return -1;
    if (s->qk_norm && (kipp_params_add(out, s->prefix, "q_norm.weight", 1, s->head_dim, 0, error) != 0 ||
                       kipp_params_add(out, s->prefix, "k_norm.weight", 1, s->head_dim, 0, error) != 0))
        return -1;
    return 0;
}

static void attention_destroy(void *part_) {
    attention_part *part = part_;
    if (part->position.part != NULL) part->position.kind->destroy(part->position.part);
    part->rt->free_weight(part->rt, &part->w_qkv);
    part->rt->free_weight(part->rt, &part->w_o);
    if (part->q_norm != NULL) part->rt->mem_free(part->rt, part->q_norm);
    if (part->k_norm != NULL) part->rt->mem_free(part->rt, part->k_norm);
    free(part);
}

static void *attention_create(const void *spec_, kipp_runtime *rt, kipp_error *error) {
    const kipp_attention_spec *s = spec_;
    if (s->n_heads == 0 || s->n_kv_heads == 0 || s->n_heads % s->n_kv_heads != 0 || s->head_dim == 0 || s->head_dim > 256) {
        kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "attention: %u query heads over %u key/value heads of size %u", s->n_heads, s->n_kv_heads, s->head_dim);
        return NULL;
    }
    attention_part *part = calloc(1, sizeof(*part));
    if (part == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    part->spec = *s;
    part->rt = rt;
    part->scale = s->scale != 0.0f ? s->scale : 1.0f / sqrtf((float)s->head_dim);
    part->position.kind = kipp_part_kind_of("position", s->position_kind, error);
    if (part->position.kind != NULL) part->position.part = part->position.kind->create(&s->rope, rt, error);
    if (part->position.part == NULL) {
        free(part);
        return NULL;
    }
    return part;
}

static int attention_load(void *part_, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    attention_part *part = part_;
    kipp_runtime *rt = part->rt;
    (void)context;
    const kipp_tensor *qkv[3] = {tensor_of(tensors, part->spec.prefix, "q_proj.weight", error),
                                 tensor_of(tensors, part->spec.prefix, "k_proj.weight", error),
                                 tensor_of(tensors, part->spec.prefix, "v_proj.weight", error)};
    const kipp_tensor *o = tensor_of(tensors, part->spec.prefix, "o_proj.weight", error);
    if (qkv[0] == NULL || qkv[1] == NULL || qkv[2] == NULL || o == NULL) return -1;
    /* rows one under the other: one product serves q, k and v, and no output element changes */
    if (rt->place_matrix(rt, qkv, 3, KIPP_LAYOUT_STREAM, &part->w_qkv, error) != 0 || rt->place_matrix(rt, &o, 1, KIPP_LAYOUT_STREAM, &part->w_o, error) != 0)
        return -1;
    if (part->spec.qk_norm) {
        const kipp_tensor *qn = tensor_of(tensors, part->spec.prefix, "q_norm.weight", error);
        const kipp_tensor *kn = tensor_of(tensors, part->spec.prefix, "k_norm.weight", error);
        if (qn == NULL || kn == NULL || rt->place_vector(rt, qn, &part->q_norm, error) != 0 || rt->place_vector(rt, kn, &part->k_norm, error) != 0)
            return -1;
    }
    return 0;
}

static void attention_cache_need(const void *spec_, kipp_kv_need *out) {
    const kipp_attention_spec *s = spec_;
    *out = (kipp_kv_need){true, s->n_kv_heads, s->head_dim, s->window, s->page_tokens};
}

static void no_state(const void *spec, kipp_state_need *out) {
    (void)spec;
    *out = (kipp_state_need){false, 0};
}

/* Causal grouped-query attention with optional per-head q/k norm, a position part and an optional window over the
 * paged cache; query head h reads key/value head h / (n_q / n_kv)  (/root/reference/src/kipp.c:2950-2993). */
static int attention_forward(void *part_, const kipp_rows *x, kipp_batch *batch, const kipp_cache_view *cache, void *state, kipp_delta *out,
                             kipp_error *error) {
    attention_part *part = part_;
    kipp_runtime *rt = part->rt;
    const kipp_attention_spec *s = &part->spec;
    (void)state;
    if (cache == NULL) return kipp_fail(error, KIPP_ERROR_INTERNAL, "attention without a cache view");
    const float *inv_freq;
    uint32_t rotary_dim;
    int interleaved;
    uint64_t same_as;
    ((const kipp_position_fn *)part->position.kind->fn)->table(part->position.part, &inv_freq, &rotary_dim, &interleaved, &same_as);
    const float *rotation = NULL;
    if (inv_freq != NULL) {
        /* made by the first layer of a forward pass that turns with these frequencies, shared by the others */
        if (batch->rotation_of != same_as) {
            if (rt->rotary_angles(rt, batch->positions, inv_freq, batch->n_tokens, rotary_dim / 2, &batch->rotation, error) != 0) return -1;
            batch->rotation_of = same_as;
        }
        rotation = batch->rotation;
    }
    const uint32_t n = batch->n_tokens;
    const size_t q_dim = (size_t)s->n_heads * s->head_dim, act = kipp_dtype_bytes(rt->act_dtype);
    const kipp_attention_geometry geometry = {s->n_heads, s->n_kv_heads, s->head_dim, s->window, part->scale};
    const float eps = s->qk_norm ? s->qk_norm_eps : 0.0f;
    void *mixed = kipp_scratch(rt, n * q_dim * act, error);
    if (mixed == NULL) return -1;
    if (rt->decode_attention != NULL && batch->n_portions == 0) {
        /* single tokens only: a table may have fewer kernels for the way from x to the mixed heads */
        bool done = false;
        kipp_rows heads = {mixed, NULL, 0, 0.0f, false};
        if (rt->decode_attention(rt, x, &part->w_qkv, cache, &part->w_o, &heads, batch, &geometry, part->q_norm, part->k_norm, eps, rotation,
                                 rotary_dim, interleaved, &done, error) != 0)
            return -1;
        if (done) return kipp_linear_defer(rt, &heads, &part->w_o, n, 8, out, error);
    }
    kipp_delta qkv;
    if (rt->linear(rt, x, &part->w_qkv, n, 4, &qkv, error) != 0) return -1;
    void *q = kipp_scratch(rt, n * q_dim * act, error);
    if (q == NULL) return -1;
    if (rt->qk_norm_rope_kv(rt, &qkv, q, cache, batch, &geometry, part->q_norm, part->k_norm, eps, rotation, rotary_dim, interleaved, error) != 0)
        return -1;
    if (rt->attention(rt, q, cache, mixed, batch, &geometry, error) != 0) return -1;
    return kipp_linear_defer(rt, &(kipp_rows){mixed, NULL, 0, 0.0f, false}, &part->w_o, n, 8, out, error);
}

static const kipp_mixer_fn attention_fn = {attention_cache_need, no_state, attention_forward, true};
static const kipp_part_kind attention_kind = {"mixer",        "attention",      sizeof(kipp_attention_spec), attention_params, attention_create,
                                              attention_load, attention_destroy, &attention_fn};

/* ------------------------------------------------------------------ feed_forward: gated_mlp */
typedef struct {
    kipp_gated_mlp_spec spec;
    kipp_runtime *rt;
    kipp_weight w_gate_up, w_down;
} gated_mlp_part;

static int gated_mlp_params(const void *spec_, kipp_param_list *out, kipp_error *error) {
    const kipp_gated_mlp_spec *s = spec_;
    if (kipp_params_add(out, s->prefix, "gate_proj.weight", 2, s->inner, s->hidden, error) != 0 ||
        kipp_params_add(out, s->prefix, "up_proj.weight", 2, s->inner, s->hidden, error) != 0 ||
        kipp_params_add(out, s->prefix, "down_proj.weight", 2, s->hidden, s->inner, error) != 0)
        return -1;
    return 0;
}

static void *gated_mlp_create(const void *spec, kipp_runtime *rt, kipp_error *error) {
    gated_mlp_part *part = calloc(1, sizeof(*part));
    if (part == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    part->spec = *(const kipp_gated_mlp_spec *)spec;
    part->rt = rt;
    return part;
}

static int gated_mlp_load(void *part_, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    gated_mlp_part *part = part_;
    (void)context;
    const kipp_tensor *gate_up[2] = {tensor_of(tensors, part->spec.prefix, "gate_proj.weight", error),
                                     tensor_of(tensors, part->spec.prefix, "up_proj.weight", error)};
    const kipp_tensor *down = tensor_of(tensors, part->spec.prefix, "down_proj.weight", error);
    if (gate_up[0] == NULL || gate_up[1] == NULL || down == NULL) return -1;
    if (part->rt->place_matrix(part->rt, gate_up, 2, KIPP_LAYOUT_STREAM_PAIRS, &part->w_gate_up, error) != 0) return -1;
    return part->rt->place_matrix(part->rt, &down, 1, KIPP_LAYOUT_STREAM, &part->w_down, error);
}

static void gated_mlp_destroy(void *part_) {
    gated_mlp_part *part = part_;
    part->rt->free_weight(part->rt, &part->w_gate_up);
    part->rt->free_weight(part->rt, &part->w_down);
    free(part);
}

/* delta = W_down (silu(W_gate x) * (W_up x))  (/root/reference/src/kipp.c:2633-2653) */
static int gated_mlp_forward(void *part_, const kipp_rows *x, kipp_batch *batch, kipp_delta *out, kipp_error *error) {
    gated_mlp_part *part = part_;
    kipp_runtime *rt = part->rt;
    const uint32_t n = batch->n_tokens;
    kipp_rows act = {kipp_scratch(rt, (size_t)n * part->spec.inner * kipp_dtype_bytes(rt->act_dtype), error), NULL, 0, 0.0f, false};
    if (act.data == NULL) return -1;
    bool done = false;
    /* both products and the activation in one kernel where the table has one */
    if (rt->gated != NULL && rt->gated(rt, x, &part->w_gate_up, &part->w_down, &act, n, &done, error) != 0) return -1;
    if (!done) {
        kipp_delta gate_up;
        if (rt->linear(rt, x, &part->w_gate_up, n, 8, &gate_up, error) != 0 || rt->swiglu(rt, &gate_up, act.data, n, part->spec.inner, error) != 0) return -1;
    }
    return kipp_linear_defer(rt, &act, &part->w_down, n, 8, out, error);
}

static const kipp_ffn_fn gated_mlp_fn = {gated_mlp_forward, true};
static const kipp_part_kind gated_mlp_kind = {"feed_forward", "gated_mlp",      sizeof(kipp_gated_mlp_spec), gated_mlp_params, gated_mlp_create,
                                              gated_mlp_load, gated_mlp_destroy, &gated_mlp_fn};

/* ------------------------------------------------------------------ block: pre_norm */
typedef struct {
    const kipp_layer_spec *spec;
    kipp_runtime *rt;
    kipp_built_part mixer_norm, mixer, ffn_norm, ffn;
    const void *mixer_spec;
    uint32_t hidden;
} pre_norm_block;

static const char *const pre_norm_roles[] = {"mixer_norm", "norm", "mixer", "mixer", "ffn_norm", "norm", "ffn", "feed_forward", NULL};

static const kipp_role_spec *role_of(const kipp_layer_spec *layer, const char *role) {
    for (uint32_t r = 0; r < layer->role_count; ++r) {
        if (strcmp(layer->roles[r].role, role) == 0) return &layer->roles[r];
    }
    return NULL;
}

static int block_params(const void *spec_, kipp_param_list *out, kipp_error *error) {
    const kipp_layer_spec *layer = spec_;
    for (uint32_t r = 0; r < layer->role_count; ++r) {
        const kipp_part_kind *kind = kipp_part_kind_of(layer->roles[r].category, layer->roles[r].kind, error);
        if (kind == NULL || kind->params(layer->roles[r].spec, out, error) != 0) return -1;
    }
    return 0;
}

static void pre_norm_destroy(void *block_) {
    pre_norm_block *block = block_;
    kipp_built_part *parts[4] = {&block->mixer_norm, &block->mixer, &block->ffn_norm, &block->ffn};
    for (int i = 0; i < 4; ++i) {
        if (parts[i]->part != NULL) parts[i]->kind->destroy(parts[i]->part);
    }
    free(block);
}

static void *pre_norm_create(const void *spec_, kipp_runtime *rt, kipp_error *error) {
    const kipp_layer_spec *layer = spec_;
    pre_norm_block *block = calloc(1, sizeof(*block));
    if (block == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    block->spec = layer;
    block->rt = rt;
    block->hidden = layer->hidden;
    kipp_built_part *parts[4] = {&block->mixer_norm, &block->mixer, &block->ffn_norm, &block->ffn};
    for (int i = 0; i < 4; ++i) {
        const kipp_role_spec *role = role_of(layer, pre_norm_roles[2 * i]);
        if (role == NULL || strcmp(role->category, pre_norm_roles[2 * i + 1]) != 0) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "a pre_norm block needs a %s in the role %s", pre_norm_roles[2 * i + 1], pre_norm_roles[2 * i]);
            pre_norm_destroy(block);
            return NULL;
        }
        parts[i]->kind = kipp_part_kind_of(role->category, role->kind, error);
        if (parts[i]->kind != NULL) parts[i]->part = parts[i]->kind->create(role->spec, rt, error);
        if (parts[i]->part == NULL) {
            pre_norm_destroy(block);
            return NULL;
        }
        if (i == 1) block->mixer_spec = role->spec;
    }
    return block;
}

static int pre_norm_load(void *block_, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    pre_norm_block *block = block_;
    kipp_built_part *parts[4] = {&block->mixer_norm, &block->mixer, &block->ffn_norm, &block->ffn};
    for (int i = 0; i < 4; ++i) {
        if (parts[i]->kind->load(parts[i]->part, tensors, context, error) != 0) return -1;
    }
    return 0;
}

/* x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x))  (/root/reference/docs/ARCHITECTURE.md:77-92).  A delta is added inside
 * the norm that follows it, so the block takes the delta of the block before as `pending` and hands its own last on. */
static int pre_norm_forward(void *block_, float *x, kipp_delta *pending, kipp_batch *batch, const kipp_cache_view *cache, void *state,
                            kipp_error *error) {
    pre_norm_block *block = block_;
    kipp_runtime *rt = block->rt;
    const uint32_t n = batch->n_tokens;
    const size_t bytes = (size_t)n * block->hidden * kipp_dtype_bytes(rt->act_dtype);
    const kipp_norm_fn *norm1 = block->mixer_norm.kind->fn, *norm2 = block->ffn_norm.kind->fn;
    const kipp_mixer_fn *mixer = block->mixer.kind->fn;
    const kipp_ffn_fn *ffn = block->ffn.kind->fn;
    /* a part that does not take rows without their scale gets finished ones: the norm is told, and what it leaves all the same is finished here */
    kipp_rows h = {kipp_scratch(rt, bytes, error), NULL, 0, 0.0f, false};
    if (h.data == NULL) return -1;
    if (norm1->forward(block->mixer_norm.part, x, kipp_delta_any(pending) ? pending : NULL, &h, n, mixer->takes_scaled_rows, error) != 0) return -1;
    if (!mixer->takes_scaled_rows && kipp_finish_rows(rt, &h, n, block->hidden, error) != 0) return -1;
    kipp_delta delta;
    if (mixer->forward(block->mixer.part, &h, batch, cache, state, &delta, error) != 0) return -1;
    kipp_rows h2 = {kipp_scratch(rt, bytes, error), NULL, 0, 0.0f, false};
    if (h2.data == NULL) return -1;
    if (norm2->forward(block->ffn_norm.part, x, &delta, &h2, n, ffn->takes_scaled_rows, error) != 0) return -1;
    if (!ffn->takes_scaled_rows && kipp_finish_rows(rt, &h2, n, block->hidden, error) != 0) return -1;
    return ffn->forward(block->ffn.part, &h2, batch, pending, error);
}

static void *pre_norm_mixer_of(void *block_, const kipp_part_kind **kind, const void **spec) {
    pre_norm_block *block = block_;
    *kind = block->mixer.kind;
    *spec = block->mixer_spec;
    return block->mixer.part;
}

static const kipp_block_fn pre_norm_fn = {pre_norm_roles, pre_norm_forward, pre_norm_mixer_of};
static const kipp_part_kind pre_norm_kind = {"block", "pre_norm", sizeof(kipp_layer_spec), block_params, pre_norm_create, pre_norm_load,
                                             pre_norm_destroy, &pre_norm_fn};

/* ------------------------------------------------------------------ embedding and head */
typedef struct {
    kipp_embedding_spec spec;
    kipp_runtime *rt;
    kipp_weight table;
} embedding_part;

static int embedding_params(const void *spec_, kipp_param_list *out, kipp_error *error) {
    const kipp_embedding_spec *s = spec_;
    return kipp_params_add(out, s->prefix, "weight", 2, s->vocab, s->hidden, error);
}

static void *embedding_create(const void *spec, kipp_runtime *rt, kipp_error *error) {
    embedding_part *part = calloc(1, sizeof(*part));
    if (part == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    part->spec = *(const kipp_embedding_spec *)spec;
    part->rt = rt;
    return part;
}

/* `context`: the head's spec (or NULL); a table that a tied head multiplies with is placed as the products want it */
static int embedding_load(void *part_, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    embedding_part *part = part_;
    const kipp_head_spec *head = context;
    const kipp_tensor *table = tensor_of(tensors, part->spec.prefix, "weight", error);
    return table == NULL ? -1
                         : part->rt->place_matrix(part->rt, &table, 1, head != NULL && head->tied ? KIPP_LAYOUT_STREAM : KIPP_LAYOUT_ROWS, &part->table, error);
}

static void embedding_destroy(void *part_) {
    embedding_part *part = part_;
    part->rt->free_weight(part->rt, &part->table);
    free(part);
}

static const kipp_part_kind embedding_kind = {"embedding",    "embedding",       sizeof(kipp_embedding_spec), embedding_params, embedding_create,
                                              embedding_load, embedding_destroy, NULL};

typedef struct {
    kipp_head_spec spec;
    kipp_runtime *rt;
    kipp_weight weight;
    bool owns;
} head_part;

static int head_params(const void *spec_, kipp_param_list *out, kipp_error *error) {
    const kipp_head_spec *s = spec_;
    return s->tied ? 0 : kipp_params_add(out, s->prefix, "weight", 2, s->vocab, s->hidden, error);
}

static void *head_create(const void *spec, kipp_runtime *rt, kipp_error *error) {
    head_part *part = calloc(1, sizeof(*part));
    if (part == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    part->spec = *(const kipp_head_spec *)spec;
    part->rt = rt;
    return part;
}

/* `context`: the embedding part; a tied head has no tensor of its own and uses its table (/root/reference/src/kipp.c:951-956) */
static int head_load(void *part_, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    head_part *part = part_;
    if (part->spec.tied) {
        part->weight = ((embedding_part *)context)->table;
        return 0;
    }
    const kipp_tensor *w = tensor_of(tensors, part->spec.prefix, "weight", error);
    if (w == NULL || part->rt->place_matrix(part->rt, &w, 1, KIPP_LAYOUT_STREAM, &part->weight, error) != 0) return -1;
    part->owns = true;
    return 0;
}

static void head_destroy(void *part_) {
    head_part *part = part_;
    if (part->owns) part->rt->free_weight(part->rt, &part->weight);
    free(part);
}

static const kipp_part_kind head_kind = {"head", "lm_head", sizeof(kipp_head_spec), head_params, head_create, head_load, head_destroy, NULL};

/* x[t] = E[token_t], no scaling (/root/reference/src/kipp.c:2579-2585) */
int kipp_embedding_forward(void *part_, const int32_t *tokens, float *out, uint32_t n, kipp_error *error) {
    embedding_part *part = part_;
    return part->rt->embed(part->rt, &part->table, tokens, out, n, error);
}

/* logits = W x, float32, no bias (/root/reference/src/kipp.c:2660-2661) */
int kipp_head_forward(void *part_, const kipp_rows *x, uint32_t rows, kipp_delta *out, kipp_error *error) {
    head_part *part = part_;
    return part->rt->linear(part->rt, x, &part->weight, rows, 1, out, error);
}

uint64_t kipp_weight_bytes(const kipp_weight *w) { return (uint64_t)w->n * w->k * (w->dtype == KIPP_F32 ? 4 : 2); }

void kipp_register_builtin_parts(void) {
    static bool done;
    if (done) return;
    done = true;
    kipp_register_part(&rms_norm_kind);
    kipp_register_part(&rope_kind);
    kipp_register_part(&none_kind);
    kipp_register_part(&attention_kind);
    kipp_register_part(&gated_mlp_kind);
    kipp_register_part(&pre_norm_kind);
    kipp_register_part(&embedding_kind);
    kipp_register_part(&head_kind);
}
