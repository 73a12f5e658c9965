/*
 * config.json -> the decoder as data, through a registry of architectures.
 *
 * The reference takes its numbers from metadata that its converter wrote from
 * the same config.json keys and checks them against a compiled-in table
 * (/root/reference/src/kipp.c:756-809, /root/reference/tools/convert_to_gguf.py:471-488).  Here
 * every size is a field of a spec; a key whose value would change the
 * computation and that is not implemented is refused, never ignored.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "internal.h"

/* ------------------------------------------------------------------ the registry */
#define KIPP_MAX_ARCHITECTURES 16
static struct {
    char name[64];
    kipp_parse_config parse;
} architectures[KIPP_MAX_ARCHITECTURES];
static size_t architecture_count;

int kipp_register_architecture(const char *name, kipp_parse_config parse) {
    for (size_t i = 0; i < architecture_count; ++i) {
        if (strcmp(architectures[i].name, name) == 0) {
            architectures[i].parse = parse;
            return 0;
        }
    }
    if (architecture_count == KIPP_MAX_ARCHITECTURES || strlen(name) >= sizeof(architectures[0].name)) return -1;
    snprintf(architectures[architecture_count].name, sizeof(architectures[0].name), "%s", name);
    architectures[architecture_count++].parse = parse;
    return 0;
}

int kipp_spec_add_role(kipp_layer_spec *layer, const char *role, const char *category, const char *kind, const void *spec,
                       size_t spec_size, kipp_error *error) {
    if (layer->role_count == KIPP_MAX_ROLES) return kipp_fail(error, KIPP_ERROR_INTERNAL, "a layer has more than %d parts", KIPP_MAX_ROLES);
    kipp_role_spec *slot = &layer->roles[layer->role_count];
    slot->spec = malloc(spec_size);
    if (slot->spec == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a part's spec");
    memcpy(slot->spec, spec, spec_size);
    snprintf(slot->role, sizeof(slot->role), "%s", role);
    snprintf(slot->category, sizeof(slot->category), "%s", category);
    snprintf(slot->kind, sizeof(slot->kind), "%s", kind);
    ++layer->role_count;
    return 0;
}

void kipp_spec_free(kipp_model_spec *spec) {
    for (uint32_t l = 0; l < spec->layer_count; ++l) {
        for (uint32_t r = 0; r < spec->layers[l].role_count; ++r) free(spec->layers[l].roles[r].spec);
    }
    free(spec->layers);
    free(spec->order);
    free(spec->final_norm);
    memset(spec, 0, sizeof(*spec));
}

int kipp_spec_from_json(const char *text, size_t length, kipp_model_spec *spec, kipp_error *error) {
    kj_doc doc;
    int rc = -1;
    kipp_register_builtin_architectures();
    memset(spec, 0, sizeof(*spec));
    if (kj_parse(text, length, &doc, error) != 0) return -1;
    const kj_node *root = kj_root(&doc);
    if (root == NULL || root->type != KJ_OBJECT) {
        kipp_fail(error, KIPP_ERROR_FORMAT, "config.json must hold a JSON object");
        goto done;
    }
    const kj_node *archs = kj_get(&doc, root, "architectures");
    const kj_node *first = kj_first(&doc, archs);
    if (archs == NULL || archs->type != KJ_ARRAY || archs->count != 1 || first->type != KJ_STRING) {
        kipp_fail(error, KIPP_ERROR_FORMAT, "config.json architectures: expected a list with one name");
        goto done;
    }
    for (size_t i = 0; i < architecture_count; ++i) {
        if (strcmp(architectures[i].name, first->string) == 0) {
            snprintf(spec->architecture, sizeof(spec->architecture), "%s", first->string);
            rc = architectures[i].parse(&doc, spec, error);
            if (rc != 0) kipp_spec_free(spec);
            goto done;
        }
    }
    {
        kipp_text known = {0};
        for (size_t i = 0; i < architecture_count; ++i) kipp_text_add(&known, "%s%s", i ? ", " : "", architectures[i].name);
        kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "architecture '%s' is not in the registry; known: %s", first->string,
                  known.data != NULL ? known.data : "(none)");
        kipp_text_free(&known);
    }
done:
    kj_free(&doc);
    return rc;
}

int kipp_spec_from_folder(const char *model_dir, kipp_model_spec *spec, kipp_error *error) {
    char path[4096];
    char *text;
    size_t length;
    if (snprintf(path, sizeof(path), "%s/config.json", model_dir) >= (int)sizeof(path))
        return kipp_fail(error, KIPP_ERROR_ARGUMENT, "the model folder's path is too long");
    if (kipp_read_file(path, &text, &length, error) != 0) return -1;
    int rc = kipp_spec_from_json(text, length, spec, error);
    free(text);
    return rc;
}

/* ------------------------------------------------------------------ Qwen3ForCausalLM */
static int need_uint(const kj_doc *doc, const kj_node *root, const char *key, uint32_t minimum, uint32_t *out, kipp_error *error) {
    const kj_node *v = kj_get(doc, root, key);
    if (v == NULL) return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json lacks the required key %s", key);
    if (v->type != KJ_NUMBER || !v->is_integer) return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json %s: expected an integer", key);
    if (v->integer < (int64_t)minimum || v->integer > (int64_t)1 << 30)
        return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json %s: must be >= %u and below 2^30, got %lld", key, minimum, (long long)v->integer);
    *out = (uint32_t)v->integer;
    return 0;
}

static int need_number(const kj_doc *doc, const kj_node *root, const char *key, double *out, kipp_error *error) {
    const kj_node *v = kj_get(doc, root, key);
    if (v == NULL) return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json lacks the required key %s", key);
    if (v->type != KJ_NUMBER) return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json %s: expected a number", key);
    *out = v->number;
    return 0;
}

static int parse_qwen3(const kj_doc *doc, kipp_model_spec *spec, kipp_error *error) {
    const kj_node *root = kj_root(doc);
    static const char *const required[] = {"vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                                           "num_key_value_heads", "rms_norm_eps", "rope_theta", "max_position_embeddings"};
    kipp_text missing = {0};
    for (size_t i = 0; i < sizeof(required) / sizeof(required[0]); ++i) {
        if (kj_get(doc, root, required[i]) == NULL) kipp_text_add(&missing, "%s%s", missing.length ? ", " : "", required[i]);
    }
    if (missing.length != 0) {
        kipp_fail(error, KIPP_ERROR_FORMAT, "config.json lacks required keys: %s", missing.data);
        kipp_text_free(&missing);
        return -1;
    }
    const kj_node *v;
    if ((v = kj_get(doc, root, "model_type")) != NULL && (v->type != KJ_STRING || strcmp(v->string, "qwen3") != 0))
        return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "config.json model_type: expected 'qwen3'");
    if ((v = kj_get(doc, root, "hidden_act")) != NULL && (v->type != KJ_STRING || strcmp(v->string, "silu") != 0))
        return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "config.json hidden_act: only 'silu' is implemented");
    if ((v = kj_get(doc, root, "attention_bias")) != NULL && !(v->type == KJ_BOOL && !v->boolean))
        return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "config.json attention_bias: projections with bias are not implemented");
    if ((v = kj_get(doc, root, "rope_scaling")) != NULL && v->type != KJ_NULL)
        return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "config.json rope_scaling: scaled rotary frequencies are not implemented");
    if ((v = kj_get(doc, root, "use_sliding_window")) != NULL && !(v->type == KJ_BOOL && !v->boolean))
        return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "config.json use_sliding_window: this architecture is run with full attention only");

    uint32_t vocab, hidden, inner, layers, heads, kv_heads, head_dim, positions;
    double eps, theta;
    if (need_uint(doc, root, "vocab_size", 1, &vocab, error) != 0 || need_uint(doc, root, "hidden_size", 1, &hidden, error) != 0 ||
        need_uint(doc, root, "intermediate_size", 1, &inner, error) != 0 || need_uint(doc, root, "num_hidden_layers", 1, &layers, error) != 0 ||
        need_uint(doc, root, "num_attention_heads", 1, &heads, error) != 0 ||
        need_uint(doc, root, "num_key_value_heads", 1, &kv_heads, error) != 0 ||
        need_uint(doc, root, "max_position_embeddings", 1, &positions, error) != 0 || need_number(doc, root, "rms_norm_eps", &eps, error) != 0 ||
        need_number(doc, root, "rope_theta", &theta, error) != 0)
        return -1;
    v = kj_get(doc, root, "head_dim");
    if (v != NULL && v->type != KJ_NULL) {
        if (need_uint(doc, root, "head_dim", 1, &head_dim, error) != 0) return -1;
    } else {
        if (hidden % heads != 0)
            return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json head_dim absent and hidden_size is not a multiple of num_attention_heads");
        head_dim = hidden / heads;
    }
    if (!(eps >= 0.0)) return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json rms_norm_eps: must be >= 0");
    if (!(theta > 0.0)) return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json rope_theta: must be positive");
    if (heads % kv_heads != 0)
        return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json num_attention_heads %u is not a multiple of num_key_value_heads %u", heads, kv_heads);
    if (head_dim > 256 || head_dim % 2 != 0)
        return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "config.json head_dim %u: the kernels take even head sizes up to 256", head_dim);
    bool tied = false;
    if ((v = kj_get(doc, root, "tie_word_embeddings")) != NULL) {
        if (v->type != KJ_BOOL) return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json tie_word_embeddings: expected true or false");
        tied = v->boolean;
    }
    if ((v = kj_get(doc, root, "eos_token_id")) != NULL && v->type != KJ_NULL) {
        const kj_node *item = v->type == KJ_ARRAY ? kj_first(doc, v) : v;
        for (; item != NULL; item = v->type == KJ_ARRAY ? kj_next(doc, item) : NULL) {
            if (item->type != KJ_NUMBER || !item->is_integer || item->integer < 0 || item->integer >= (int64_t)vocab)
                return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json eos_token_id: not a token of the vocabulary");
            if (spec->stop_token_count == KIPP_MAX_STOP_TOKENS)
                return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "config.json eos_token_id: more than %u stop tokens", KIPP_MAX_STOP_TOKENS);
            spec->stop_tokens[spec->stop_token_count++] = (uint32_t)item->integer;
        }
    }

    spec->hidden = hidden;
    spec->vocab = vocab;
    spec->max_position = positions;
    spec->embedding = (kipp_embedding_spec){vocab, hidden, "model.embed_tokens."};
    spec->head = (kipp_head_spec){vocab, hidden, tied, "lm_head."};
    spec->layers = calloc(layers, sizeof(kipp_layer_spec));
    spec->order = calloc(layers, sizeof(kipp_layer_run));
    kipp_rms_norm_spec *final_norm = calloc(1, sizeof(kipp_rms_norm_spec));
    if (spec->layers == NULL || spec->order == NULL || final_norm == NULL) {
        free(final_norm);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for %u layers", layers);
    }
    spec->layer_count = spec->run_count = layers;
    final_norm->width = hidden;
    final_norm->eps = (float)eps;
    snprintf(final_norm->prefix, sizeof(final_norm->prefix), "model.norm.");
    spec->final_norm = final_norm;
    snprintf(spec->final_norm_kind, sizeof(spec->final_norm_kind), "rms_norm");
    /* per layer: input norm, attention with per-head q/k norm and rotary encoding, post-attention norm, SwiGLU
     * (/root/reference/src/kipp.c:2588-2655) */
    for (uint32_t l = 0; l < layers; ++l) {
        kipp_layer_spec *layer = &spec->layers[l];
        kipp_rms_norm_spec norm = {hidden, (float)eps, ""};
        kipp_attention_spec attn;
        kipp_gated_mlp_spec mlp = {hidden, inner, ""};
        snprintf(layer->block, sizeof(layer->block), "pre_norm");
        layer->hidden = hidden;
        memset(&attn, 0, sizeof(attn));
        attn.hidden = hidden;
        attn.n_heads = heads;
        attn.n_kv_heads = kv_heads;
        attn.head_dim = head_dim;
        attn.qk_norm = true;
        attn.qk_norm_eps = (float)eps;
        snprintf(attn.position_kind, sizeof(attn.position_kind), "rope");
        attn.rope = (kipp_rope_spec){head_dim, theta, head_dim, 0};
        snprintf(attn.prefix, sizeof(attn.prefix), "model.layers.%u.self_attn.", l);
        snprintf(norm.prefix, sizeof(norm.prefix), "model.layers.%u.input_layernorm.", l);
        if (kipp_spec_add_role(layer, "mixer_norm", "norm", "rms_norm", &norm, sizeof(norm), error) != 0) return -1;
        if (kipp_spec_add_role(layer, "mixer", "mixer", "attention", &attn, sizeof(attn), error) != 0) return -1;
        snprintf(norm.prefix, sizeof(norm.prefix), "model.layers.%u.post_attention_layernorm.", l);
        if (kipp_spec_add_role(layer, "ffn_norm", "norm", "rms_norm", &norm, sizeof(norm), error) != 0) return -1;
        snprintf(mlp.prefix, sizeof(mlp.prefix), "model.layers.%u.mlp.", l);
        if (kipp_spec_add_role(layer, "ffn", "feed_forward", "gated_mlp", &mlp, sizeof(mlp), error) != 0) return -1;
        spec->order[l] = (kipp_layer_run){l, -1};
    }
    kipp_model_info *info = &spec->info;
    info->block_count = layers;
    info->embedding_length = hidden;
    info->feed_forward_length = inner;
    info->attention_head_count = heads;
    info->attention_head_count_kv = kv_heads;
    info->attention_head_dim = head_dim;
    info->vocab_size = vocab;
    info->context_length = positions;
    info->rope_theta = (float)theta;
    info->rms_norm_eps = (float)eps;
    info->tied_embeddings = tied;
    return 0;
}

void kipp_register_builtin_architectures(void) {
    static bool done;
    if (done) return;
    done = true;
    kipp_register_architecture("Qwen3ForCausalLM", parse_qwen3);
}
