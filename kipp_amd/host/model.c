/*
 * A model: the spec read from config.json, the tensors bound by name, the parts
 * built from the spec through the registries, the cache manager, and the forward
 * pass over one flattened batch (/root/reference/src/kipp.c:1293-1384 opens the
 * reference's model; :2588-2661 is its forward pass).
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "backend.h"
#include "internal.h"

/* ------------------------------------------------------------------ what the model needs of the file */
int kipp_model_params(const kipp_model_spec *spec, kipp_param_list *out, kipp_error *error) {
    const kipp_part_kind *kind = kipp_part_kind_of("embedding", "embedding", error);
    if (kind == NULL || kind->params(&spec->embedding, out, error) != 0) return -1;
    for (uint32_t l = 0; l < spec->layer_count; ++l) {
        kind = kipp_part_kind_of("block", spec->layers[l].block, error);
        if (kind == NULL || kind->params(&spec->layers[l], out, error) != 0) return -1;
    }
    kind = kipp_part_kind_of("norm", spec->final_norm_kind, error);
    if (kind == NULL || kind->params(spec->final_norm, out, error) != 0) return -1;
    kind = kipp_part_kind_of("head", "lm_head", error);
    if (kind == NULL || kind->params(&spec->head, out, error) != 0) return -1;
    return 0;
}

/* Names of a category of the one error, as many as fit its share of the message. */
static void list_names(kipp_text *text, const char *title, char **names, size_t count, size_t budget) {
    if (count == 0) return;
    kipp_text_add(text, "\n  %s (%zu): ", title, count);
    size_t start = text->length, shown = 0;
    for (; shown < count; ++shown) {
        if (text->length - start + strlen(names[shown]) + 24 > budget && shown > 0) break;
        kipp_text_add(text, "%s%s", shown ? ", " : "", names[shown]);
    }
    if (shown < count) kipp_text_add(text, ", ... and %zu more", count - shown);
}

static int compare_names(const void *a, const void *b) { return strcmp(*(char *const *)a, *(char *const *)b); }

/*
 * ONE error that lists every missing tensor, every unexpected tensor and every wrong shape or type (the reference
 * stops at the first: /root/reference/src/kipp.c:859-906, 997-1002).
 */
int kipp_check_tensors(const char *where, kipp_tensor_file *found, const kipp_param_list *expected, kipp_error *error) {
    size_t capacity = expected->count + found->tensor_count + 1;
    char **missing = calloc(capacity, sizeof(char *)), **unexpected = calloc(capacity, sizeof(char *)), **wrong = calloc(capacity, sizeof(char *));
    size_t n_missing = 0, n_unexpected = 0, n_wrong = 0;
    int rc = 0;
    if (missing == NULL || unexpected == NULL || wrong == NULL) {
        rc = kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        goto done;
    }
    for (size_t t = 0; t < found->tensor_count; ++t) found->tensors[t].bound = false;
    for (size_t e = 0; e < expected->count; ++e) {
        const kipp_param *p = &expected->items[e];
        kipp_tensor *t = kipp_tensors_find(found, p->name);
        if (t == NULL) {
            missing[n_missing++] = strdup(p->name);
            continue;
        }
        t->bound = true;
        bool shape_ok = t->ndim == p->ndim && t->shape[0] == p->shape[0] && (p->ndim < 2 || t->shape[1] == p->shape[1]);
        char line[384];
        if (!shape_ok) {
            char got[96] = "(", want[64];
            for (uint32_t d = 0; d < t->ndim; ++d) snprintf(got + strlen(got), sizeof(got) - strlen(got), "%s%llu", d ? ", " : "", (unsigned long long)t->shape[d]);
            if (p->ndim == 2) snprintf(want, sizeof(want), "(%llu, %llu)", (unsigned long long)p->shape[0], (unsigned long long)p->shape[1]);
            else snprintf(want, sizeof(want), "(%llu)", (unsigned long long)p->shape[0]);
            snprintf(line, sizeof(line), "%s: shape %s), expected %s", p->name, got, want);
            wrong[n_wrong++] = strdup(line);
        } else if (t->dtype < 0) {
            snprintf(line, sizeof(line), "%s: type %s, expected BF16, F16 or F32", p->name, t->dtype_name);
            wrong[n_wrong++] = strdup(line);
        }
    }
    for (size_t t = 0; t < found->tensor_count; ++t) {
        if (!found->tensors[t].bound) unexpected[n_unexpected++] = strdup(found->tensors[t].name);
    }
    if (n_missing + n_unexpected + n_wrong != 0) {
        kipp_text text = {0};
        qsort(missing, n_missing, sizeof(char *), compare_names);
        qsort(unexpected, n_unexpected, sizeof(char *), compare_names);
        kipp_text_add(&text, "weights in %s do not match the configuration:", where);
        size_t share = (sizeof(error->message) - 300) / ((n_missing != 0) + (n_unexpected != 0) + (n_wrong != 0));
        list_names(&text, "missing tensors", missing, n_missing, share);
        list_names(&text, "unexpected tensors", unexpected, n_unexpected, share);
        list_names(&text, "wrong shape or type", wrong, n_wrong, share);
        rc = kipp_fail(error, KIPP_ERROR_FORMAT, "%s", text.data != NULL ? text.data : "weights do not match the configuration");
        kipp_text_free(&text);
    }
done:
    for (size_t i = 0; i < n_missing; ++i) free(missing[i]);
    for (size_t i = 0; i < n_unexpected; ++i) free(unexpected[i]);
    for (size_t i = 0; i < n_wrong; ++i) free(wrong[i]);
    free(missing);
    free(unexpected);
    free(wrong);
    return rc;
}

/* ------------------------------------------------------------------ open and close */
static void model_free(kipp_model *model) {
    if (model == NULL) return;
    free(model->batch.h_all);
    if (model->rt != NULL) {
        for (size_t i = 0; i < model->graph_count; ++i) {
            if (model->graphs[i].graph != NULL) model->rt->graph_free(model->rt, model->graphs[i].graph);
        }
        free(model->graphs);
        if (model->batch.d_all != NULL && !model->rt->on_host) model->rt->mem_free(model->rt, model->batch.d_all);
        if (model->batch.d_all != NULL && model->rt->on_host) free(model->batch.d_all);
        free(model->batch.tables);
        if (model->cache.rt != NULL) kipp_cache_free(&model->cache);
        if (model->head.part != NULL) model->head.kind->destroy(model->head.part);
        if (model->final_norm.part != NULL) model->final_norm.kind->destroy(model->final_norm.part);
        if (model->blocks != NULL) {
            for (uint32_t l = 0; l < model->spec.layer_count; ++l) {
                if (model->blocks[l].part != NULL) model->blocks[l].kind->destroy(model->blocks[l].part);
            }
        }
        if (model->embedding.part != NULL) model->embedding.kind->destroy(model->embedding.part);
        kipp_runtime_destroy(model->rt);
    }
    free(model->blocks);
    free(model->sessions);
    kipp_tensors_close(&model->tensors);
    kipp_spec_free(&model->spec);
    free(model);
}

int kipp_model_open(const char *model_dir, kipp_model **out_model, kipp_error *error) {
    kipp_model_open_config config;
    memset(&config, 0, sizeof(config));
    config.share_prefixes = 1;
    return kipp_model_open_ex(model_dir, &config, out_model, error);
}

int kipp_model_open_backend(const char *model_dir, kipp_path path, kipp_model **out_model, kipp_error *error) {
    kipp_model_open_config config;
    memset(&config, 0, sizeof(config));
    config.share_prefixes = 1;
    config.path = path;
    return kipp_model_open_ex(model_dir, &config, out_model, error);
}

int kipp_model_open_pooled(const char *model_dir, kipp_path path, uint32_t kv_pool_pages, kipp_model **out_model, kipp_error *error) {
    kipp_error_clear(error);
    if (kv_pool_pages == 0) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "a pool of no pages");
    kipp_model_open_config config;
    memset(&config, 0, sizeof(config));
    config.share_prefixes = 1;
    config.path = path;
    config.kv_pool_pages = kv_pool_pages;
    return kipp_model_open_ex(model_dir, &config, out_model, error);
}

int kipp_model_open_ex(const char *model_dir, const kipp_model_open_config *config, kipp_model **out_model, kipp_error *error) {
    kipp_error_clear(error);
    if (model_dir == NULL || config == NULL || out_model == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "model folder, configuration and result must be given");
    *out_model = NULL;
    kipp_model *model = calloc(1, sizeof(*model));
    if (model == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    model->config = *config;
    model->fail_forward_after = -1;
    if (model->config.page_tokens == 0) model->config.page_tokens = 16;
    if (model->config.max_sessions == 0) model->config.max_sessions = 64;
    if (model->config.max_step_tokens == 0) model->config.max_step_tokens = 2048;
    kipp_param_list params = {0};
    kipp_kv_need *kv_needs = NULL;
    kipp_state_need *state_needs = NULL;
    if (kipp_spec_from_folder(model_dir, &model->spec, error) != 0) goto fail;
    if (kipp_tensors_open(model_dir, &model->tensors, error) != 0) goto fail;
    if (kipp_model_params(&model->spec, &params, error) != 0) goto fail;
    if (kipp_check_tensors(model_dir, &model->tensors, &params, error) != 0) goto fail;
    switch (config->path) {
        case KIPP_PATH_CPU_FP32: model->rt = kipp_runtime_cpu(error); break;
        case KIPP_PATH_GPU_BF16:
        case KIPP_PATH_GPU_FP32: model->rt = kipp_runtime_hip(config->path, config->device, config->kernel_dir, error); break;
        default: kipp_fail(error, KIPP_ERROR_ARGUMENT, "unknown path %d", (int)config->path);
    }
    if (model->rt == NULL) goto fail;
    kipp_runtime *rt = model->rt;

    /* the parts, by the kinds the spec names */
    const kipp_model_spec *spec = &model->spec;
    model->blocks = calloc(spec->layer_count ? spec->layer_count : 1, sizeof(kipp_built_part));
    if (model->blocks == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        goto fail;
    }
    model->embedding.kind = kipp_part_kind_of("embedding", "embedding", error);
    if (model->embedding.kind == NULL || (model->embedding.part = model->embedding.kind->create(&spec->embedding, rt, error)) == NULL) goto fail;
    if (model->embedding.kind->load(model->embedding.part, &model->tensors, (void *)&spec->head, error) != 0) goto fail;
    for (uint32_t l = 0; l < spec->layer_count; ++l) {
        model->blocks[l].kind = kipp_part_kind_of("block", spec->layers[l].block, error);
        if (model->blocks[l].kind == NULL || (model->blocks[l].part = model->blocks[l].kind->create(&spec->layers[l], rt, error)) == NULL) goto fail;
        if (model->blocks[l].kind->load(model->blocks[l].part, &model->tensors, NULL, error) != 0) goto fail;
    }
    model->final_norm.kind = kipp_part_kind_of("norm", spec->final_norm_kind, error);
    if (model->final_norm.kind == NULL || (model->final_norm.part = model->final_norm.kind->create(spec->final_norm, rt, error)) == NULL) goto fail;
    if (model->final_norm.kind->load(model->final_norm.part, &model->tensors, NULL, error) != 0) goto fail;
    model->head.kind = kipp_part_kind_of("head", "lm_head", error);
    if (model->head.kind == NULL || (model->head.part = model->head.kind->create(&spec->head, rt, error)) == NULL) goto fail;
    if (model->head.kind->load(model->head.part, &model->tensors, model->embedding.part, error) != 0) goto fail;
    for (size_t p = 0; p < params.count; ++p) {
        uint64_t n = params.items[p].shape[0] * (params.items[p].ndim == 2 ? params.items[p].shape[1] : 1);
        const kipp_tensor *t = kipp_tensors_find(&model->tensors, params.items[p].name);
        bool narrow = rt->act_dtype == KIPP_BF16 && params.items[p].ndim == 2 && t != NULL && t->dtype == KIPP_BF16;
        model->weight_bytes += n * (narrow ? 2 : 4);
    }

    /* what every run of the order keeps, asked of its mixer */
    kv_needs = calloc(spec->run_count ? spec->run_count : 1, sizeof(kipp_kv_need));
    state_needs = calloc(spec->run_count ? spec->run_count : 1, sizeof(kipp_state_need));
    if (kv_needs == NULL || state_needs == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        goto fail;
    }
    for (uint32_t run = 0; run < spec->run_count; ++run) {
        const kipp_layer_run *entry = &spec->order[run];
        if (entry->layer >= spec->layer_count || entry->cache_of >= (int32_t)run ||
            (entry->cache_of >= 0 && spec->order[entry->cache_of].cache_of >= 0)) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "order[%u] names a layer that does not exist, or a cache that is not an earlier run's own", run);
            goto fail;
        }
        const kipp_block_fn *block_fn = model->blocks[entry->layer].kind->fn;
        const kipp_part_kind *mixer_kind;
        const void *mixer_spec;
        block_fn->mixer_of(model->blocks[entry->layer].part, &mixer_kind, &mixer_spec);
        const kipp_mixer_fn *mixer_fn = mixer_kind->fn;
        mixer_fn->cache_need(mixer_spec, &kv_needs[run]);
        mixer_fn->state_need(mixer_spec, &state_needs[run]);
    }
    uint32_t pool_pages = config->kv_pool_pages != 0 ? config->kv_pool_pages
                                                     : (spec->max_position + model->config.page_tokens - 1) / model->config.page_tokens;
    model->config.kv_pool_pages = pool_pages;
    if (kipp_cache_init(&model->cache, rt, kv_needs, state_needs, spec->order, spec->run_count, model->config.page_tokens, pool_pages,
                        model->config.max_sessions, spec->max_position, config->share_prefixes != 0, config->page_order, error) != 0)
        goto fail;
    model->batch.tables = calloc(model->cache.group_count ? model->cache.group_count : 1, sizeof(int32_t *));
    if (model->batch.tables == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        goto fail;
    }
    free(params.items);
    free(kv_needs);
    free(state_needs);
    *out_model = model;
    return 0;
fail:
    free(params.items);
    free(kv_needs);
    free(state_needs);
    model_free(model);
    return -1;
}

int kipp_model_close(kipp_model *model, kipp_error *error) {
    if (model == NULL) return 0;
    if (model->session_count != 0) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "%zu sessions of the model are still alive", model->session_count);
    model_free(model);
    return 0;
}

int kipp_model_get_info(const kipp_model *model, kipp_model_info *out_info) {
    if (model == NULL || out_info == NULL) return -1;
    *out_info = model->spec.info;
    out_info->architecture = model->spec.architecture;
    out_info->path = model->rt->path;
    out_info->stop_token_count = model->spec.stop_token_count;
    memcpy(out_info->stop_tokens, model->spec.stop_tokens, sizeof(out_info->stop_tokens));
    out_info->page_tokens = model->cache.page_tokens;
    out_info->cache_groups = model->cache.group_count;
    out_info->mapped_bytes = model->tensors.mapped_bytes;
    out_info->weight_bytes = model->weight_bytes;
    out_info->cache_bytes = 0;
    for (uint32_t g = 0; g < model->cache.group_count; ++g) out_info->cache_bytes += 2 * model->cache.groups[g].slab_bytes * model->cache.groups[g].run_count;
    return 0;
}

void kipp_test_fail_forward_after(kipp_model *model, int skip) { model->fail_forward_after = skip; }

int kipp_model_is_stop_token(const kipp_model *model, uint32_t token) {
    for (uint32_t i = 0; i < model->spec.stop_token_count; ++i) {
        if (model->spec.stop_tokens[i] == token) return 1;
    }
    return 0;
}

int kipp_model_kv_pool_stats(const kipp_model *model, uint32_t group, kipp_kv_pool_stats_public *out_stats) {
    if (model == NULL || out_stats == NULL || group >= model->cache.group_count) return -1;
    const kipp_pool *pool = &model->cache.groups[group].pool;
    *out_stats = (kipp_kv_pool_stats_public){pool->page_count, pool->free_count, pool->reused_total, pool->evicted_total};
    return 0;
}

/* ------------------------------------------------------------------ the forward pass */
int kipp_model_forward(kipp_model *model, kipp_batch *batch, float **out_logits, kipp_error *error) {
    kipp_runtime *rt = model->rt;
    const kipp_model_spec *spec = &model->spec;
    const uint32_t n = batch->n_tokens;
    *out_logits = NULL;
    batch->rotation = NULL;
    batch->rotation_of = 0;
    batch->item_seq = batch->item_tile = NULL;
    batch->items_of = 0;
    batch->n_items = 0;
    batch->decode_workspace[0] = NULL;
    float *x = kipp_scratch(rt, (size_t)n * spec->hidden * sizeof(float), error);
    if (x == NULL || kipp_embedding_forward(model->embedding.part, batch->tokens, x, n, error) != 0) return -1;
    kipp_delta pending = {NULL, 0, NULL, NULL, 0, 0, false};
    for (uint32_t run = 0; run < spec->run_count; ++run) {
        const kipp_built_part *block = &model->blocks[spec->order[run].layer];
        kipp_cache_view view;
        bool has_view = kipp_cache_view_of(&model->cache, run, spec->order[run].cache_of, &view);
        if (((const kipp_block_fn *)block->kind->fn)->forward(block->part, x, &pending, batch, has_view ? &view : NULL, model->cache.states[run], error) != 0)
            return -1;
    }
    if (batch->n_want == 0) return 0; /* a portion of a prompt whose logits nobody needs: no final norm, no head */
    const kipp_norm_fn *final_norm = model->final_norm.kind->fn;
    kipp_rows normed = {kipp_scratch(rt, (size_t)batch->n_want * spec->hidden * kipp_dtype_bytes(rt->act_dtype), error), NULL, 0, 0.0f, false};
    if (normed.data == NULL) return -1;
    if (batch->want_every_row) {
        /* every row in order (a step of single tokens): no gather, the last delta is added inside the norm, and the head's
         * product may apply the norm's scale */
        if (final_norm->forward(model->final_norm.part, x, kipp_delta_any(&pending) ? &pending : NULL, &normed, n, true, error) != 0) return -1;
    } else {
        if (kipp_delta_any(&pending) && rt->residual_add(rt, x, &pending, n, spec->hidden, error) != 0) return -1;
        float *rows = kipp_scratch(rt, (size_t)batch->n_want * spec->hidden * sizeof(float), error);
        if (rows == NULL) return -1;
        if (rt->gather_rows(rt, x, batch->want_rows, rows, batch->n_want, spec->hidden, error) != 0) return -1;
        if (final_norm->forward(model->final_norm.part, rows, NULL, &normed, batch->n_want, true, error) != 0) return -1;
    }
    kipp_delta logits;
    if (kipp_head_forward(model->head.part, &normed, batch->n_want, &logits, error) != 0) return -1;
    if (logits.parts != 1) return kipp_fail(error, KIPP_ERROR_INTERNAL, "the head's product came in %d parts", logits.parts);
    *out_logits = logits.data;
    return 0;
}
