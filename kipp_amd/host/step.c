/*
 * Sessions and THE step function.
 *
 * kipp_step runs one batch: for every item a session's next tokens, portions of
 * prompts beside single decoded tokens, cut anywhere.  It validates, claims the
 * pages of every item or of none, flattens the batch (one upload of all integers),
 * runs the model over exactly these tokens from the cache that earlier steps
 * left, reads back the logits at the wanted places, and only then records the
 * tokens in the sessions (/root/reference/src/kipp.c:3984-4082 is the reference's batched
 * call: one row an item there, any places here).  Every other way to evaluate
 * (a session alone, a batch with the last row each, rows one by one) is a call
 * of it.
 */
#include <stdlib.h>
#include <string.h>

#include "backend.h"
#include "internal.h"

/* ------------------------------------------------------------------ sessions */
int kipp_session_create(kipp_model *model, uint32_t capacity, kipp_session **out_session, kipp_error *error) {
    kipp_error_clear(error);
    if (model == NULL || out_session == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "model and result must be given");
    *out_session = NULL;
    if (capacity > model->spec.max_position)
        return kipp_fail(error, KIPP_ERROR_RANGE, "a capacity of %u tokens exceeds the model's %u positions", capacity, model->spec.max_position);
    if (model->session_count == model->session_capacity) {
        size_t grown = model->session_capacity == 0 ? 16 : model->session_capacity * 2;
        kipp_session **list = realloc(model->sessions, grown * sizeof(kipp_session *));
        if (list == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        model->sessions = list;
        model->session_capacity = grown;
    }
    kipp_session *session = calloc(1, sizeof(*session));
    if (session == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    session->model = model;
    if (kipp_cache_open(&model->cache, session, capacity, error) != 0) {
        kipp_cache_close(&model->cache, session);
        free(session);
        return -1;
    }
    model->sessions[model->session_count++] = session;
    *out_session = session;
    return 0;
}

void kipp_session_destroy(kipp_session *session) {
    if (session == NULL) return;
    kipp_model *model = session->model;
    kipp_cache_close(&model->cache, session); /* publishes its full pages where sharing is on, then frees */
    for (size_t i = 0; i < model->session_count; ++i) {
        if (model->sessions[i] == session) {
            model->sessions[i] = model->sessions[--model->session_count];
            break;
        }
    }
    free(session);
}

int kipp_session_reset(kipp_session *session, kipp_error *error) {
    kipp_error_clear(error);
    if (session == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no session");
    kipp_cache *cache = &session->model->cache;
    kipp_cache_clear(cache, session);
    for (uint32_t run = 0; run < cache->run_count; ++run) {
        if (cache->states[run] != NULL) {
            size_t bytes = (size_t)cache->state_needs[run].bytes;
            if (cache->rt->mem_zero(cache->rt, (char *)cache->states[run] + (size_t)session->slot * bytes, bytes, error) != 0) return -1;
        }
    }
    return 0;
}

int kipp_session_truncate(kipp_session *session, uint32_t length, kipp_error *error) {
    kipp_error_clear(error);
    if (session == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no session");
    return kipp_cache_truncate(&session->model->cache, session, length, error);
}

int kipp_session_get_info(const kipp_session *session, kipp_session_info *out_info) {
    if (session == NULL || out_info == NULL) return -1;
    const kipp_cache *cache = &session->model->cache;
    out_info->capacity = session->capacity;
    out_info->length = session->length;
    out_info->adopted_tokens = session->adopted_tokens;
    out_info->cache_bytes = 0;
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        const kipp_cache_group *group = &cache->groups[g];
        uint64_t page_bytes = 2ull * group->run_count * group->need.n_kv_heads * group->page_tokens * group->need.head_dim *
                              kipp_dtype_bytes(cache->rt->act_dtype);
        for (uint32_t block = 0; block < session->table_lengths[g]; ++block) {
            if (session->tables[g][block] >= 0) out_info->cache_bytes += page_bytes;
        }
    }
    return 0;
}

int kipp_session_match_prefix(kipp_session *session, const uint32_t *tokens, size_t token_count, uint32_t *matched_tokens,
                              kipp_error *error) {
    kipp_error_clear(error);
    uint32_t matched = 0;
    if (session == NULL || (tokens == NULL && token_count != 0)) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "session and tokens must be given");
    int rc = kipp_cache_adopt(&session->model->cache, session, tokens, token_count, &matched, error);
    if (matched_tokens != NULL) *matched_tokens = matched;
    return rc;
}

/* ------------------------------------------------------------------ the batch */
#define KIPP_GRAPH_CONTEXT 1024u /* contexts of recorded steps are rounded up to multiples of this */
#define KIPP_GRAPH_ROWS 64u      /* most single tokens of a recorded step */
#define KIPP_GRAPH_SHAPES 64u    /* recordings kept */

static int batch_room(kipp_model *model, size_t ints, kipp_error *error) {
    kipp_batch *batch = &model->batch;
    kipp_runtime *rt = model->rt;
    if (ints <= batch->capacity) return 0;
    size_t capacity = batch->capacity == 0 ? 4096 : batch->capacity;
    while (capacity < ints) capacity *= 2;
    int32_t *host = realloc(batch->h_all, capacity * sizeof(int32_t));
    if (host == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a batch of %zu integers", ints);
    batch->h_all = host;
    if (rt->on_host) {
        int32_t *mirror = realloc(batch->d_all, capacity * sizeof(int32_t));
        if (mirror == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a batch of %zu integers", ints);
        batch->d_all = mirror;
    } else {
        if (batch->d_all != NULL) rt->mem_free(rt, batch->d_all);
        batch->d_all = rt->mem_alloc(rt, capacity * sizeof(int32_t), error);
        if (batch->d_all == NULL) {
            batch->capacity = 0;
            return -1;
        }
    }
    batch->capacity = capacity;
    return 0;
}

/* Flattens the items: the tokens of every item one after the other, with what each operation needs to find a token's
 * sequence, position and pages; all integers go to where the path computes in one copy. */
static int build_batch(kipp_model *model, const kipp_step_item *items, size_t item_count, bool rounded, kipp_error *error) {
    kipp_batch *batch = &model->batch;
    const kipp_cache *cache = &model->cache;
    size_t n_tokens = 0, n_want = 0, n_decode = 0;
    uint32_t max_blocks = 1, max_decode_ctx = 0;
    for (size_t i = 0; i < item_count; ++i) {
        n_tokens += items[i].token_count;
        n_want += items[i].want_count;
        if (items[i].token_count == 1) {
            ++n_decode;
            if (items[i].session->length + 1 > max_decode_ctx) max_decode_ctx = items[i].session->length + 1;
        }
        for (uint32_t g = 0; g < cache->group_count; ++g) {
            if (items[i].session->table_lengths[g] > max_blocks) max_blocks = items[i].session->table_lengths[g];
        }
    }
    if (rounded) {
        /* a step that may be recorded: the width of the tables and the longest context are rounded up, so that the launches'
         * shapes, and with them the recording, serve every step of the same class (a row's own position still bounds what
         * it reads) */
        uint32_t width = 16;
        while (width < max_blocks) width *= 2;
        max_blocks = width;
        max_decode_ctx = (max_decode_ctx + KIPP_GRAPH_CONTEXT - 1) / KIPP_GRAPH_CONTEXT * KIPP_GRAPH_CONTEXT;
    }
    size_t n = item_count, tables = (size_t)cache->group_count * n * max_blocks;
    size_t ints = 3 * n_tokens + 4 * n + n_want + n_decode + tables;
    if (n_tokens > INT32_MAX / 4 || ints > INT32_MAX) return kipp_fail(error, KIPP_ERROR_RANGE, "a step of %zu tokens is too large", n_tokens);
    if (batch_room(model, ints, error) != 0) return -1;
    int32_t *h = batch->h_all, *d = batch->d_all;
    size_t at = 0;
#define KIPP_SECTION(host_name, dev_name, count) \
    int32_t *host_name = h + at;                 \
    batch->dev_name = d + at;                    \
    at += (count)
    KIPP_SECTION(h_tokens, tokens, n_tokens);
    KIPP_SECTION(h_positions, positions, n_tokens);
    KIPP_SECTION(h_seq_of, seq_of_token, n_tokens);
    KIPP_SECTION(h_q_start, q_start, n);
    KIPP_SECTION(h_q_len, q_len, n);
    KIPP_SECTION(h_ctx_len, ctx_len, n);
    KIPP_SECTION(h_slots, slots, n);
    KIPP_SECTION(h_want, want_rows, n_want);
    KIPP_SECTION(h_decode, decode_rows, n_decode);
#undef KIPP_SECTION
    for (uint32_t g = 0; g < cache->group_count; ++g) batch->tables[g] = d + at + (size_t)g * n * max_blocks;
    int32_t *h_tables = h + at;
    size_t row = 0, want_at = 0, decode_at = 0;
    for (size_t i = 0; i < item_count; ++i) {
        const kipp_session *session = items[i].session;
        h_q_start[i] = (int32_t)row;
        h_q_len[i] = (int32_t)items[i].token_count;
        h_ctx_len[i] = (int32_t)(session->length + items[i].token_count);
        h_slots[i] = (int32_t)session->slot;
        if (items[i].token_count == 1) h_decode[decode_at++] = (int32_t)row;
        for (size_t w = 0; w < items[i].want_count; ++w) h_want[want_at++] = (int32_t)(row + items[i].want[w]);
        for (size_t t = 0; t < items[i].token_count; ++t, ++row) {
            h_tokens[row] = (int32_t)items[i].tokens[t];
            h_positions[row] = (int32_t)(session->length + t);
            h_seq_of[row] = (int32_t)i;
        }
        for (uint32_t g = 0; g < cache->group_count; ++g) {
            int32_t *table = h_tables + ((size_t)g * n + i) * max_blocks;
            for (uint32_t b = 0; b < max_blocks; ++b) {
                int32_t page = b < session->table_lengths[g] ? session->tables[g][b] : 0;
                table[b] = page >= 0 ? page : 0; /* a page the window has passed is never read */
            }
        }
    }
    batch->h_q_start = h_q_start;
    batch->h_q_len = h_q_len;
    batch->h_ctx_len = h_ctx_len;
    batch->n_tokens = (uint32_t)n_tokens;
    batch->n_seqs = (uint32_t)n;
    batch->n_want = (uint32_t)n_want;
    batch->want_every_row = n_want == n_tokens;
    for (size_t w = 0; w < n_want && batch->want_every_row; ++w) batch->want_every_row = h_want[w] == (int32_t)w;
    batch->n_decode = (uint32_t)n_decode;
    batch->n_portions = (uint32_t)(n - n_decode);
    batch->max_decode_ctx = max_decode_ctx;
    batch->max_blocks = max_blocks;
    return model->rt->upload(model->rt, d, h, ints * sizeof(int32_t), error);
}

/* ------------------------------------------------------------------ the step */
/* The forward pass of the batch, and with `choose` the index of the largest logit of every wanted row beside it (the lowest
 * among equals): what comes back is then one number a row. */
static int forward_and_choose(kipp_model *model, bool choose, float **logits, int32_t **chosen, kipp_error *error) {
    kipp_scratch_reset(model->rt);
    *chosen = NULL;
    if (kipp_model_forward(model, &model->batch, logits, error) != 0) return -1;
    if (!choose || model->batch.n_want == 0) return 0;
    *chosen = kipp_scratch(model->rt, (size_t)model->batch.n_want * sizeof(int32_t), error);
    if (*chosen == NULL) return -1;
    return model->rt->argmax(model->rt, *logits, *chosen, model->batch.n_want, model->spec.vocab, error);
}

/* Recordings kept: KIPP_GRAPH_SHAPES, or what KIPP_AMD_GRAPH_SHAPES says (tests make it small). */
static size_t graph_shapes(void) {
    const char *text = getenv("KIPP_AMD_GRAPH_SHAPES");
    long n = text != NULL ? strtol(text, NULL, 10) : 0;
    return n >= 1 && n <= 4096 ? (size_t)n : KIPP_GRAPH_SHAPES;
}

/* Runs the batch.  `single` (tokens one a session, all wanted, their shape rounded by build_batch): a shape that has come
 * before is recorded, and from then on run again from the recording.  Every buffer a recording names keeps its place:
 * weights, pages and state slots for the model's life, the step's workspace because a step takes it in the same order from
 * the same start, the batch's integers and the table's own buffers until they grow (then the recording is made again). */
static int run_step(kipp_model *model, bool single, bool choose, float **logits, int32_t **chosen, kipp_error *error) {
    kipp_runtime *rt = model->rt;
    const kipp_batch *batch = &model->batch;
    if (!single) return forward_and_choose(model, choose, logits, chosen, error);
    const uint64_t key = ((uint64_t)batch->n_tokens << 48) | ((uint64_t)batch->max_blocks << 24) | ((uint64_t)(batch->max_decode_ctx / KIPP_GRAPH_CONTEXT) << 1) |
                         (choose ? 1u : 0u);
    kipp_step_graph *entry = NULL;
    for (size_t i = 0; i < model->graph_count && entry == NULL; ++i) {
        if (model->graphs[i].key == key) entry = &model->graphs[i];
    }
    if (entry == NULL && model->graph_count >= graph_shapes()) {
        /* more shapes than are kept: the one used longest ago makes room */
        entry = &model->graphs[0];
        for (size_t i = 1; i < model->graph_count; ++i) {
            if (model->graphs[i].used < entry->used) entry = &model->graphs[i];
        }
        if (entry->graph != NULL) rt->graph_free(rt, entry->graph);
        *entry = (kipp_step_graph){key, 0, false, NULL, NULL, 0, NULL, NULL, 0};
    }
    if (entry == NULL) {
        if (model->graph_count == model->graph_capacity) {
            size_t capacity = model->graph_capacity == 0 ? 8 : model->graph_capacity * 2;
            kipp_step_graph *grown = realloc(model->graphs, capacity * sizeof(kipp_step_graph));
            if (grown == NULL) return forward_and_choose(model, choose, logits, chosen, error);
            model->graphs = grown;
            model->graph_capacity = capacity;
        }
        entry = &model->graphs[model->graph_count++];
        *entry = (kipp_step_graph){key, 0, false, NULL, NULL, 0, NULL, NULL, 0};
    }
    entry->used = ++model->graph_clock;
    if (entry->graph != NULL && (entry->batch_base != batch->d_all || entry->generation != rt->generation)) {
        rt->graph_free(rt, entry->graph); /* a buffer it names has moved */
        entry->graph = NULL;
    }
    if (entry->graph == NULL && entry->seen >= 1 && !entry->refused) {
        /* the shape has run once as it is (whatever it needed to make is made): record it now */
        kipp_error why;
        void *graph = NULL;
        if (rt->graph_begin(rt, &why) == 0) {
            int rc = forward_and_choose(model, choose, logits, chosen, &why);
            if (rt->graph_end(rt, rc == 0, &graph, &why) != 0) graph = NULL;
        }
        if (graph == NULL) {
            entry->refused = true; /* run as it is, now and from now on */
            if (rt->after_failed_step != NULL) rt->after_failed_step(rt);
        } else {
            entry->graph = graph;
            entry->batch_base = batch->d_all;
            entry->generation = rt->generation;
            entry->logits = *logits;
            entry->chosen = *chosen;
        }
    }
    if (entry->graph != NULL) {
        *logits = entry->logits;
        *chosen = entry->chosen;
        ++model->graph_replays;
        return rt->graph_launch(rt, entry->graph, error);
    }
    ++entry->seen;
    return forward_and_choose(model, choose, logits, chosen, error);
}

uint64_t kipp_test_graph_replays(const kipp_model *model) { return model != NULL ? model->graph_replays : 0; }

/* For tests: work lists of prompt portions whose keys were cut over more workgroups since the model was opened. */
uint64_t kipp_test_cut_attention_steps(const kipp_model *model) { return model != NULL ? model->rt->cut_attention_steps : 0; }

typedef struct {
    const uint32_t *targets; /* one a wanted place */
    double *nll;
    size_t capacity;
} nll_request;
static int step_common(kipp_model *model, const kipp_step_item *items, size_t item_count, float *logits, size_t logits_capacity, uint32_t *best,
                       size_t best_capacity, const kipp_sample_params *choices, const double *uniform, const nll_request *scored, kipp_error *error);

int kipp_step(kipp_model *model, const kipp_step_item *items, size_t item_count, float *logits, size_t logits_capacity,
              kipp_error *error) {
    return step_common(model, items, item_count, logits, logits_capacity, NULL, 0, NULL, NULL, NULL, error);
}

int kipp_step_sample_logits(kipp_model *model, const kipp_step_item *items, size_t item_count, const kipp_sample_params *params,
                            const double *uniform, uint32_t *tokens, size_t token_capacity, float *logits, size_t logits_capacity,
                            kipp_error *error) {
    uint32_t none;
    kipp_error_clear(error);
    if (model != NULL && model->rt->sample == NULL) return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "this path has no sampler of its own");
    if (params == NULL || uniform == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "parameters and draws must be given");
    if (tokens == NULL && token_capacity != 0) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no room for the tokens");
    return step_common(model, items, item_count, logits, logits != NULL ? logits_capacity : 0, tokens != NULL ? tokens : &none,
                       tokens != NULL ? token_capacity : 0, params, uniform, NULL, error);
}

int kipp_step_sample(kipp_model *model, const kipp_step_item *items, size_t item_count, const kipp_sample_params *params,
                     const double *uniform, uint32_t *tokens, size_t token_capacity, kipp_error *error) {
    return kipp_step_sample_logits(model, items, item_count, params, uniform, tokens, token_capacity, NULL, 0, error);
}

int kipp_step_nll(kipp_model *model, const kipp_step_item *items, size_t item_count, const uint32_t *targets, double *nll, size_t nll_capacity,
                  kipp_error *error) {
    kipp_error_clear(error);
    if (targets == NULL || nll == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "targets and room for the results must be given");
    const nll_request scored = {targets, nll, nll_capacity};
    return step_common(model, items, item_count, NULL, 0, NULL, 0, NULL, NULL, &scored, error);
}

int kipp_step_argmax(kipp_model *model, const kipp_step_item *items, size_t item_count, uint32_t *tokens, size_t token_capacity,
                     kipp_error *error) {
    uint32_t none; /* a step that wants nothing may come without room */
    if (tokens == NULL && token_capacity != 0) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no room for the tokens");
    return step_common(model, items, item_count, NULL, 0, tokens != NULL ? tokens : &none, tokens != NULL ? token_capacity : 0, NULL, NULL, NULL, error);
}

/* `best` NULL: the wanted rows of logits go to `logits` (room for `logits_capacity` floats); else one token for every wanted
 * row goes to `best` (room for `best_capacity` of them), found where the path computes: the index of the largest logit, or
 * with `choices` what kipp_sample_ex would choose with each row's parameters and draw, and then `logits`, if given, gets the
 * rows as the model left them (before a bias or a penalty changed them) as well.  With `scored` neither: every wanted row's
 * -log softmax at its target goes there. */
static int step_common(kipp_model *model, const kipp_step_item *items, size_t item_count, float *logits, size_t logits_capacity, uint32_t *best,
                       size_t best_capacity, const kipp_sample_params *choices, const double *uniform, const nll_request *scored, kipp_error *error) {
    kipp_error_clear(error);
    if (model == NULL || (items == NULL && item_count != 0)) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "model and items must be given");
    if (item_count == 0) return 0;
    if (item_count > KIPP_EVAL_BATCH_LIMIT) return kipp_fail(error, KIPP_ERROR_RANGE, "%zu items are more than a step takes (%u)", item_count, KIPP_EVAL_BATCH_LIMIT);
    const uint32_t vocab = model->spec.vocab;
    size_t wanted = 0, claimed = 0, total = 0;
    int rc = -1;
    for (size_t i = 0; i < item_count; ++i) {
        const kipp_step_item *item = &items[i];
        if (item->session == NULL || item->session->model != model) {
            kipp_fail(error, KIPP_ERROR_ARGUMENT, "item %zu: its session is not one of this model", i);
            goto unmark;
        }
        if (item->session->in_step) {
            kipp_fail(error, KIPP_ERROR_ARGUMENT, "item %zu: a session appears twice in one step", i);
            goto unmark;
        }
        item->session->in_step = true;
        if (item->token_count == 0 || item->tokens == NULL) {
            kipp_fail(error, KIPP_ERROR_ARGUMENT, "item %zu: an entry needs at least one token", i);
            goto unmark;
        }
        for (size_t t = 0; t < item->token_count; ++t) {
            if (item->tokens[t] >= vocab) {
                kipp_fail(error, KIPP_ERROR_RANGE, "item %zu: token %u is outside the vocabulary of %u", i, item->tokens[t], vocab);
                goto unmark;
            }
        }
        for (size_t w = 0; w < item->want_count; ++w) {
            if (item->want == NULL || item->want[w] >= item->token_count) {
                kipp_fail(error, KIPP_ERROR_RANGE, "item %zu: a wanted place is not among its %zu tokens", i, item->token_count);
                goto unmark;
            }
        }
        wanted += item->want_count;
        total += item->token_count;
    }
    if (total > model->config.max_step_tokens) {
        kipp_fail(error, KIPP_ERROR_RANGE, "a step of %zu tokens exceeds max_step_tokens = %u", total, model->config.max_step_tokens);
        goto unmark;
    }
    size_t floats = 0;
    if (best != NULL && (wanted > best_capacity || wanted > INT32_MAX)) {
        kipp_fail(error, KIPP_ERROR_ARGUMENT, "%zu wanted places do not fit the %zu indices given", wanted, best_capacity);
        goto unmark;
    }
    if (scored != NULL) {
        if (wanted > scored->capacity || wanted > INT32_MAX) {
            kipp_fail(error, KIPP_ERROR_ARGUMENT, "%zu wanted places do not fit the %zu results given", wanted, scored->capacity);
            goto unmark;
        }
        for (size_t w = 0; w < wanted; ++w) {
            if (scored->targets[w] >= vocab) {
                kipp_fail(error, KIPP_ERROR_RANGE, "wanted place %zu: target %u is outside the vocabulary of %u", w, scored->targets[w], vocab);
                goto unmark;
            }
        }
    } else if (best != NULL && logits == NULL) {
        floats = 0;
    } else if (kipp_mul_size(wanted, vocab, &floats) != 0 || floats > logits_capacity || (wanted != 0 && logits == NULL)) {
        kipp_fail(error, KIPP_ERROR_ARGUMENT, "%zu wanted rows of %u logits do not fit the %zu floats given", wanted, vocab, logits_capacity);
        goto unmark;
    }
    /* pages for every item, or for none */
    for (; claimed < item_count; ++claimed) {
        if (kipp_cache_reserve_one(&model->cache, items[claimed].session, items[claimed].token_count, error) != 0) goto unclaim;
    }
    if (model->fail_forward_after >= 0 && model->fail_forward_after-- == 0) {
        kipp_fail(error, KIPP_ERROR_INTERNAL, "the forward pass was told to fail (a test's switch)");
        goto unclaim;
    }
    /* single tokens that all want their logits: the shape comes again and again, so it is recorded once and run as a graph */
    bool single = model->rt->graph_begin != NULL && item_count <= KIPP_GRAPH_ROWS && wanted == item_count;
    for (size_t i = 0; i < item_count && single; ++i) single = items[i].token_count == 1;
    if (build_batch(model, items, item_count, single, error) != 0) goto unclaim; /* rounded whether or not steps are recorded: the same launches either way */
    float *device_logits = NULL;
    int32_t *chosen = NULL;
    if (run_step(model, single && !model->config.eager_steps, best != NULL && choices == NULL, &device_logits, &chosen, error) != 0) goto unclaim;
    if (best != NULL && logits != NULL && model->rt->download(model->rt, logits, device_logits, floats * sizeof(float), error) != 0) goto unclaim;
    if (choices != NULL && wanted != 0) {
        for (size_t w = 0; w < wanted; ++w) { /* what kipp_sample_ex refuses */
            const kipp_sample_params *p = &choices[w];
            if (p->temperature > 0.0f && !(p->top_p > 0.0f && p->top_p <= 1.0f && p->min_p >= 0.0f && p->min_p <= 1.0f && uniform[w] >= 0.0 && uniform[w] < 1.0)) {
                kipp_fail(error, KIPP_ERROR_ARGUMENT, "wanted place %zu: top_p in (0, 1], min_p in [0, 1] and a draw in [0, 1)", w);
                goto unclaim;
            }
        }
        if (model->rt->sample(model->rt, device_logits, choices, uniform, &chosen, (uint32_t)wanted, vocab, error) != 0) goto unclaim;
    }
    /* reading back (even nothing) waits for the step's work: what it wrote into the pages is there when it returns */
    if (scored != NULL && wanted != 0) {
        if (model->rt->row_nll(model->rt, device_logits, scored->targets, scored->nll, (uint32_t)wanted, vocab, error) != 0) goto unclaim;
    } else if (best != NULL && wanted != 0) {
        if (model->rt->download(model->rt, best, chosen, wanted * sizeof(int32_t), error) != 0) goto unclaim;
    } else if (model->rt->download(model->rt, logits, device_logits, floats * sizeof(float), error) != 0) {
        goto unclaim;
    }
    for (size_t i = 0; i < item_count; ++i) kipp_cache_commit(&model->cache, items[i].session, items[i].tokens, items[i].token_count);
    rc = 0;
    goto unmark;
unclaim:
    if (model->rt->after_failed_step != NULL) model->rt->after_failed_step(model->rt);
    for (size_t i = 0; i < claimed; ++i) kipp_cache_trim(&model->cache, items[i].session); /* the step did not happen: its pages go back */
unmark:
    for (size_t i = 0; i < item_count; ++i) {
        if (items[i].session != NULL && items[i].session->model == model) items[i].session->in_step = false;
    }
    return rc;
}

/* ------------------------------------------------------------------ the other ways to evaluate */
int kipp_session_eval_scored(kipp_session *session, const uint32_t *tokens, size_t token_count, float *logits, uint32_t rows,
                             kipp_error *error) {
    if (session == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no session");
    if (rows == 0 || rows > token_count) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "rows must be 1 .. token_count");
    uint32_t *want = malloc(rows * sizeof(uint32_t));
    if (want == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    for (uint32_t r = 0; r < rows; ++r) want[r] = (uint32_t)(token_count - rows + r);
    kipp_step_item item = {session, tokens, token_count, want, rows};
    int rc = kipp_step(session->model, &item, 1, logits, (size_t)rows * session->model->spec.vocab, error);
    free(want);
    return rc;
}

int kipp_session_eval_n(kipp_session *session, const uint32_t *tokens, size_t token_count, float *logits, uint32_t rows,
                        kipp_error *error) {
    if (session == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no session");
    if (rows == 0 || rows > token_count) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "rows must be 1 .. token_count");
    /* on the 32-bit paths every output element is summed in an order that depends on its own row alone: one step gives
     * the bits of single-token evaluation.  Under bfloat16 a portion takes other kernels than a single token, so the
     * wanted tokens run one by one behind the rest. */
    if (session->model->rt->act_dtype == KIPP_F32 || rows == 1) return kipp_session_eval_scored(session, tokens, token_count, logits, rows, error);
    const uint32_t vocab = session->model->spec.vocab, before = session->length;
    size_t head = token_count - rows;
    if (head > 0) {
        kipp_step_item item = {session, tokens, head, NULL, 0};
        if (kipp_step(session->model, &item, 1, NULL, 0, error) != 0) return -1;
    }
    const uint32_t zero = 0;
    for (uint32_t r = 0; r < rows; ++r) {
        kipp_step_item item = {session, tokens + head + r, 1, &zero, 1};
        if (kipp_step(session->model, &item, 1, logits + (size_t)r * vocab, vocab, error) != 0) {
            kipp_error keep;
            if (error != NULL) keep = *error;
            kipp_cache_truncate(&session->model->cache, session, before, NULL); /* all or nothing, as one step would be */
            if (error != NULL) *error = keep;
            return -1;
        }
    }
    return 0;
}

int kipp_session_eval(kipp_session *session, const uint32_t *tokens, size_t token_count, float *logits, size_t logits_count,
                      kipp_error *error) {
    if (session == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no session");
    if (logits_count < session->model->spec.vocab) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "logits must hold %u floats", session->model->spec.vocab);
    return kipp_session_eval_scored(session, tokens, token_count, logits, 1, error);
}

int kipp_model_eval(kipp_model *model, const uint32_t *tokens, size_t token_count, float *logits, size_t logits_count, kipp_error *error) {
    kipp_error_clear(error);
    if (model == NULL || tokens == NULL || logits == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "model, tokens and logits must be given");
    if (token_count == 0 || token_count > KIPP_MODEL_EVAL_LIMIT)
        return kipp_fail(error, KIPP_ERROR_RANGE, "between 1 and %u tokens, not %zu", KIPP_MODEL_EVAL_LIMIT, token_count);
    if (logits_count < model->spec.vocab) return kipp_fail(error, KIPP_ERROR_RANGE, "logits must hold %u floats", model->spec.vocab);
    kipp_session *session = NULL;
    if (kipp_session_create(model, (uint32_t)token_count, &session, error) != 0) return -1;
    const int rc = kipp_session_eval_scored(session, tokens, token_count, logits, 1, error);
    kipp_session_destroy(session);
    return rc;
}

int kipp_eval_batch(kipp_model *model, kipp_batch_item *items, size_t item_count, kipp_error *error) {
    kipp_error_clear(error);
    if (model == NULL || (items == NULL && item_count != 0)) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "model and items must be given");
    if (item_count == 0) return 0;
    if (item_count > KIPP_EVAL_BATCH_LIMIT) return kipp_fail(error, KIPP_ERROR_RANGE, "%zu items are more than a batch takes (%u)", item_count, KIPP_EVAL_BATCH_LIMIT);
    const uint32_t vocab = model->spec.vocab;
    kipp_step_item *step = calloc(item_count, sizeof(kipp_step_item));
    uint32_t *want = malloc(item_count * sizeof(uint32_t));
    float *rows = malloc(item_count * (size_t)vocab * sizeof(float));
    int rc = -1;
    if (step == NULL || want == NULL || rows == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        goto done;
    }
    for (size_t i = 0; i < item_count; ++i) {
        if (items[i].token_count == 0 || items[i].logits == NULL) {
            kipp_fail(error, KIPP_ERROR_ARGUMENT, "item %zu: tokens and room for logits must be given", i);
            goto done;
        }
        want[i] = (uint32_t)(items[i].token_count - 1);
        step[i] = (kipp_step_item){items[i].session, items[i].tokens, items[i].token_count, &want[i], 1};
    }
    rc = kipp_step(model, step, item_count, rows, item_count * (size_t)vocab, error);
    if (rc == 0) {
        for (size_t i = 0; i < item_count; ++i) memcpy(items[i].logits, rows + i * vocab, (size_t)vocab * sizeof(float));
    }
done:
    free(step);
    free(want);
    free(rows);
    return rc;
}

/* ------------------------------------------------------------------ hooks for tests */
size_t kipp_test_session_pages(const kipp_session *session, uint32_t group, int32_t *out_pages, size_t capacity) {
    if (session == NULL || group >= session->model->cache.group_count) return 0;
    size_t n = session->table_lengths[group] < capacity ? session->table_lengths[group] : capacity;
    memcpy(out_pages, session->tables[group], n * sizeof(int32_t));
    return n;
}

/* Reverses the session's block tables and moves the pages' contents along, so that every position lies in another
 * page than before (/root/reference/src/kipp.c:4135-4165 does the same to prove reads and writes under a mapping that is
 * not the identity).  Only for sessions whose pages are all their own. */
int kipp_test_scramble_session_kv(kipp_session *session, kipp_error *error) {
    kipp_error_clear(error);
    if (session == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "no session");
    kipp_cache *cache = &session->model->cache;
    kipp_runtime *rt = cache->rt;
    if (session->adopted_tokens != 0) return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "adopted pages are shared and stay where they are");
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        kipp_cache_group *group = &cache->groups[g];
        uint32_t count = session->table_lengths[g];
        size_t page_bytes = (size_t)group->need.n_kv_heads * group->page_tokens * group->need.head_dim * kipp_dtype_bytes(rt->act_dtype);
        void *spare = rt->mem_alloc(rt, page_bytes, error);
        if (spare == NULL) return -1;
        for (uint32_t lo = 0, hi = count ? count - 1 : 0; lo < hi; ++lo, --hi) {
            int32_t a = session->tables[g][lo], b = session->tables[g][hi];
            if (a < 0 || b < 0) continue;
            for (uint32_t r = 0; r < group->run_count; ++r) {
                void *slabs[2] = {group->k[r], group->v[r]};
                for (int s = 0; s < 2; ++s) {
                    char *pa = (char *)slabs[s] + (size_t)a * page_bytes, *pb = (char *)slabs[s] + (size_t)b * page_bytes;
                    if (rt->copy(rt, spare, pa, page_bytes, error) != 0 || rt->copy(rt, pa, pb, page_bytes, error) != 0 ||
                        rt->copy(rt, pb, spare, page_bytes, error) != 0) {
                        rt->mem_free(rt, spare);
                        return -1;
                    }
                }
            }
            session->tables[g][lo] = b;
            session->tables[g][hi] = a;
        }
        rt->mem_free(rt, spare);
    }
    return 0;
}
