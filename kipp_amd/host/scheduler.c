/*
 * The scheduler above the step function (kipp_amd.h says what it promises; the
 * policy is the reference's server loop, /root/reference/src/kipp_server.c:1623-1893
 * admission, :1900-2125 stepping, :2081-2088 a batch that fails).
 *
 * A request is a session of the model plus its progress.  Requests publish their
 * full pages as they go, and a waiting request whose prompt begins like that of
 * a request that is still running its prompt waits until those pages are there
 * and adopts them instead of computing them again.  Admission reserves: a request
 * is admitted only if every pool still has what it may claim plus what every
 * running request may still claim (in a group with a window: the distance to the
 * most it ever holds at once), so pages never run out in the middle of a
 * generation; when they are short, requests wait, in order.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "internal.h"
#include "backend.h"

#define RECENT_WINDOW 64 /* tokens the penalties look back over (/root/reference/src/kipp_server.c:848) */

typedef enum { WAITING, PREFILL, DECODE, FINISHED } request_state;

typedef struct request {
    uint64_t id;
    uint32_t *prompt;
    uint32_t prompt_count, max_new_tokens;
    kipp_sample_params params;
    uint32_t *bias_tokens;
    float *bias_values;
    uint64_t rng;
    uint32_t stop_tokens[KIPP_MAX_STOP_TOKENS];
    uint32_t stop_token_count;
    request_state state;
    uint32_t fed; /* prompt tokens already in the cache */
    uint32_t *output;
    uint32_t output_count;
    uint32_t next_token;
    uint32_t recent[RECENT_WINDOW];
    uint32_t recent_count; /* how many of the last generated tokens `recent` holds, oldest first */
    kipp_finish_reason reason;
    char error[256];
    kipp_session *session;
    double arrived, first_token_at;
    bool has_first;
    float *last_logits;
    struct request *next; /* in its list: waiting (arrival order), running (admission order), finished */
} request;

struct kipp_scheduler {
    kipp_model *model;
    uint32_t max_step_tokens, prefill_chunk, max_running;
    request *waiting, *waiting_tail, *running, *finished;
    uint32_t running_count;
    bool keep_last_logits;
    kipp_scheduler_stats stats;
    /* room for one step */
    kipp_step_item *items;
    request **item_requests;
    uint32_t *wants;
    float *logits;
    uint32_t *chosen;
    kipp_sample_params *choices; /* with the device sampler: every wanted row's parameters, */
    double *draws;               /* and its draw */
    size_t logits_rows;
    bool device_sampler; /* the path has a sampler of its own and KIPP_AMD_SAMPLER does not say "host" */
};

static double now_seconds(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

static void request_free(request *r) {
    free(r->prompt);
    free(r->output);
    free(r->bias_tokens);
    free(r->bias_values);
    free(r->last_logits);
    free(r);
}

static request *find_in(request *list, uint64_t id) {
    for (request *r = list; r != NULL; r = r->next) {
        if (r->id == id) return r;
    }
    return NULL;
}

static void unlink_from(request **list, request *r) {
    for (request **link = list; *link != NULL; link = &(*link)->next) {
        if (*link == r) {
            *link = r->next;
            r->next = NULL;
            return;
        }
    }
}

static void append_to(request **list, request *r) {
    request **link = list;
    while (*link != NULL) link = &(*link)->next;
    *link = r;
    r->next = NULL;
}

int kipp_scheduler_create(kipp_model *model, const kipp_scheduler_config *config, kipp_scheduler **out_scheduler, kipp_error *error) {
    kipp_error_clear(error);
    if (model == NULL || out_scheduler == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "model and result must be given");
    kipp_scheduler *s = calloc(1, sizeof(*s));
    if (s == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    s->model = model;
    s->max_step_tokens = config != NULL && config->max_step_tokens ? config->max_step_tokens : 2048;
    s->prefill_chunk = config != NULL && config->prefill_chunk ? config->prefill_chunk : 512;
    s->max_running = config != NULL && config->max_running ? config->max_running : model->config.max_sessions;
    s->keep_last_logits = config != NULL && config->keep_last_logits != 0;
    if (s->max_step_tokens > model->config.max_step_tokens) s->max_step_tokens = model->config.max_step_tokens;
    if (s->max_running > model->config.max_sessions) s->max_running = model->config.max_sessions;
    if (s->max_running > KIPP_EVAL_BATCH_LIMIT) s->max_running = KIPP_EVAL_BATCH_LIMIT;
    s->items = calloc(s->max_running, sizeof(kipp_step_item));
    s->item_requests = calloc(s->max_running, sizeof(request *));
    s->wants = calloc(s->max_running, sizeof(uint32_t));
    s->logits_rows = s->max_running;
    s->logits = malloc(s->logits_rows * (size_t)model->spec.vocab * sizeof(float));
    s->chosen = malloc(s->logits_rows * sizeof(uint32_t));
    s->choices = malloc(s->logits_rows * sizeof(kipp_sample_params));
    s->draws = malloc(s->logits_rows * sizeof(double));
    const char *sampler = getenv("KIPP_AMD_SAMPLER");
    s->device_sampler = model->rt->sample != NULL && !(sampler != NULL && strcmp(sampler, "host") == 0);
    if (s->items == NULL || s->item_requests == NULL || s->wants == NULL || s->logits == NULL || s->chosen == NULL || s->choices == NULL || s->draws == NULL) {
        kipp_scheduler_destroy(s);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for the scheduler's step");
    }
    *out_scheduler = s;
    return 0;
}

void kipp_scheduler_destroy(kipp_scheduler *s) {
    if (s == NULL) return;
    request *lists[3] = {s->waiting, s->running, s->finished};
    for (int l = 0; l < 3; ++l) {
        for (request *r = lists[l], *next; r != NULL; r = next) {
            next = r->next;
            if (r->session != NULL) kipp_session_destroy(r->session);
            request_free(r);
        }
    }
    free(s->items);
    free(s->item_requests);
    free(s->wants);
    free(s->logits);
    free(s->chosen);
    free(s->choices);
    free(s->draws);
    free(s);
}

/* Most tokens one request brings in a step. */
static uint32_t largest_step(const kipp_scheduler *s) { return s->prefill_chunk < s->max_step_tokens ? s->prefill_chunk : s->max_step_tokens; }

/* Most tokens the cache will ever hold for it: the last chosen token is never run. */
static uint32_t budget_tokens(const request *r) { return r->prompt_count + (r->max_new_tokens > 0 ? r->max_new_tokens - 1 : 0); }

/* The most pages group `g` may still have to hand the request beyond those it holds now (`session` NULL: nothing yet). */
static uint32_t pages_bound(const kipp_scheduler *s, const kipp_session *session, uint32_t g, uint32_t budget) {
    const kipp_cache_group *group = &s->model->cache.groups[g];
    uint32_t have = session != NULL ? session->table_lengths[g] : 0;
    uint32_t blocks = (budget + group->page_tokens - 1) / group->page_tokens;
    uint32_t need = blocks > have ? blocks - have : 0;
    if (group->need.window != 0) {
        uint32_t most = (group->need.window - 1 + largest_step(s) + group->page_tokens - 1) / group->page_tokens + 1, held = 0;
        for (uint32_t b = 0; b < have; ++b) held += session->tables[g][b] >= 0;
        uint32_t room = most > held ? most - held : 0;
        if (room < need) need = room;
    }
    return need;
}

int kipp_scheduler_add(kipp_scheduler *s, const kipp_request *in, kipp_error *error) {
    kipp_error_clear(error);
    if (s == NULL || in == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "scheduler and request must be given");
    const kipp_model *model = s->model;
    /* an id names one request at a time: a second one would replace the first one's result */
    if (find_in(s->waiting, in->id) != NULL || find_in(s->running, in->id) != NULL || find_in(s->finished, in->id) != NULL) {
        ++s->stats.refused;
        return kipp_fail(error, KIPP_ERROR_ARGUMENT, "request %llu is already waiting, running, or finished and not collected", (unsigned long long)in->id);
    }
    if (in->prompt_count == 0 || in->prompt == NULL) {
        ++s->stats.refused;
        return kipp_fail(error, KIPP_ERROR_ARGUMENT, "request %llu: empty prompt", (unsigned long long)in->id);
    }
    if (in->prompt_count > model->spec.max_position || in->max_new_tokens > model->spec.max_position - in->prompt_count) {
        ++s->stats.refused;
        return kipp_fail(error, KIPP_ERROR_RANGE, "request %llu: prompt %zu + max_new_tokens %u exceeds the model's %u positions",
                         (unsigned long long)in->id, in->prompt_count, in->max_new_tokens, model->spec.max_position);
    }
    for (size_t t = 0; t < in->prompt_count; ++t) {
        if (in->prompt[t] >= model->spec.vocab) {
            ++s->stats.refused;
            return kipp_fail(error, KIPP_ERROR_RANGE, "request %llu: token %u is outside the vocabulary", (unsigned long long)in->id, in->prompt[t]);
        }
    }
    if (in->stop_token_count > KIPP_MAX_STOP_TOKENS) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "more than %u stop tokens", KIPP_MAX_STOP_TOKENS);
    if (in->params.temperature > 0.0f && (!(in->params.top_p > 0.0f && in->params.top_p <= 1.0f) || in->params.min_p < 0.0f || in->params.min_p > 1.0f))
        return kipp_fail(error, KIPP_ERROR_ARGUMENT, "top_p must be in (0, 1] and min_p in [0, 1]");
    request probe;
    memset(&probe, 0, sizeof(probe));
    probe.prompt_count = (uint32_t)in->prompt_count;
    probe.max_new_tokens = in->max_new_tokens;
    for (uint32_t g = 0; g < model->cache.group_count; ++g) {
        uint32_t most = pages_bound(s, NULL, g, budget_tokens(&probe));
        if (most > model->cache.groups[g].pool.page_count) {
            ++s->stats.refused;
            return kipp_fail(error, KIPP_ERROR_RANGE, "request %llu: needs %u pages of group %u, more than its pool's %u", (unsigned long long)in->id,
                             most, g, model->cache.groups[g].pool.page_count);
        }
    }
    request *r = calloc(1, sizeof(*r));
    if (r == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    r->id = in->id;
    r->prompt_count = (uint32_t)in->prompt_count;
    r->max_new_tokens = in->max_new_tokens;
    r->params = in->params;
    r->prompt = malloc(in->prompt_count * sizeof(uint32_t));
    r->output = malloc((in->max_new_tokens ? in->max_new_tokens : 1) * sizeof(uint32_t));
    r->last_logits = s->keep_last_logits ? malloc((size_t)model->spec.vocab * sizeof(float)) : NULL;
    bool ok = r->prompt != NULL && r->output != NULL && (r->last_logits != NULL || !s->keep_last_logits);
    if (ok && in->params.logit_bias_count != 0) {
        r->bias_tokens = malloc(in->params.logit_bias_count * sizeof(uint32_t));
        r->bias_values = malloc(in->params.logit_bias_count * sizeof(float));
        ok = r->bias_tokens != NULL && r->bias_values != NULL;
        if (ok) {
            memcpy(r->bias_tokens, in->params.logit_bias_tokens, in->params.logit_bias_count * sizeof(uint32_t));
            memcpy(r->bias_values, in->params.logit_bias_values, in->params.logit_bias_count * sizeof(float));
        }
    }
    if (!ok) {
        request_free(r);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a request of %zu tokens", in->prompt_count);
    }
    memcpy(r->prompt, in->prompt, in->prompt_count * sizeof(uint32_t));
    r->params.logit_bias_tokens = r->bias_tokens;
    r->params.logit_bias_values = r->bias_values;
    r->params.recent_tokens = NULL;
    r->params.recent_count = 0;
    r->rng = in->seed != 0 ? in->seed : 1; /* 0 mapped to 1 (/root/reference/src/kipp_server.c:1852-1862) */
    r->stop_token_count = in->stop_token_count;
    memcpy(r->stop_tokens, in->stop_tokens, sizeof(r->stop_tokens));
    r->state = WAITING;
    r->arrived = now_seconds();
    append_to(&s->waiting, r);
    ++s->stats.requests;
    return 0;
}

static void finish(kipp_scheduler *s, request *r, kipp_finish_reason reason) {
    r->state = FINISHED;
    r->reason = reason;
    if (find_in(s->running, r->id) == r) {
        unlink_from(&s->running, r);
        --s->running_count;
    } else {
        unlink_from(&s->waiting, r);
    }
    if (r->session != NULL) {
        kipp_session_destroy(r->session); /* publishes what is left to publish, gives every page and the slot back */
        r->session = NULL;
    }
    append_to(&s->finished, r);
    ++s->stats.finished;
    if (reason == KIPP_FINISH_FAILED) ++s->stats.failed;
    else if (r->has_first) s->stats.decode_seconds_sum += now_seconds() - r->first_token_at;
}

int kipp_scheduler_cancel(kipp_scheduler *s, uint64_t id, kipp_error *error) {
    kipp_error_clear(error);
    request *r = find_in(s->waiting, id);
    if (r == NULL) r = find_in(s->running, id);
    if (r == NULL) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "request %llu is neither waiting nor running", (unsigned long long)id);
    finish(s, r, KIPP_FINISH_CANCELLED);
    return 0;
}

int kipp_scheduler_idle(const kipp_scheduler *s) { return s->waiting == NULL && s->running == NULL; }

/* Is a running request about to publish pages that `r` could adopt? */
static bool worth_waiting(const kipp_scheduler *s, const request *r) {
    if (!s->model->cache.share) return false;
    const uint32_t page = s->model->cache.page_tokens;
    for (const request *other = s->running; other != NULL; other = other->next) {
        if (other->state != PREFILL) continue;
        uint32_t n = r->prompt_count - 1 < other->prompt_count ? r->prompt_count - 1 : other->prompt_count, common = 0;
        while (common < n && r->prompt[common] == other->prompt[common]) ++common;
        if (common / page > other->fed / page) return true;
    }
    return false;
}

static int admit(kipp_scheduler *s, kipp_error *error) {
    kipp_cache *cache = &s->model->cache;
    while (s->waiting != NULL && s->running_count < s->max_running) {
        request *r = s->waiting;
        if (worth_waiting(s, r)) {
            ++s->stats.waits_for_prefix;
            return 0;
        }
        if (kipp_session_create(s->model, budget_tokens(r) > 0 ? budget_tokens(r) : 1, &r->session, error) != 0) {
            if (error != NULL && error->code == KIPP_ERROR_RANGE) { /* every slot is taken by sessions that are not ours: wait */
                kipp_error_clear(error);
                ++s->stats.waits_for_pages;
                return 0;
            }
            return -1;
        }
        r->session->publish_early = cache->share;
        uint32_t matched = 0;
        if (cache->share && kipp_cache_adopt(cache, r->session, r->prompt, r->prompt_count, &matched, error) != 0) return -1;
        bool fits = true;
        for (uint32_t g = 0; g < cache->group_count && fits; ++g) {
            uint64_t promised = pages_bound(s, r->session, g, budget_tokens(r));
            for (const request *other = s->running; other != NULL; other = other->next) promised += pages_bound(s, other->session, g, budget_tokens(other));
            fits = promised <= cache->groups[g].pool.free_count;
        }
        if (!fits) {
            kipp_session_destroy(r->session); /* undo; stays first in line */
            r->session = NULL;
            ++s->stats.waits_for_pages;
            return 0;
        }
        s->waiting = r->next;
        r->next = NULL;
        append_to(&s->running, r);
        ++s->running_count;
        r->fed = matched;
        r->state = PREFILL;
        s->stats.prefix_tokens_reused += matched;
        s->stats.queue_wait_seconds_sum += now_seconds() - r->arrived;
        ++s->stats.queue_wait_count;
    }
    return 0;
}

static void remember(request *r, uint32_t token) {
    if (r->recent_count == RECENT_WINDOW) {
        memmove(r->recent, r->recent + 1, (RECENT_WINDOW - 1) * sizeof(uint32_t));
        --r->recent_count;
    }
    r->recent[r->recent_count++] = token;
}

static void accept(kipp_scheduler *s, request *r, uint32_t token, kipp_produced *out, size_t capacity, size_t *count) {
    if (r->max_new_tokens == 0) {
        finish(s, r, KIPP_FINISH_LENGTH);
        return;
    }
    for (uint32_t i = 0; i < r->stop_token_count; ++i) {
        if (r->stop_tokens[i] == token) {
            finish(s, r, KIPP_FINISH_STOP); /* not kept, not fed back */
            return;
        }
    }
    if (!r->has_first) {
        r->has_first = true;
        r->first_token_at = now_seconds();
        s->stats.ttft_seconds_sum += r->first_token_at - r->arrived;
        ++s->stats.ttft_count;
    }
    r->output[r->output_count++] = token;
    remember(r, token);
    if (out != NULL && *count < capacity) out[*count] = (kipp_produced){r->id, token};
    ++*count;
    ++s->stats.generated_tokens;
    if (r->output_count >= r->max_new_tokens) {
        finish(s, r, KIPP_FINISH_LENGTH);
        return;
    }
    r->next_token = token;
    r->state = DECODE;
}

int kipp_scheduler_step(kipp_scheduler *s, kipp_produced *out, size_t capacity, size_t *out_count, kipp_error *error) {
    kipp_error_clear(error);
    size_t produced = 0;
    if (out_count != NULL) *out_count = 0;
    if (admit(s, error) != 0) return -1;
    /* the plan: every decoding request's next token first, then portions of prompts in arrival order while the budget lasts */
    uint32_t budget = s->max_step_tokens, n = 0, wanted = 0;
    for (request *r = s->running; r != NULL; r = r->next) {
        if (r->state != DECODE || budget == 0) continue;
        s->wants[n] = 0;
        s->items[n] = (kipp_step_item){r->session, &r->next_token, 1, &s->wants[n], 1};
        s->item_requests[n++] = r;
        --budget;
        ++wanted;
    }
    for (request *r = s->running; r != NULL; r = r->next) {
        if (r->state != PREFILL || budget == 0) continue;
        uint32_t left = r->prompt_count - r->fed, take = left < s->prefill_chunk ? left : s->prefill_chunk;
        if (take > budget) take = budget;
        bool last = take == left;
        s->wants[n] = take - 1;
        s->items[n] = (kipp_step_item){r->session, r->prompt + r->fed, take, &s->wants[n], last ? 1 : 0};
        s->item_requests[n++] = r;
        budget -= take;
        wanted += last;
    }
    if (n == 0) return 0;
    /* where every wanted place is chosen by the largest logit alone, the choice is made beside the logits */
    bool greedy = !s->keep_last_logits;
    for (uint32_t i = 0; i < n && greedy; ++i) {
        const kipp_sample_params *p = &s->item_requests[i]->params;
        greedy = s->items[i].want_count == 0 || (p->temperature <= 0.0f && p->frequency_penalty == 0.0f && p->presence_penalty == 0.0f &&
                                                 (p->repetition_penalty == 1.0f || p->repetition_penalty == 0.0f) && p->logit_bias_count == 0);
    }
    /* else, where the path has a sampler of its own, every row is chosen there as well: a row's bias and penalties change it
     * where it lies, and a sampled row gets the draw that kipp_sample_ex would take from the request's generator now
     * (parameters it would refuse go to it, so that it does) */
    bool beside = !greedy && s->device_sampler;
    uint32_t rows = 0;
    for (uint32_t i = 0; i < n && beside; ++i) {
        const kipp_sample_params *p = &s->item_requests[i]->params;
        if (s->items[i].want_count == 0) continue;
        beside = p->temperature <= 0.0f || (p->top_p > 0.0f && p->top_p <= 1.0f && p->min_p >= 0.0f && p->min_p <= 1.0f && s->item_requests[i]->rng != 0);
    }
    for (uint32_t i = 0; i < n && beside; ++i) {
        request *r = s->item_requests[i];
        if (s->items[i].want_count == 0) continue;
        s->choices[rows] = r->params;
        s->choices[rows].recent_tokens = r->recent;
        s->choices[rows].recent_count = r->recent_count;
        s->draws[rows++] = r->params.temperature > 0.0f ? kipp_rng_uniform(&r->rng) : 0.0;
    }
    greedy = greedy || beside; /* from here on: the tokens are in s->chosen */
    kipp_error step_error;
    int step_rc = beside   ? kipp_step_sample_logits(s->model, s->items, n, s->choices, s->draws, s->chosen, s->logits_rows,
                                                     s->keep_last_logits ? s->logits : NULL, s->logits_rows * (size_t)s->model->spec.vocab, &step_error)
                  : greedy ? kipp_step_argmax(s->model, s->items, n, s->chosen, s->logits_rows, &step_error)
                           : kipp_step(s->model, s->items, n, s->logits, s->logits_rows * (size_t)s->model->spec.vocab, &step_error);
    if (step_rc != 0) {
        /* the batch failed as a unit: every request that had tokens in it fails; those that were not in it go on */
        ++s->stats.failed_steps;
        for (uint32_t i = 0; i < n; ++i) {
            snprintf(s->item_requests[i]->error, sizeof(s->item_requests[i]->error), "%s: %.200s", kipp_error_code_name(step_error.code), step_error.message);
            finish(s, s->item_requests[i], KIPP_FINISH_FAILED);
        }
        return 0;
    }
    ++s->stats.steps;
    const uint32_t vocab = s->model->spec.vocab;
    uint32_t row = 0;
    for (uint32_t i = 0; i < n; ++i) {
        request *r = s->item_requests[i];
        if (r->state == PREFILL) {
            r->fed += (uint32_t)s->items[i].token_count;
            s->stats.prompt_tokens += s->items[i].token_count;
        }
        if (s->items[i].want_count == 0) continue;
        if (greedy) {
            if (r->last_logits != NULL) memcpy(r->last_logits, s->logits + (size_t)row * vocab, (size_t)vocab * sizeof(float));
            accept(s, r, s->chosen[row++], out, capacity, &produced);
            continue;
        }
        const float *logits = s->logits + (size_t)row++ * vocab;
        if (r->last_logits != NULL) memcpy(r->last_logits, logits, (size_t)vocab * sizeof(float));
        kipp_sample_params params = r->params;
        params.recent_tokens = r->recent;
        params.recent_count = r->recent_count;
        uint32_t token = 0;
        if (kipp_sample_ex(logits, vocab, &params, &r->rng, &token, error) != 0) {
            snprintf(r->error, sizeof(r->error), "sampling: %.200s", error != NULL ? error->message : "");
            kipp_error_clear(error);
            finish(s, r, KIPP_FINISH_FAILED);
            continue;
        }
        accept(s, r, token, out, capacity, &produced);
    }
    if (out_count != NULL) *out_count = produced;
    return 0;
}

int kipp_scheduler_result(const kipp_scheduler *s, uint64_t id, kipp_result *out_result) {
    const request *r = find_in(s->finished, id);
    if (r == NULL) r = find_in(s->running, id);
    if (r == NULL) r = find_in(s->waiting, id);
    if (r == NULL || out_result == NULL) return -1;
    *out_result = (kipp_result){r->id, r->state == FINISHED ? r->reason : KIPP_FINISH_NONE, r->output, r->output_count, r->error};
    return 0;
}

const float *kipp_scheduler_last_logits(const kipp_scheduler *s, uint64_t id) {
    const request *r = find_in(s->finished, id);
    if (r == NULL) r = find_in(s->running, id);
    return r != NULL && (r->has_first || r->state == FINISHED) ? r->last_logits : NULL;
}

int kipp_scheduler_collect(kipp_scheduler *s, uint64_t id) {
    request *r = find_in(s->finished, id);
    if (r == NULL) return -1;
    unlink_from(&s->finished, r);
    request_free(r);
    return 0;
}

int kipp_scheduler_get_stats(const kipp_scheduler *s, kipp_scheduler_stats *out_stats) {
    if (s == NULL || out_stats == NULL) return -1;
    *out_stats = s->stats;
    return 0;
}
