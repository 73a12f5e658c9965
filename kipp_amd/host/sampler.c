/*
 * Token choice on the host, in the order and the float widths of the reference's
 * sampler (/root/reference/src/kipp.c:3386-3559; parameters /root/reference/src/kipp.h:278-291):
 * logit bias; repetition, presence and frequency penalties over the recent
 * tokens, each distinct token once; argmax with the lowest index winning ties;
 * temperature <= 0 returns it and leaves the generator untouched; else scale by
 * 1/T, keep candidates within 20 of the maximum, order them descending (equal
 * logits: lower id first), top-k, weights expf(l - max) summed in double, min-p,
 * top-p (shortest beginning with mass >= top_p * total, at least one), one draw
 * of xorshift64*.  It is also the scalar reference of the device sampler.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "internal.h"

/* /root/reference/src/kipp.c:3322-3333 */
double kipp_rng_uniform(uint64_t *state) {
    uint64_t x = *state;
    x ^= x >> 12;
    x ^= x << 25;
    x ^= x >> 27;
    *state = x;
    return (double)((x * 2685821657736338717ull) >> 11) / 9007199254740992.0;
}

typedef struct {
    float logit;
    uint32_t token;
} candidate;

static bool before(const candidate *a, const candidate *b) { return a->logit > b->logit || (a->logit == b->logit && a->token < b->token); }

/* heap sort: the order is total (no two candidates share a token), so any correct sort gives the same sequence */
static void sift(candidate *items, size_t root, size_t count) {
    for (;;) {
        size_t child = 2 * root + 1;
        if (child >= count) return;
        if (child + 1 < count && before(&items[child], &items[child + 1])) ++child; /* the later of the two */
        if (!before(&items[root], &items[child])) return;
        candidate t = items[root];
        items[root] = items[child];
        items[child] = t;
        root = child;
    }
}

static void order_candidates(candidate *items, size_t count) {
    for (size_t i = count / 2; i-- > 0;) sift(items, i, count);
    for (size_t end = count; end-- > 1;) {
        candidate t = items[0];
        items[0] = items[end];
        items[end] = t;
        sift(items, 0, end);
    }
}

int kipp_sample_ex(const float *logits, size_t logits_count, const kipp_sample_params *params, uint64_t *rng_state,
                   uint32_t *out_token, kipp_error *error) {
    kipp_error_clear(error);
    if (logits == NULL || logits_count == 0 || params == NULL || out_token == NULL)
        return kipp_fail(error, KIPP_ERROR_ARGUMENT, "logits, parameters and result must be given");
    if (logits_count > UINT32_MAX) return kipp_fail(error, KIPP_ERROR_RANGE, "too many logits");
    const float *values = logits;
    float *changed = NULL;
    bool penalties = params->frequency_penalty != 0.0f || params->presence_penalty != 0.0f ||
                     (params->repetition_penalty != 0.0f && params->repetition_penalty != 1.0f);
    if (params->logit_bias_count != 0 || (penalties && params->recent_count != 0)) {
        changed = malloc(logits_count * sizeof(float));
        if (changed == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        memcpy(changed, logits, logits_count * sizeof(float));
        for (size_t i = 0; i < params->logit_bias_count; ++i) {
            if (params->logit_bias_tokens[i] < logits_count) changed[params->logit_bias_tokens[i]] += params->logit_bias_values[i];
        }
        if (penalties) {
            for (size_t i = 0; i < params->recent_count; ++i) {
                uint32_t token = params->recent_tokens[i];
                bool seen = false;
                if (token >= logits_count) continue;
                for (size_t j = 0; j < i && !seen; ++j) seen = params->recent_tokens[j] == token;
                if (seen) continue; /* each distinct token once */
                size_t count = 0;
                for (size_t j = 0; j < params->recent_count; ++j) count += params->recent_tokens[j] == token;
                float v = changed[token];
                if (params->repetition_penalty != 0.0f && params->repetition_penalty != 1.0f)
                    v = v > 0.0f ? v / params->repetition_penalty : v * params->repetition_penalty;
                v -= params->presence_penalty;
                v -= params->frequency_penalty * (float)count;
                changed[token] = v;
            }
        }
        values = changed;
    }
    size_t best = 0;
    for (size_t i = 1; i < logits_count; ++i) {
        if (values[i] > values[best]) best = i;
    }
    int rc = 0;
    if (params->temperature <= 0.0f) {
        *out_token = (uint32_t)best;
        goto done;
    }
    if (!(params->top_p > 0.0f && params->top_p <= 1.0f)) {
        rc = kipp_fail(error, KIPP_ERROR_ARGUMENT, "top_p must be greater than 0 and at most 1");
        goto done;
    }
    if (params->min_p < 0.0f || params->min_p > 1.0f) {
        rc = kipp_fail(error, KIPP_ERROR_ARGUMENT, "min_p must be between 0 and 1");
        goto done;
    }
    if (rng_state == NULL || *rng_state == 0) {
        rc = kipp_fail(error, KIPP_ERROR_ARGUMENT, "sampling requires a nonzero RNG state");
        goto done;
    }
    {
        const float inverse_temperature = 1.0f / params->temperature;
        const float top = values[best] * inverse_temperature, cutoff = top - 20.0f;
        size_t count = 0;
        for (size_t i = 0; i < logits_count; ++i) count += values[i] * inverse_temperature >= cutoff;
        candidate *items = malloc((count ? count : 1) * sizeof(candidate));
        if (items == NULL) {
            rc = kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
            goto done;
        }
        count = 0;
        for (size_t i = 0; i < logits_count; ++i) {
            float scaled = values[i] * inverse_temperature;
            if (scaled >= cutoff) items[count++] = (candidate){scaled, (uint32_t)i};
        }
        order_candidates(items, count);
        if (params->top_k != 0 && params->top_k < count) count = params->top_k;
        double total = 0.0;
        for (size_t i = 0; i < count; ++i) {
            items[i].logit = expf(items[i].logit - top);
            total += items[i].logit;
        }
        if (params->min_p > 0.0f && count > 0) {
            double threshold = (double)params->min_p * items[0].logit;
            size_t keep = count;
            for (size_t i = 1; i < count; ++i) {
                if (items[i].logit < threshold) {
                    keep = i;
                    break;
                }
            }
            count = keep;
            total = 0.0;
            for (size_t i = 0; i < count; ++i) total += items[i].logit;
        }
        double target = (double)params->top_p * total, kept = 0.0;
        size_t nucleus = 0;
        while (nucleus < count && kept < target) kept += items[nucleus++].logit;
        if (nucleus == 0) {
            nucleus = 1;
            kept = items[0].logit;
        }
        double draw = kipp_rng_uniform(rng_state) * kept, cumulative = 0.0;
        uint32_t token = items[nucleus - 1].token;
        for (size_t i = 0; i < nucleus; ++i) {
            cumulative += items[i].logit;
            if (draw < cumulative) {
                token = items[i].token;
                break;
            }
        }
        *out_token = token;
        free(items);
    }
done:
    free(changed);
    return rc;
}

int kipp_sample(const float *logits, size_t logits_count, float temperature, float top_p, uint64_t *rng_state, uint32_t *out_token,
                kipp_error *error) {
    kipp_sample_params params;
    memset(&params, 0, sizeof(params));
    params.temperature = temperature;
    params.top_p = top_p;
    params.repetition_penalty = 1.0f;
    return kipp_sample_ex(logits, logits_count, &params, rng_state, out_token, error);
}
