/*
 * The host logic of the C library under AddressSanitizer and UndefinedBehaviorSanitizer
 * (the reference builds its own host the same way, /root/reference/Makefile): the JSON reader, checked sizes,
 * the page pool and the cache manager under random orders of sessions, a model folder opened
 * and stepped on the scalar path under several cuttings with scrambled block tables, the error paths
 * of the step function, the scheduler over few pages with cancellations and a failed step, and the sampler.
 * The GPU's table is not part of this build.
 *
 *   host_test MODEL_DIR [MODEL_DIR ...] [--toy TOY_DIR]      exit code 0 and a last line "ok <checks>" on success
 *
 * TOY_DIR holds a model of an architecture that this file defines and registers itself (a mixer with state of its own).
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "backend.h"
#include "internal.h"

static int checks, failures;
#define CHECK(cond)                                                            \
    do {                                                                       \
        ++checks;                                                              \
        if (!(cond)) {                                                         \
            ++failures;                                                        \
            fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
        }                                                                      \
    } while (0)

static uint64_t rng_state = 0x9e3779b97f4a7c15ull;
static uint32_t rnd(uint32_t below) {
    rng_state ^= rng_state >> 12;
    rng_state ^= rng_state << 25;
    rng_state ^= rng_state >> 27;
    return (uint32_t)(((rng_state * 2685821657736338717ull) >> 33) % below);
}

static void test_json(void) {
    kj_doc doc;
    kipp_error error;
    const char *good = "{\"a\": [1, 2.5, -3e2, true, null], \"b\": {\"c\": \"x\\u00e9\\ud83d\\ude00\\n\"}, \"d\": 9007199254740993}";
    CHECK(kj_parse(good, strlen(good), &doc, &error) == 0);
    const kj_node *root = kj_root(&doc), *a = kj_get(&doc, root, "a");
    CHECK(root->type == KJ_OBJECT && root->count == 3 && a != NULL && a->type == KJ_ARRAY && a->count == 5);
    const kj_node *item = kj_first(&doc, a);
    CHECK(item->is_integer && item->integer == 1);
    item = kj_next(&doc, item);
    CHECK(!item->is_integer && item->number == 2.5);
    item = kj_next(&doc, item);
    CHECK(!item->is_integer && item->number == -300.0);
    item = kj_next(&doc, item);
    CHECK(item->type == KJ_BOOL && item->boolean);
    item = kj_next(&doc, item);
    CHECK(item->type == KJ_NULL && kj_next(&doc, item) == NULL);
    const kj_node *c = kj_get(&doc, kj_get(&doc, root, "b"), "c");
    CHECK(c != NULL && strcmp(c->string, "x\xc3\xa9\xf0\x9f\x98\x80\n") == 0 && c->string_length == 8);
    CHECK(kj_get(&doc, root, "d")->is_integer && kj_get(&doc, root, "d")->integer == 9007199254740993ll);
    CHECK(kj_get(&doc, root, "nope") == NULL);
    kj_free(&doc);
    static const char *const bad[] = {"", "{", "{\"a\": 1,}", "{\"a\": 1} x", "{\"a\": 1, \"a\": 2}", "[01]", "[1.]", "[.5]", "[1e]", "[NaN]",
                                      "[Infinity]", "\"\\ud800\"", "\"\\udc00\"", "\"\\u12\"", "\"a\nb\"", "\"\\x\"", "[1 2]", "{1: 2}", "{\"a\" 1}",
                                      "'a'", "[\"\\u0000\"]", "tru", "[1e999]", "-", "\"abc"};
    for (size_t i = 0; i < sizeof(bad) / sizeof(bad[0]); ++i) {
        CHECK(kj_parse(bad[i], strlen(bad[i]), &doc, &error) != 0);
        CHECK(error.code == KIPP_ERROR_FORMAT);
    }
    char deep[200];
    memset(deep, '[', 70);
    memset(deep + 70, ']', 70);
    CHECK(kj_parse(deep, 140, &doc, &error) != 0);
    memset(deep, '[', 60);
    memset(deep + 60, ']', 60);
    CHECK(kj_parse(deep, 120, &doc, &error) == 0);
    kj_free(&doc);
    /* a text that is not nul-terminated at its length */
    char *exact = malloc(7);
    memcpy(exact, "[1, 23]", 7);
    CHECK(kj_parse(exact, 7, &doc, &error) == 0 && kj_root(&doc)->count == 2);
    kj_free(&doc);
    CHECK(kj_parse(exact, 6, &doc, &error) != 0);
    free(exact);
}

static void test_sizes(void) {
    size_t out = 0;
    CHECK(kipp_add_size(SIZE_MAX - 1, 1, &out) == 0 && out == SIZE_MAX);
    CHECK(kipp_add_size(SIZE_MAX, 1, &out) != 0);
    CHECK(kipp_mul_size(SIZE_MAX / 2, 2, &out) == 0 && kipp_mul_size(SIZE_MAX / 2 + 1, 2, &out) != 0 && kipp_mul_size(0, SIZE_MAX, &out) == 0);
    CHECK(kipp_test_float_to_bf16(1.0f) == 0x3f80 && kipp_test_float_to_bf16(-2.0f) == 0xc000); /* /root/reference/tests/kipp_test.c:56-62 */
    CHECK(isinf(kipp_test_bf16_to_float(0x7f80)) && kipp_test_bf16_to_float(kipp_test_float_to_bf16(1.00390625f)) == 1.0f);
    CHECK(kipp_test_float_to_bf16(1.01171875f) == 0x3f82); /* 1 + 3/256: a tie, to the even neighbour above */
}

/* /root/reference/tests/kipp_test.c:3092-3392 has the reference's pool scenarios; these are their invariants under random orders */
static void test_pool(void) {
    kipp_pool pool;
    kipp_error error;
    const uint32_t pages = 13, page_tokens = 4;
    CHECK(kipp_pool_init(&pool, pages, page_tokens, NULL, &error) == 0);
    uint32_t held[64], n_held = 0, tokens[4];
    for (int round = 0; round < 4000; ++round) {
        uint32_t action = rnd(10);
        if (action < 4) {
            uint32_t page = kipp_pool_alloc(&pool);
            CHECK((page == KIPP_NO_PAGE) == (pool.free_count == 0 && page == KIPP_NO_PAGE));
            if (page != KIPP_NO_PAGE) held[n_held++] = page;
        } else if (action < 7 && n_held > 0) {
            uint32_t at = rnd(n_held);
            CHECK(kipp_pool_release(&pool, held[at]) == 0);
            held[at] = held[--n_held];
        } else if (action < 9 && n_held > 0) {
            uint32_t at = rnd(n_held);
            for (int i = 0; i < 4; ++i) tokens[i] = rnd(2);
            if (!kipp_pool_is_indexed(&pool, held[at]) && pool.pages[held[at]].ref_count == 1) kipp_pool_seal(&pool, held[at], rnd(2), tokens);
        } else if (n_held < 60) {
            uint32_t sequence[9], got[2];
            for (int i = 0; i < 9; ++i) sequence[i] = rnd(2);
            uint32_t matched = kipp_pool_prefix_match(&pool, sequence, 9, got, 2, NULL);
            CHECK(matched <= 2);
            for (uint32_t i = 0; i < matched; ++i) held[n_held++] = got[i];
        }
        if (kipp_pool_check(&pool, &error) != 0) {
            CHECK(0);
            fprintf(stderr, "%s\n", error.message);
            break;
        }
        uint32_t referenced = 0;
        for (uint32_t p = 0; p < pages; ++p) referenced += pool.pages[p].ref_count;
        CHECK(referenced == n_held && pool.free_count <= pages);
    }
    CHECK(kipp_pool_release(&pool, 99) != 0);
    while (n_held > 0) kipp_pool_release(&pool, held[--n_held]);
    CHECK(pool.free_count == pages);
    kipp_pool_free(&pool);
    /* a collision: the same forced hash for different tokens is told apart by the tokens */
    CHECK(kipp_pool_init(&pool, 4, 2, NULL, &error) == 0);
    pool.force_hash = true;
    pool.forced_hash = 7;
    uint32_t a = kipp_pool_alloc(&pool), b = kipp_pool_alloc(&pool), ta[2] = {1, 2}, tb[2] = {3, 4}, find[3] = {3, 4, 9}, got[1];
    kipp_pool_seal(&pool, a, 0, ta);
    kipp_pool_seal(&pool, b, 0, tb);
    CHECK(kipp_pool_prefix_match(&pool, find, 3, got, 1, NULL) == 1 && got[0] == b);
    kipp_pool_free(&pool);
    uint32_t twice[3] = {0, 1, 1};
    CHECK(kipp_pool_init(&pool, 3, 2, twice, &error) != 0);
    CHECK(kipp_pool_init(&pool, 0, 2, NULL, &error) != 0);
}

static int same_bits(const float *a, const float *b, size_t n) { return memcmp(a, b, n * sizeof(float)) == 0; }

/* One model folder on the scalar path: the whole sequence in one step, then the same tokens in portions beside a second
 * session, with the tables reversed on the way; the logits must be the same bits. */
static void test_model(const char *folder) {
    kipp_model *model = NULL;
    kipp_error error;
    kipp_model_open_config config;
    memset(&config, 0, sizeof(config));
    config.path = KIPP_PATH_CPU_FP32;
    config.page_tokens = 4;
    config.kv_pool_pages = 40;
    config.max_sessions = 3;
    config.share_prefixes = 1;
    if (kipp_model_open_ex(folder, &config, &model, &error) != 0) {
        fprintf(stderr, "cannot open %s: %s\n", folder, error.message);
        CHECK(0);
        return;
    }
    kipp_model_info info;
    CHECK(kipp_model_get_info(model, &info) == 0 && info.vocab_size > 0 && info.cache_groups == 1);
    const uint32_t vocab = info.vocab_size, n = 37;
    uint32_t tokens[64], other[64], want[64];
    for (uint32_t i = 0; i < 64; ++i) {
        tokens[i] = rnd(vocab);
        other[i] = rnd(vocab);
        want[i] = i;
    }
    float *whole = malloc((size_t)n * vocab * sizeof(float)), *cut = malloc((size_t)n * vocab * sizeof(float)),
          *spare = malloc((size_t)64 * vocab * sizeof(float));
    kipp_session *a = NULL, *b = NULL, *c = NULL, *d = NULL;
    CHECK(kipp_session_create(model, 0, &a, &error) == 0);
    kipp_step_item item = {a, tokens, n, want, n};
    CHECK(kipp_step(model, &item, 1, whole, (size_t)n * vocab, &error) == 0);
    for (size_t i = 0; i < (size_t)n * vocab; ++i) {
        if (!isfinite(whole[i])) {
            CHECK(0);
            break;
        }
    }
    kipp_session_info sinfo;
    CHECK(kipp_session_get_info(a, &sinfo) == 0 && sinfo.length == n && sinfo.cache_bytes > 0);
    CHECK(kipp_session_reset(a, &error) == 0); /* publishes 9 full pages */
    CHECK(kipp_session_create(model, 0, &b, &error) == 0 && kipp_session_create(model, 0, &c, &error) == 0);
    CHECK(kipp_session_create(model, 0, &d, &error) != 0 && error.code == KIPP_ERROR_RANGE); /* three slots */
    /* portions of `a` (which adopts nothing: its first portion is run) beside portions and single tokens of `b` */
    static const uint32_t portions[] = {5, 2, 9, 1, 1, 7, 3, 1, 8};
    uint32_t fed = 0, fed_b = 0;
    for (size_t p = 0; p < sizeof(portions) / sizeof(portions[0]); ++p) {
        uint32_t take_b = 1 + rnd(4);
        kipp_step_item items[2] = {{b, other + fed_b, take_b, want, p % 2 ? take_b : 0}, {a, tokens + fed, portions[p], want, portions[p]}};
        size_t rows_b = items[0].want_count;
        CHECK(kipp_step(model, items, 2, spare, (size_t)64 * vocab, &error) == 0);
        memcpy(cut + (size_t)fed * vocab, spare + rows_b * vocab, (size_t)portions[p] * vocab * sizeof(float));
        fed += portions[p];
        fed_b += take_b;
        if (p % 3 == 1) CHECK(kipp_test_scramble_session_kv(a, &error) == 0 && kipp_test_scramble_session_kv(b, &error) == 0);
        CHECK(kipp_cache_check(&model->cache, model->sessions, model->session_count, &error) == 0);
    }
    CHECK(fed == n && same_bits(whole, cut, (size_t)n * vocab));
    /* a session that adopts the published beginning continues with the same bits */
    uint32_t matched = 0;
    CHECK(kipp_session_match_prefix(c, tokens, n, &matched, &error) == 0 && matched == 36);
    CHECK(kipp_test_scramble_session_kv(c, &error) != 0 && error.code == KIPP_ERROR_UNSUPPORTED);
    CHECK(kipp_session_eval(c, tokens + matched, n - matched, spare, vocab, &error) == 0 && same_bits(spare, whole + (size_t)(n - 1) * vocab, vocab));
    /* error paths leave everything as it was */
    kipp_kv_pool_stats_public before, after;
    kipp_model_kv_pool_stats(model, 0, &before);
    uint32_t bad_token = vocab, place = 5;
    kipp_step_item bad = {a, &bad_token, 1, want, 1};
    CHECK(kipp_step(model, &bad, 1, spare, vocab, &error) != 0 && error.code == KIPP_ERROR_RANGE);
    bad = (kipp_step_item){a, tokens, 2, &place, 1};
    CHECK(kipp_step(model, &bad, 1, spare, vocab, &error) != 0);
    bad = (kipp_step_item){a, tokens, 2, want, 2};
    CHECK(kipp_step(model, &bad, 1, spare, vocab, &error) != 0 && error.code == KIPP_ERROR_ARGUMENT); /* room for one row only */
    kipp_step_item twice[2] = {{a, tokens, 1, want, 1}, {a, tokens, 1, want, 1}};
    CHECK(kipp_step(model, twice, 2, spare, 2 * (size_t)vocab, &error) != 0);
    kipp_model_kv_pool_stats(model, 0, &after);
    CHECK(before.free_blocks == after.free_blocks && kipp_session_get_info(a, &sinfo) == 0 && sinfo.length == n);
    CHECK(kipp_session_truncate(a, 10, &error) == 0 && kipp_session_truncate(a, 11, &error) != 0);
    CHECK(kipp_session_eval_n(a, tokens + 10, 5, spare, 3, &error) == 0 && same_bits(spare, whole + (size_t)12 * vocab, (size_t)3 * vocab));
    CHECK(kipp_model_close(model, &error) != 0); /* sessions are alive */
    kipp_session_destroy(a);
    kipp_session_destroy(b);
    kipp_session_destroy(c);
    kipp_model_kv_pool_stats(model, 0, &after);
    CHECK(after.free_blocks == after.total_blocks && after.reused_blocks_total >= 9);
    /* rows scored in the step that makes them: -log softmax at the next token, from the logits of the whole sequence */
    {
        kipp_session *e = NULL;
        double each[64], sum = 0.0, want_sum = 0.0;
        CHECK(kipp_session_create(model, 0, &e, &error) == 0);
        kipp_step_item scored_item = {e, tokens, n, want, n - 1};
        CHECK(kipp_step_nll(model, &scored_item, 1, tokens + 1, each, 64, &error) == 0);
        for (uint32_t r = 0; r + 1 < n; ++r) {
            const float *row = whole + (size_t)r * vocab;
            float top = row[0];
            double total = 0.0;
            for (uint32_t t = 1; t < vocab; ++t) top = row[t] > top ? row[t] : top;
            for (uint32_t t = 0; t < vocab; ++t) total += exp((double)row[t] - (double)top);
            want_sum += (double)top + log(total) - (double)row[tokens[r + 1]];
            sum += each[r];
        }
        CHECK(fabs(sum - want_sum) < 1e-9 && sum > 0.0);
        CHECK(kipp_step_nll(model, &scored_item, 1, tokens + 1, each, 3, &error) != 0 && error.code == KIPP_ERROR_ARGUMENT);
        uint32_t far_target = vocab;
        kipp_step_item one = {e, tokens, 1, want, 1};
        CHECK(kipp_step_nll(model, &one, 1, &far_target, each, 64, &error) != 0 && error.code == KIPP_ERROR_RANGE);
        /* the scalar path has no sampler of its own; the generator's draws are kipp_sample_ex's */
        kipp_sample_params greedy_params;
        memset(&greedy_params, 0, sizeof(greedy_params));
        double draw = 0.0;
        uint32_t token = 0;
        CHECK(kipp_step_sample(model, &one, 1, &greedy_params, &draw, &token, 1, &error) != 0 && error.code == KIPP_ERROR_UNSUPPORTED);
        uint64_t state = 88172645463325252ull, twin = state;
        double u = kipp_rng_uniform(&state);
        CHECK(u >= 0.0 && u < 1.0 && state != twin);
        kipp_session_destroy(e);
    }
    /* evaluation through a session of its own: the bits of the whole sequence, nothing held afterwards, three slots free again */
    CHECK(kipp_model_eval(model, tokens, n, spare, vocab, &error) == 0 && same_bits(spare, whole + (size_t)(n - 1) * vocab, vocab));
    CHECK(kipp_model_eval(model, tokens, n, spare, vocab - 1, &error) != 0 && error.code == KIPP_ERROR_RANGE);
    CHECK(kipp_model_eval(model, tokens, 0, spare, vocab, &error) != 0 && error.code == KIPP_ERROR_RANGE);
    CHECK(kipp_model_eval(model, tokens, KIPP_MODEL_EVAL_LIMIT + 1, spare, vocab, &error) != 0 && error.code == KIPP_ERROR_RANGE);
    kipp_model_kv_pool_stats(model, 0, &after);
    CHECK(after.free_blocks == after.total_blocks && model->session_count == 0);
    CHECK(kipp_model_close(model, &error) == 0);
    /* the short ways to open: a path alone, a path and a pool */
    CHECK(strcmp(kipp_backend_name(KIPP_PATH_CPU_FP32), kipp_path_name(KIPP_PATH_CPU_FP32)) == 0);
    CHECK(kipp_model_open_pooled(folder, KIPP_PATH_CPU_FP32, 0, &model, &error) != 0 && error.code == KIPP_ERROR_ARGUMENT);
    CHECK(kipp_model_open_pooled(folder, KIPP_PATH_CPU_FP32, 7, &model, &error) == 0);
    if (model != NULL) {
        kipp_model_kv_pool_stats(model, 0, &after);
        CHECK(after.total_blocks == 7 && kipp_model_get_info(model, &info) == 0 && info.path == KIPP_PATH_CPU_FP32);
        CHECK(kipp_model_eval(model, tokens, n, spare, vocab, &error) == 0 && same_bits(spare, whole + (size_t)(n - 1) * vocab, vocab));
        CHECK(kipp_model_close(model, &error) == 0);
    }
    CHECK(kipp_model_open_backend(folder, KIPP_PATH_CPU_FP32, &model, &error) == 0);
    if (model != NULL) {
        CHECK(kipp_model_get_info(model, &info) == 0 && info.path == KIPP_PATH_CPU_FP32 && info.page_tokens == 16);
        CHECK(kipp_model_close(model, &error) == 0);
    }
    free(whole);
    free(cut);
    free(spare);
    /* a folder that is not there, and one without weights */
    CHECK(kipp_model_open_ex("/nonexistent/kipp", &config, &model, &error) != 0 && error.code == KIPP_ERROR_IO && model == NULL);
}

static void test_sampler(void) {
    kipp_error error;
    uint32_t token = 99;
    uint64_t state = 1;
    float logits[5] = {0.5f, 2.0f, 2.0f, -1.0f, 1.5f};
    CHECK(kipp_sample(logits, 5, 0.0f, 1.0f, NULL, &token, &error) == 0 && token == 1); /* greedy never touches the generator */
    CHECK(kipp_sample(logits, 5, 1.0f, 1.0f, NULL, &token, &error) != 0 && error.code == KIPP_ERROR_ARGUMENT);
    CHECK(kipp_sample(logits, 5, 1.0f, 1.5f, &state, &token, &error) != 0);
    int seen[5] = {0};
    for (int i = 0; i < 2000; ++i) {
        CHECK(kipp_sample(logits, 5, 1.0f, 1.0f, &state, &token, &error) == 0 && token < 5);
        ++seen[token];
    }
    CHECK(seen[1] > seen[0] && seen[2] > seen[3] && seen[3] > 0);
    kipp_sample_params params;
    memset(&params, 0, sizeof(params));
    params.temperature = 1.0f;
    params.top_p = 1.0f;
    params.top_k = 1;
    for (int i = 0; i < 50; ++i) CHECK(kipp_sample_ex(logits, 5, &params, &state, &token, &error) == 0 && token == 1); /* top_k = 1 is the argmax */
    uint32_t recent[3] = {1, 1, 7}, bias_tokens[2] = {3, 9};
    float bias_values[2] = {10.0f, 1.0f};
    params.temperature = 0.0f;
    params.repetition_penalty = 2.0f;
    params.recent_tokens = recent;
    params.recent_count = 3;
    CHECK(kipp_sample_ex(logits, 5, &params, NULL, &token, &error) == 0 && token == 2); /* token 1 halved, tokens beyond the vocabulary ignored */
    params.logit_bias_tokens = bias_tokens;
    params.logit_bias_values = bias_values;
    params.logit_bias_count = 2;
    CHECK(kipp_sample_ex(logits, 5, &params, NULL, &token, &error) == 0 && token == 3);
    CHECK(strcmp(kipp_error_code_name(KIPP_ERROR_RANGE), "range") == 0 && strcmp(kipp_path_name(KIPP_PATH_CPU_FP32), "cpu-fp32") == 0);
}

/* vectors of the reference's own unit tests for the scalar operations (/root/reference/tests/kipp_test.c:88-175) */
static void test_scalar_operations(void) {
    float x[2] = {3.0f, 4.0f}, w[2] = {1.0f, 1.0f}, out[2];
    kipp_test_rms_norm(x, w, out, 2, 0.0f);
    CHECK(fabsf(out[0] - 3.0f / sqrtf(12.5f)) < 1e-6f && fabsf(out[1] - 4.0f / sqrtf(12.5f)) < 1e-6f);
    float matrix[6] = {1, 2, 3, -1, 0.5f, 0}, input[3] = {2, -1, 0.5f}, product[2];
    kipp_test_matvec(matrix, input, product, 2, 3);
    CHECK(product[0] == 1.5f && product[1] == -2.5f);
    float head[4] = {1, 2, 3, 4};
    kipp_test_rope(head, 4, 1, 10000.0f);
    float c = cosf(1.0f), s = sinf(1.0f), c2 = cosf(0.01f), s2 = sinf(0.01f);
    CHECK(fabsf(head[0] - (c - 3 * s)) < 1e-6f && fabsf(head[1] - (2 * c2 - 4 * s2)) < 1e-6f && fabsf(head[2] - (3 * c + s)) < 1e-6f &&
          fabsf(head[3] - (4 * c2 + 2 * s2)) < 1e-6f);
    float values[3] = {1, 2, 3};
    kipp_test_softmax(values, 3);
    CHECK(fabsf(values[0] + values[1] + values[2] - 1.0f) < 1e-6f && values[0] < values[1] && values[1] < values[2]);
    CHECK(kipp_test_silu(0.0f) == 0.0f && fabsf(kipp_test_silu(1.0f) - 0.7310586f) < 1e-6f);
    /* two tokens, 32 query heads over 8 key/value heads, q = k = 0, v0 = 1, v1 = 3: 1 then 2 */
    enum { T = 2, NQ = 32, NKV = 8, D = 128 };
    static float q[T * NQ * D], k[T * NKV * D], v[T * NKV * D], o[T * NQ * D];
    for (int i = 0; i < NKV * D; ++i) {
        v[i] = 1.0f;
        v[NKV * D + i] = 3.0f;
    }
    kipp_test_causal_gqa(q, k, v, o, T, NQ, NKV, D);
    CHECK(o[0] == 1.0f && o[NQ * D - 1] == 1.0f && o[NQ * D] == 2.0f && o[2 * NQ * D - 1] == 2.0f);
}

/* The scheduler over few pages: random requests, some sharing a beginning, cancellations and one failed step.  Greedy
 * output must not depend on the company: each request is run again alone and gives the same tokens. */
static void test_scheduler(const char *folder) {
    kipp_model *model = NULL;
    kipp_error error;
    kipp_model_open_config config;
    memset(&config, 0, sizeof(config));
    config.path = KIPP_PATH_CPU_FP32;
    config.page_tokens = 4;
    config.kv_pool_pages = 24;
    config.max_sessions = 4;
    config.share_prefixes = 1;
    if (kipp_model_open_ex(folder, &config, &model, &error) != 0) {
        CHECK(0);
        return;
    }
    kipp_model_info info;
    kipp_model_get_info(model, &info);
    enum { REQUESTS = 14, LONGEST = 40 };
    static uint32_t prompts[REQUESTS][LONGEST], outputs[REQUESTS][16];
    size_t lengths[REQUESTS], output_counts[REQUESTS];
    uint32_t budgets[REQUESTS];
    kipp_finish_reason reasons[REQUESTS];
    kipp_scheduler *scheduler = NULL;
    kipp_scheduler_config sconfig = {11, 6, 0, 1};
    CHECK(kipp_scheduler_create(model, &sconfig, &scheduler, &error) == 0);
    kipp_request request;
    for (int r = 0; r < REQUESTS; ++r) {
        lengths[r] = 3 + rnd(LONGEST - 3);
        for (size_t i = 0; i < lengths[r]; ++i) prompts[r][i] = r % 3 == 2 && i < 17 ? prompts[r - 1][i] : rnd(info.vocab_size);
        if (r % 3 == 2 && lengths[r - 1] < 17) lengths[r] = lengths[r - 1]; /* the copied part must exist */
        budgets[r] = 1 + rnd(12);
    }
    int added = 0, steps = 0;
    while (added < REQUESTS || !kipp_scheduler_idle(scheduler)) {
        for (int k = rnd(3); k > 0 && added < REQUESTS; --k, ++added) {
            memset(&request, 0, sizeof(request));
            request.id = 100 + added;
            request.prompt = prompts[added];
            request.prompt_count = lengths[added];
            request.max_new_tokens = budgets[added];
            request.params.repetition_penalty = 1.0f;
            CHECK(kipp_scheduler_add(scheduler, &request, &error) == 0);
            CHECK(kipp_scheduler_add(scheduler, &request, &error) != 0); /* the id is known */
        }
        if (steps == 9) kipp_test_fail_forward_after(model, 0);
        if (steps == 5) kipp_scheduler_cancel(scheduler, 100, &error);
        kipp_produced produced[8];
        size_t count = 0;
        CHECK(kipp_scheduler_step(scheduler, produced, 8, &count, &error) == 0 && count <= 4);
        CHECK(kipp_cache_check(&model->cache, model->sessions, model->session_count, &error) == 0);
        if (++steps > 2000) {
            CHECK(0);
            break;
        }
    }
    kipp_scheduler_stats stats;
    CHECK(kipp_scheduler_get_stats(scheduler, &stats) == 0 && stats.requests == REQUESTS && stats.failed_steps == 1 && stats.failed >= 1);
    for (int r = 0; r < REQUESTS; ++r) {
        kipp_result result;
        CHECK(kipp_scheduler_result(scheduler, 100 + r, &result) == 0 && result.reason != KIPP_FINISH_NONE);
        reasons[r] = result.reason;
        output_counts[r] = result.output_count;
        CHECK(result.output_count <= budgets[r]);
        memcpy(outputs[r], result.output, result.output_count * sizeof(uint32_t));
        if (result.reason == KIPP_FINISH_LENGTH) CHECK(result.output_count == budgets[r] && kipp_scheduler_last_logits(scheduler, 100 + r) != NULL);
        if (result.reason == KIPP_FINISH_FAILED) CHECK(result.error[0] != '\0');
        CHECK(kipp_scheduler_collect(scheduler, 100 + r) == 0 && kipp_scheduler_result(scheduler, 100 + r, &result) != 0);
    }
    kipp_kv_pool_stats_public pool;
    kipp_model_kv_pool_stats(model, 0, &pool);
    CHECK(pool.free_blocks == pool.total_blocks);
    /* alone, one after the other: the same tokens as far as the first run got */
    for (int r = 0; r < REQUESTS; ++r) {
        memset(&request, 0, sizeof(request));
        request.id = r;
        request.prompt = prompts[r];
        request.prompt_count = lengths[r];
        request.max_new_tokens = budgets[r];
        request.params.repetition_penalty = 1.0f;
        CHECK(kipp_scheduler_add(scheduler, &request, &error) == 0);
        while (!kipp_scheduler_idle(scheduler)) {
            kipp_produced produced[4];
            size_t count;
            CHECK(kipp_scheduler_step(scheduler, produced, 4, &count, &error) == 0);
        }
        kipp_result result;
        CHECK(kipp_scheduler_result(scheduler, r, &result) == 0 && result.reason == KIPP_FINISH_LENGTH && result.output_count >= output_counts[r]);
        CHECK(memcmp(result.output, outputs[r], output_counts[r] * sizeof(uint32_t)) == 0);
        if (reasons[r] == KIPP_FINISH_LENGTH) CHECK(result.output_count == output_counts[r]);
    }
    /* destroyed with work in hand: what runs is cancelled and its pages come back */
    memset(&request, 0, sizeof(request));
    request.id = 999;
    request.prompt = prompts[0];
    request.prompt_count = lengths[0];
    request.max_new_tokens = 5;
    request.params.repetition_penalty = 1.0f;
    CHECK(kipp_scheduler_add(scheduler, &request, &error) == 0);
    kipp_produced one[4];
    size_t count;
    CHECK(kipp_scheduler_step(scheduler, one, 4, &count, &error) == 0);
    kipp_scheduler_destroy(scheduler);
    kipp_model_kv_pool_stats(model, 0, &pool);
    CHECK(pool.free_blocks == pool.total_blocks);
    CHECK(kipp_model_close(model, &error) == 0);
}

/* ------------------------------------------------------------------------------------------------------------------
 * A toy architecture that exists in this file alone: every second layer mixes by the mean of what its session has seen
 * so far, which it keeps as state of fixed size (no pages).  Registered from here, built, loaded and stepped by the
 * library as it is: nothing in the library knows it. */
typedef struct {
    uint32_t hidden;
    char prefix[KIPP_NAME];
} toy_mean_spec;

typedef struct {
    toy_mean_spec spec;
    kipp_runtime *rt;
    kipp_weight w;
} toy_mean_part;

static int toy_mean_params(const void *spec_, kipp_param_list *out, kipp_error *error) {
    const toy_mean_spec *spec = spec_;
    return kipp_params_add(out, spec->prefix, "w.weight", 2, spec->hidden, spec->hidden, error);
}

static void *toy_mean_create(const void *spec, struct kipp_runtime *rt, kipp_error *error) {
    toy_mean_part *part = calloc(1, sizeof(*part));
    if (part == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    part->spec = *(const toy_mean_spec *)spec;
    part->rt = rt;
    return part;
}

static int toy_mean_load(void *part_, const kipp_tensor_file *tensors, void *context, kipp_error *error) {
    toy_mean_part *part = part_;
    char name[KIPP_NAME + 32];
    (void)context;
    snprintf(name, sizeof(name), "%sw.weight", part->spec.prefix);
    const kipp_tensor *w = kipp_tensors_find(tensors, name);
    if (w == NULL) return kipp_fail(error, KIPP_ERROR_FORMAT, "missing tensor '%s'", name);
    return part->rt->place_matrix(part->rt, &w, 1, KIPP_LAYOUT_ROWS, &part->w, error);
}

static void toy_mean_destroy(void *part_) {
    toy_mean_part *part = part_;
    part->rt->free_weight(part->rt, &part->w);
    free(part);
}

static void toy_mean_cache_need(const void *spec, kipp_kv_need *out) {
    (void)spec;
    memset(out, 0, sizeof(*out)); /* no pages */
}

static void toy_mean_state_need(const void *spec_, kipp_state_need *out) {
    const toy_mean_spec *spec = spec_;
    *out = (kipp_state_need){true, ((uint64_t)spec->hidden + 1) * sizeof(float)}; /* the sum of its inputs, and their number */
}

/* delta[t] = W mean(x[0..t] of the session); the sums live in the session's slot and go on from step to step */
static int toy_mean_forward(void *part_, const kipp_rows *x, kipp_batch *batch, const kipp_cache_view *cache, void *state, kipp_delta *out,
                            kipp_error *error) {
    toy_mean_part *part = part_;
    kipp_runtime *rt = part->rt;
    const uint32_t h = part->spec.hidden;
    (void)cache;
    if (!rt->on_host || state == NULL) return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "the toy mixer computes on the host path only");
    float *mean = kipp_scratch(rt, (size_t)batch->n_tokens * h * sizeof(float), error);
    if (mean == NULL) return -1;
    const float *rows = x->data;
    for (uint32_t i = 0; i < batch->n_seqs; ++i) {
        float *slot = (float *)state + (size_t)batch->slots[i] * (h + 1);
        for (int32_t t = batch->q_start[i]; t < batch->q_start[i] + batch->q_len[i]; ++t) {
            slot[h] += 1.0f;
            for (uint32_t c = 0; c < h; ++c) {
                slot[c] += rows[(size_t)t * h + c];
                mean[(size_t)t * h + c] = slot[c] / slot[h];
            }
        }
    }
    return rt->linear(rt, &(kipp_rows){mean, NULL, 0, 0.0f, false}, &part->w, batch->n_tokens, 1, out, error);
}

static const kipp_mixer_fn toy_mean_fn = {toy_mean_cache_need, toy_mean_state_need, toy_mean_forward, false};
static const kipp_part_kind toy_mean_kind = {"mixer", "toy_mean", sizeof(toy_mean_spec), toy_mean_params, toy_mean_create, toy_mean_load,
                                             toy_mean_destroy, &toy_mean_fn};

static uint32_t toy_uint(const kj_doc *doc, const char *key) {
    const kj_node *v = kj_get(doc, kj_root(doc), key);
    return v != NULL && v->type == KJ_NUMBER && v->is_integer && v->integer > 0 ? (uint32_t)v->integer : 0;
}

/* config.json of "ToyMeanForCausalLM": even layers attend (two heads, rotary), odd layers take the toy mixer */
static int parse_toy(const kj_doc *doc, kipp_model_spec *spec, kipp_error *error) {
    uint32_t vocab = toy_uint(doc, "vocab_size"), hidden = toy_uint(doc, "hidden_size"), inner = toy_uint(doc, "intermediate_size"),
             layers = toy_uint(doc, "num_hidden_layers"), positions = toy_uint(doc, "max_position_embeddings");
    if (vocab == 0 || hidden == 0 || inner == 0 || layers == 0 || positions == 0 || hidden % 2 != 0)
        return kipp_fail(error, KIPP_ERROR_FORMAT, "config.json of the toy architecture lacks a size");
    spec->hidden = hidden;
    spec->vocab = vocab;
    spec->max_position = positions;
    spec->embedding = (kipp_embedding_spec){vocab, hidden, "model.embed_tokens."};
    spec->head = (kipp_head_spec){vocab, hidden, true, "lm_head."};
    spec->layers = calloc(layers, sizeof(kipp_layer_spec));
    spec->order = calloc(layers, sizeof(kipp_layer_run));
    kipp_rms_norm_spec *final_norm = calloc(1, sizeof(kipp_rms_norm_spec));
    if (spec->layers == NULL || spec->order == NULL || final_norm == NULL) {
        free(final_norm);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    }
    spec->layer_count = spec->run_count = layers;
    *final_norm = (kipp_rms_norm_spec){hidden, 1e-5f, "model.norm."};
    spec->final_norm = final_norm;
    snprintf(spec->final_norm_kind, sizeof(spec->final_norm_kind), "rms_norm");
    for (uint32_t l = 0; l < layers; ++l) {
        kipp_layer_spec *layer = &spec->layers[l];
        kipp_rms_norm_spec norm = {hidden, 1e-5f, ""};
        kipp_gated_mlp_spec mlp = {hidden, inner, ""};
        snprintf(layer->block, sizeof(layer->block), "pre_norm");
        layer->hidden = hidden;
        snprintf(norm.prefix, sizeof(norm.prefix), "model.layers.%u.input_layernorm.", l);
        if (kipp_spec_add_role(layer, "mixer_norm", "norm", "rms_norm", &norm, sizeof(norm), error) != 0) return -1;
        if (l % 2 == 1) {
            toy_mean_spec toy = {hidden, ""};
            snprintf(toy.prefix, sizeof(toy.prefix), "model.layers.%u.mixer.", l);
            if (kipp_spec_add_role(layer, "mixer", "mixer", "toy_mean", &toy, sizeof(toy), error) != 0) return -1;
        } else {
            kipp_attention_spec attn;
            memset(&attn, 0, sizeof(attn));
            attn.hidden = hidden;
            attn.n_heads = 2;
            attn.n_kv_heads = 1;
            attn.head_dim = hidden / 2;
            snprintf(attn.position_kind, sizeof(attn.position_kind), "rope");
            attn.rope = (kipp_rope_spec){hidden / 2, 10000.0, hidden / 2, 0};
            snprintf(attn.prefix, sizeof(attn.prefix), "model.layers.%u.self_attn.", l);
            if (kipp_spec_add_role(layer, "mixer", "mixer", "attention", &attn, sizeof(attn), error) != 0) return -1;
        }
        snprintf(norm.prefix, sizeof(norm.prefix), "model.layers.%u.post_attention_layernorm.", l);
        if (kipp_spec_add_role(layer, "ffn_norm", "norm", "rms_norm", &norm, sizeof(norm), error) != 0) return -1;
        snprintf(mlp.prefix, sizeof(mlp.prefix), "model.layers.%u.mlp.", l);
        if (kipp_spec_add_role(layer, "ffn", "feed_forward", "gated_mlp", &mlp, sizeof(mlp), error) != 0) return -1;
        spec->order[l] = (kipp_layer_run){l, -1};
    }
    spec->info.block_count = layers;
    spec->info.embedding_length = hidden;
    spec->info.vocab_size = vocab;
    spec->info.context_length = positions;
    spec->info.tied_embeddings = true;
    return 0;
}

/* The toy model's folder (written by the caller: config.json with architectures ["ToyMeanForCausalLM"], tensors by the names
 * the parts declare): whole prompts, portions beside another session's, and a slot taken again all give the same bits; what
 * the state cannot do is refused. */
static void test_toy_architecture(const char *folder) {
    kipp_model *model = NULL;
    kipp_error error;
    kipp_model_open_config config;
    memset(&config, 0, sizeof(config));
    config.path = KIPP_PATH_CPU_FP32;
    config.page_tokens = 4;
    config.kv_pool_pages = 24;
    config.max_sessions = 2;
    config.share_prefixes = 1; /* asked for, and switched off by the model itself: state cannot be adopted */
    CHECK(kipp_model_open_ex(folder, &config, &model, &error) != 0 && error.code == KIPP_ERROR_UNSUPPORTED); /* nobody knows the architecture yet */
    CHECK(kipp_register_part(&toy_mean_kind) == 0 && kipp_register_architecture("ToyMeanForCausalLM", parse_toy) == 0);
    if (kipp_model_open_ex(folder, &config, &model, &error) != 0) {
        fprintf(stderr, "cannot open the toy model %s: %s\n", folder, error.message);
        CHECK(0);
        return;
    }
    kipp_model_info info;
    CHECK(kipp_model_get_info(model, &info) == 0 && info.cache_groups == 1 && strcmp(info.architecture, "ToyMeanForCausalLM") == 0);
    const uint32_t vocab = info.vocab_size, n = 21;
    uint32_t tokens[32], other[32], want[32];
    for (uint32_t i = 0; i < 32; ++i) {
        tokens[i] = rnd(vocab);
        other[i] = rnd(vocab);
        want[i] = i;
    }
    float *whole = malloc((size_t)n * vocab * sizeof(float)), *cut = malloc((size_t)n * vocab * sizeof(float)),
          *spare = malloc((size_t)32 * vocab * sizeof(float));
    kipp_session *a = NULL, *b = NULL, *c = NULL;
    CHECK(kipp_session_create(model, 0, &a, &error) == 0);
    kipp_step_item item = {a, tokens, n, want, n};
    CHECK(kipp_step(model, &item, 1, whole, (size_t)n * vocab, &error) == 0);
    uint32_t matched = 7;
    CHECK(kipp_session_truncate(a, 5, &error) != 0 && error.code == KIPP_ERROR_UNSUPPORTED);                    /* state cannot be rolled back */
    CHECK(kipp_session_match_prefix(a, tokens, n, &matched, &error) != 0 && error.code == KIPP_ERROR_UNSUPPORTED); /* nor adopted */
    kipp_session_destroy(a);
    /* portions of b beside portions of c: each session's sums stay its own */
    CHECK(kipp_session_create(model, 0, &b, &error) == 0 && kipp_session_create(model, 0, &c, &error) == 0);
    static const uint32_t portions[] = {5, 1, 1, 7, 2, 5};
    uint32_t fed = 0, fed_c = 0;
    for (size_t p = 0; p < sizeof(portions) / sizeof(portions[0]); ++p) {
        uint32_t take_c = 1 + rnd(3);
        kipp_step_item items[2] = {{c, other + fed_c, take_c, want, 0}, {b, tokens + fed, portions[p], want, portions[p]}};
        CHECK(kipp_step(model, items, 2, spare, (size_t)32 * vocab, &error) == 0);
        memcpy(cut + (size_t)fed * vocab, spare, (size_t)portions[p] * vocab * sizeof(float));
        fed += portions[p];
        fed_c += take_c;
    }
    CHECK(fed == n && same_bits(whole, cut, (size_t)n * vocab));
    /* the slot that b leaves is c's successor's: it starts from zero again */
    kipp_session_destroy(b);
    CHECK(kipp_session_create(model, 0, &b, &error) == 0);
    item = (kipp_step_item){b, tokens, n, want, n};
    CHECK(kipp_step(model, &item, 1, cut, (size_t)n * vocab, &error) == 0 && same_bits(whole, cut, (size_t)n * vocab));
    /* the mixer does count: the same last token behind another beginning has other logits */
    kipp_session_destroy(b);
    CHECK(kipp_session_create(model, 0, &b, &error) == 0);
    other[n - 1] = tokens[n - 1];
    item = (kipp_step_item){b, other, n, want + n - 1, 1};
    CHECK(kipp_step(model, &item, 1, spare, vocab, &error) == 0 && !same_bits(spare, whole + (size_t)(n - 1) * vocab, vocab));
    kipp_session_destroy(b);
    kipp_session_destroy(c);
    CHECK(kipp_model_close(model, &error) == 0);
    free(whole);
    free(cut);
    free(spare);
}

int main(int argc, char **argv) {
    test_json();
    test_sizes();
    test_pool();
    test_sampler();
    test_scalar_operations();
    int models = argc;
    for (int i = 1; i < argc; ++i) {
        if (strcmp(argv[i], "--toy") == 0 && i + 1 < argc) {
            test_toy_architecture(argv[i + 1]);
            models = i;
        }
    }
    for (int i = 1; i < models; ++i) test_model(argv[i]);
    for (int i = 1; i < models; ++i) test_scheduler(argv[i]);
    if (failures != 0) {
        fprintf(stderr, "%d of %d checks failed\n", failures, checks);
        return 1;
    }
    printf("ok %d\n", checks);
    return 0;
}
