/*
 * kipp_amd: the C interface of the engine, in the manner of the reference's
 * kipp.h (/root/reference/src/kipp.h:99-295): a model opened from a folder
 * (config.json + safetensors), sessions that each hold one timeline of tokens in
 * the paged cache, evaluation of one session, of a batch of sessions, and of a
 * mixed step (portions of prompts beside single tokens, logits at any places),
 * a sampler, and an error record that every call fills on failure.
 *
 * Every function that returns int returns 0 on success and -1 on failure, with
 * the reason in `error` (which may be NULL).  Nothing here is thread-safe
 * beyond "one thread at a time per model".
 *
 * Paths (kipp_path): the GPU in bfloat16 (the kernels serving uses), the GPU
 * in true 32-bit, and a scalar 32-bit path on the host that needs no GPU: the
 * oracle of the other two, block tables and pages included.
 */
#ifndef KIPP_AMD_H
#define KIPP_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KIPP_AMD_VERSION "0.4.0"
#define KIPP_MAX_STOP_TOKENS 8u
#define KIPP_EVAL_BATCH_LIMIT 256u

typedef struct kipp_model kipp_model;
typedef struct kipp_session kipp_session;

typedef enum {
    KIPP_OK = 0,
    KIPP_ERROR_ARGUMENT,
    KIPP_ERROR_IO,
    KIPP_ERROR_FORMAT,
    KIPP_ERROR_UNSUPPORTED,
    KIPP_ERROR_MEMORY,
    KIPP_ERROR_RANGE,
    KIPP_ERROR_INTERNAL
} kipp_error_code;

/* The message is long enough for the one error that lists every missing,
 * unexpected and wrongly shaped tensor of a model folder. */
typedef struct {
    kipp_error_code code;
    char message[2048];
} kipp_error;

typedef enum {
    KIPP_PATH_GPU_BF16 = 0, /* bfloat16 weights and cache, float32 residual stream, norms and softmax */
    KIPP_PATH_GPU_FP32 = 1, /* everything float32 on the GPU, products by plain FMA */
    KIPP_PATH_CPU_FP32 = 2  /* scalar float32 on the host: the oracle */
} kipp_path;

typedef struct {
    kipp_path path;
    uint32_t page_tokens;     /* tokens a page; 0: 16 */
    uint32_t kv_pool_pages;   /* pages of every cache group's pool; 0: one context length of pages */
    uint32_t max_sessions;    /* sessions alive at a time; 0: 64 */
    uint32_t max_step_tokens; /* most tokens one step brings (sizes the workspace); 0: 2048 */
    int share_prefixes;       /* sessions publish full pages when they end; fresh sessions may adopt them */
    int device;               /* GPU ordinal */
    const char *kernel_dir;   /* folder of the built kernel libraries; NULL: $KIPP_AMD_KERNELS, else beside this library */
    const uint32_t *page_order; /* NULL, or kv_pool_pages page ids: the order in which a fresh pool hands out its pages */
    int eager_steps;          /* nonzero: no step is recorded and run again as a graph (gpu-bf16 records its steps of single tokens) */
} kipp_model_open_config;

typedef struct {
    const char *architecture; /* architectures[0] of config.json */
    kipp_path path;
    uint32_t block_count;
    uint32_t embedding_length;
    uint32_t feed_forward_length;
    uint32_t attention_head_count;
    uint32_t attention_head_count_kv;
    uint32_t attention_head_dim;
    uint32_t vocab_size;
    uint32_t context_length;
    float rope_theta;
    float rms_norm_eps;
    int tied_embeddings;
    uint32_t stop_tokens[KIPP_MAX_STOP_TOKENS];
    uint32_t stop_token_count;
    uint32_t page_tokens;
    uint32_t cache_groups;
    uint64_t mapped_bytes; /* bytes of the model files that are mapped */
    uint64_t weight_bytes; /* bytes the weights take where the path computes */
    uint64_t cache_bytes;  /* bytes of all cache pools */
} kipp_model_info;

typedef struct {
    uint32_t capacity;
    uint32_t length;
    uint32_t adopted_tokens;
    uint64_t cache_bytes; /* bytes of the pages it holds, over all groups */
} kipp_session_info;

int kipp_model_open(const char *model_dir, kipp_model **out_model, kipp_error *error);
int kipp_model_open_ex(const char *model_dir, const kipp_model_open_config *config, kipp_model **out_model, kipp_error *error);
/* Every other field as kipp_model_open leaves it, on the given path (/root/reference/src/kipp.h:110-111). */
int kipp_model_open_backend(const char *model_dir, kipp_path path, kipp_model **out_model, kipp_error *error);
/* The same with a pool of `kv_pool_pages` pages (not 0) for every cache group, shared by all sessions, which publish and
 * adopt beginnings (/root/reference/src/kipp.h:112-122). */
int kipp_model_open_pooled(const char *model_dir, kipp_path path, uint32_t kv_pool_pages, kipp_model **out_model, kipp_error *error);
/* Refuses while sessions are alive (/root/reference/src/kipp.c:1340-1344). */
int kipp_model_close(kipp_model *model, kipp_error *error);
int kipp_model_get_info(const kipp_model *model, kipp_model_info *out_info);
int kipp_model_is_stop_token(const kipp_model *model, uint32_t token);
const char *kipp_path_name(kipp_path path);
const char *kipp_backend_name(kipp_path path); /* the reference's name for the same (/root/reference/src/kipp.h:145) */
/* Evaluation without a session of the caller's: up to KIPP_MODEL_EVAL_LIMIT tokens through a session of its own, which
 * is destroyed before the call returns (it needs one free session and the pages for the tokens; where sharing is on its
 * full pages stay published like any ended session's); the logits of the last token, `logits_count` at least the
 * vocabulary (/root/reference/src/kipp.h:159-166). */
#define KIPP_MODEL_EVAL_LIMIT 256u
int kipp_model_eval(kipp_model *model, const uint32_t *tokens, size_t token_count, float *logits, size_t logits_count, kipp_error *error);

/* A session holds up to `capacity` tokens (0: the model's context length). */
int kipp_session_create(kipp_model *model, uint32_t capacity, kipp_session **out_session, kipp_error *error);
/* Publishes its full pages (where sharing is on), gives every page back; the session starts again at length 0. */
int kipp_session_reset(kipp_session *session, kipp_error *error);
/* Keeps the first `length` tokens; never below what was adopted. */
int kipp_session_truncate(kipp_session *session, uint32_t length, kipp_error *error);
void kipp_session_destroy(kipp_session *session);
int kipp_session_get_info(const kipp_session *session, kipp_session_info *out_info);
/* Appends the tokens and writes the logits of the last one ([vocab] floats). */
int kipp_session_eval(kipp_session *session, const uint32_t *tokens, size_t token_count, float *logits, size_t logits_count,
                      kipp_error *error);
/* The logits of the last `rows` tokens, each row the bits that evaluating its token alone gives. */
int kipp_session_eval_n(kipp_session *session, const uint32_t *tokens, size_t token_count, float *logits, uint32_t rows,
                        kipp_error *error);
/* The same rows from one step: within tolerance of eval_n under bfloat16, the same bits on the 32-bit paths. */
int kipp_session_eval_scored(kipp_session *session, const uint32_t *tokens, size_t token_count, float *logits, uint32_t rows,
                             kipp_error *error);
/* On a fresh session: adopt the longest published beginning of `tokens`, whole pages, at most (count - 1) / page. */
int kipp_session_match_prefix(kipp_session *session, const uint32_t *tokens, size_t token_count, uint32_t *matched_tokens,
                              kipp_error *error);

typedef struct {
    uint32_t total_blocks;
    uint32_t free_blocks;
    uint64_t reused_blocks_total;
    uint64_t evicted_blocks_total;
} kipp_kv_pool_stats_public;

/* The pool of cache group `group` (0 for a model with one). */
int kipp_model_kv_pool_stats(const kipp_model *model, uint32_t group, kipp_kv_pool_stats_public *out_stats);

typedef struct {
    kipp_session *session;
    const uint32_t *tokens;
    size_t token_count;
    float *logits; /* at least vocab_size values: the last token's */
} kipp_batch_item;

int kipp_eval_batch(kipp_model *model, kipp_batch_item *items, size_t item_count, kipp_error *error);

/* One entry of a step: a session's next tokens and the places among them whose logits are wanted. */
typedef struct {
    kipp_session *session;
    const uint32_t *tokens;
    size_t token_count;
    const uint32_t *want; /* places 0 .. token_count - 1, in the order their rows are written */
    size_t want_count;    /* may be 0: a portion of a prompt whose logits nobody needs */
} kipp_step_item;

/*
 * THE step function: all items are one batch, portions of prompts beside single
 * tokens, cut anywhere; it runs only the tokens it is given, from the cache
 * that earlier steps left, and writes float32 logits [sum of want_count][vocab]
 * in the order of the items and of their `want`.  All or nothing: on failure
 * no session has changed and every page claimed for the step is back.
 */
int kipp_step(kipp_model *model, const kipp_step_item *items, size_t item_count, float *logits, size_t logits_capacity,
              kipp_error *error);
/* The same step, answered with the index of the largest logit at every wanted place (the lowest index among equals,
 * /root/reference/src/kipp.c:3459-3464), found where the path computes: greedy decoding then reads back one number a
 * place instead of a row of logits. */
int kipp_step_argmax(kipp_model *model, const kipp_step_item *items, size_t item_count, uint32_t *tokens, size_t token_capacity,
                     kipp_error *error);

int kipp_sample(const float *logits, size_t logits_count, float temperature, float top_p, uint64_t *rng_state, uint32_t *out_token,
                kipp_error *error);

typedef struct {
    float temperature;
    float top_p;              /* nucleus mass in (0, 1]; 1 disables */
    uint32_t top_k;           /* keep k highest; 0 disables */
    float min_p;              /* keep prob >= min_p * max_prob; 0 disables */
    float frequency_penalty;  /* logit -= count * penalty */
    float presence_penalty;   /* logit -= penalty if present */
    float repetition_penalty; /* divide positive / multiply negative logits; 0 or 1 disables */
    const uint32_t *recent_tokens;
    size_t recent_count;
    const uint32_t *logit_bias_tokens;
    const float *logit_bias_values;
    size_t logit_bias_count;
} kipp_sample_params;

int kipp_sample_ex(const float *logits, size_t logits_count, const kipp_sample_params *params, uint64_t *rng_state,
                   uint32_t *out_token, kipp_error *error);

/* kipp_step with one token for every wanted place, chosen where the path computes, with the meaning of kipp_sample_ex:
 * `params` has one entry a wanted place, in the order of the items and their places (bias and recent tokens included:
 * they change the row where it lies, in kipp_sample_ex's order and with its float operations), `uniform` for each the
 * one draw in [0, 1) that kipp_sample_ex would take from its generator (not looked at where temperature <= 0: the
 * largest logit).  Only a number a row comes back.  KIPP_ERROR_UNSUPPORTED on a path that has no sampler of its own
 * (the scalar one: take kipp_step and kipp_sample_ex). */
int kipp_step_sample(kipp_model *model, const kipp_step_item *items, size_t item_count, const kipp_sample_params *params,
                     const double *uniform, uint32_t *tokens, size_t token_capacity, kipp_error *error);
/* The same, and the wanted rows of logits as the model left them (before a bias or a penalty changed them) as well. */
int kipp_step_sample_logits(kipp_model *model, const kipp_step_item *items, size_t item_count, const kipp_sample_params *params,
                            const double *uniform, uint32_t *tokens, size_t token_capacity, float *logits, size_t logits_capacity,
                            kipp_error *error);
/* kipp_step with, for every wanted place, what its row of logits gives for a target token: nll[w] = -log softmax(row)[targets[w]]
 * (the row's maximum in float32, the exponentials and their sum in float64: what a perplexity run adds up,
 * /root/reference/src/kipp_cli.c:759-778), computed where the path computes; `targets` has one token a wanted place, in the
 * order of the items and their places.  Only a number a row comes back. */
int kipp_step_nll(kipp_model *model, const kipp_step_item *items, size_t item_count, const uint32_t *targets, double *nll, size_t nll_capacity,
                  kipp_error *error);
/* The next draw of a generator, as kipp_sample_ex takes it (/root/reference/src/kipp.c:3322-3333): in [0, 1); the state must not be 0. */
double kipp_rng_uniform(uint64_t *rng_state);

/*
 * The scheduler above the step function: it admits requests, cuts prompts into
 * portions under a token budget, decodes, finishes and frees (the reference's
 * server loop lifted out of its HTTP code, /root/reference/src/kipp_server.c:1623-1893
 * admission, :1900-2125 stepping).  Waiting requests are admitted strictly in
 * arrival order; pages are reserved at admission, so a running request never
 * fails for pages and a short pool delays requests, in order; one step is one
 * call of kipp_step with every decoding request's next token first and portions
 * of prompts in arrival order behind them; a step that fails fails the requests
 * that had tokens in it, and the queue moves on.
 */
typedef struct kipp_scheduler kipp_scheduler;

typedef struct {
    uint32_t max_step_tokens; /* token budget of one step; 0: 2048 */
    uint32_t prefill_chunk;   /* largest portion of a prompt in one step; 0: 512 */
    uint32_t max_running;     /* requests running at a time; 0: as many as the model has session slots */
    int keep_last_logits;     /* keep, for every request, the logits row its last token was chosen from (kipp_scheduler_last_logits) */
} kipp_scheduler_config;

typedef struct {
    uint64_t id;
    const uint32_t *prompt;
    size_t prompt_count;
    uint32_t max_new_tokens;
    kipp_sample_params params; /* recent_tokens is ignored: the scheduler keeps the last 64 generated tokens itself */
    uint64_t seed;             /* of the request's own generator; 0 is taken as 1 */
    uint32_t stop_tokens[KIPP_MAX_STOP_TOKENS];
    uint32_t stop_token_count;
} kipp_request;

typedef enum {
    KIPP_FINISH_NONE = 0,
    KIPP_FINISH_LENGTH,    /* max_new_tokens reached */
    KIPP_FINISH_STOP,      /* a stop token was chosen: neither kept nor fed back */
    KIPP_FINISH_CANCELLED,
    KIPP_FINISH_FAILED     /* a step it had tokens in failed */
} kipp_finish_reason;

typedef struct {
    uint64_t id;
    uint32_t token;
} kipp_produced;

typedef struct {
    uint64_t id;
    kipp_finish_reason reason; /* KIPP_FINISH_NONE: still waiting or running */
    const uint32_t *output;    /* what it has generated so far; valid until the next call on the scheduler */
    size_t output_count;
    const char *error;         /* what the failed step said, else "" */
} kipp_result;

typedef struct {
    uint64_t requests, refused, finished, failed, failed_steps;
    uint64_t prompt_tokens, generated_tokens, prefix_tokens_reused, steps, waits_for_pages, waits_for_prefix;
    /* sums of seconds with their counts, as the reference's server exports them (/root/reference/src/kipp_server.c:71-84) */
    double queue_wait_seconds_sum;
    uint64_t queue_wait_count;
    double ttft_seconds_sum;
    uint64_t ttft_count;
    double decode_seconds_sum;
} kipp_scheduler_stats;

int kipp_scheduler_create(kipp_model *model, const kipp_scheduler_config *config, kipp_scheduler **out_scheduler, kipp_error *error);
/* Cancels what is waiting or running, then frees. */
void kipp_scheduler_destroy(kipp_scheduler *scheduler);
/* Refused (-1) if it can never run: empty prompt, a token outside the vocabulary, prompt + max_new_tokens beyond the
 * model's positions or the pool, an id that is still known. */
int kipp_scheduler_add(kipp_scheduler *scheduler, const kipp_request *request, kipp_error *error);
int kipp_scheduler_cancel(kipp_scheduler *scheduler, uint64_t id, kipp_error *error);
/* Admit, run one batch, choose tokens.  Writes the (request, token) pairs that became known, at most `capacity`. */
int kipp_scheduler_step(kipp_scheduler *scheduler, kipp_produced *out, size_t capacity, size_t *out_count, kipp_error *error);
int kipp_scheduler_idle(const kipp_scheduler *scheduler);
/* A request by its id, whatever its state; -1 if the id is not known. */
int kipp_scheduler_result(const kipp_scheduler *scheduler, uint64_t id, kipp_result *out_result);
/* Forget a finished request (its id may come again). */
int kipp_scheduler_collect(kipp_scheduler *scheduler, uint64_t id);
int kipp_scheduler_get_stats(const kipp_scheduler *scheduler, kipp_scheduler_stats *out_stats);
/* The logits row the last token of request `id` was chosen from (vocab floats), or NULL: for a caller that prints them. */
const float *kipp_scheduler_last_logits(const kipp_scheduler *scheduler, uint64_t id);

const char *kipp_error_code_name(kipp_error_code code);

/*
 * Hooks for tests (always compiled; the reference guards its own with
 * KIPP_TESTING, /root/reference/src/kipp.h:299-340): each scalar operation of
 * the host path alone, and ways to disturb a model's cache so that a test can
 * show that the comparison with the plain implementation would notice.
 */
float kipp_test_bf16_to_float(uint16_t value);
uint16_t kipp_test_float_to_bf16(float value);
int kipp_test_checked_add_size(size_t left, size_t right, size_t *result);
int kipp_test_checked_multiply_size(size_t left, size_t right, size_t *result);
void kipp_test_rms_norm(const float *input, const float *weight, float *output, size_t length, float epsilon);
void kipp_test_matvec(const float *weight, const float *input, float *output, size_t rows, size_t columns);
void kipp_test_matvec_bf16(const uint16_t *weight, const float *input, float *output, size_t rows, size_t columns);
void kipp_test_rope(float *head, size_t head_dim, uint32_t position, float theta);
void kipp_test_softmax(float *values, size_t count);
float kipp_test_silu(float value);
void kipp_test_causal_gqa(const float *query, const float *key, const float *value, float *output, size_t token_count,
                          size_t query_head_count, size_t kv_head_count, size_t head_dim);
uint64_t kipp_test_chain_hash(uint64_t parent, const uint32_t *tokens, size_t count);
/* Reverse the block table of a session that holds pages (contents move with it): results must not change. */
int kipp_test_scramble_session_kv(kipp_session *session, kipp_error *error);
/* The model's next `skip` forward passes run; the one after them fails with an error of its own.  skip < 0: never. */
void kipp_test_fail_forward_after(kipp_model *model, int skip);
/* Pages a session holds in a group, in table order; returns how many were written (at most `capacity`). */
size_t kipp_test_session_pages(const kipp_session *session, uint32_t group, int32_t *out_pages, size_t capacity);

#ifdef __cplusplus
}
#endif

#endif
