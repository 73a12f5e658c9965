/*
 * The command line of the C host, in the manner of the reference's `kipp`
 * (/root/reference/src/kipp_cli.c:571-610 options, :1057-1067 capacity, :1145-1217 output):
 * evaluate a prompt, generate --decode tokens through the scheduler, print the
 * final top-N logits and one KIPP_METRIC line.  The prompt is token ids (this
 * engine has no tokenizer).
 *
 *   kipp --model DIR --tokens 5,17,3 --decode 16 [--path gpu-bf16|gpu-fp32|cpu-fp32]
 *   kipp --model DIR --ppl tokens.u32 --ppl-window 512        perplexity over a token file (:646-801)
 */
#include <errno.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "kipp_amd.h"

static void usage(FILE *out) {
    fputs("usage: kipp --model DIR (--tokens 5,17,3 | --tokens-file F.u32 | --ppl F.u32) [options]\n"
          "  --path gpu-bf16|gpu-fp32|cpu-fp32   execution path, never a fallback (default gpu-bf16)\n"
          "  --decode N          tokens to generate (default 0)\n"
          "  --temperature F     0 = greedy argmax (default)\n"
          "  --top-p F           nucleus mass, 0 < F <= 1 (default 1)\n"
          "  --top-k N           keep N highest logits (0 = off)\n"
          "  --min-p F           min prob vs top, 0 <= F <= 1 (0 = off)\n"
          "  --seed N            nonzero sampling seed (default 1)\n"
          "  --top N             final top-N logits to print, 1..100 (default 10)\n"
          "  --stop-token N      token that ends decoding (may repeat; default: eos_token_id of config.json)\n"
          "  --max-context N     most tokens the session may hold (default: the model's positions)\n"
          "  --page N            tokens per cache page (default 16)\n"
          "  --kv-pages N        pages in the pool (default: enough for this run)\n"
          "  --kv-mib F          size of the pool in MiB instead\n"
          "  --prefill-chunk N   largest portion of a prompt in one step (default 512)\n"
          "  --max-step-tokens N token budget of one step (default 2048)\n"
          "  --ppl FILE          perplexity over a file of little-endian uint32 tokens\n"
          "  --ppl-window N      tokens of one window; each starts from an empty context (default 2048)\n"
          "  --ppl-limit N       score at most N tokens of the file (0 = all)\n"
          "  --kernels DIR       folder of the built kernel libraries\n",
          out);
}

static double seconds(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

static int parse_tokens(const char *text, uint32_t **out, size_t *count) {
    size_t capacity = 64, n = 0;
    uint32_t *tokens = malloc(capacity * sizeof(uint32_t));
    if (tokens == NULL) return -1;
    const char *at = text;
    while (*at != '\0') {
        while (*at == ',' || *at == ' ') ++at;
        if (*at == '\0') break;
        char *end;
        errno = 0;
        unsigned long value = strtoul(at, &end, 10);
        if (end == at || errno != 0 || value > 0xfffffffful) {
            free(tokens);
            return -1;
        }
        if (n == capacity) {
            uint32_t *grown = realloc(tokens, (capacity *= 2) * sizeof(uint32_t));
            if (grown == NULL) {
                free(tokens);
                return -1;
            }
            tokens = grown;
        }
        tokens[n++] = (uint32_t)value;
        at = end;
    }
    *out = tokens;
    *count = n;
    return 0;
}

static int read_token_file(const char *path, uint32_t **out, size_t *count) {
    FILE *f = fopen(path, "rb");
    if (f == NULL) return -1;
    fseek(f, 0, SEEK_END);
    long size = ftell(f);
    fseek(f, 0, SEEK_SET);
    if (size < 0 || size % 4 != 0) {
        fclose(f);
        return -1;
    }
    unsigned char *raw = malloc(size ? (size_t)size : 1);
    uint32_t *tokens = malloc(size ? (size_t)size : 4);
    if (raw == NULL || tokens == NULL || fread(raw, 1, (size_t)size, f) != (size_t)size) {
        free(raw);
        free(tokens);
        fclose(f);
        return -1;
    }
    fclose(f);
    for (long i = 0; i < size / 4; ++i)
        tokens[i] = (uint32_t)raw[4 * i] | (uint32_t)raw[4 * i + 1] << 8 | (uint32_t)raw[4 * i + 2] << 16 | (uint32_t)raw[4 * i + 3] << 24; /* little-endian */
    free(raw);
    *out = tokens;
    *count = (size_t)(size / 4);
    return 0;
}

/* Perplexity: windows of `window` tokens that do not overlap, each from an empty session, no burn-in; a window of W tokens
 * scores its W - 1 targets.  Portions of `chunk` tokens, every row scored in the step that makes it (kipp_step_nll); sums in double. */
static int run_perplexity(kipp_model *model, const kipp_model_info *info, const uint32_t *stream, size_t token_count, size_t window,
                          size_t chunk) {
    int status = 1;
    kipp_error error;
    kipp_session *session = NULL;
    (void)info;
    double *nll_of = malloc(chunk * sizeof(double));
    uint32_t *want = malloc(chunk * sizeof(uint32_t));
    if (nll_of == NULL || want == NULL) {
        fprintf(stderr, "kipp: ppl: unable to allocate a portion's results\n");
        free(nll_of);
        free(want);
        return 1;
    }
    for (size_t r = 0; r < chunk; ++r) want[r] = (uint32_t)r;
    if (kipp_session_create(model, (uint32_t)window, &session, &error) != 0) {
        fprintf(stderr, "kipp: ppl: session: %s\n", error.message);
        goto done;
    }
    const size_t windows = (token_count + window - 1) / window;
    size_t scored = 0;
    double nll = 0.0;
    const double started = seconds();
    for (size_t w = 0; w < windows; ++w) {
        const uint32_t *tokens = stream + w * window;
        const size_t length = token_count - w * window < window ? token_count - w * window : window;
        if (length < 2) break; /* a tail of one token has nothing to score */
        if (kipp_session_reset(session, &error) != 0) {
            fprintf(stderr, "kipp: ppl: reset: %s\n", error.message);
            goto done;
        }
        for (size_t at = 0; at < length; at += chunk) {
            const size_t n = length - at < chunk ? length - at : chunk;
            /* row r predicts the token behind it, if that lies inside the window: the rows wanted are the first `rows`, their
             * targets the tokens from at + 1 on; each row's -log softmax at its target is computed where the logits lie */
            const size_t rows = at + n < length ? n : n - 1;
            kipp_step_item item = {session, tokens + at, n, want, rows};
            if (kipp_step_nll(model, &item, 1, tokens + at + 1, nll_of, chunk, &error) != 0) {
                fprintf(stderr, "kipp: ppl: eval: %s\n", error.message);
                goto done;
            }
            for (size_t r = 0; r < rows; ++r) nll += nll_of[r];
            scored += rows;
        }
        fprintf(stderr, "ppl: window %zu/%zu ppl=%.4f\n", w + 1, windows, exp(nll / (double)scored));
    }
    fprintf(stderr, "KIPP_PPL backend=%s tokens=%zu scored=%zu window=%zu nll=%.9f ppl=%.6f seconds=%.3f\n", kipp_path_name(info->path),
            token_count, scored, window, nll, exp(nll / (double)scored), seconds() - started);
    status = 0;
done:
    kipp_session_destroy(session);
    free(nll_of);
    free(want);
    return status;
}

int main(int argc, char **argv) {
    const char *model_dir = NULL, *tokens_text = NULL, *tokens_file = NULL, *kernels = NULL, *path_name = "gpu-bf16", *ppl_file = NULL;
    unsigned long ppl_window = 2048, ppl_limit = 0;
    unsigned long decode = 0, top_k = 0, top_n = 10, page = 16, kv_pages = 0, prefill_chunk = 512, max_step_tokens = 2048, max_context = 0;
    unsigned long long seed = 1;
    double temperature = 0.0, top_p = 1.0, min_p = 0.0, kv_mib = 0.0;
    uint32_t stops[KIPP_MAX_STOP_TOKENS];
    uint32_t stop_count = 0;
    int stops_given = 0;
    for (int i = 1; i < argc; ++i) {
        const char *arg = argv[i];
        if (strcmp(arg, "--help") == 0 || strcmp(arg, "-h") == 0) {
            usage(stdout);
            return 0;
        }
        if (i + 1 >= argc) {
            fprintf(stderr, "kipp: %s needs a value\n", arg);
            return 2;
        }
        const char *value = argv[++i];
        if (strcmp(arg, "--model") == 0) model_dir = value;
        else if (strcmp(arg, "--tokens") == 0) tokens_text = value;
        else if (strcmp(arg, "--tokens-file") == 0) tokens_file = value;
        else if (strcmp(arg, "--path") == 0 || strcmp(arg, "--backend") == 0) path_name = value;
        else if (strcmp(arg, "--kernels") == 0) kernels = value;
        else if (strcmp(arg, "--ppl") == 0) ppl_file = value;
        else if (strcmp(arg, "--ppl-window") == 0) ppl_window = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--ppl-limit") == 0) ppl_limit = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--decode") == 0) decode = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--temperature") == 0) temperature = strtod(value, NULL);
        else if (strcmp(arg, "--top-p") == 0) top_p = strtod(value, NULL);
        else if (strcmp(arg, "--top-k") == 0) top_k = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--min-p") == 0) min_p = strtod(value, NULL);
        else if (strcmp(arg, "--seed") == 0) seed = strtoull(value, NULL, 10);
        else if (strcmp(arg, "--top") == 0) top_n = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--max-context") == 0) max_context = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--page") == 0) page = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--kv-pages") == 0) kv_pages = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--kv-mib") == 0) kv_mib = strtod(value, NULL);
        else if (strcmp(arg, "--prefill-chunk") == 0) prefill_chunk = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--max-step-tokens") == 0) max_step_tokens = strtoul(value, NULL, 10);
        else if (strcmp(arg, "--stop-token") == 0) {
            stops_given = 1;
            if (stop_count == KIPP_MAX_STOP_TOKENS) {
                fprintf(stderr, "kipp: more than %u stop tokens\n", KIPP_MAX_STOP_TOKENS);
                return 2;
            }
            stops[stop_count++] = (uint32_t)strtoul(value, NULL, 10);
        } else {
            fprintf(stderr, "kipp: unknown option %s\n", arg);
            usage(stderr);
            return 2;
        }
    }
    kipp_path path;
    if (strcmp(path_name, "gpu-bf16") == 0) path = KIPP_PATH_GPU_BF16;
    else if (strcmp(path_name, "gpu-fp32") == 0) path = KIPP_PATH_GPU_FP32;
    else if (strcmp(path_name, "cpu-fp32") == 0) path = KIPP_PATH_CPU_FP32;
    else {
        fprintf(stderr, "kipp: path '%s' is not built into this engine (gpu-bf16, gpu-fp32, cpu-fp32)\n", path_name);
        return 2;
    }
    if (model_dir == NULL) {
        fprintf(stderr, "kipp: --model is required\n");
        return 2;
    }
    if (top_n < 1 || top_n > 100) {
        fprintf(stderr, "kipp: --top must be between 1 and 100\n");
        return 2;
    }
    if (seed == 0) {
        fprintf(stderr, "kipp: --seed must be nonzero\n");
        return 2;
    }
    if (page == 0 || prefill_chunk == 0 || max_step_tokens == 0) {
        fprintf(stderr, "kipp: --page, --prefill-chunk and --max-step-tokens must be positive\n");
        return 2;
    }
    uint32_t *tokens = NULL;
    size_t token_count = 0;
    if (ppl_file != NULL) {
        if (tokens_text != NULL || tokens_file != NULL || decode != 0) {
            fprintf(stderr, "kipp: --ppl cannot be combined with --tokens, --tokens-file or --decode\n");
            return 2;
        }
        if (ppl_window < 2) {
            fprintf(stderr, "kipp: --ppl-window must be at least 2\n");
            return 2;
        }
        if (read_token_file(ppl_file, &tokens, &token_count) != 0) {
            fprintf(stderr, "kipp: ppl: '%s' is not a uint32 token file\n", ppl_file);
            return 2;
        }
        if (ppl_limit != 0 && ppl_limit < token_count) token_count = ppl_limit;
        if (token_count < 2) {
            fprintf(stderr, "kipp: ppl: need at least two tokens to score\n");
            free(tokens);
            return 2;
        }
    } else if ((tokens_text == NULL) == (tokens_file == NULL)) {
        fprintf(stderr, "kipp: give --tokens or --tokens-file\n");
        return 2;
    } else if ((tokens_text != NULL ? parse_tokens(tokens_text, &tokens, &token_count) : read_token_file(tokens_file, &tokens, &token_count)) != 0) {
        fprintf(stderr, "kipp: the prompt must be token ids (5,17,3, or a file of little-endian uint32)\n");
        return 2;
    }
    if (token_count == 0) {
        fprintf(stderr, "kipp: the prompt is empty\n");
        free(tokens);
        return 2;
    }

    int rc = 1;
    kipp_error error;
    kipp_model *model = NULL;
    kipp_scheduler *scheduler = NULL;
    kipp_model_open_config config;
    memset(&config, 0, sizeof(config));
    config.path = path;
    config.page_tokens = (uint32_t)page;
    config.max_sessions = 1;
    config.max_step_tokens = (uint32_t)max_step_tokens;
    config.kernel_dir = kernels;
    size_t capacity = ppl_file != NULL ? ppl_window : token_count + decode;
    if (ppl_file != NULL && max_step_tokens < prefill_chunk) config.max_step_tokens = (uint32_t)prefill_chunk;
    config.kv_pool_pages = kv_pages != 0 ? (uint32_t)kv_pages : (uint32_t)((capacity + page - 1) / page);
    if (kv_mib > 0.0) {
        /* what a page takes is asked of a model with a pool of one page: bytes of all groups' slabs for that page and its spare */
        kipp_model *probe = NULL;
        kipp_model_open_config small = config;
        kipp_model_info probe_info;
        small.path = KIPP_PATH_CPU_FP32;
        small.kv_pool_pages = 1;
        if (kipp_model_open_ex(model_dir, &small, &probe, &error) != 0) {
            fprintf(stderr, "kipp: model: %s\n", error.message);
            goto done;
        }
        kipp_model_get_info(probe, &probe_info);
        kipp_model_close(probe, NULL);
        uint64_t per_page = probe_info.cache_bytes / 2 / (path == KIPP_PATH_GPU_BF16 ? 2 : 1);
        uint64_t pages = per_page != 0 ? (uint64_t)(kv_mib * 1024.0 * 1024.0) / per_page : 0;
        if (pages == 0 || pages > 0xfffffffful / 4) {
            fprintf(stderr, "kipp: --kv-mib %g holds no page of %llu bytes, or too many\n", kv_mib, (unsigned long long)per_page);
            goto done;
        }
        config.kv_pool_pages = (uint32_t)pages;
    }
    if (kipp_model_open_ex(model_dir, &config, &model, &error) != 0) {
        fprintf(stderr, "kipp: model: %s\n", error.message);
        goto done;
    }
    kipp_model_info info;
    kipp_model_get_info(model, &info);
    if (ppl_file != NULL) {
        if (ppl_window > info.context_length) {
            fprintf(stderr, "kipp: --ppl-window must be between 2 and %u\n", info.context_length);
            goto done;
        }
        for (size_t i = 0; i < token_count; ++i) {
            if (tokens[i] >= info.vocab_size) {
                fprintf(stderr, "kipp: ppl: token %zu is out of range\n", i);
                goto done;
            }
        }
        rc = run_perplexity(model, &info, tokens, token_count, ppl_window, prefill_chunk);
        goto done;
    }
    /* the session holds prompt + decode tokens, within the context length (/root/reference/src/kipp_cli.c:1057-1067) */
    size_t limit = max_context != 0 && max_context < info.context_length ? max_context : info.context_length;
    if (token_count > limit || decode > limit - token_count) {
        fprintf(stderr, "kipp: session: %zu prompt tokens and %lu to decode exceed the context of %zu tokens\n", token_count, decode, limit);
        goto done;
    }
    fprintf(stderr, "kipp: evaluating %zu token%s on %s\n", token_count, token_count == 1 ? "" : "s", kipp_path_name(path));
    kipp_scheduler_config sconfig = {(uint32_t)max_step_tokens, (uint32_t)prefill_chunk, 1, 1};
    if (kipp_scheduler_create(model, &sconfig, &scheduler, &error) != 0) {
        fprintf(stderr, "kipp: scheduler: %s\n", error.message);
        goto done;
    }
    kipp_request request;
    memset(&request, 0, sizeof(request));
    request.id = 1;
    request.prompt = tokens;
    request.prompt_count = token_count;
    request.max_new_tokens = (uint32_t)(decode > 0 ? decode : 1); /* --decode 0 still evaluates the prompt: one row of logits */
    request.params.temperature = (float)temperature;
    request.params.top_p = (float)top_p;
    request.params.top_k = (uint32_t)top_k;
    request.params.min_p = (float)min_p;
    request.params.repetition_penalty = 1.0f;
    request.seed = seed;
    if (stops_given) {
        memcpy(request.stop_tokens, stops, sizeof(stops));
        request.stop_token_count = stop_count;
    } else {
        memcpy(request.stop_tokens, info.stop_tokens, sizeof(request.stop_tokens));
        request.stop_token_count = info.stop_token_count;
    }
    if (kipp_scheduler_add(scheduler, &request, &error) != 0) {
        fprintf(stderr, "kipp: request: %s\n", error.message);
        goto done;
    }
    double started = seconds(), prefill_seconds = 0.0;
    size_t shown = 0;
    int first = 1;
    if (decode > 0) fputs("generated\t", stdout);
    while (!kipp_scheduler_idle(scheduler)) {
        kipp_produced produced[4];
        size_t count = 0;
        if (kipp_scheduler_step(scheduler, produced, 4, &count, &error) != 0) {
            fprintf(stderr, "\nkipp: step: %s\n", error.message);
            goto done;
        }
        kipp_result result;
        kipp_scheduler_result(scheduler, 1, &result);
        if (first && (count > 0 || result.reason != KIPP_FINISH_NONE)) {
            first = 0;
            prefill_seconds = seconds() - started; /* the prompt is in and its last row chose the first token */
            started = seconds();
        }
        if (decode > 0) {
            for (size_t i = 0; i < count; ++i, ++shown) printf("%s%u", shown ? " " : "", produced[i].token);
            fflush(stdout);
        }
    }
    double decode_seconds = seconds() - started;
    if (decode > 0) fputc('\n', stdout);
    kipp_result result;
    kipp_scheduler_result(scheduler, 1, &result);
    if (result.reason == KIPP_FINISH_FAILED) {
        fprintf(stderr, "kipp: generation failed: %s\n", result.error);
        goto done;
    }
    const float *row = kipp_scheduler_last_logits(scheduler, 1);
    if (row != NULL) {
        /* the top-N of the last row that counts: rank, token id, logit (equal logits: lower id first) */
        unsigned char *taken = calloc(info.vocab_size, 1);
        for (unsigned long rank = 1; taken != NULL && rank <= top_n && rank <= info.vocab_size; ++rank) {
            uint32_t best = 0;
            int have = 0;
            for (uint32_t t = 0; t < info.vocab_size; ++t) {
                if (!taken[t] && (!have || row[t] > row[best])) {
                    best = t;
                    have = 1;
                }
            }
            taken[best] = 1;
            printf("%lu\t%u\t%.9g\n", rank, best, (double)row[best]);
        }
        free(taken);
    }
    size_t decoded = decode > 0 && result.output_count > 0 ? result.output_count - 1 : 0;
    fprintf(stderr, "KIPP_METRIC backend=%s prefill_tokens=%zu prefill_seconds=%.9f decode_tokens=%zu decode_seconds=%.9f\n", kipp_path_name(path),
            token_count, prefill_seconds, decoded, decode_seconds);
    rc = 0;
done:
    kipp_scheduler_destroy(scheduler);
    if (model != NULL) kipp_model_close(model, NULL);
    free(tokens);
    return rc;
}
