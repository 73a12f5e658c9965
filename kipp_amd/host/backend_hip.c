/*
 * The GPU's table of operations: the launchers of the kernel libraries
 * (csrc/<name>.hip, each built into its own shared library) on buffers from
 * hipMalloc, one stream of the default priority, in bfloat16 (the kernels that
 * serving uses) or in true float32 (plain FMA products, the generic attention).
 * The libraries are opened at their first use; one that is missing, or a launch
 * that a kernel refuses, is an error with its name: there is no other path
 * behind any operation.
 *
 * Which file holds a kernel: <kernel_dir>/MANIFEST lists "<name>[.<constants>] <file>"
 * for the current builds (written by kipp_amd.csrc.build); without it the folder
 * is searched for libkipp_<name>[.<constants>].<10 hex digits>.so and the newest is taken.
 */
#define __HIP_PLATFORM_AMD__ 1
#include <dirent.h>
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include "backend.h"

#define PREFILL_MAX_BLOCKS 4096 /* table entries of one sequence the kernel for portions stages */

typedef int (*fn_embed)(const void *, int, const int32_t *, float *, int, int, hipStream_t);
typedef int (*fn_rmsnorm)(float *, const void *, int, int, const float *, void *, int, int, int, float, hipStream_t);
typedef int (*fn_residual_add)(float *, const void *, int, int, size_t, hipStream_t);
typedef int (*fn_swiglu)(const void *, int, int, void *, int, int, int, int, hipStream_t);
typedef int (*fn_cast)(const void *, int, void *, int, size_t, hipStream_t);
typedef int (*fn_gather_rows)(const void *, const int32_t *, void *, int, int, hipStream_t);
typedef int (*fn_fill_zero)(void *, size_t, hipStream_t);
typedef int (*fn_rotary_angles)(const int32_t *, const float *, float *, int, int, hipStream_t);
typedef int (*fn_qk_norm_rope_kv)(const void *, int, void *, int, void *, void *, int, const int32_t *, const int32_t *, const int32_t *, int,
                                  const float *, const float *, float, const float *, const float *, int, int, int, int, int, int, int, int,
                                  int, hipStream_t);
typedef int (*fn_attention_generic)(const void *, int, const void *, const void *, int, void *, int, const int32_t *, const int32_t *,
                                    const int32_t *, int, int, int, int, int, int, float, int, hipStream_t);
typedef int (*fn_attention_prefill)(const void *, const void *, const void *, void *, const int32_t *, const int32_t *, const int32_t *,
                                    const int32_t *, const int32_t *, const int32_t *, int, int, int, int, int, int, float, int, int,
                                    const int32_t *, int, float *, float *, int, const int32_t *, const int32_t *, int, hipStream_t);
typedef int (*fn_attention_decode)(const void *, const void *, const void *, void *, float *, float *, const int32_t *, const int32_t *,
                                   const int32_t *, const int32_t *, int, int, int, int, int, int, float, int, int, int, int32_t *,
                                   hipStream_t);
typedef int (*fn_int_void)(void);
typedef int (*fn_gemm_f32)(const float *, const void *, int, float *, int, int, int, hipStream_t);
typedef int (*fn_skinny_parts)(int, int, int);
typedef int (*fn_gemm_skinny)(const void *, const void *, float *, int, int, int, int, int, const float *, int, float, float *, const float *,
                              void *, float *, int, int, hipStream_t);
typedef int (*fn_rows_parts)(int, int, int, int);
typedef int (*fn_gemm_rows)(const void *, const void *, float *, int, int, int, int, int, int, hipStream_t);
typedef int (*fn_gemm_rows_swiglu)(const void *, const void *, void *, int, int, int, int, hipStream_t);
typedef int (*fn_skinny_swiglu)(const void *, const void *, void *, int, int, int, int, const float *, int, float, int, int, hipStream_t);
typedef int (*fn_int_int)(int);
typedef int (*fn_int3)(int, int, int);
typedef int (*fn_scale_rows)(const void *, const float *, void *, int, int, int, int, float, int, hipStream_t);
typedef int (*fn_tile_weight)(const void *, void *, int, int, int, hipStream_t);
typedef int (*fn_argmax)(const float *, int32_t *, int, int, float *, hipStream_t);
typedef int (*fn_sample)(const float *, int, int, const float *, const int32_t *, const float *, const float *, const double *, int32_t *,
                         hipStream_t);
typedef int (*fn_row_nll)(const float *, int, int, const int32_t *, double *, hipStream_t);
typedef int (*fn_adjust_logits)(float *, int, int, const int32_t *, const int32_t *, const int32_t *, const float *, const float *,
                                const float *, const float *, hipStream_t);
typedef int (*fn_attention_decode_fused)(const float *, int, int, const float *, const float *, float, const float *, const float *, int, void *,
                                         void *, void *, float *, float *, const int32_t *, const int32_t *, const int32_t *, const int32_t *, int,
                                         int, int, int, int, int, float, int, int, int, int32_t *, int, hipStream_t);
typedef int (*fn_ring_takes)(int, int, int, int);
typedef int (*fn_tiles_parts)(int, int, int, int, int);
typedef int (*fn_gemm_tiles)(const void *, const void *, void *, int, int, int, int, int, int, hipStream_t);

typedef struct {
    uint32_t head_dim, group;
    void *prefill_lib, *decode_lib;
    fn_attention_prefill prefill;
    fn_attention_decode decode;
    fn_attention_decode_fused decode_fused;
    fn_ring_takes ring_takes;
    int prefill_rows, split, split_min, fused_ok, fused_slabs;
} attention_variant;

typedef struct {
    int device;
    hipStream_t stream;
    char kernel_dir[3072];
    void *libs[12];
    size_t lib_count;
    fn_embed embed;
    fn_rmsnorm rmsnorm;
    fn_residual_add residual_add;
    fn_swiglu swiglu;
    fn_cast cast;
    fn_gather_rows gather_rows;
    fn_fill_zero fill_zero;
    fn_rotary_angles rotary_angles;
    fn_qk_norm_rope_kv qk_norm_rope_kv;
    fn_attention_generic attention_generic;
    fn_gemm_f32 gemm_f32;
    fn_skinny_parts skinny_parts;
    fn_gemm_skinny gemm_skinny;
    fn_rows_parts rows_parts;
    fn_gemm_rows gemm_rows;
    fn_gemm_rows_swiglu gemm_rows_swiglu;
    fn_int3 rows_swiglu_pays;
    fn_tiles_parts tiles_parts;
    fn_gemm_tiles gemm_tiles;
    fn_skinny_swiglu gemm_skinny_swiglu;
    fn_int_int skinny_sumsq_stride;
    fn_scale_rows scale_rows;
    fn_tile_weight tile_weight;
    fn_argmax argmax;
    fn_int_int argmax_scratch_floats;
    fn_sample sample;
    fn_adjust_logits adjust_logits;
    fn_row_nll row_nll;
    void *pinned;               /* SMALL_DOWNLOAD bytes of pinned host memory */
    unsigned char *sample_host; /* what the sampler of a step is told, packed by field */
    unsigned char *sample_device; /* the same on the GPU, behind the tokens chosen */
    size_t sample_bytes;        /* room of both */
    bool fuse;             /* few rows: residual add and norm ride on the products around them, decode attention starts from the QKV product */
    bool steps_major;      /* rows that one few-rows product writes for the next: in the order that product reads fastest */
    bool merge_in_kernel;  /* decode attention: the splits of a head are merged by the last of their workgroups to finish */
    int32_t *arrivals;     /* its counts of finished splits, zero between launches */
    size_t arrivals_count;
    attention_variant variants[8];
    size_t variant_count;
    uint64_t generic_attention_launches; /* bfloat16 attention that fell to the generic kernel */
    int compute_units;     /* of the device, for plans that fill it */
} hip_state;

static int hip_bad(kipp_error *error, hipError_t code, const char *what) {
    return kipp_fail(error, code == hipErrorOutOfMemory ? KIPP_ERROR_MEMORY : KIPP_ERROR_INTERNAL, "%s: %s", what, hipGetErrorString(code));
}

/* ------------------------------------------------------------------ finding and opening the libraries */
static int find_library(const hip_state *st, const char *key, char *path, size_t path_size, kipp_error *error) {
    char manifest[4096], line[1024];
    snprintf(manifest, sizeof(manifest), "%s/MANIFEST", st->kernel_dir);
    FILE *f = fopen(manifest, "r");
    if (f != NULL) {
        size_t key_length = strlen(key);
        while (fgets(line, sizeof(line), f) != NULL) {
            if (strncmp(line, key, key_length) == 0 && line[key_length] == ' ') {
                char *name = line + key_length + 1;
                name[strcspn(name, "\r\n")] = '\0';
                snprintf(path, path_size, "%s/%s", st->kernel_dir, name);
                fclose(f);
                if (access(path, R_OK) == 0) return 0;
                return kipp_fail(error, KIPP_ERROR_IO, "%s names %s for %s, which is not there: build the kernels again", manifest, name, key);
            }
        }
        fclose(f);
    }
    /* no manifest, or it does not know the key: libkipp_<key>.<10 hex digits>.so, the newest */
    DIR *dir = opendir(st->kernel_dir);
    if (dir == NULL) return kipp_fail(error, KIPP_ERROR_IO, "the folder of the kernel libraries, %s, cannot be read", st->kernel_dir);
    char prefix[256];
    snprintf(prefix, sizeof(prefix), "libkipp_%s.", key);
    size_t prefix_length = strlen(prefix);
    time_t newest = 0;
    bool any = false;
    struct dirent *entry;
    while ((entry = readdir(dir)) != NULL) {
        const char *name = entry->d_name;
        if (strncmp(name, prefix, prefix_length) != 0 || strlen(name) != prefix_length + 13 || strcmp(name + prefix_length + 10, ".so") != 0) continue;
        char candidate[4096];
        struct stat info;
        snprintf(candidate, sizeof(candidate), "%s/%s", st->kernel_dir, name);
        if (stat(candidate, &info) == 0 && (!any || info.st_mtime > newest)) {
            any = true;
            newest = info.st_mtime;
            snprintf(path, path_size, "%s", candidate);
        }
    }
    closedir(dir);
    if (!any)
        return kipp_fail(error, KIPP_ERROR_IO, "no kernel library for %s in %s: build it first (python -m kipp_amd.csrc.build)", key, st->kernel_dir);
    return 0;
}

static void *open_library(hip_state *st, const char *key, kipp_error *error) {
    char path[4096];
    if (find_library(st, key, path, sizeof(path), error) != 0) return NULL;
    void *lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (lib == NULL) kipp_fail(error, KIPP_ERROR_IO, "cannot load %s: %s", path, dlerror());
    return lib;
}

static void *symbol(void *lib, const char *name, kipp_error *error) {
    void *fn = dlsym(lib, name);
    if (fn == NULL) kipp_fail(error, KIPP_ERROR_INTERNAL, "a kernel library lacks %s", name);
    return fn;
}

#define KIPP_SYM(lib, field, name)                                   \
    do {                                                             \
        *(void **)(&st->field) = symbol(lib, name, error);           \
        if (st->field == NULL) return -1;                            \
    } while (0)

static int open_common(hip_state *st, kipp_error *error) {
    static const char *const names[] = {"elementwise", "rope_kv", "attention_generic", "gemm_f32", "gemm_skinny", "gemm_rows", "gemm_tiles", "sampling"};
    void *libs[8];
    for (size_t i = 0; i < 8; ++i) {
        libs[i] = open_library(st, names[i], error);
        if (libs[i] == NULL) return -1;
        st->libs[st->lib_count++] = libs[i];
    }
    KIPP_SYM(libs[0], embed, "kipp_embed");
    KIPP_SYM(libs[0], rmsnorm, "kipp_rmsnorm");
    KIPP_SYM(libs[0], residual_add, "kipp_residual_add");
    KIPP_SYM(libs[0], swiglu, "kipp_swiglu");
    KIPP_SYM(libs[0], cast, "kipp_cast");
    KIPP_SYM(libs[0], gather_rows, "kipp_gather_rows");
    KIPP_SYM(libs[0], fill_zero, "kipp_fill_zero");
    KIPP_SYM(libs[1], rotary_angles, "kipp_rotary_angles");
    KIPP_SYM(libs[1], qk_norm_rope_kv, "kipp_qk_norm_rope_kv");
    KIPP_SYM(libs[2], attention_generic, "kipp_paged_attention_generic");
    KIPP_SYM(libs[3], gemm_f32, "kipp_gemm_f32");
    KIPP_SYM(libs[4], skinny_parts, "kipp_gemm_skinny_parts");
    KIPP_SYM(libs[4], gemm_skinny, "kipp_gemm_skinny");
    KIPP_SYM(libs[5], rows_parts, "kipp_gemm_rows_parts");
    KIPP_SYM(libs[5], gemm_rows, "kipp_gemm_rows");
    KIPP_SYM(libs[5], gemm_rows_swiglu, "kipp_gemm_rows_swiglu");
    KIPP_SYM(libs[5], rows_swiglu_pays, "kipp_gemm_rows_swiglu_pays");
    KIPP_SYM(libs[6], tiles_parts, "kipp_gemm_tiles_parts");
    KIPP_SYM(libs[6], gemm_tiles, "kipp_gemm_tiles");
    KIPP_SYM(libs[0], scale_rows, "kipp_scale_rows");
    KIPP_SYM(libs[0], tile_weight, "kipp_tile_weight");
    KIPP_SYM(libs[4], gemm_skinny_swiglu, "kipp_gemm_skinny_swiglu");
    KIPP_SYM(libs[4], skinny_sumsq_stride, "kipp_gemm_skinny_sumsq_stride");
    KIPP_SYM(libs[7], argmax, "kipp_argmax");
    KIPP_SYM(libs[7], argmax_scratch_floats, "kipp_argmax_scratch_floats");
    KIPP_SYM(libs[7], sample, "kipp_sample");
    KIPP_SYM(libs[7], adjust_logits, "kipp_adjust_logits");
    KIPP_SYM(libs[7], row_nll, "kipp_row_nll");
    return 0;
}

static attention_variant *variant_of(hip_state *st, uint32_t head_dim, uint32_t group, kipp_error *error) {
    for (size_t i = 0; i < st->variant_count; ++i) {
        if (st->variants[i].head_dim == head_dim && st->variants[i].group == group) return &st->variants[i];
    }
    if (st->variant_count == sizeof(st->variants) / sizeof(st->variants[0])) {
        kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "more attention geometries in one model than this table keeps");
        return NULL;
    }
    attention_variant *v = &st->variants[st->variant_count];
    char key[96];
    memset(v, 0, sizeof(*v));
    v->head_dim = head_dim;
    v->group = group;
    snprintf(key, sizeof(key), "attention_prefill.HEAD_DIM%u", head_dim);
    if ((v->prefill_lib = open_library(st, key, error)) == NULL) return NULL;
    snprintf(key, sizeof(key), "attention_decode.GROUP%u.HEAD_DIM%u", group, head_dim);
    if ((v->decode_lib = open_library(st, key, error)) == NULL) return NULL;
    *(void **)(&v->prefill) = symbol(v->prefill_lib, "kipp_attention_prefill", error);
    *(void **)(&v->decode) = symbol(v->decode_lib, "kipp_attention_decode", error);
    *(void **)(&v->decode_fused) = symbol(v->decode_lib, "kipp_attention_decode_fused", error);
    *(void **)(&v->ring_takes) = symbol(v->decode_lib, "kipp_attention_decode_ring_takes", error);
    fn_int_void rows = NULL, split = NULL, split_min = NULL, fused_ok = NULL, fused_slabs = NULL;
    *(void **)(&rows) = symbol(v->prefill_lib, "kipp_attention_prefill_rows", error);
    *(void **)(&split) = symbol(v->decode_lib, "kipp_attention_decode_split", error);
    *(void **)(&split_min) = symbol(v->decode_lib, "kipp_attention_decode_split_min", error);
    *(void **)(&fused_ok) = symbol(v->decode_lib, "kipp_attention_decode_fused_ok", error);
    *(void **)(&fused_slabs) = symbol(v->decode_lib, "kipp_attention_decode_fused_slabs", error);
    if (v->prefill == NULL || v->decode == NULL || v->decode_fused == NULL || v->ring_takes == NULL || rows == NULL || split == NULL ||
        split_min == NULL || fused_ok == NULL || fused_slabs == NULL)
        return NULL;
    v->prefill_rows = rows();
    v->split = split();
    v->split_min = split_min();
    v->fused_ok = fused_ok();
    v->fused_slabs = fused_slabs();
    ++st->variant_count;
    return v;
}

/* ------------------------------------------------------------------ memory */
static void hip_destroy(kipp_runtime *rt) {
    hip_state *st = rt->state;
    if (st != NULL) {
        hipStreamSynchronize(st->stream);
        if (st->arrivals != NULL) hipFree(st->arrivals);
        if (st->sample_device != NULL) hipFree(st->sample_device);
        if (st->pinned != NULL) hipHostFree(st->pinned);
        free(st->sample_host);
        if (st->stream != NULL) hipStreamDestroy(st->stream);
        /* the libraries stay loaded: their kernels may be registered with the HIP runtime until the process ends */
        free(st);
    }
    free(rt);
}

static void *hip_alloc(kipp_runtime *rt, size_t bytes, kipp_error *error) {
    hip_state *st = rt->state;
    void *memory = NULL;
    hipError_t code = hipMalloc(&memory, bytes ? bytes : 256);
    if (code != hipSuccess) {
        hip_bad(error, code, "hipMalloc");
        return NULL;
    }
    code = hipMemsetAsync(memory, 0, bytes ? bytes : 256, st->stream);
    if (code != hipSuccess) {
        hipFree(memory);
        hip_bad(error, code, "hipMemsetAsync");
        return NULL;
    }
    return memory;
}

static void hip_free(kipp_runtime *rt, void *memory) {
    hip_state *st = rt->state;
    hipStreamSynchronize(st->stream); /* nothing in flight may still use it */
    hipFree(memory);
}

static int hip_zero(kipp_runtime *rt, void *memory, size_t bytes, kipp_error *error) {
    hip_state *st = rt->state;
    hipError_t code = hipMemsetAsync(memory, 0, bytes, st->stream);
    return code == hipSuccess ? 0 : hip_bad(error, code, "hipMemsetAsync");
}

static int hip_upload(kipp_runtime *rt, void *to, const void *from_host, size_t bytes, kipp_error *error) {
    hip_state *st = rt->state;
    if (bytes == 0) return 0;
    /* from pageable memory: the call returns once the bytes have left the host buffer */
    hipError_t code = hipMemcpyAsync(to, from_host, bytes, hipMemcpyHostToDevice, st->stream);
    return code == hipSuccess ? 0 : hip_bad(error, code, "copy to the GPU");
}

#define SMALL_DOWNLOAD 4096 /* bytes that come back through pinned memory of the runtime's own (a step's chosen tokens) */

static int hip_download(kipp_runtime *rt, void *to_host, const void *from, size_t bytes, kipp_error *error) {
    hip_state *st = rt->state;
    hipError_t code = hipSuccess;
    /* a copy into pageable memory is staged by the runtime and waited for inside the call; the few bytes of a decode step
     * come through a pinned buffer instead: the copy is queued behind the step and one wait covers both */
    if (bytes != 0 && bytes <= SMALL_DOWNLOAD && st->pinned == NULL && hipHostMalloc(&st->pinned, SMALL_DOWNLOAD, hipHostMallocDefault) != hipSuccess)
        st->pinned = NULL; /* without it: straight to the caller's memory, as for the large copies */
    void *target = bytes != 0 && bytes <= SMALL_DOWNLOAD && st->pinned != NULL ? st->pinned : to_host;
    if (bytes != 0) code = hipMemcpyAsync(target, from, bytes, hipMemcpyDeviceToHost, st->stream);
    if (code == hipSuccess) code = hipStreamSynchronize(st->stream);
    if (code == hipSuccess && target != to_host) memcpy(to_host, target, bytes);
    return code == hipSuccess ? 0 : hip_bad(error, code, "copy from the GPU (or a kernel before it)");
}

static int hip_copy(kipp_runtime *rt, void *to, const void *from, size_t bytes, kipp_error *error) {
    hip_state *st = rt->state;
    hipError_t code = hipMemcpyAsync(to, from, bytes, hipMemcpyDeviceToDevice, st->stream);
    return code == hipSuccess ? 0 : hip_bad(error, code, "copy on the GPU");
}

static int refused(kipp_error *error, const char *what, int code);

/* ------------------------------------------------------------------ placement */
static float half_to_float(uint16_t bits) {
    uint32_t sign = (uint32_t)(bits & 0x8000u) << 16, exponent = (bits >> 10) & 0x1f, fraction = bits & 0x3ffu, wide;
    if (exponent == 0) {
        if (fraction == 0) wide = sign;
        else {
            int shift = 0;
            while (!(fraction & 0x400u)) {
                fraction <<= 1;
                ++shift;
            }
            wide = sign | ((uint32_t)(127 - 15 + 1 - shift) << 23) | ((fraction & 0x3ffu) << 13);
        }
    } else if (exponent == 31) wide = sign | 0x7f800000u | (fraction << 13);
    else wide = sign | ((exponent + 127 - 15) << 23) | (fraction << 13);
    float value;
    memcpy(&value, &wide, sizeof(value));
    return value;
}

/* The tensor's values as float32 in a buffer of the host (freed by the caller). */
static float *widened(const kipp_tensor *tensor, size_t count, kipp_error *error) {
    float *wide = malloc(count ? count * sizeof(float) : 4);
    if (wide == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory widening %s", tensor->name);
        return NULL;
    }
    if (tensor->dtype == KIPP_F32) memcpy(wide, tensor->data, count * sizeof(float));
    else {
        const uint16_t *narrow = tensor->data;
        for (size_t i = 0; i < count; ++i) {
            if (tensor->dtype == KIPP_BF16) {
                uint32_t bits = (uint32_t)narrow[i] << 16;
                memcpy(&wide[i], &bits, sizeof(float));
            } else {
                wide[i] = half_to_float(narrow[i]);
            }
        }
    }
    return wide;
}

static int hip_place_matrix(kipp_runtime *rt, const kipp_tensor *const *pieces, size_t piece_count, kipp_weight_layout layout, kipp_weight *out,
                            kipp_error *error) {
    hip_state *st = rt->state;
    uint64_t rows = 0, columns = pieces[0]->shape[1];
    bool keep_bf16 = rt->act_dtype == KIPP_BF16;
    for (size_t p = 0; p < piece_count; ++p) {
        rows += pieces[p]->shape[0];
        keep_bf16 = keep_bf16 && pieces[p]->dtype == KIPP_BF16; /* pieces of different types, and everything on the 32-bit path, are widened */
    }
    size_t count, bytes;
    if (rows > INT32_MAX || columns > INT32_MAX || kipp_mul_size((size_t)rows, (size_t)columns, &count) != 0 ||
        kipp_mul_size(count, keep_bf16 ? 2 : 4, &bytes) != 0)
        return kipp_fail(error, KIPP_ERROR_RANGE, "a matrix of %llu x %llu is too large", (unsigned long long)rows, (unsigned long long)columns);
    char *data = hip_alloc(rt, bytes, error);
    if (data == NULL) return -1;
    size_t at = 0;
    for (size_t p = 0; p < piece_count; ++p) {
        size_t n = (size_t)(pieces[p]->shape[0] * pieces[p]->shape[1]);
        int rc;
        if (keep_bf16 || pieces[p]->dtype == KIPP_F32) {
            rc = hip_upload(rt, data + at, pieces[p]->data, n * (keep_bf16 ? 2 : 4), error); /* straight out of the mapped file */
        } else {
            float *wide = widened(pieces[p], n, error);
            rc = wide == NULL ? -1 : hip_upload(rt, data + at, wide, n * 4, error);
            if (rc == 0) rc = hip_download(rt, NULL, NULL, 0, error); /* the copy has left the buffer before it is freed */
            free(wide);
        }
        if (rc != 0) {
            hip_free(rt, data);
            return -1;
        }
        at += n * (keep_bf16 ? 2 : 4);
    }
    *out = (kipp_weight){data, keep_bf16 ? KIPP_BF16 : KIPP_F32, (uint32_t)rows, (uint32_t)columns, NULL, false};
    /* Decode reads every weight once a step and is bound by that read, which is a fifth faster from the streaming layout;
     * products of many rows read the rows.  The price is the matrix held twice. */
    bool pairs = layout == KIPP_LAYOUT_STREAM_PAIRS && piece_count == 2 && pieces[0]->shape[0] == pieces[1]->shape[0];
    if (keep_bf16 && layout != KIPP_LAYOUT_ROWS && columns % 32 == 0 && columns > 0 && rows > 0) {
        size_t inner = pairs ? (size_t)(rows / 2) : 0, tile_count = pairs ? (inner + 7) / 8 : ((size_t)rows + 15) / 16, tile_bytes;
        if (kipp_mul_size(tile_count * 32, (size_t)columns, &tile_bytes) != 0) {
            hip_free(rt, data);
            return kipp_fail(error, KIPP_ERROR_RANGE, "a matrix of %llu x %llu is too large", (unsigned long long)rows, (unsigned long long)columns);
        }
        void *tiles = hip_alloc(rt, tile_bytes, error);
        int rc = tiles == NULL ? -1 : st->tile_weight(data, tiles, (int)rows, (int)columns, (int)inner, st->stream);
        if (rc != 0) {
            if (tiles != NULL) {
                hip_free(rt, tiles);
                refused(error, "tile_weight", rc);
            }
            hip_free(rt, data);
            return -1;
        }
        out->tiles = tiles;
        out->pairs = pairs;
    }
    return 0;
}

static int hip_place_vector(kipp_runtime *rt, const kipp_tensor *tensor, float **out, kipp_error *error) {
    size_t n = (size_t)tensor->shape[0];
    float *wide = widened(tensor, n, error);
    if (wide == NULL) return -1;
    float *data = hip_alloc(rt, n * sizeof(float), error);
    int rc = data == NULL ? -1 : hip_upload(rt, data, wide, n * sizeof(float), error);
    if (rc == 0) rc = hip_download(rt, NULL, NULL, 0, error);
    free(wide);
    if (rc != 0) {
        if (data != NULL) hip_free(rt, data);
        return -1;
    }
    *out = data;
    return 0;
}

static void hip_free_weight(kipp_runtime *rt, kipp_weight *weight) {
    if (weight->data != NULL) hip_free(rt, weight->data);
    if (weight->tiles != NULL) hip_free(rt, weight->tiles);
    weight->data = weight->tiles = NULL;
}

/* ------------------------------------------------------------------ operations */
static int refused(kipp_error *error, const char *what, int code) {
    return kipp_fail(error, KIPP_ERROR_INTERNAL, "%s: launch failed or arguments refused (code %d)", what, code);
}

static int hip_embed(kipp_runtime *rt, const kipp_weight *table, const int32_t *tokens, float *out, uint32_t n, kipp_error *error) {
    hip_state *st = rt->state;
    int rc = st->embed(table->data, table->dtype, tokens, out, (int)n, (int)table->k, st->stream);
    return rc == 0 ? 0 : refused(error, "embed", rc);
}

#define FEW_ROWS 12           /* up to these the kernel in which every wave reads its rows of x itself is the faster one, and has the fused ends */
#define STAGED_ROWS 192       /* up to these the kernel that stages x through LDS; beyond, the one built for hundreds of rows where it takes the shape */
#define FUSE_NORM_X_BYTES 40e6 /* most bytes of x the workgroups of an unsplit product may read together for the fused norm to pay */

/* The few-rows kernel takes this product (and with it the ends that spare a decode step its norm kernels). */
static bool few_rows(const kipp_runtime *rt, const kipp_weight *w, uint32_t m) {
    return rt->act_dtype == KIPP_BF16 && w->dtype == KIPP_BF16 && m <= FEW_ROWS && w->k % 8 == 0 && w->k >= 32;
}

static bool hip_defers(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w, uint32_t m) {
    const hip_state *st = rt->state;
    return st->fuse && x->sumsq == NULL && few_rows(rt, w, m) && !w->pairs;
}

static int hip_scale_rows(kipp_runtime *rt, const kipp_rows *in, void *out, uint32_t rows, uint32_t width, kipp_error *error) {
    hip_state *st = rt->state;
    int rc = st->scale_rows(in->data, in->sumsq, out, (int)rows, (int)width, in->sumsq_parts, (in->sumsq_parts + 3) / 4 * 4, in->eps,
                            in->steps_major ? 1 : 0, st->stream);
    return rc == 0 ? 0 : refused(error, "scale_rows", rc);
}

static int hip_rmsnorm(kipp_runtime *rt, float *x, kipp_delta *delta, const float *weight, kipp_rows *out, uint32_t rows, uint32_t width,
                       float eps, bool may_leave_scale, kipp_error *error) {
    hip_state *st = rt->state;
    out->sumsq = NULL;
    if (delta != NULL && delta->parts == 0 && delta->w != NULL) {
        /* A product that has not been launched: its kernel adds it to x and prepares the norm of the new x.  That kernel is
         * not split over workgroups; where the product alone would be, each of its N / 16 workgroups reads all of its
         * operand instead of a part, which costs more than the norm's kernel once that is some tens of megabytes. */
        const kipp_weight *w = delta->w;
        const int N = (int)w->n, K = (int)w->k, most = delta->max_parts > 8 ? 8 : (delta->max_parts < 1 ? 1 : delta->max_parts);
        bool fused = st->fuse && few_rows(rt, w, delta->m) && !w->pairs && delta->m == rows && w->n == width &&
                     !(st->skinny_parts(N, K, most) > 1 && (double)((N + 15) / 16) * rows * K * 2 > FUSE_NORM_X_BYTES);
        if (fused) {
            const int stride = st->skinny_sumsq_stride(N);
            float *sumsq = kipp_scratch(rt, (size_t)rows * (size_t)stride * sizeof(float), error);
            void *unscaled = may_leave_scale ? out->data : kipp_scratch(rt, (size_t)rows * width * 2, error);
            if (sumsq == NULL || unscaled == NULL) return -1;
            const bool tiled = w->tiles != NULL;
            /* the rows go to a few-rows product (or to the kernel that finishes them): in the order those read fastest */
            const bool major = st->steps_major && N % 32 == 0 && rows > 1;
            int rc = st->gemm_skinny(delta->x, tiled ? w->tiles : w->data, NULL, (int)rows, N, K, 1, tiled ? 1 : 0, NULL, 0, 0.0f, x, weight, unscaled,
                                     sumsq, delta->x_steps_major ? 1 : 0, major ? 1 : 0, st->stream);
            if (rc != 0) return refused(error, "gemm_skinny (with the residual's end)", rc);
            *delta = (kipp_delta){NULL, 0, NULL, NULL, 0, 0, false};
            const kipp_rows left = {unscaled, sumsq, (N + 15) / 16, eps, major};
            if (may_leave_scale) {
                *out = left;
                return 0;
            }
            return hip_scale_rows(rt, &left, out->data, rows, width, error);
        }
        if (kipp_settle(rt, delta, error) != 0) return -1;
    }
    const bool any = delta != NULL && delta->parts > 0;
    int rc = st->rmsnorm(x, any ? delta->data : NULL, KIPP_F32, any ? delta->parts : 1, weight, out->data, rt->act_dtype, (int)rows, (int)width, eps,
                         st->stream);
    return rc == 0 ? 0 : refused(error, "rmsnorm", rc);
}

static int hip_residual_add(kipp_runtime *rt, float *x, kipp_delta *delta, uint32_t rows, uint32_t width, kipp_error *error) {
    hip_state *st = rt->state;
    if (kipp_settle(rt, delta, error) != 0) return -1;
    int rc = st->residual_add(x, delta->data, KIPP_F32, delta->parts, (size_t)rows * width, st->stream);
    return rc == 0 ? 0 : refused(error, "residual_add", rc);
}

/* x . w^T.  bfloat16 x bfloat16: up to 12 rows the kernel in which every wave streams its rows of w against all of x (it also
 * applies a scale that the rows still lack), up to 192 rows the one that stages x through LDS, both from the streaming layout
 * where the weight has it; beyond those the tiled matrix-core kernel (K a multiple of 32) or the staged one over runs of 256
 * rows; a shape none of them takes (K no multiple of 8, or below 32) and every float32 weight go through the plain float32
 * product. */
static int hip_linear(kipp_runtime *rt, const kipp_rows *rows_in, const kipp_weight *w, uint32_t m, int max_parts, kipp_delta *out, kipp_error *error) {
    hip_state *st = rt->state;
    const int M = (int)m, N = (int)w->n, K = (int)w->k;
    size_t count;
    if (kipp_mul_size(m, w->n, &count) != 0 || count > SIZE_MAX / 64) return kipp_fail(error, KIPP_ERROR_RANGE, "a product's size overflows");
    if (max_parts < 1) max_parts = 1;
    kipp_rows finished = *rows_in;
    if (finished.sumsq != NULL && !few_rows(rt, w, m) && kipp_finish_rows(rt, &finished, m, w->k, error) != 0) return -1;
    if (finished.steps_major && !few_rows(rt, w, m)) return kipp_fail(error, KIPP_ERROR_INTERNAL, "rows in steps-major order for a product that does not read it");
    const void *x = finished.data;
    /* paired tiles give the columns in another order: only the product that ends in the activation reads them */
    const bool tiled = w->tiles != NULL && !w->pairs;
    const void *streamed = tiled ? w->tiles : w->data;
    int rc;
#define KIPP_DELTA(y, parts) ((kipp_delta){(y), (parts), NULL, NULL, 0, 0, false})
    if (w->dtype == KIPP_BF16 && rt->act_dtype == KIPP_BF16 && K % 8 == 0 && K >= 32) {
        if (M <= FEW_ROWS) {
            int most = max_parts > 8 ? 8 : max_parts, parts = st->skinny_parts(N, K, most);
            float *y = parts >= 1 ? kipp_scratch(rt, (size_t)parts * count * 4, error) : NULL;
            if (y == NULL) return parts >= 1 ? -1 : refused(error, "gemm_skinny (its cut)", parts);
            rc = st->gemm_skinny(x, streamed, y, M, N, K, most, tiled ? 1 : 0, finished.sumsq, finished.sumsq_parts, finished.eps, NULL, NULL, NULL,
                                 NULL, finished.steps_major ? 1 : 0, 0, st->stream);
            *out = KIPP_DELTA(y, parts);
            return rc == 0 ? 0 : refused(error, "gemm_skinny", rc);
        }
        const bool tiles_take = K % 32 == 0 && (uint64_t)(M > N ? M : N) * (uint64_t)K * 2 < ((uint64_t)1 << 32);
        if (M <= STAGED_ROWS || (M <= 256 && !tiles_take)) {
            int most = max_parts > 12 ? 12 : max_parts, parts = st->rows_parts(M, N, K, most);
            float *y = parts >= 1 ? kipp_scratch(rt, (size_t)parts * count * 4, error) : NULL;
            if (y == NULL) return parts >= 1 ? -1 : refused(error, "gemm_rows (its cut)", parts);
            rc = st->gemm_rows(x, streamed, y, M, N, K, most, tiled ? 1 : 0, 0, st->stream);
            *out = KIPP_DELTA(y, parts);
            return rc == 0 ? 0 : refused(error, "gemm_rows", rc);
        }
        if (tiles_take) {
            int most = max_parts > 4 ? 4 : max_parts, parts = st->tiles_parts(M, N, K, 0, most);
            float *y = parts >= 1 ? kipp_scratch(rt, (size_t)parts * count * 4, error) : NULL;
            if (y == NULL) return parts >= 1 ? -1 : refused(error, "gemm_tiles (its cut)", parts);
            rc = st->gemm_tiles(x, w->data, y, M, N, K, 0, most, 0, st->stream);
            *out = KIPP_DELTA(y, parts);
            return rc == 0 ? 0 : refused(error, "gemm_tiles", rc);
        }
        float *y = kipp_scratch(rt, count * 4, error);
        if (y == NULL) return -1;
        for (int row = 0; row < M; row += 256) {
            int rows = M - row < 256 ? M - row : 256;
            rc = st->gemm_rows((const char *)x + (size_t)row * K * 2, streamed, y + (size_t)row * N, rows, N, K, 1, tiled ? 1 : 0, 0, st->stream);
            if (rc != 0) return refused(error, "gemm_rows", rc);
        }
        *out = KIPP_DELTA(y, 1);
        return 0;
    }
    const float *wide = x;
    if (rt->act_dtype == KIPP_BF16) {
        float *cast = kipp_scratch(rt, (size_t)m * w->k * 4, error);
        if (cast == NULL) return -1;
        rc = st->cast(x, KIPP_BF16, cast, KIPP_F32, (size_t)m * w->k, st->stream);
        if (rc != 0) return refused(error, "cast", rc);
        wide = cast;
    }
    float *y = kipp_scratch(rt, count * 4, error);
    if (y == NULL) return -1;
    rc = st->gemm_f32(wide, w->data, w->dtype, y, M, N, K, st->stream);
    *out = KIPP_DELTA(y, 1);
    return rc == 0 ? 0 : refused(error, "gemm_f32", rc);
}

/* Few rows against [gate; up]: both products and the activation in one kernel (and the norm's scale, if it was left to us).
 * Up to 192 rows: the product streamed from the paired tiles, whose columns come out gate tile by gate tile, then the activation
 * over those pairs.  Beyond: the matrix-core kernel with the activation as its end. */
static int hip_gated(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w, const kipp_weight *reader, kipp_rows *act, uint32_t m, bool *done,
                     kipp_error *error) {
    hip_state *st = rt->state;
    *done = false;
    if (rt->act_dtype != KIPP_BF16 || w->dtype != KIPP_BF16 || w->n % 2 != 0 || w->k % 8 != 0 || w->k < 32 || (w->tiles != NULL && !w->pairs)) return 0;
    const bool tiled = w->tiles != NULL;
    const int M = (int)m, K = (int)w->k, inner = (int)(w->n / 2);
    if (m <= FEW_ROWS) {
        /* the activation goes to `reader` alone: in the order its product reads fastest, if that is a few-rows product too */
        const bool major = st->steps_major && reader != NULL && few_rows(rt, reader, m) && !reader->pairs && inner % 32 == 0 && m > 1;
        int rc = st->gemm_skinny_swiglu(x->data, tiled ? w->tiles : w->data, act->data, M, (int)w->n, K, tiled ? 1 : 0, x->sumsq, x->sumsq_parts, x->eps,
                                        x->steps_major ? 1 : 0, major ? 1 : 0, st->stream);
        if (rc != 0) return refused(error, "gemm_skinny_swiglu", rc);
        act->steps_major = major;
        *done = true;
        return 0;
    }
    kipp_rows finished = *x;
    if (m > STAGED_ROWS) {
        /* many rows: both products and the activation in one pass of the matrix-core kernel (one rounding, after the activation) */
        if (K % 32 != 0 || (uint64_t)(M > (int)w->n ? M : (int)w->n) * (uint64_t)K * 2 >= ((uint64_t)1 << 32)) return 0;
        if (kipp_finish_rows(rt, &finished, m, w->k, error) != 0) return -1;
        int rc = st->gemm_tiles(finished.data, w->data, act->data, M, (int)w->n, K, 1, 1, 0, st->stream);
        if (rc != 0) return refused(error, "gemm_tiles (with the activation's end)", rc);
        *done = true;
        return 0;
    }
    if (!tiled) return 0;
    if (kipp_finish_rows(rt, &finished, m, w->k, error) != 0) return -1;
    if (K % 32 == 0 && st->rows_swiglu_pays(M, (int)w->n, K)) {
        /* a few dozen rows against a weight with rows enough for every compute unit: the activation at the product's end */
        int rc = st->gemm_rows_swiglu(finished.data, w->tiles, act->data, M, (int)w->n, K, 0, st->stream);
        if (rc != 0) return refused(error, "gemm_rows_swiglu", rc);
        *done = true;
        return 0;
    }
    const int width = 16 * ((inner + 7) / 8); /* columns of the product from paired tiles: 16 for every 8 outputs */
    int parts = st->rows_parts(M, width, K, 12);
    float *y = parts >= 1 ? kipp_scratch(rt, (size_t)parts * m * (size_t)width * sizeof(float), error) : NULL;
    if (y == NULL) return parts >= 1 ? -1 : refused(error, "gemm_rows (its cut)", parts);
    int rc = st->gemm_rows(finished.data, w->tiles, y, M, width, K, 12, 1, 0, st->stream);
    if (rc != 0) return refused(error, "gemm_rows (paired tiles)", rc);
    rc = st->swiglu(y, KIPP_F32, parts, act->data, rt->act_dtype, M, inner, 1, st->stream);
    if (rc != 0) return refused(error, "swiglu (pairs)", rc);
    *done = true;
    return 0;
}

/* Memory of its own for what follows a step's logits (the sampler's parameters and tokens, targets and their results): host
 * and GPU hold `bytes` each, and keep their place until more is asked for. */
static int sample_room(hip_state *st, size_t bytes, kipp_error *error) {
    if (bytes <= st->sample_bytes) return 0;
    size_t room = bytes < 16384 ? 16384 : 2 * bytes;
    unsigned char *host = realloc(st->sample_host, room);
    if (host == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    st->sample_host = host;
    st->sample_bytes = 0;
    if (st->sample_device != NULL) {
        hipStreamSynchronize(st->stream);
        hipFree(st->sample_device);
        st->sample_device = NULL;
    }
    hipError_t code = hipMalloc((void **)&st->sample_device, room);
    if (code != hipSuccess) return hip_bad(error, code, "hipMalloc");
    st->sample_bytes = room;
    return 0;
}

static int hip_row_nll(kipp_runtime *rt, const float *logits, const uint32_t *targets, double *out, uint32_t rows, uint32_t vocab, kipp_error *error) {
    hip_state *st = rt->state;
    if (rows == 0) return 0;
    const size_t result_bytes = (size_t)rows * 8, target_bytes = (size_t)rows * 4;
    if (sample_room(st, result_bytes + target_bytes, error) != 0) return -1;
    memcpy(st->sample_host + result_bytes, targets, target_bytes);
    hipError_t code = hipMemcpyAsync(st->sample_device + result_bytes, st->sample_host + result_bytes, target_bytes, hipMemcpyHostToDevice, st->stream);
    if (code != hipSuccess) return hip_bad(error, code, "copy to the GPU");
    int rc = st->row_nll(logits, (int)rows, (int)vocab, (const int32_t *)(st->sample_device + result_bytes), (double *)st->sample_device, st->stream);
    if (rc != 0) return refused(error, "row_nll", rc);
    code = hipMemcpyAsync(out, st->sample_device, result_bytes, hipMemcpyDeviceToHost, st->stream);
    if (code == hipSuccess) code = hipStreamSynchronize(st->stream);
    return code == hipSuccess ? 0 : hip_bad(error, code, "copy from the GPU (or a kernel before it)");
}

/* The device sampler over the rows of a step.  What it is told goes up in one copy, packed by field: the sampler's
 * parameters ([temperature | top_p | min_p | top_k] of 4 bytes a row, then the draws of 8), and, where a row has a bias or
 * penalties, the entries that the kernel before it walks ([begin (rows + 1) | biases | repetition | presence | frequency |
 * tokens | values]: a row's biases in their order, then its distinct recent tokens with their counts, as kipp_sample_ex
 * goes through them).  All of it lies in memory of its own that stays where it is until it must grow: the step's workspace is
 * not touched (a recorded step's logits lie there), and a call that follows a recording allocates nothing. */
static int hip_sample(kipp_runtime *rt, float *logits, const kipp_sample_params *params, const double *uniform, int32_t **out, uint32_t rows,
                      uint32_t vocab, kipp_error *error) {
    hip_state *st = rt->state;
    if (rows == 0) return 0;
    if (vocab >= (1u << 24)) return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "the device sampler takes vocabularies below 2^24");
    size_t entries = 0;
    for (uint32_t r = 0; r < rows; ++r) {
        const kipp_sample_params *p = &params[r];
        const bool penalties = p->frequency_penalty != 0.0f || p->presence_penalty != 0.0f || (p->repetition_penalty != 0.0f && p->repetition_penalty != 1.0f);
        entries += p->logit_bias_count + (penalties ? p->recent_count : 0); /* at most: tokens outside the vocabulary and repeated ones drop out */
    }
    const size_t out_bytes = ((size_t)rows * 4 + 15) / 16 * 16, pack_bytes = (size_t)rows * 24;
    const size_t adjust_words = entries != 0 ? 5 * (size_t)rows + 1 + 2 * entries : 0;
    const size_t bytes = out_bytes + pack_bytes + adjust_words * 4;
    if (sample_room(st, bytes, error) != 0) return -1;
    /* host and device hold the same layout; nothing of the first out_bytes goes up */
    unsigned char *h = st->sample_host + out_bytes, *d = st->sample_device + out_bytes;
    float *f32 = (float *)h;
    int32_t *i32 = (int32_t *)(h + (size_t)rows * 12);
    double *f64 = (double *)(h + (size_t)rows * 16);
    int32_t *begin = (int32_t *)(h + pack_bytes), *biases = begin + rows + 1;
    float *penalty = (float *)(biases + rows); /* [repetition | presence | frequency] */
    int32_t *token = (int32_t *)(penalty + 3 * (size_t)rows);
    float *value = (float *)(token + entries);
    size_t at = 0;
    for (uint32_t r = 0; r < rows; ++r) {
        const kipp_sample_params *p = &params[r];
        const bool sampled = p->temperature > 0.0f;
        f32[r] = sampled ? p->temperature : 0.0f;
        f32[rows + r] = sampled ? p->top_p : 1.0f;
        f32[2 * rows + r] = sampled ? p->min_p : 0.0f;
        i32[r] = sampled && p->top_k < (uint32_t)INT32_MAX ? (int32_t)p->top_k : 0;
        f64[r] = sampled ? uniform[r] : 0.0;
        if (entries == 0) continue;
        begin[r] = (int32_t)at;
        for (size_t b = 0; b < p->logit_bias_count; ++b) {
            if (p->logit_bias_tokens[b] >= vocab) continue;
            token[at] = (int32_t)p->logit_bias_tokens[b];
            value[at++] = p->logit_bias_values[b];
        }
        biases[r] = (int32_t)at - begin[r];
        penalty[r] = p->repetition_penalty;
        penalty[rows + r] = p->presence_penalty;
        penalty[2 * (size_t)rows + r] = p->frequency_penalty;
        const bool penalties = p->frequency_penalty != 0.0f || p->presence_penalty != 0.0f || (p->repetition_penalty != 0.0f && p->repetition_penalty != 1.0f);
        for (size_t i = 0; penalties && i < p->recent_count; ++i) {
            const uint32_t t = p->recent_tokens[i];
            bool seen = t >= vocab;
            for (size_t j = 0; j < i && !seen; ++j) seen = p->recent_tokens[j] == t;
            if (seen) continue; /* each distinct token once */
            size_t count = 0;
            for (size_t j = 0; j < p->recent_count; ++j) count += p->recent_tokens[j] == t;
            token[at] = (int32_t)t;
            value[at++] = (float)count;
        }
    }
    if (entries != 0) begin[rows] = (int32_t)at;
    hipError_t code = hipMemcpyAsync(d, h, pack_bytes + adjust_words * 4, hipMemcpyHostToDevice, st->stream);
    if (code != hipSuccess) return hip_bad(error, code, "copy to the GPU");
    if (at != 0) {
        const int32_t *d_begin = (const int32_t *)(d + pack_bytes), *d_biases = d_begin + rows + 1;
        const float *d_penalty = (const float *)(d_biases + rows);
        const int32_t *d_token = (const int32_t *)(d_penalty + 3 * (size_t)rows);
        int rc = st->adjust_logits(logits, (int)rows, (int)vocab, d_begin, d_biases, d_token, (const float *)(d_token + entries), d_penalty,
                                   d_penalty + rows, d_penalty + 2 * (size_t)rows, st->stream);
        if (rc != 0) return refused(error, "adjust_logits", rc);
    }
    *out = (int32_t *)st->sample_device;
    int rc = st->sample(logits, (int)rows, (int)vocab, (const float *)d, (const int32_t *)(d + (size_t)rows * 12), (const float *)d + rows,
                        (const float *)d + 2 * rows, (const double *)(d + (size_t)rows * 16), *out, st->stream);
    return rc == 0 ? 0 : refused(error, "sample", rc);
}

static int hip_argmax(kipp_runtime *rt, const float *logits, int32_t *out, uint32_t rows, uint32_t vocab, kipp_error *error) {
    hip_state *st = rt->state;
    float *scratch = kipp_scratch(rt, (size_t)st->argmax_scratch_floats((int)rows) * sizeof(float), error);
    if (scratch == NULL) return -1;
    int rc = st->argmax(logits, out, (int)rows, (int)vocab, scratch, st->stream);
    return rc == 0 ? 0 : refused(error, "argmax", rc);
}

static int hip_swiglu(kipp_runtime *rt, const kipp_delta *gate_up, void *out, uint32_t rows, uint32_t inner, kipp_error *error) {
    hip_state *st = rt->state;
    int rc = st->swiglu(gate_up->data, KIPP_F32, gate_up->parts, out, rt->act_dtype, (int)rows, (int)inner, 0, st->stream);
    return rc == 0 ? 0 : refused(error, "swiglu", rc);
}

static int hip_rotary_angles(kipp_runtime *rt, const int32_t *positions, const float *inv_freq, uint32_t n, uint32_t half,
                             const float **out_rotation, kipp_error *error) {
    hip_state *st = rt->state;
    float *angles = kipp_scratch(rt, (size_t)n * 2 * half * sizeof(float), error);
    if (angles == NULL) return -1;
    int rc = st->rotary_angles(positions, inv_freq, angles, (int)n, (int)half, st->stream);
    *out_rotation = angles;
    return rc == 0 ? 0 : refused(error, "rotary_angles", rc);
}

static int hip_qk_norm_rope_kv(kipp_runtime *rt, const kipp_delta *qkv, void *q_out, const kipp_cache_view *cache, const kipp_batch *batch,
                               const kipp_attention_geometry *g, const float *q_norm_w, const float *k_norm_w, float eps,
                               const float *rotation, uint32_t rotary_dim, int interleaved, kipp_error *error) {
    hip_state *st = rt->state;
    int rc = st->qk_norm_rope_kv(qkv->data, KIPP_F32, q_out, rt->act_dtype, cache->k, cache->v, rt->act_dtype, batch->positions,
                                 batch->seq_of_token, batch->tables[cache->group], (int)batch->max_blocks, q_norm_w, k_norm_w, eps, NULL, rotation,
                                 (int)rotary_dim, interleaved, (int)batch->n_tokens, (int)g->n_q, (int)g->n_kv, (int)g->head_dim,
                                 (int)cache->page_tokens, cache->writable ? 1 : 0, qkv->parts, st->stream);
    return rc == 0 ? 0 : refused(error, "qk_norm_rope_kv", rc);
}

static int compare_items(const void *a, const void *b) {
    const int32_t *x = a, *y = b; /* (keys, entry, tile, cut): the longest key range first, then in order */
    if (x[0] != y[0]) return x[0] > y[0] ? -1 : 1;
    if (x[1] != y[1]) return x[1] < y[1] ? -1 : 1;
    if (x[2] != y[2]) return x[2] < y[2] ? -1 : 1;
    return x[3] < y[3] ? -1 : (x[3] > y[3]);
}

#define PREFILL_MIN_CUT 512 /* fewest keys of a cut of the keys (below, the merge costs more than the cut gains) */

/* The work list of the kernel for portions: (entry, tile of its query rows) for every entry that brings more than one
 * token, the longest key range first.  A workgroup walks all keys its tile sees.  Where the tiles times the heads are
 * fewer workgroups than two a compute unit and the contexts are long (a portion of a few hundred rows behind thousands of
 * keys), the keys are cut as well, at multiples of a length chosen so that the GPU is filled about twice: an item is then
 * (entry, tile, cut), and the cuts of a row are merged in order afterwards.  Made by the first attention of a forward pass,
 * shared by the others of the same geometry. */
static int prefill_work(kipp_runtime *rt, kipp_batch *batch, int tile_rows, const kipp_attention_geometry *g, kipp_error *error) {
    hip_state *st = rt->state;
    const uint64_t made_for = ((uint64_t)g->n_q << 40) ^ ((uint64_t)g->head_dim << 24) ^ ((uint64_t)g->window << 1) ^ 1u;
    if (batch->item_seq != NULL && batch->items_of == made_for) return 0;
    size_t tiles = 0;
    int longest = 0;
    for (uint32_t i = 0; i < batch->n_seqs; ++i) {
        if (batch->h_q_len[i] <= 1) continue;
        tiles += (size_t)(batch->h_q_len[i] + tile_rows - 1) / (size_t)tile_rows;
        if (batch->h_ctx_len[i] > longest) longest = batch->h_ctx_len[i]; /* the last tile's last key + 1 */
    }
    int cut_keys = 0;
    const size_t workgroups = tiles * g->n_q, units = (size_t)st->compute_units;
    if (g->window == 0 && tiles != 0 && workgroups < 2 * units) {
        const size_t want = (2 * units + workgroups - 1) / workgroups;
        cut_keys = (int)((((size_t)longest + want - 1) / want + 63) / 64 * 64);
        if (cut_keys < PREFILL_MIN_CUT) cut_keys = PREFILL_MIN_CUT;
        if (longest <= cut_keys) cut_keys = 0;
    }
    size_t count = 0, merged = 0;
    for (uint32_t i = 0; i < batch->n_seqs; ++i) {
        int n = batch->h_q_len[i], ctx = batch->h_ctx_len[i];
        if (n <= 1) continue;
        for (int t = 0; t * tile_rows < n; ++t) {
            int last_row = (t + 1) * tile_rows < n ? (t + 1) * tile_rows : n;
            count += cut_keys ? (size_t)((ctx - n + last_row - 1) / cut_keys + 1) : 1;
            merged += (size_t)(last_row - t * tile_rows);
        }
    }
    const size_t ints = (count ? count : 1) * 3 + (merged ? merged : 1) * 2;
    int32_t *items = malloc((count ? count : 1) * 4 * sizeof(int32_t)), *lists = malloc(ints * sizeof(int32_t));
    if (items == NULL || lists == NULL) {
        free(items);
        free(lists);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
    }
    int32_t *rows_of = lists + 3 * count, *cuts_of = rows_of + merged;
    size_t at = 0, row_at = 0;
    uint32_t most = 1;
    for (uint32_t i = 0; i < batch->n_seqs; ++i) {
        int n = batch->h_q_len[i], ctx = batch->h_ctx_len[i];
        if (n <= 1) continue;
        for (int t = 0; t * tile_rows < n; ++t) {
            int last_row = (t + 1) * tile_rows < n ? (t + 1) * tile_rows : n;
            int last = ctx - n + last_row - 1; /* the last key the tile sees */
            int cuts = cut_keys ? last / cut_keys + 1 : 1;
            for (int c = 0; c < cuts; ++c, ++at) {
                int end = cut_keys && (c + 1) * cut_keys < last + 1 ? (c + 1) * cut_keys : last + 1;
                items[4 * at] = cut_keys ? end - c * cut_keys : last; /* the keys it walks (uncut: the last key, as good an order) */
                items[4 * at + 1] = (int32_t)i;
                items[4 * at + 2] = t;
                items[4 * at + 3] = c;
            }
            if ((uint32_t)cuts > most) most = (uint32_t)cuts;
            for (int r = t * tile_rows; r < last_row; ++r, ++row_at) {
                rows_of[row_at] = batch->h_q_start[i] + r;
                cuts_of[row_at] = cuts;
            }
        }
    }
    qsort(items, count, 4 * sizeof(int32_t), compare_items);
    for (size_t i = 0; i < count; ++i) {
        lists[i] = items[4 * i + 1];
        lists[count + i] = items[4 * i + 2];
        lists[2 * count + i] = items[4 * i + 3];
    }
    int32_t *device = kipp_scratch(rt, ints * sizeof(int32_t), error);
    int rc = device == NULL ? -1 : hip_upload(rt, device, lists, ints * sizeof(int32_t), error);
    free(items);
    free(lists);
    if (rc != 0) return -1;
    batch->item_seq = device;
    batch->item_tile = device + count;
    batch->item_cut = device + 2 * count;
    batch->merge_rows = device + 3 * count;
    batch->merge_cuts = batch->merge_rows + merged;
    batch->n_items = (uint32_t)count;
    batch->n_merge = (uint32_t)merged;
    batch->cut_keys = (uint32_t)cut_keys;
    batch->most_cuts = most;
    batch->cut_acc = batch->cut_ml = NULL;
    if (cut_keys) {
        ++rt->cut_attention_steps;
        const size_t slots = (size_t)batch->n_tokens * g->n_q * most;
        batch->cut_acc = kipp_scratch(rt, slots * g->head_dim * sizeof(float), error);
        batch->cut_ml = kipp_scratch(rt, slots * 2 * sizeof(float), error);
        if (batch->cut_acc == NULL || batch->cut_ml == NULL) return -1;
    }
    batch->items_of = made_for;
    return 0;
}

/* Counts of finished splits for `count` (token, key/value head) pairs: zero between launches (the workgroup that merges sets
 * its count back), kept from step to step, zeroed again after a step that failed.  NULL: the merge is a launch of its own. */
static int arrivals_for(kipp_runtime *rt, size_t count, int32_t **out, kipp_error *error) {
    hip_state *st = rt->state;
    *out = NULL;
    if (!st->merge_in_kernel) return 0;
    if (st->arrivals_count < count) {
        if (rt->recording) return kipp_fail(error, KIPP_ERROR_MEMORY, "the counts of finished splits would grow while a step is recorded");
        size_t grown = count < 65536 ? 65536 : count;
        ++rt->generation; /* recordings hold the old address */
        hipStreamSynchronize(st->stream);
        if (st->arrivals != NULL) hipFree(st->arrivals);
        st->arrivals = NULL;
        st->arrivals_count = 0;
        hipError_t code = hipMalloc((void **)&st->arrivals, grown * sizeof(int32_t));
        if (code != hipSuccess) return hip_bad(error, code, "hipMalloc");
        int rc = st->fill_zero(st->arrivals, grown, st->stream);
        if (rc != 0) return refused(error, "fill_zero", rc);
        st->arrivals_count = grown;
    }
    *out = st->arrivals;
    return 0;
}

/* Partial results of the splits, shared by the layers of one geometry within the step. */
static int decode_workspace(kipp_runtime *rt, kipp_batch *batch, const attention_variant *v, const kipp_attention_geometry *g, size_t *max_splits,
                            int *grid, kipp_error *error) {
    *max_splits = (batch->max_decode_ctx + (size_t)v->split_min - 1) / (size_t)v->split_min + 1;
    const size_t key = ((size_t)g->n_q << 32) ^ ((size_t)g->head_dim << 16) ^ *max_splits;
    if (batch->decode_workspace[0] == NULL || batch->decode_workspace_key != key) {
        size_t rows = (size_t)batch->n_decode * g->n_q * *max_splits;
        batch->decode_workspace[0] = kipp_scratch(rt, rows * g->head_dim * sizeof(float), error);
        batch->decode_workspace[1] = kipp_scratch(rt, rows * 2 * sizeof(float), error);
        if (batch->decode_workspace[0] == NULL || batch->decode_workspace[1] == NULL) return -1;
        batch->decode_workspace_key = key;
    }
    uint32_t span = g->window != 0 && g->window < batch->max_decode_ctx ? g->window : batch->max_decode_ctx;
    size_t need = (span + (size_t)v->split - 1) / (size_t)v->split + (g->window != 0 ? 1 : 0);
    *grid = (int)(need < 1 ? 1 : (need > *max_splits ? *max_splits : need));
    return 0;
}

static bool attention_fast(const kipp_runtime *rt, const kipp_attention_geometry *g, const kipp_cache_view *cache, const kipp_batch *batch) {
    const uint32_t group = g->n_q / g->n_kv, page = cache->page_tokens;
    return rt->act_dtype == KIPP_BF16 && g->head_dim % 16 == 0 && group <= 16 && (page & (page - 1)) == 0 && batch->max_blocks <= PREFILL_MAX_BLOCKS;
}

#define FUSED_DECODE_ROWS 16   /* up to this many single tokens take the decode attention that starts from the QKV product ... */
#define FUSED_DECODE_KEYS 8192 /* ... while their contexts are shorter than this (beyond, every split's workgroup would prepare the queries again) */

/* Single tokens only: the QKV product in at most four slabs, then norm, rotation, cache write and attention in one kernel,
 * for a few tokens and wherever the kernel that walks whole contexts or long ranges runs. */
static int hip_decode_attention(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w_qkv, const kipp_cache_view *cache,
                                const kipp_weight *reader, kipp_rows *out, kipp_batch *batch, const kipp_attention_geometry *g,
                                const float *q_norm_w, const float *k_norm_w, float eps, const float *rotation, uint32_t rotary_dim,
                                int interleaved, bool *done, kipp_error *error) {
    hip_state *st = rt->state;
    *done = false;
    const uint32_t n = batch->n_tokens;
    if (!st->fuse || !attention_fast(rt, g, cache, batch) || batch->n_portions != 0 || batch->n_decode != n || interleaved) return 0;
    if (g->head_dim % 128 != 0 || g->head_dim > 256 || (rotation != NULL && rotary_dim != g->head_dim)) return 0;
    attention_variant *v = variant_of(st, g->head_dim, g->n_q / g->n_kv, error);
    if (v == NULL) return -1;
    if (!v->fused_ok) return 0;
    size_t max_splits;
    int grid;
    uint32_t span = g->window != 0 && g->window < batch->max_decode_ctx ? g->window : batch->max_decode_ctx;
    int splits = (int)((span + (size_t)v->split - 1) / (size_t)v->split) + (g->window != 0 ? 1 : 0);
    if (!((n <= FUSED_DECODE_ROWS && batch->max_decode_ctx < FUSED_DECODE_KEYS) ||
          v->ring_takes((int)n, (int)g->n_kv, (int)cache->page_tokens, splits < 1 ? 1 : splits)))
        return 0;
    kipp_delta qkv;
    if (hip_linear(rt, x, w_qkv, n, v->fused_slabs, &qkv, error) != 0) return -1;
    int32_t *arrivals;
    if (decode_workspace(rt, batch, v, g, &max_splits, &grid, error) != 0 || arrivals_for(rt, (size_t)n * g->n_q, &arrivals, error) != 0) return -1;
    /* the mixed heads go to `reader` alone: in the order its product reads fastest, if that is a few-rows product */
    const bool major = st->steps_major && reader != NULL && few_rows(rt, reader, n) && !reader->pairs && n > 1;
    int rc = v->decode_fused(qkv.data, qkv.parts, (int)n, q_norm_w, k_norm_w, eps, NULL, rotation, cache->writable ? 1 : 0, cache->k, cache->v,
                             out->data, batch->decode_workspace[0], batch->decode_workspace[1], batch->decode_rows, batch->positions,
                             batch->seq_of_token, batch->tables[cache->group], (int)batch->max_blocks, (int)n, (int)g->n_q, (int)g->n_kv,
                             (int)g->head_dim, (int)cache->page_tokens, g->scale, (int)g->window, grid, (int)max_splits, arrivals, major ? 1 : 0,
                             st->stream);
    if (rc != 0) return refused(error, "attention_decode_fused", rc);
    out->steps_major = major;
    *done = true;
    return 0;
}

static int hip_attention(kipp_runtime *rt, const void *q, const kipp_cache_view *cache, void *out, kipp_batch *batch,
                         const kipp_attention_geometry *g, kipp_error *error) {
    hip_state *st = rt->state;
    const uint32_t group = g->n_q / g->n_kv, page = cache->page_tokens;
    const int32_t *table = batch->tables[cache->group];
    int rc;
    const bool fast = attention_fast(rt, g, cache, batch);
    if (!fast) {
        /* the float32 path, and geometries the matrix-core kernels refuse (head sizes that are no multiple of 16, more than
         * 16 query heads a key/value head, pages that are no power of two) */
        if (rt->act_dtype == KIPP_BF16) ++st->generic_attention_launches;
        rc = st->attention_generic(q, rt->act_dtype, cache->k, cache->v, rt->act_dtype, out, rt->act_dtype, batch->positions, batch->seq_of_token,
                                   table, (int)batch->max_blocks, (int)batch->n_tokens, (int)g->n_q, (int)g->n_kv, (int)g->head_dim, (int)page,
                                   g->scale, (int)g->window, st->stream);
        return rc == 0 ? 0 : refused(error, "paged_attention_generic", rc);
    }
    attention_variant *v = variant_of(st, g->head_dim, group, error);
    if (v == NULL) return -1;
    if (batch->n_portions != 0) {
        if (prefill_work(rt, batch, v->prefill_rows, g, error) != 0) return -1;
        const bool cut = batch->cut_keys != 0;
        rc = v->prefill(q, cache->k, cache->v, out, batch->item_seq, batch->item_tile, batch->q_start, batch->q_len, batch->positions, table,
                        (int)batch->max_blocks, (int)batch->n_items, (int)g->n_q, (int)g->n_kv, (int)g->head_dim, (int)page, g->scale,
                        (int)g->window, v->prefill_rows, cut ? batch->item_cut : NULL, (int)batch->cut_keys, batch->cut_acc, batch->cut_ml,
                        cut ? (int)batch->most_cuts : 0, cut ? batch->merge_rows : NULL, cut ? batch->merge_cuts : NULL,
                        cut ? (int)batch->n_merge : 0, st->stream);
        if (rc != 0) return refused(error, "attention_prefill", rc);
    }
    if (batch->n_decode != 0) {
        size_t max_splits;
        int grid;
        int32_t *arrivals;
        if (decode_workspace(rt, batch, v, g, &max_splits, &grid, error) != 0 || arrivals_for(rt, (size_t)batch->n_decode * g->n_q, &arrivals, error) != 0)
            return -1;
        rc = v->decode(q, cache->k, cache->v, out, batch->decode_workspace[0], batch->decode_workspace[1], batch->decode_rows, batch->positions,
                       batch->seq_of_token, table, (int)batch->max_blocks, (int)batch->n_decode, (int)g->n_q, (int)g->n_kv, (int)g->head_dim,
                       (int)page, g->scale, (int)g->window, grid, (int)max_splits, arrivals, st->stream);
        if (rc != 0) return refused(error, "attention_decode", rc);
    }
    return 0;
}

/* A step that failed may have left counts of finished splits behind: zero them, so that the next launch merges when it should. */
static void hip_after_failed_step(kipp_runtime *rt) {
    hip_state *st = rt->state;
    hipStreamSynchronize(st->stream);
    (void)hipGetLastError();
    if (st->arrivals != NULL) st->fill_zero(st->arrivals, st->arrivals_count, st->stream);
}

/* ------------------------------------------------------------------ recorded steps (HIP graphs) */
static int hip_graph_begin(kipp_runtime *rt, kipp_error *error) {
    hip_state *st = rt->state;
    hipError_t code = hipStreamBeginCapture(st->stream, hipStreamCaptureModeThreadLocal);
    if (code != hipSuccess) return hip_bad(error, code, "hipStreamBeginCapture");
    rt->recording = true;
    return 0;
}

static int hip_graph_end(kipp_runtime *rt, bool keep, void **out_graph, kipp_error *error) {
    hip_state *st = rt->state;
    hipGraph_t graph = NULL;
    hipError_t code = hipStreamEndCapture(st->stream, &graph);
    rt->recording = false;
    *out_graph = NULL;
    if (code != hipSuccess || graph == NULL || !keep) {
        if (graph != NULL) hipGraphDestroy(graph);
        (void)hipGetLastError();
        return keep ? hip_bad(error, code, "hipStreamEndCapture") : 0;
    }
    hipGraphExec_t exec = NULL;
    code = hipGraphInstantiate(&exec, graph, NULL, NULL, 0);
    hipGraphDestroy(graph);
    if (code != hipSuccess) return hip_bad(error, code, "hipGraphInstantiate");
    *out_graph = exec;
    return 0;
}

static int hip_graph_launch(kipp_runtime *rt, void *graph, kipp_error *error) {
    hip_state *st = rt->state;
    hipError_t code = hipGraphLaunch((hipGraphExec_t)graph, st->stream);
    return code == hipSuccess ? 0 : hip_bad(error, code, "hipGraphLaunch");
}

static void hip_graph_free(kipp_runtime *rt, void *graph) {
    hip_state *st = rt->state;
    hipStreamSynchronize(st->stream);
    hipGraphExecDestroy((hipGraphExec_t)graph);
}

static int hip_gather_rows(kipp_runtime *rt, const float *x, const int32_t *index, float *out, uint32_t n, uint32_t width, kipp_error *error) {
    hip_state *st = rt->state;
    int rc = st->gather_rows(x, index, out, (int)n, (int)width, st->stream);
    return rc == 0 ? 0 : refused(error, "gather_rows", rc);
}

/* ------------------------------------------------------------------ making the table */
static void default_kernel_dir(char *out, size_t size) {
    const char *env = getenv("KIPP_AMD_KERNELS");
    if (env != NULL && env[0] != '\0') {
        snprintf(out, size, "%s", env);
        return;
    }
    Dl_info info;
    out[0] = '\0';
    if (dladdr((void *)default_kernel_dir, &info) != 0 && info.dli_fname != NULL) {
        /* this library lies in <package>/host/_lib; the kernels in <package>/csrc/_lib */
        char here[3000];
        snprintf(here, sizeof(here), "%s", info.dli_fname);
        char *slash = strrchr(here, '/');
        if (slash != NULL) {
            *slash = '\0';
            snprintf(out, size, "%s/../../csrc/_lib", here);
        }
    }
}

kipp_runtime *kipp_runtime_hip(kipp_path path, int device, const char *kernel_dir, kipp_error *error) {
    int count = 0;
    hipError_t code = hipGetDeviceCount(&count);
    if (code != hipSuccess || count <= 0) {
        kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "no GPU visible: the paths gpu-bf16 and gpu-fp32 run on a gfx950 GPU only (cpu-fp32 needs none)");
        return NULL;
    }
    if (device < 0 || device >= count) {
        kipp_fail(error, KIPP_ERROR_ARGUMENT, "GPU %d of %d", device, count);
        return NULL;
    }
    kipp_runtime *rt = calloc(1, sizeof(*rt));
    hip_state *st = calloc(1, sizeof(*st));
    if (rt == NULL || st == NULL) {
        free(rt);
        free(st);
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        return NULL;
    }
    rt->state = st;
    st->device = device;
    /* KIPP_AMD_FUSE=0: every norm and the rotation as kernels of their own, also for few rows; KIPP_AMD_DECODE_MERGE=launch:
     * the splits of decode attention are merged by a launch of its own, which needs no ordering between workgroups */
    const char *fuse = getenv("KIPP_AMD_FUSE"), *merge = getenv("KIPP_AMD_DECODE_MERGE");
    st->fuse = path == KIPP_PATH_GPU_BF16 && !(fuse != NULL && strcmp(fuse, "0") == 0);
    st->merge_in_kernel = !(merge != NULL && strcmp(merge, "launch") == 0);
    const char *major = getenv("KIPP_AMD_STEPS_MAJOR");
    st->steps_major = st->fuse && !(major != NULL && strcmp(major, "0") == 0);
    if (kernel_dir != NULL && kernel_dir[0] != '\0') snprintf(st->kernel_dir, sizeof(st->kernel_dir), "%s", kernel_dir);
    else default_kernel_dir(st->kernel_dir, sizeof(st->kernel_dir));
    if ((code = hipSetDevice(device)) != hipSuccess || (code = hipStreamCreate(&st->stream)) != hipSuccess) {
        hip_bad(error, code, "hipSetDevice / hipStreamCreate");
        free(st);
        free(rt);
        return NULL;
    }
    if (hipDeviceGetAttribute(&st->compute_units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || st->compute_units <= 0)
        st->compute_units = 256;
    if (open_common(st, error) != 0) {
        hipStreamDestroy(st->stream);
        free(st);
        free(rt);
        return NULL;
    }
    rt->name = path == KIPP_PATH_GPU_BF16 ? "gpu-bf16" : "gpu-fp32";
    rt->path = path;
    rt->act_dtype = path == KIPP_PATH_GPU_BF16 ? KIPP_BF16 : KIPP_F32;
    rt->on_host = false;
    rt->destroy = hip_destroy;
    rt->mem_alloc = hip_alloc;
    rt->mem_free = hip_free;
    rt->mem_zero = hip_zero;
    rt->upload = hip_upload;
    rt->download = hip_download;
    rt->copy = hip_copy;
    rt->place_matrix = hip_place_matrix;
    rt->place_vector = hip_place_vector;
    rt->free_weight = hip_free_weight;
    rt->embed = hip_embed;
    rt->rmsnorm = hip_rmsnorm;
    rt->residual_add = hip_residual_add;
    rt->linear = hip_linear;
    rt->swiglu = hip_swiglu;
    rt->rotary_angles = hip_rotary_angles;
    rt->qk_norm_rope_kv = hip_qk_norm_rope_kv;
    rt->attention = hip_attention;
    rt->gather_rows = hip_gather_rows;
    rt->defers = hip_defers;
    rt->scale_rows = hip_scale_rows;
    rt->gated = hip_gated;
    rt->decode_attention = hip_decode_attention;
    rt->argmax = hip_argmax;
    rt->sample = hip_sample;
    rt->row_nll = hip_row_nll;
    rt->after_failed_step = hip_after_failed_step;
    if (path == KIPP_PATH_GPU_BF16) { /* the 32-bit path is for checking, not for speed: its steps run as they are */
        rt->graph_begin = hip_graph_begin;
        rt->graph_end = hip_graph_end;
        rt->graph_launch = hip_graph_launch;
        rt->graph_free = hip_graph_free;
    }
    return rt;
}
