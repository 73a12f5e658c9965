/* What both tables of operations share: the step's workspace and small helpers. */
#include <stdlib.h>
#include <string.h>

#include "backend.h"

#define KIPP_CHUNK ((size_t)32 << 20)

size_t kipp_dtype_bytes(int dtype) { return dtype == KIPP_F32 ? 4 : 2; }

/* The workspace is a list of chunks that are made when a step first needs them and kept: a step takes memory from
 * the start of the list again, so a steady stream of steps allocates nothing. */
void *kipp_scratch(kipp_runtime *rt, size_t bytes, kipp_error *error) {
    bytes = (bytes + 255) & ~(size_t)255;
    if (bytes == 0) bytes = 256;
    while (rt->workspace.current < rt->workspace.count) {
        if (rt->workspace.sizes[rt->workspace.current] - rt->workspace.used >= bytes) {
            void *at = (char *)rt->workspace.chunks[rt->workspace.current] + rt->workspace.used;
            rt->workspace.used += bytes;
            return at;
        }
        ++rt->workspace.current;
        rt->workspace.used = 0;
    }
    if (rt->recording) {
        /* memory cannot be made while operations are recorded: the caller drops the recording and runs the step as it is */
        kipp_fail(error, KIPP_ERROR_MEMORY, "the step's workspace would grow while a step is recorded");
        return NULL;
    }
    size_t size = bytes > KIPP_CHUNK ? bytes : KIPP_CHUNK;
    void **chunks = realloc(rt->workspace.chunks, (rt->workspace.count + 1) * sizeof(void *));
    if (chunks != NULL) rt->workspace.chunks = chunks;
    size_t *sizes = chunks != NULL ? realloc(rt->workspace.sizes, (rt->workspace.count + 1) * sizeof(size_t)) : NULL;
    if (sizes != NULL) rt->workspace.sizes = sizes;
    if (chunks == NULL || sizes == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for the step's workspace");
        return NULL;
    }
    void *chunk = rt->mem_alloc(rt, size, error);
    if (chunk == NULL) return NULL;
    rt->workspace.chunks[rt->workspace.count] = chunk;
    rt->workspace.sizes[rt->workspace.count] = size;
    rt->workspace.current = rt->workspace.count++;
    rt->workspace.used = bytes;
    return chunk;
}

void kipp_scratch_reset(kipp_runtime *rt) {
    rt->workspace.current = 0;
    rt->workspace.used = 0;
}

int kipp_settle(kipp_runtime *rt, kipp_delta *delta, kipp_error *error) {
    if (delta->parts > 0 || delta->w == NULL) return 0;
    const kipp_rows x = {(void *)delta->x, NULL, 0, 0.0f, delta->x_steps_major};
    const kipp_weight *w = delta->w;
    delta->w = NULL; /* what linear writes is a delta that has been launched */
    return rt->linear(rt, &x, w, delta->m, delta->max_parts, delta, error);
}

int kipp_finish_rows(kipp_runtime *rt, kipp_rows *rows, uint32_t m, uint32_t width, kipp_error *error) {
    if (rows->sumsq == NULL) return 0;
    if (rt->scale_rows == NULL) return kipp_fail(error, KIPP_ERROR_INTERNAL, "rows without their scale on a path that leaves none");
    void *out = kipp_scratch(rt, (size_t)m * width * kipp_dtype_bytes(rt->act_dtype), error);
    if (out == NULL || rt->scale_rows(rt, rows, out, m, width, error) != 0) return -1;
    *rows = (kipp_rows){out, NULL, 0, 0.0f, false};
    return 0;
}

int kipp_linear_defer(kipp_runtime *rt, const kipp_rows *x, const kipp_weight *w, uint32_t m, int max_parts, kipp_delta *out, kipp_error *error) {
    if (rt->defers != NULL && x->sumsq == NULL && rt->defers(rt, x, w, m)) {
        *out = (kipp_delta){NULL, 0, x->data, w, m, max_parts, x->steps_major};
        return 0;
    }
    return rt->linear(rt, x, w, m, max_parts, out, error);
}

void kipp_runtime_destroy(kipp_runtime *rt) {
    if (rt == NULL) return;
    for (size_t i = 0; i < rt->workspace.count; ++i) rt->mem_free(rt, rt->workspace.chunks[i]);
    free(rt->workspace.chunks);
    free(rt->workspace.sizes);
    rt->destroy(rt);
}

#ifdef KIPP_NO_HIP
/* A build without the GPU's table (the host logic alone, as the sanitizer build is): the GPU paths say so. */
kipp_runtime *kipp_runtime_hip(kipp_path path, int device, const char *kernel_dir, kipp_error *error) {
    (void)path;
    (void)device;
    (void)kernel_dir;
    kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "this build of the library has no GPU paths (cpu-fp32 only)");
    return NULL;
}
#endif
