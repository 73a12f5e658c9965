/* The error record, checked size arithmetic and a growing text
 * (/root/reference/src/kipp.c:201-248 has the reference's `fail` and checked sizes). */
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "internal.h"

int kipp_fail(kipp_error *error, kipp_error_code code, const char *format, ...) {
    if (error != NULL) {
        va_list args;
        error->code = code;
        va_start(args, format);
        vsnprintf(error->message, sizeof(error->message), format, args);
        va_end(args);
    }
    return -1;
}

void kipp_error_clear(kipp_error *error) {
    if (error != NULL) {
        error->code = KIPP_OK;
        error->message[0] = '\0';
    }
}

int kipp_add_size(size_t left, size_t right, size_t *result) {
    if (left > SIZE_MAX - right) return -1;
    *result = left + right;
    return 0;
}

int kipp_mul_size(size_t left, size_t right, size_t *result) {
    if (right != 0 && left > SIZE_MAX / right) return -1;
    *result = left * right;
    return 0;
}

const char *kipp_error_code_name(kipp_error_code code) {
    switch (code) {
        case KIPP_OK: return "ok";
        case KIPP_ERROR_ARGUMENT: return "argument";
        case KIPP_ERROR_IO: return "io";
        case KIPP_ERROR_FORMAT: return "format";
        case KIPP_ERROR_UNSUPPORTED: return "unsupported";
        case KIPP_ERROR_MEMORY: return "memory";
        case KIPP_ERROR_RANGE: return "range";
        case KIPP_ERROR_INTERNAL: return "internal";
    }
    return "unknown";
}

const char *kipp_path_name(kipp_path path) {
    switch (path) {
        case KIPP_PATH_GPU_BF16: return "gpu-bf16";
        case KIPP_PATH_GPU_FP32: return "gpu-fp32";
        case KIPP_PATH_CPU_FP32: return "cpu-fp32";
    }
    return "unknown";
}

const char *kipp_backend_name(kipp_path path) { return kipp_path_name(path); }

void kipp_text_add(kipp_text *text, const char *format, ...) {
    if (text->failed) return;
    for (;;) {
        va_list args;
        size_t room = text->capacity - text->length;
        int wrote;
        va_start(args, format);
        wrote = vsnprintf(text->data != NULL ? text->data + text->length : NULL, text->data != NULL ? room : 0, format, args);
        va_end(args);
        if (wrote < 0) {
            text->failed = true;
            return;
        }
        if (text->data != NULL && (size_t)wrote < room) {
            text->length += (size_t)wrote;
            return;
        }
        size_t capacity = text->capacity == 0 ? 256 : text->capacity * 2;
        while (capacity < text->length + (size_t)wrote + 1) capacity *= 2;
        char *grown = realloc(text->data, capacity);
        if (grown == NULL) {
            text->failed = true;
            return;
        }
        text->data = grown;
        text->capacity = capacity;
        text->data[text->length] = '\0';
    }
}

void kipp_text_free(kipp_text *text) {
    free(text->data);
    memset(text, 0, sizeof(*text));
}

int kipp_test_checked_add_size(size_t left, size_t right, size_t *result) { return kipp_add_size(left, right, result); }
int kipp_test_checked_multiply_size(size_t left, size_t right, size_t *result) { return kipp_mul_size(left, right, result); }
