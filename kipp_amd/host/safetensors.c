/*
 * safetensors, read in place: an 8-byte little-endian header length, a JSON
 * header {name: {dtype, shape, data_offsets}}, then the payload; offsets count
 * from the payload's start (as the reference's converter reads it,
 * /root/reference/tools/convert_to_gguf.py:282-343).  A file is mapped read-only and
 * tensors point into the mapping; a folder holds model.safetensors, or the shards
 * that model.safetensors.index.json names in its weight_map.
 *
 * Checked here (format errors of the file itself; whether the tensors are the
 * ones the model needs is the loader's question): the header fits the file,
 * every entry has dtype, shape and two offsets, the span equals
 * product(shape) x element size, lies inside the payload and overlaps no other
 * (/root/reference/src/kipp.c:1032-1061 has the reference's overlap and range checks).
 */
#include <errno.h>
#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "internal.h"

#define KIPP_MAX_HEADER ((uint64_t)100 << 20)

static const struct {
    const char *name;
    int code;
    uint32_t bytes;
} dtypes[] = {{"F32", KIPP_F32, 4}, {"BF16", KIPP_BF16, 2}, {"F16", KIPP_F16, 2}, {"F64", -1, 8}, {"I64", -1, 8}, {"I32", -1, 4},
              {"I16", -1, 2},       {"I8", -1, 1},          {"U8", -1, 1},        {"BOOL", -1, 1}};

typedef struct {
    uint64_t begin, end;
    size_t tensor;
} span;

static int compare_spans(const void *a, const void *b) {
    const span *x = a, *y = b;
    if (x->begin != y->begin) return x->begin < y->begin ? -1 : 1;
    if (x->end != y->end) return x->end < y->end ? -1 : 1;
    return 0;
}

static int add_tensor(kipp_tensor_file *file, const kipp_tensor *tensor, kipp_error *error) {
    if (file->tensor_count == file->tensor_capacity) {
        size_t capacity = file->tensor_capacity == 0 ? 64 : file->tensor_capacity * 2;
        kipp_tensor *grown = realloc(file->tensors, capacity * sizeof(kipp_tensor));
        if (grown == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for the tensor directory");
        file->tensors = grown;
        file->tensor_capacity = capacity;
    }
    file->tensors[file->tensor_count++] = *tensor;
    return 0;
}

/* Maps one file and adds its tensors; `only_of` (may be NULL) is the weight_map of an index: a tensor is taken
 * only if the map names this shard for it. */
static int open_one(kipp_tensor_file *file, const char *path, const char *shard, const kj_doc *index_doc, const kj_node *weight_map,
                    kipp_error *error) {
    struct stat st;
    int fd = open(path, O_RDONLY);
    if (fd < 0) return kipp_fail(error, KIPP_ERROR_IO, "cannot open %s: %s", path, strerror(errno));
    if (fstat(fd, &st) != 0 || st.st_size < 0) {
        close(fd);
        return kipp_fail(error, KIPP_ERROR_IO, "cannot stat %s", path);
    }
    uint64_t size = (uint64_t)st.st_size;
    if (size < 8) {
        close(fd);
        return kipp_fail(error, KIPP_ERROR_FORMAT, "%s: truncated before the header length", path);
    }
    void *mapping = mmap(NULL, (size_t)size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (mapping == MAP_FAILED) return kipp_fail(error, KIPP_ERROR_IO, "cannot map %s: %s", path, strerror(errno));
    {
        void **maps = realloc(file->mappings, (file->mapping_count + 1) * sizeof(void *));
        size_t *sizes = maps != NULL ? realloc(file->mapping_sizes, (file->mapping_count + 1) * sizeof(size_t)) : NULL;
        if (maps != NULL) file->mappings = maps;
        if (sizes != NULL) file->mapping_sizes = sizes;
        if (maps == NULL || sizes == NULL) {
            munmap(mapping, (size_t)size);
            return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        }
        file->mappings[file->mapping_count] = mapping;
        file->mapping_sizes[file->mapping_count++] = (size_t)size;
        file->mapped_bytes += size;
    }
    const unsigned char *bytes = mapping;
    uint64_t header_length = 0;
    for (int i = 7; i >= 0; --i) header_length = (header_length << 8) | bytes[i];
    if (header_length > KIPP_MAX_HEADER || header_length > size - 8)
        return kipp_fail(error, KIPP_ERROR_FORMAT, "%s: header length %llu does not fit the file (%llu bytes)", path,
                         (unsigned long long)header_length, (unsigned long long)size);
    uint64_t base = 8 + header_length, payload = size - base;
    kj_doc doc;
    kipp_error inner;
    if (kj_parse((const char *)bytes + 8, (size_t)header_length, &doc, &inner) != 0)
        return kipp_fail(error, KIPP_ERROR_FORMAT, "%s: header is not valid JSON (%.200s)", path, inner.message);
    int rc = -1;
    span *spans = NULL;
    size_t span_count = 0;
    const kj_node *root = kj_root(&doc);
    if (root == NULL || root->type != KJ_OBJECT) {
        kipp_fail(error, KIPP_ERROR_FORMAT, "%s: header must be a JSON object", path);
        goto done;
    }
    spans = malloc((root->count + 1) * sizeof(span));
    if (spans == NULL) {
        kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        goto done;
    }
    size_t first_new = file->tensor_count;
    for (const kj_node *entry = kj_first(&doc, root); entry != NULL; entry = kj_next(&doc, entry)) {
        if (strcmp(entry->key, "__metadata__") == 0) continue;
        const char *name = entry->key;
        if (weight_map != NULL) {
            const kj_node *owner = kj_get(index_doc, weight_map, name);
            if (owner == NULL || owner->type != KJ_STRING || strcmp(owner->string, shard) != 0) continue;
        }
        const kj_node *dtype = kj_get(&doc, entry, "dtype"), *shape = kj_get(&doc, entry, "shape"),
                      *offsets = kj_get(&doc, entry, "data_offsets");
        if (entry->type != KJ_OBJECT || dtype == NULL || dtype->type != KJ_STRING || shape == NULL || shape->type != KJ_ARRAY ||
            offsets == NULL || offsets->type != KJ_ARRAY || offsets->count != 2) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: entry '%s' is malformed", path, name);
            goto done;
        }
        kipp_tensor tensor;
        memset(&tensor, 0, sizeof(tensor));
        if (strlen(name) >= sizeof(tensor.name)) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: a tensor name is longer than %zu bytes", path, sizeof(tensor.name) - 1);
            goto done;
        }
        snprintf(tensor.name, sizeof(tensor.name), "%s", name);
        uint32_t width = 0;
        tensor.dtype = -2;
        for (size_t i = 0; i < sizeof(dtypes) / sizeof(dtypes[0]); ++i) {
            if (strcmp(dtypes[i].name, dtype->string) == 0) {
                tensor.dtype = dtypes[i].code;
                width = dtypes[i].bytes;
            }
        }
        if (tensor.dtype == -2) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensor '%s' has unsupported dtype '%.20s'", path, name, dtype->string);
            goto done;
        }
        snprintf(tensor.dtype_name, sizeof(tensor.dtype_name), "%s", dtype->string);
        if (shape->count > 4) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensor '%s' has %u dimensions", path, name, shape->count);
            goto done;
        }
        size_t count = 1;
        for (const kj_node *dim = kj_first(&doc, shape); dim != NULL; dim = kj_next(&doc, dim)) {
            if (dim->type != KJ_NUMBER || !dim->is_integer || dim->integer < 0 || kipp_mul_size(count, (size_t)dim->integer, &count) != 0) {
                kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensor '%s' has a bad shape", path, name);
                goto done;
            }
            tensor.shape[tensor.ndim++] = (uint64_t)dim->integer;
        }
        const kj_node *b = kj_first(&doc, offsets), *e = kj_next(&doc, b);
        if (b->type != KJ_NUMBER || !b->is_integer || e->type != KJ_NUMBER || !e->is_integer || b->integer < 0 || e->integer < b->integer ||
            (uint64_t)e->integer > payload) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensor '%s' lies outside the file", path, name);
            goto done;
        }
        size_t need;
        if (kipp_mul_size(count, width, &need) != 0 || (uint64_t)(e->integer - b->integer) != need) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensor '%s' spans %lld bytes but its shape of %s needs %zu", path, name,
                      (long long)(e->integer - b->integer), dtype->string, count * (size_t)width);
            goto done;
        }
        tensor.data = bytes + base + (uint64_t)b->integer;
        tensor.bytes = need;
        if (kipp_tensors_find(file, name) != NULL) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensor '%s' is already there from another shard", path, name);
            goto done;
        }
        if (add_tensor(file, &tensor, error) != 0) goto done;
        spans[span_count++] = (span){(uint64_t)b->integer, (uint64_t)e->integer, file->tensor_count - 1};
    }
    qsort(spans, span_count, sizeof(span), compare_spans);
    for (size_t i = 1; i < span_count; ++i) {
        if (spans[i].begin < spans[i - 1].end) {
            kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensors '%s' and '%s' overlap", path, file->tensors[spans[i - 1].tensor].name,
                      file->tensors[spans[i].tensor].name);
            goto done;
        }
    }
    (void)first_new;
    rc = 0;
done:
    free(spans);
    kj_free(&doc);
    return rc;
}

int kipp_tensors_open(const char *model_dir, kipp_tensor_file *out, kipp_error *error) {
    char index_path[4096], path[4096];
    memset(out, 0, sizeof(*out));
    if (snprintf(index_path, sizeof(index_path), "%s/model.safetensors.index.json", model_dir) >= (int)sizeof(index_path))
        return kipp_fail(error, KIPP_ERROR_ARGUMENT, "the model folder's path is too long");
    if (access(index_path, R_OK) == 0) {
        char *text;
        size_t length;
        kj_doc doc;
        if (kipp_read_file(index_path, &text, &length, error) != 0) return -1;
        if (kj_parse(text, length, &doc, error) != 0) {
            free(text);
            return -1;
        }
        int rc = 0;
        const kj_node *map = kj_get(&doc, kj_root(&doc), "weight_map");
        if (map == NULL || map->type != KJ_OBJECT) rc = kipp_fail(error, KIPP_ERROR_FORMAT, "%s: no weight_map", index_path);
        /* every shard once, in the order in which the map first names it */
        for (const kj_node *entry = kj_first(&doc, map); rc == 0 && entry != NULL; entry = kj_next(&doc, entry)) {
            bool seen = false;
            if (entry->type != KJ_STRING || strchr(entry->string, '/') != NULL) {
                rc = kipp_fail(error, KIPP_ERROR_FORMAT, "%s: weight_map['%s'] is not a file name", index_path, entry->key);
                break;
            }
            for (const kj_node *before = kj_first(&doc, map); before != entry; before = kj_next(&doc, before)) {
                if (before->type == KJ_STRING && strcmp(before->string, entry->string) == 0) seen = true;
            }
            if (seen) continue;
            if (snprintf(path, sizeof(path), "%s/%s", model_dir, entry->string) >= (int)sizeof(path))
                rc = kipp_fail(error, KIPP_ERROR_ARGUMENT, "a shard's path is too long");
            else
                rc = open_one(out, path, entry->string, &doc, map, error);
        }
        if (rc == 0) {
            kipp_text absent = {0};
            for (const kj_node *entry = kj_first(&doc, map); entry != NULL; entry = kj_next(&doc, entry)) {
                if (kipp_tensors_find(out, entry->key) == NULL) kipp_text_add(&absent, "%s%s", absent.length ? ", " : "", entry->key);
            }
            if (absent.length != 0) rc = kipp_fail(error, KIPP_ERROR_FORMAT, "%s: tensors listed but absent from their shard: %s", index_path, absent.data);
            kipp_text_free(&absent);
        }
        kj_free(&doc);
        free(text);
        if (rc != 0) kipp_tensors_close(out);
        return rc;
    }
    snprintf(path, sizeof(path), "%s/model.safetensors", model_dir);
    if (access(path, R_OK) != 0)
        return kipp_fail(error, KIPP_ERROR_IO, "%s: neither model.safetensors nor model.safetensors.index.json", model_dir);
    if (open_one(out, path, NULL, NULL, NULL, error) != 0) {
        kipp_tensors_close(out);
        return -1;
    }
    return 0;
}

void kipp_tensors_close(kipp_tensor_file *file) {
    for (size_t i = 0; i < file->mapping_count; ++i) munmap(file->mappings[i], file->mapping_sizes[i]);
    free(file->mappings);
    free(file->mapping_sizes);
    free(file->tensors);
    memset(file, 0, sizeof(*file));
}

kipp_tensor *kipp_tensors_find(const kipp_tensor_file *file, const char *name) {
    for (size_t i = 0; i < file->tensor_count; ++i) {
        if (strcmp(file->tensors[i].name, name) == 0) return &file->tensors[i];
    }
    return NULL;
}
