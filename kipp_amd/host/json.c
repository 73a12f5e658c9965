/*
 * A strict JSON reader for config.json and safetensors headers (the reference
 * reads its own with /root/reference/src/kipp_json.c).  The whole document becomes one
 * array of nodes plus one block of decoded strings.  Strict: one value and
 * nothing behind it, no duplicate keys, no control characters inside strings,
 * no leading zeros, no NaN or Infinity, surrogates must pair, at most 64 levels.
 */
#include <errno.h>
#include <fcntl.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include "internal.h"

#define KJ_MAX_DEPTH 64

typedef struct {
    const char *text;
    size_t length, at;
    kj_doc *doc;
    kipp_error *error;
} kj_reader;

static int kj_bad(kj_reader *r, const char *what) {
    return kipp_fail(r->error, KIPP_ERROR_FORMAT, "JSON: %s at byte %zu", what, r->at);
}

static void kj_space(kj_reader *r) {
    while (r->at < r->length) {
        char c = r->text[r->at];
        if (c != ' ' && c != '\t' && c != '\n' && c != '\r') break;
        ++r->at;
    }
}

static int kj_new_node(kj_reader *r, uint32_t *index) {
    kj_doc *doc = r->doc;
    if (doc->count == doc->capacity) {
        size_t capacity = doc->capacity == 0 ? 64 : doc->capacity * 2;
        kj_node *grown = realloc(doc->nodes, capacity * sizeof(kj_node));
        if (grown == NULL) return kipp_fail(r->error, KIPP_ERROR_MEMORY, "JSON: out of memory");
        doc->nodes = grown;
        doc->capacity = capacity;
    }
    if (doc->count >= UINT32_MAX) return kj_bad(r, "too many values");
    *index = (uint32_t)doc->count++;
    memset(&doc->nodes[*index], 0, sizeof(kj_node));
    return 0;
}

static int kj_hex4(kj_reader *r, uint32_t *value) {
    if (r->length - r->at < 4) return kj_bad(r, "short \\u escape");
    *value = 0;
    for (int i = 0; i < 4; ++i) {
        char c = r->text[r->at++];
        uint32_t digit;
        if (c >= '0' && c <= '9') digit = (uint32_t)(c - '0');
        else if (c >= 'a' && c <= 'f') digit = (uint32_t)(c - 'a' + 10);
        else if (c >= 'A' && c <= 'F') digit = (uint32_t)(c - 'A' + 10);
        else return kj_bad(r, "bad \\u escape");
        *value = *value * 16 + digit;
    }
    return 0;
}

/* Decodes a string (the reader stands behind its opening quote) into the strings block, which was
 * reserved to the length of the whole text before parsing: a decoded string is never longer than its source,
 * so pointers into the block stay valid. */
static int kj_string(kj_reader *r, const char **out, size_t *out_length) {
    kj_doc *doc = r->doc;
    char *begin = doc->strings + doc->strings_length, *to = begin;
    for (;;) {
        if (r->at >= r->length) return kj_bad(r, "unterminated string");
        unsigned char c = (unsigned char)r->text[r->at++];
        if (c == '"') break;
        if (c < 0x20) return kj_bad(r, "control character in a string");
        if (c != '\\') {
            *to++ = (char)c;
            continue;
        }
        if (r->at >= r->length) return kj_bad(r, "unterminated escape");
        c = (unsigned char)r->text[r->at++];
        switch (c) {
            case '"': *to++ = '"'; break;
            case '\\': *to++ = '\\'; break;
            case '/': *to++ = '/'; break;
            case 'b': *to++ = '\b'; break;
            case 'f': *to++ = '\f'; break;
            case 'n': *to++ = '\n'; break;
            case 'r': *to++ = '\r'; break;
            case 't': *to++ = '\t'; break;
            case 'u': {
                uint32_t code, low;
                if (kj_hex4(r, &code) != 0) return -1;
                if (code >= 0xdc00 && code <= 0xdfff) return kj_bad(r, "lone low surrogate");
                if (code >= 0xd800 && code <= 0xdbff) {
                    if (r->length - r->at < 2 || r->text[r->at] != '\\' || r->text[r->at + 1] != 'u') return kj_bad(r, "lone high surrogate");
                    r->at += 2;
                    if (kj_hex4(r, &low) != 0) return -1;
                    if (low < 0xdc00 || low > 0xdfff) return kj_bad(r, "bad surrogate pair");
                    code = 0x10000 + ((code - 0xd800) << 10) + (low - 0xdc00);
                }
                if (code == 0) return kj_bad(r, "NUL inside a string");
                if (code < 0x80) *to++ = (char)code;
                else if (code < 0x800) {
                    *to++ = (char)(0xc0 | (code >> 6));
                    *to++ = (char)(0x80 | (code & 0x3f));
                } else if (code < 0x10000) {
                    *to++ = (char)(0xe0 | (code >> 12));
                    *to++ = (char)(0x80 | ((code >> 6) & 0x3f));
                    *to++ = (char)(0x80 | (code & 0x3f));
                } else {
                    *to++ = (char)(0xf0 | (code >> 18));
                    *to++ = (char)(0x80 | ((code >> 12) & 0x3f));
                    *to++ = (char)(0x80 | ((code >> 6) & 0x3f));
                    *to++ = (char)(0x80 | (code & 0x3f));
                }
                break;
            }
            default: return kj_bad(r, "unknown escape");
        }
    }
    *to++ = '\0';
    *out = begin;
    *out_length = (size_t)(to - begin) - 1;
    doc->strings_length += (size_t)(to - begin);
    return 0;
}

static int kj_number(kj_reader *r, kj_node *node) {
    size_t begin = r->at;
    bool integer = true;
    if (r->at < r->length && r->text[r->at] == '-') ++r->at;
    if (r->at >= r->length) return kj_bad(r, "number expected");
    if (r->text[r->at] == '0') {
        ++r->at;
        if (r->at < r->length && r->text[r->at] >= '0' && r->text[r->at] <= '9') return kj_bad(r, "leading zero");
    } else if (r->text[r->at] >= '1' && r->text[r->at] <= '9') {
        while (r->at < r->length && r->text[r->at] >= '0' && r->text[r->at] <= '9') ++r->at;
    } else {
        return kj_bad(r, "number expected");
    }
    if (r->at < r->length && r->text[r->at] == '.') {
        integer = false;
        ++r->at;
        if (r->at >= r->length || r->text[r->at] < '0' || r->text[r->at] > '9') return kj_bad(r, "digits expected behind the point");
        while (r->at < r->length && r->text[r->at] >= '0' && r->text[r->at] <= '9') ++r->at;
    }
    if (r->at < r->length && (r->text[r->at] == 'e' || r->text[r->at] == 'E')) {
        integer = false;
        ++r->at;
        if (r->at < r->length && (r->text[r->at] == '+' || r->text[r->at] == '-')) ++r->at;
        if (r->at >= r->length || r->text[r->at] < '0' || r->text[r->at] > '9') return kj_bad(r, "digits expected in the exponent");
        while (r->at < r->length && r->text[r->at] >= '0' && r->text[r->at] <= '9') ++r->at;
    }
    char buffer[64];
    size_t length = r->at - begin;
    if (length >= sizeof(buffer)) return kj_bad(r, "number too long");
    memcpy(buffer, r->text + begin, length);
    buffer[length] = '\0';
    errno = 0;
    node->type = KJ_NUMBER;
    node->number = strtod(buffer, NULL);
    if (!isfinite(node->number)) return kj_bad(r, "number out of range");
    if (integer) {
        errno = 0;
        long long value = strtoll(buffer, NULL, 10);
        if (errno == 0) {
            node->is_integer = true;
            node->integer = (int64_t)value;
        }
    }
    return 0;
}

static int kj_value(kj_reader *r, uint32_t *out_index, int depth);

static int kj_container(kj_reader *r, uint32_t self, bool object, int depth) {
    uint32_t last = 0, count = 0;
    char close = object ? '}' : ']';
    kj_space(r);
    if (r->at < r->length && r->text[r->at] == close) {
        ++r->at;
        return 0;
    }
    for (;;) {
        const char *key = NULL;
        size_t key_length = 0;
        uint32_t child;
        kj_space(r);
        if (object) {
            if (r->at >= r->length || r->text[r->at] != '"') return kj_bad(r, "a key expected");
            ++r->at;
            if (kj_string(r, &key, &key_length) != 0) return -1;
            for (uint32_t at = r->doc->nodes[self].first; at != 0; at = r->doc->nodes[at].next) {
                if (strcmp(r->doc->nodes[at].key, key) == 0) return kj_bad(r, "duplicate key");
            }
            kj_space(r);
            if (r->at >= r->length || r->text[r->at] != ':') return kj_bad(r, "':' expected");
            ++r->at;
        }
        if (kj_value(r, &child, depth + 1) != 0) return -1;
        r->doc->nodes[child].key = key;
        if (last == 0) r->doc->nodes[self].first = child;
        else r->doc->nodes[last].next = child;
        last = child;
        r->doc->nodes[self].count = ++count;
        kj_space(r);
        if (r->at >= r->length) return kj_bad(r, "unterminated array or object");
        if (r->text[r->at] == ',') {
            ++r->at;
            continue;
        }
        if (r->text[r->at] == close) {
            ++r->at;
            return 0;
        }
        return kj_bad(r, "',' or a closing bracket expected");
    }
}

static bool kj_literal(kj_reader *r, const char *word) {
    size_t length = strlen(word);
    if (r->length - r->at < length || memcmp(r->text + r->at, word, length) != 0) return false;
    r->at += length;
    return true;
}

static int kj_value(kj_reader *r, uint32_t *out_index, int depth) {
    uint32_t index;
    if (depth > KJ_MAX_DEPTH) return kj_bad(r, "nested too deeply");
    kj_space(r);
    if (r->at >= r->length) return kj_bad(r, "a value expected");
    if (kj_new_node(r, &index) != 0) return -1;
    *out_index = index;
    char c = r->text[r->at];
    if (c == '{' || c == '[') {
        ++r->at;
        r->doc->nodes[index].type = c == '{' ? KJ_OBJECT : KJ_ARRAY;
        return kj_container(r, index, c == '{', depth);
    }
    if (c == '"') {
        const char *string;
        size_t length;
        ++r->at;
        if (kj_string(r, &string, &length) != 0) return -1;
        r->doc->nodes[index].type = KJ_STRING;
        r->doc->nodes[index].string = string;
        r->doc->nodes[index].string_length = length;
        return 0;
    }
    if (kj_literal(r, "true")) {
        r->doc->nodes[index].type = KJ_BOOL;
        r->doc->nodes[index].boolean = true;
        return 0;
    }
    if (kj_literal(r, "false")) {
        r->doc->nodes[index].type = KJ_BOOL;
        return 0;
    }
    if (kj_literal(r, "null")) {
        r->doc->nodes[index].type = KJ_NULL;
        return 0;
    }
    {
        kj_node node;
        memset(&node, 0, sizeof(node));
        if (kj_number(r, &node) != 0) return -1;
        r->doc->nodes[index] = node;
    }
    return 0;
}

int kj_parse(const char *text, size_t length, kj_doc *doc, kipp_error *error) {
    kj_reader r = {text, length, 0, doc, error};
    uint32_t root;
    memset(doc, 0, sizeof(*doc));
    /* node 0 is never a child (0 means "none" in the links): a placeholder stands there, the root is node 1 */
    doc->strings_capacity = length + 1;
    doc->strings = malloc(doc->strings_capacity);
    if (doc->strings == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "JSON: out of memory");
    if (kj_new_node(&r, &root) != 0 || kj_value(&r, &root, 0) != 0) {
        kj_free(doc);
        return -1;
    }
    kj_space(&r);
    if (r.at != length) {
        kj_bad(&r, "something follows the value");
        kj_free(doc);
        return -1;
    }
    return 0;
}

void kj_free(kj_doc *doc) {
    free(doc->nodes);
    free(doc->strings);
    memset(doc, 0, sizeof(*doc));
}

const kj_node *kj_root(const kj_doc *doc) { return doc->count > 1 ? &doc->nodes[1] : NULL; }

const kj_node *kj_first(const kj_doc *doc, const kj_node *parent) {
    return parent != NULL && parent->first != 0 ? &doc->nodes[parent->first] : NULL;
}

const kj_node *kj_next(const kj_doc *doc, const kj_node *child) {
    return child != NULL && child->next != 0 ? &doc->nodes[child->next] : NULL;
}

const kj_node *kj_get(const kj_doc *doc, const kj_node *object, const char *key) {
    if (object == NULL || object->type != KJ_OBJECT) return NULL;
    for (const kj_node *child = kj_first(doc, object); child != NULL; child = kj_next(doc, child)) {
        if (strcmp(child->key, key) == 0) return child;
    }
    return NULL;
}

int kipp_read_file(const char *path, char **out_text, size_t *out_length, kipp_error *error) {
    struct stat st;
    int fd = open(path, O_RDONLY);
    if (fd < 0) return kipp_fail(error, KIPP_ERROR_IO, "cannot open %s: %s", path, strerror(errno));
    if (fstat(fd, &st) != 0 || st.st_size < 0 || (uint64_t)st.st_size > (uint64_t)1 << 30) {
        close(fd);
        return kipp_fail(error, KIPP_ERROR_IO, "cannot read %s: not a file of reasonable size", path);
    }
    size_t length = (size_t)st.st_size, got = 0;
    char *text = malloc(length + 1);
    if (text == NULL) {
        close(fd);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory reading %s", path);
    }
    while (got < length) {
        ssize_t n = read(fd, text + got, length - got);
        if (n <= 0) {
            close(fd);
            free(text);
            return kipp_fail(error, KIPP_ERROR_IO, "cannot read %s", path);
        }
        got += (size_t)n;
    }
    close(fd);
    text[length] = '\0';
    *out_text = text;
    *out_length = length;
    return 0;
}
