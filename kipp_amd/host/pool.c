/*
 * Bookkeeping of one pool of pages: who holds a page, which pages are free,
 * and which pages carry known content.
 *
 * A page is either held (ref count > 0) or on the free list, which runs from
 * the least to the most recently released page; `alloc` takes the oldest.  A
 * full page can be sealed: its tokens and the hash chained from the pages
 * before it go into an index (buckets of chained pages), so that a later
 * session with the same beginning adopts the page instead of computing it
 * again.  A sealed page that became free stays in the index until it is taken
 * for new content; a hit is always verified by the tokens, never by the hash
 * alone (/root/reference/src/kipp_kv_pool.c:13-22, 48-64, 176-190, 202-304).
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "internal.h"

#define FNV_OFFSET 1469598103934665603ull
#define FNV_PRIME 1099511628211ull

uint64_t kipp_pool_chain_hash(uint64_t parent, const uint32_t *tokens, size_t count) {
    uint64_t h = FNV_OFFSET;
    for (int shift = 0; shift < 64; shift += 8) h = (h ^ ((parent >> shift) & 0xff)) * FNV_PRIME;
    for (size_t i = 0; i < count; ++i) {
        for (int shift = 0; shift < 32; shift += 8) h = (h ^ ((tokens[i] >> shift) & 0xff)) * FNV_PRIME;
    }
    return h;
}

uint64_t kipp_test_chain_hash(uint64_t parent, const uint32_t *tokens, size_t count) { return kipp_pool_chain_hash(parent, tokens, count); }

static uint64_t pool_hash(const kipp_pool *pool, uint64_t parent, const uint32_t *tokens) {
    return pool->force_hash ? pool->forced_hash : kipp_pool_chain_hash(parent, tokens, pool->page_tokens);
}

static void free_list_push(kipp_pool *pool, uint32_t page) {
    kipp_page *p = &pool->pages[page];
    p->prev_free = pool->free_tail;
    p->next_free = KIPP_NO_PAGE;
    if (pool->free_tail != KIPP_NO_PAGE) pool->pages[pool->free_tail].next_free = page;
    else pool->free_head = page;
    pool->free_tail = page;
    p->on_free_list = true;
    ++pool->free_count;
}

static void free_list_remove(kipp_pool *pool, uint32_t page) {
    kipp_page *p = &pool->pages[page];
    if (p->prev_free != KIPP_NO_PAGE) pool->pages[p->prev_free].next_free = p->next_free;
    else pool->free_head = p->next_free;
    if (p->next_free != KIPP_NO_PAGE) pool->pages[p->next_free].prev_free = p->prev_free;
    else pool->free_tail = p->prev_free;
    p->prev_free = p->next_free = KIPP_NO_PAGE;
    p->on_free_list = false;
    --pool->free_count;
}

/* 0 .. n - 1 in an order in which neighbours lie far apart (steps of about 0.618 n, coprime to n): sequences of
 * equal length that arrive together would otherwise lie at equal, often power-of-two distances in memory, and
 * kernels that walk them in step would find every sequence's current page in the same memory channel. */
static uint32_t gcd32(uint32_t a, uint32_t b) {
    while (b != 0) {
        uint32_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

int kipp_pool_init(kipp_pool *pool, uint32_t page_count, uint32_t page_tokens, const uint32_t *order, kipp_error *error) {
    memset(pool, 0, sizeof(*pool));
    if (page_count == 0 || page_tokens == 0 || page_count >= KIPP_NO_PAGE / 2)
        return kipp_fail(error, KIPP_ERROR_ARGUMENT, "a pool needs at least one page of at least one token");
    size_t token_slots;
    if (kipp_mul_size(page_count, page_tokens, &token_slots) != 0 || token_slots > SIZE_MAX / sizeof(uint32_t))
        return kipp_fail(error, KIPP_ERROR_RANGE, "the pool's size overflows");
    pool->page_count = page_count;
    pool->page_tokens = page_tokens;
    pool->bucket_count = 2;
    while (pool->bucket_count < 2 * (uint64_t)page_count) pool->bucket_count *= 2;
    pool->pages = calloc(page_count, sizeof(kipp_page));
    pool->tokens = calloc(token_slots, sizeof(uint32_t));
    pool->buckets = malloc(pool->bucket_count * sizeof(uint32_t));
    bool *seen = calloc(page_count, sizeof(bool));
    if (pool->pages == NULL || pool->tokens == NULL || pool->buckets == NULL || seen == NULL) {
        free(seen);
        kipp_pool_free(pool);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a pool of %u pages", page_count);
    }
    for (uint32_t b = 0; b < pool->bucket_count; ++b) pool->buckets[b] = KIPP_NO_PAGE;
    pool->free_head = pool->free_tail = KIPP_NO_PAGE;
    uint32_t step = (uint32_t)((double)page_count * 0.6180339887);
    if (step == 0) step = 1;
    while (gcd32(step, page_count) != 1) ++step;
    for (uint32_t i = 0; i < page_count; ++i) {
        uint32_t page = order != NULL ? order[i] : (uint32_t)(((uint64_t)i * step) % page_count);
        if (page >= page_count || seen[page]) {
            free(seen);
            kipp_pool_free(pool);
            return kipp_fail(error, KIPP_ERROR_ARGUMENT, "the order of a pool's pages must name every page once");
        }
        seen[page] = true;
        pool->pages[page].hash_next = KIPP_NO_PAGE;
        free_list_push(pool, page);
    }
    free(seen);
    return 0;
}

void kipp_pool_free(kipp_pool *pool) {
    free(pool->pages);
    free(pool->tokens);
    free(pool->buckets);
    memset(pool, 0, sizeof(*pool));
}

static void index_remove(kipp_pool *pool, uint32_t page) {
    kipp_page *p = &pool->pages[page];
    if (!p->indexed) return;
    uint32_t *link = &pool->buckets[p->hash & (pool->bucket_count - 1)];
    while (*link != KIPP_NO_PAGE && *link != page) link = &pool->pages[*link].hash_next;
    if (*link == page) *link = p->hash_next;
    p->hash_next = KIPP_NO_PAGE;
    p->indexed = false;
}

static uint32_t index_lookup(const kipp_pool *pool, uint64_t hash, const uint32_t *tokens) {
    for (uint32_t at = pool->buckets[hash & (pool->bucket_count - 1)]; at != KIPP_NO_PAGE; at = pool->pages[at].hash_next) {
        if (pool->pages[at].hash == hash &&
            memcmp(pool->tokens + (size_t)at * pool->page_tokens, tokens, pool->page_tokens * sizeof(uint32_t)) == 0)
            return at;
    }
    return KIPP_NO_PAGE;
}

uint32_t kipp_pool_alloc(kipp_pool *pool) {
    uint32_t page = pool->free_head;
    if (page == KIPP_NO_PAGE) return KIPP_NO_PAGE;
    free_list_remove(pool, page);
    if (pool->pages[page].indexed) {
        index_remove(pool, page);
        ++pool->evicted_total;
    }
    pool->pages[page].ref_count = 1;
    return page;
}

void kipp_pool_retain(kipp_pool *pool, uint32_t page) {
    if (pool->pages[page].ref_count == 0) free_list_remove(pool, page);
    ++pool->pages[page].ref_count;
}

int kipp_pool_release(kipp_pool *pool, uint32_t page) {
    if (page >= pool->page_count || pool->pages[page].ref_count == 0) return -1;
    if (--pool->pages[page].ref_count == 0) free_list_push(pool, page);
    return 0;
}

bool kipp_pool_is_indexed(const kipp_pool *pool, uint32_t page) { return pool->pages[page].indexed; }

uint64_t kipp_pool_seal(kipp_pool *pool, uint32_t page, uint64_t parent, const uint32_t *tokens) {
    uint64_t hash = pool_hash(pool, parent, tokens);
    kipp_page *p = &pool->pages[page];
    if (p->ref_count == 0 || p->indexed) return hash; /* the caller's mistake; nothing is published */
    if (index_lookup(pool, hash, tokens) == KIPP_NO_PAGE) {
        memcpy(pool->tokens + (size_t)page * pool->page_tokens, tokens, pool->page_tokens * sizeof(uint32_t));
        p->hash = hash;
        p->indexed = true;
        uint32_t *bucket = &pool->buckets[hash & (pool->bucket_count - 1)];
        p->hash_next = *bucket;
        *bucket = page;
    }
    return hash;
}

uint32_t kipp_pool_prefix_match(kipp_pool *pool, const uint32_t *tokens, size_t count, uint32_t *out_pages, uint32_t capacity,
                                uint64_t *out_chain) {
    size_t limit = count == 0 ? 0 : (count - 1) / pool->page_tokens; /* one token is always left to run */
    uint64_t parent = 0;
    uint32_t matched = 0;
    for (size_t block = 0; block < limit && matched < capacity; ++block) {
        const uint32_t *chunk = tokens + block * pool->page_tokens;
        uint64_t hash = pool_hash(pool, parent, chunk);
        uint32_t page = index_lookup(pool, hash, chunk);
        if (page == KIPP_NO_PAGE) break;
        kipp_pool_retain(pool, page);
        ++pool->reused_total;
        out_pages[matched++] = page;
        parent = hash;
    }
    if (out_chain != NULL) *out_chain = parent;
    return matched;
}

int kipp_pool_check(const kipp_pool *pool, kipp_error *error) {
    uint32_t on_list = 0;
    for (uint32_t at = pool->free_head, prev = KIPP_NO_PAGE; at != KIPP_NO_PAGE; prev = at, at = pool->pages[at].next_free) {
        if (pool->pages[at].ref_count != 0 || !pool->pages[at].on_free_list || pool->pages[at].prev_free != prev)
            return kipp_fail(error, KIPP_ERROR_INTERNAL, "page %u is on the free list but held, or the list is broken", at);
        if (++on_list > pool->page_count) return kipp_fail(error, KIPP_ERROR_INTERNAL, "the free list has a cycle");
    }
    if (on_list != pool->free_count) return kipp_fail(error, KIPP_ERROR_INTERNAL, "the free list holds %u pages, the count says %u", on_list, pool->free_count);
    for (uint32_t page = 0; page < pool->page_count; ++page) {
        const kipp_page *p = &pool->pages[page];
        if ((p->ref_count > 0) == p->on_free_list)
            return kipp_fail(error, KIPP_ERROR_INTERNAL, "page %u: ref %u, on the free list: %d", page, p->ref_count, (int)p->on_free_list);
        if (p->indexed) {
            uint32_t at = pool->buckets[p->hash & (pool->bucket_count - 1)];
            while (at != KIPP_NO_PAGE && at != page) at = pool->pages[at].hash_next;
            if (at != page) return kipp_fail(error, KIPP_ERROR_INTERNAL, "page %u says it is indexed but its bucket does not hold it", page);
        }
    }
    return 0;
}
