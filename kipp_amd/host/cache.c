/*
 * The cache manager: pages of keys and values for every session, per group of
 * layer runs, and slots of fixed-size state.
 *
 * Runs of the layer order with the same need (heads, head size, window, page
 * size) form a group; a group has its own pool of pages, its own block table
 * in every session, and one key and one value slab for each of its runs, laid
 * out [page][kv head][slot in page][head_dim].  A group with a window gives
 * pages back as soon as the window has passed them; every group gives all
 * pages back when the session ends.  A run whose mixer keeps state of fixed
 * size gets a row of [slots + 1][bytes] instead, zeroed when a session claims
 * its slot.
 *
 * Claims are all-or-nothing (/root/reference/src/kipp.c:3616-3635, 4043-4072).  Full
 * pages are published when a session ends or is reset, never earlier, so shared
 * pages are complete and truncation only touches private ones
 * (/root/reference/src/kipp.c:3647-3670, 3755-3767).
 */
#include <stdlib.h>
#include <string.h>

#include "backend.h"
#include "internal.h"

static bool same_need(const kipp_kv_need *a, const kipp_kv_need *b) {
    return a->n_kv_heads == b->n_kv_heads && a->head_dim == b->head_dim && a->window == b->window && a->page_tokens == b->page_tokens;
}

int kipp_cache_init(kipp_cache *cache, kipp_runtime *rt, const kipp_kv_need *kv_needs, const kipp_state_need *state_needs,
                    const kipp_layer_run *order, uint32_t run_count, uint32_t page_tokens, uint32_t pool_pages, uint32_t max_sessions,
                    uint32_t max_position, bool share, const uint32_t *page_order, kipp_error *error) {
    memset(cache, 0, sizeof(*cache));
    cache->rt = rt;
    cache->run_count = run_count;
    cache->page_tokens = page_tokens;
    cache->max_sessions = max_sessions;
    cache->max_position = max_position;
    cache->run_group = malloc(run_count * sizeof(int32_t));
    cache->run_in_group = malloc(run_count * sizeof(int32_t));
    cache->groups = calloc(run_count ? run_count : 1, sizeof(kipp_cache_group));
    cache->state_needs = calloc(run_count ? run_count : 1, sizeof(kipp_state_need));
    cache->states = calloc(run_count ? run_count : 1, sizeof(void *));
    cache->free_slots = malloc((size_t)max_sessions * sizeof(uint32_t));
    if (!cache->run_group || !cache->run_in_group || !cache->groups || !cache->state_needs || !cache->states || !cache->free_slots) {
        kipp_cache_free(cache);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for the cache manager");
    }
    for (uint32_t s = 0; s < max_sessions; ++s) cache->free_slots[s] = max_sessions - 1 - s;
    cache->free_slot_count = max_sessions;
    bool any_state = false, any_window = false, one_page_size = true;
    for (uint32_t run = 0; run < run_count; ++run) {
        cache->run_group[run] = cache->run_in_group[run] = -1;
        cache->state_needs[run] = state_needs[run];
        any_state = any_state || state_needs[run].any;
        if (order[run].cache_of >= 0 || !kv_needs[run].any) continue;
        uint32_t g = 0;
        while (g < cache->group_count && !same_need(&cache->groups[g].need, &kv_needs[run])) ++g;
        if (g == cache->group_count) {
            kipp_cache_group *group = &cache->groups[cache->group_count++];
            group->index = g;
            group->need = kv_needs[run];
            group->page_tokens = kv_needs[run].page_tokens ? kv_needs[run].page_tokens : page_tokens;
            group->runs = malloc(run_count * sizeof(uint32_t));
            if (group->runs == NULL) {
                kipp_cache_free(cache);
                return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a cache group");
            }
            any_window = any_window || group->need.window != 0;
            one_page_size = one_page_size && group->page_tokens == cache->groups[0].page_tokens;
        }
        cache->run_group[run] = (int32_t)g;
        cache->run_in_group[run] = (int32_t)cache->groups[g].run_count;
        cache->groups[g].runs[cache->groups[g].run_count++] = run;
    }
    /* sharing needs every token of a beginning in pages that are kept, and pages that hold the same tokens in every group */
    cache->share = share && !any_state && !any_window && one_page_size && cache->group_count > 0;
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        kipp_cache_group *group = &cache->groups[g];
        /* a group whose pages have another size gets as many as hold the same tokens */
        uint64_t pages = ((uint64_t)pool_pages * page_tokens + group->page_tokens - 1) / group->page_tokens;
        if (pages == 0 || pages > UINT32_MAX / 4) {
            kipp_cache_free(cache);
            return kipp_fail(error, KIPP_ERROR_RANGE, "a pool of %llu pages", (unsigned long long)pages);
        }
        const uint32_t *order_of_pages = page_order != NULL && pages == pool_pages ? page_order : NULL;
        if (kipp_pool_init(&group->pool, (uint32_t)pages, group->page_tokens, order_of_pages, error) != 0) {
            kipp_cache_free(cache);
            return -1;
        }
        group->k = calloc(group->run_count, sizeof(void *));
        group->v = calloc(group->run_count, sizeof(void *));
        size_t elements, bytes;
        /* one page more than the pool hands out: a place for rows that only fill a batch up */
        if (group->k == NULL || group->v == NULL || kipp_mul_size((size_t)pages + 1, group->need.n_kv_heads, &elements) != 0 ||
            kipp_mul_size(elements, (size_t)group->page_tokens * group->need.head_dim, &elements) != 0 ||
            kipp_mul_size(elements, kipp_dtype_bytes(rt->act_dtype), &bytes) != 0) {
            kipp_cache_free(cache);
            return kipp_fail(error, KIPP_ERROR_RANGE, "the cache's byte size overflows");
        }
        group->slab_bytes = bytes;
        for (uint32_t r = 0; r < group->run_count; ++r) {
            /* zeroed: masked slots must hold finite values */
            group->k[r] = rt->mem_alloc(rt, bytes, error);
            group->v[r] = group->k[r] != NULL ? rt->mem_alloc(rt, bytes, error) : NULL;
            if (group->v[r] == NULL) {
                kipp_cache_free(cache);
                return -1;
            }
        }
    }
    for (uint32_t run = 0; run < run_count; ++run) {
        if (!state_needs[run].any) continue;
        size_t bytes;
        if (kipp_mul_size((size_t)max_sessions + 1, (size_t)state_needs[run].bytes, &bytes) != 0 ||
            (cache->states[run] = rt->mem_alloc(rt, bytes, error)) == NULL) {
            kipp_cache_free(cache);
            return error != NULL && error->code != KIPP_OK ? -1 : kipp_fail(error, KIPP_ERROR_RANGE, "the state slots' size overflows");
        }
    }
    return 0;
}

void kipp_cache_free(kipp_cache *cache) {
    kipp_runtime *rt = cache->rt;
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        kipp_cache_group *group = &cache->groups[g];
        for (uint32_t r = 0; r < group->run_count; ++r) {
            if (group->k != NULL && group->k[r] != NULL) rt->mem_free(rt, group->k[r]);
            if (group->v != NULL && group->v[r] != NULL) rt->mem_free(rt, group->v[r]);
        }
        free(group->k);
        free(group->v);
        free(group->runs);
        kipp_pool_free(&group->pool);
    }
    if (cache->states != NULL) {
        for (uint32_t run = 0; run < cache->run_count; ++run) {
            if (cache->states[run] != NULL) rt->mem_free(rt, cache->states[run]);
        }
    }
    free(cache->groups);
    free(cache->run_group);
    free(cache->run_in_group);
    free(cache->state_needs);
    free(cache->states);
    free(cache->free_slots);
    memset(cache, 0, sizeof(*cache));
}

bool kipp_cache_view_of(const kipp_cache *cache, uint32_t run, int32_t cache_of, kipp_cache_view *out) {
    uint32_t source = cache_of >= 0 ? (uint32_t)cache_of : run;
    int32_t g = cache->run_group[source];
    if (g < 0) return false;
    const kipp_cache_group *group = &cache->groups[g];
    out->group = (uint32_t)g;
    out->k = group->k[cache->run_in_group[source]];
    out->v = group->v[cache->run_in_group[source]];
    out->page_tokens = group->page_tokens;
    out->page_count = group->pool.page_count;
    out->writable = cache_of < 0;
    return true;
}

static uint32_t blocks_for(uint32_t tokens, uint32_t page_tokens) { return (tokens + page_tokens - 1) / page_tokens; }

int kipp_cache_open(kipp_cache *cache, kipp_session *session, uint32_t capacity, kipp_error *error) {
    if (cache->free_slot_count == 0) return kipp_fail(error, KIPP_ERROR_RANGE, "all %u session slots are taken", cache->max_sessions);
    if (capacity == 0 || capacity > cache->max_position) capacity = cache->max_position;
    session->capacity = capacity;
    session->length = session->adopted_tokens = 0;
    session->tokens = malloc((size_t)capacity * sizeof(uint32_t));
    session->tables = calloc(cache->group_count ? cache->group_count : 1, sizeof(int32_t *));
    session->table_lengths = calloc(cache->group_count ? cache->group_count : 1, sizeof(uint32_t));
    session->adopted = calloc(cache->group_count ? cache->group_count : 1, sizeof(uint32_t));
    bool ok = session->tokens && session->tables && session->table_lengths && session->adopted;
    for (uint32_t g = 0; ok && g < cache->group_count; ++g) {
        session->tables[g] = malloc((size_t)blocks_for(capacity, cache->groups[g].page_tokens) * sizeof(int32_t) + sizeof(int32_t));
        ok = session->tables[g] != NULL;
    }
    if (!ok) {
        kipp_cache_close(cache, session);
        return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory for a session of %u tokens", capacity);
    }
    session->slot = cache->free_slots[--cache->free_slot_count];
    ++cache->live_sessions;
    for (uint32_t run = 0; run < cache->run_count; ++run) {
        if (cache->states[run] != NULL) {
            size_t bytes = (size_t)cache->state_needs[run].bytes;
            if (cache->rt->mem_zero(cache->rt, (char *)cache->states[run] + (size_t)session->slot * bytes, bytes, error) != 0) return -1;
        }
    }
    return 0;
}

int kipp_cache_adopt(kipp_cache *cache, kipp_session *session, const uint32_t *tokens, size_t count, uint32_t *matched,
                     kipp_error *error) {
    *matched = 0;
    if (!cache->share) return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "this model's sessions do not share pages");
    if (session->length != 0) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "only a fresh session adopts a beginning");
    if (count > session->capacity) count = session->capacity;
    uint32_t keep = UINT32_MAX;
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        uint32_t capacity = blocks_for(session->capacity, cache->groups[g].page_tokens);
        uint32_t got = kipp_pool_prefix_match(&cache->groups[g].pool, tokens, count, (uint32_t *)session->tables[g], capacity, NULL);
        session->table_lengths[g] = got;
        if (got < keep) keep = got;
    }
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        while (session->table_lengths[g] > keep) kipp_pool_release(&cache->groups[g].pool, (uint32_t)session->tables[g][--session->table_lengths[g]]);
        session->adopted[g] = keep;
    }
    session->adopted_tokens = session->length = keep * cache->page_tokens;
    memcpy(session->tokens, tokens, (size_t)session->length * sizeof(uint32_t));
    session->published = keep;
    session->chain = 0;
    for (uint32_t block = 0; block < keep; ++block) {
        const kipp_pool *pool = &cache->groups[0].pool;
        session->chain = pool->force_hash ? pool->forced_hash : kipp_pool_chain_hash(session->chain, tokens + (size_t)block * cache->page_tokens, cache->page_tokens);
    }
    *matched = session->length;
    return 0;
}

int kipp_cache_reserve_one(kipp_cache *cache, kipp_session *session, size_t count, kipp_error *error) {
    if (count == 0) return kipp_fail(error, KIPP_ERROR_ARGUMENT, "a step entry needs at least one token");
    if (count > session->capacity - session->length)
        return kipp_fail(error, KIPP_ERROR_RANGE, "%zu more tokens exceed the session's capacity of %u (it holds %u)", count,
                         session->capacity, session->length);
    uint32_t new_length = session->length + (uint32_t)count;
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        kipp_cache_group *group = &cache->groups[g];
        uint32_t blocks = blocks_for(new_length, group->page_tokens);
        while (session->table_lengths[g] < blocks) {
            uint32_t page = kipp_pool_alloc(&group->pool);
            if (page == KIPP_NO_PAGE) {
                kipp_cache_trim(cache, session);
                return kipp_fail(error, KIPP_ERROR_RANGE, "KV pool exhausted: group %u has no free page", g);
            }
            session->tables[g][session->table_lengths[g]++] = (int32_t)page;
        }
    }
    return 0;
}

void kipp_cache_trim(kipp_cache *cache, kipp_session *session) {
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        uint32_t blocks = blocks_for(session->length, cache->groups[g].page_tokens);
        while (session->table_lengths[g] > blocks) {
            int32_t page = session->tables[g][--session->table_lengths[g]];
            if (page >= 0) kipp_pool_release(&cache->groups[g].pool, (uint32_t)page);
        }
    }
}

void kipp_cache_commit(kipp_cache *cache, kipp_session *session, const uint32_t *tokens, size_t count) {
    memcpy(session->tokens + session->length, tokens, count * sizeof(uint32_t));
    session->length += (uint32_t)count;
    if (session->publish_early && cache->share) {
        while ((session->published + 1) * cache->page_tokens <= session->length) {
            const uint32_t *chunk = session->tokens + (size_t)session->published * cache->page_tokens;
            uint64_t hash = session->chain;
            for (uint32_t g = 0; g < cache->group_count; ++g)
                hash = kipp_pool_seal(&cache->groups[g].pool, (uint32_t)session->tables[g][session->published], session->chain, chunk);
            session->chain = hash;
            ++session->published;
        }
    }
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        kipp_cache_group *group = &cache->groups[g];
        if (group->need.window == 0) continue;
        /* the next query sees keys from length - window + 1 on: pages wholly before that go back */
        uint32_t first_needed = session->length + 1 > group->need.window ? session->length + 1 - group->need.window : 0;
        uint32_t passed = first_needed / group->page_tokens;
        for (uint32_t block = 0; block < passed && block < session->table_lengths[g]; ++block) {
            if (session->tables[g][block] >= 0) {
                kipp_pool_release(&group->pool, (uint32_t)session->tables[g][block]);
                session->tables[g][block] = -1;
            }
        }
    }
}

int kipp_cache_truncate(kipp_cache *cache, kipp_session *session, uint32_t length, kipp_error *error) {
    if (length > session->length) return kipp_fail(error, KIPP_ERROR_RANGE, "cannot truncate %u tokens to %u", session->length, length);
    for (uint32_t run = 0; run < cache->run_count; ++run) {
        if (cache->state_needs[run].any) return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "per-session state cannot be rolled back");
    }
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        if (cache->groups[g].need.window != 0) return kipp_fail(error, KIPP_ERROR_UNSUPPORTED, "a windowed group cannot be rolled back");
    }
    uint32_t floor = session->published * cache->page_tokens > session->adopted_tokens ? session->published * cache->page_tokens : session->adopted_tokens;
    if (length < floor) return kipp_fail(error, KIPP_ERROR_RANGE, "cannot truncate below the %u adopted or published tokens", floor);
    session->length = length;
    kipp_cache_trim(cache, session);
    return 0;
}

void kipp_cache_clear(kipp_cache *cache, kipp_session *session) {
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        kipp_cache_group *group = &cache->groups[g];
        if (cache->share) {
            uint64_t parent = 0;
            uint32_t full = session->length / group->page_tokens;
            for (uint32_t block = 0; block < full && block < session->table_lengths[g]; ++block) {
                const uint32_t *chunk = session->tokens + (size_t)block * group->page_tokens;
                uint32_t page = (uint32_t)session->tables[g][block];
                if (block < session->adopted[g] || kipp_pool_is_indexed(&group->pool, page))
                    parent = group->pool.force_hash ? group->pool.forced_hash : kipp_pool_chain_hash(parent, chunk, group->page_tokens);
                else
                    parent = kipp_pool_seal(&group->pool, page, parent, chunk);
            }
        }
        for (uint32_t block = 0; block < session->table_lengths[g]; ++block) {
            if (session->tables[g][block] >= 0) kipp_pool_release(&group->pool, (uint32_t)session->tables[g][block]);
        }
        session->table_lengths[g] = 0;
        session->adopted[g] = 0;
    }
    session->length = session->adopted_tokens = 0;
    session->published = 0;
    session->chain = 0;
}

void kipp_cache_close(kipp_cache *cache, kipp_session *session) {
    if (session->tables != NULL && session->table_lengths != NULL && session->adopted != NULL && session->tokens != NULL) {
        bool complete = true;
        for (uint32_t g = 0; g < cache->group_count; ++g) complete = complete && session->tables[g] != NULL;
        if (complete) {
            kipp_cache_clear(cache, session);
            cache->free_slots[cache->free_slot_count++] = session->slot;
            --cache->live_sessions;
        }
    }
    if (session->tables != NULL) {
        for (uint32_t g = 0; g < cache->group_count; ++g) free(session->tables[g]);
    }
    free(session->tables);
    free(session->table_lengths);
    free(session->adopted);
    free(session->tokens);
    session->tables = NULL;
    session->table_lengths = session->adopted = session->tokens = NULL;
}

int kipp_cache_check(const kipp_cache *cache, kipp_session *const *sessions, size_t session_count, kipp_error *error) {
    for (uint32_t g = 0; g < cache->group_count; ++g) {
        const kipp_pool *pool = &cache->groups[g].pool;
        if (kipp_pool_check(pool, error) != 0) return -1;
        uint32_t *named = calloc(pool->page_count, sizeof(uint32_t));
        if (named == NULL) return kipp_fail(error, KIPP_ERROR_MEMORY, "out of memory");
        for (size_t s = 0; s < session_count; ++s) {
            for (uint32_t block = 0; block < sessions[s]->table_lengths[g]; ++block) {
                if (sessions[s]->tables[g][block] >= 0) ++named[sessions[s]->tables[g][block]];
            }
        }
        for (uint32_t page = 0; page < pool->page_count; ++page) {
            if (named[page] != pool->pages[page].ref_count) {
                kipp_fail(error, KIPP_ERROR_INTERNAL, "group %u page %u: named %u times, held %u times", g, page, named[page], pool->pages[page].ref_count);
                free(named);
                return -1;
            }
        }
        free(named);
    }
    if (cache->live_sessions + cache->free_slot_count != cache->max_sessions) return kipp_fail(error, KIPP_ERROR_INTERNAL, "a session slot was lost");
    return 0;
}
