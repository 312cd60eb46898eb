// Expert offload runtime: asynchronous slab copies on a side stream and the
// LRU policy of one eviction group.  The policy object is plain host code (no
// GPU calls) so it can be tested on a machine without a GPU.
//
// Behaviour follows the reference's ExpertCache (src/expert_cache.py:20-52,
// 120-201): requested experts are marked used first, resident experts are
// served before misses, every miss evicts the least recently used resident
// expert of the group and becomes the most recently used one.
#include <hip/hip_runtime_api.h>

#include <list>
#include <new>
#include <vector>

#include "hqq_mi355x.h"

struct hqq_lru {
    int32_t n_experts;
    int32_t slots;
    std::vector<int32_t> slot_of;   // expert -> device slot or -1
    std::vector<int32_t> expert_in; // slot -> expert or -1
    std::list<int32_t> order;       // resident experts, least recently used first
    std::vector<std::list<int32_t>::iterator> pos;
    int64_t hits = 0, misses = 0;
};

extern "C" {

int hqq_slab_h2d_async(void *dst_device, const void *src_pinned, size_t bytes, void *copy_stream, void *done_event)
{
    if (!dst_device || !src_pinned)
        return HQQ_E_NULL;
    if (bytes == 0)
        return HQQ_OK;
    hipError_t e = hipMemcpyAsync(dst_device, src_pinned, bytes, hipMemcpyHostToDevice, (hipStream_t)copy_stream);
    if (e != hipSuccess)
        return (int)e;
    if (done_event) {
        e = hipEventRecord((hipEvent_t)done_event, (hipStream_t)copy_stream);
        if (e != hipSuccess)
            return (int)e;
    }
    return HQQ_OK;
}

int hqq_stream_wait_event(void *stream, void *event)
{
    if (!event)
        return HQQ_E_NULL;
    hipError_t e = hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0);
    return e == hipSuccess ? HQQ_OK : (int)e;
}

hqq_lru *hqq_lru_create(int32_t n_experts, int32_t slots)
{
    if (n_experts <= 0 || slots <= 0)
        return nullptr;
    hqq_lru *c = new (std::nothrow) hqq_lru;
    if (!c)
        return nullptr;
    c->n_experts = n_experts;
    c->slots = slots;
    c->slot_of.assign(n_experts, -1);
    c->expert_in.assign(slots, -1);
    c->pos.resize(n_experts);
    return c;
}

void hqq_lru_destroy(hqq_lru *c) { delete c; }

int hqq_lru_add_resident(hqq_lru *c, int32_t e)
{
    if (!c || e < 0 || e >= c->n_experts || c->slot_of[e] >= 0)
        return HQQ_E_CACHE;
    for (int32_t s = 0; s < c->slots; ++s)
        if (c->expert_in[s] < 0) {
            c->expert_in[s] = e;
            c->slot_of[e] = s;
            c->pos[e] = c->order.insert(c->order.end(), e);
            return s;
        }
    return HQQ_E_CACHE; // "Cache is full"
}

int hqq_lru_plan(hqq_lru *c, const int32_t *experts, int32_t n, int32_t *order, int32_t *slot, int32_t *victim)
{
    if (!c || !experts || !order || !slot || !victim)
        return HQQ_E_NULL;
    if (n < 0)
        return HQQ_E_CACHE;
    int32_t n_miss = 0;
    for (int32_t i = 0; i < n; ++i) {
        const int32_t e = experts[i];
        if (e < 0 || e >= c->n_experts)
            return HQQ_E_CACHE;
        for (int32_t k = 0; k < i; ++k)
            if (experts[k] == e)
                return HQQ_E_CACHE; // duplicates
        n_miss += c->slot_of[e] < 0;
    }
    if (n_miss > 0 && (int32_t)c->order.size() == 0)
        return HQQ_E_CACHE; // "No evictable experts"
    // resident first, stable; mark all used before any eviction
    int32_t w = 0;
    for (int32_t i = 0; i < n; ++i)
        if (c->slot_of[experts[i]] >= 0)
            order[w++] = experts[i];
    const int32_t n_hit = w;
    for (int32_t i = 0; i < n; ++i)
        if (c->slot_of[experts[i]] < 0)
            order[w++] = experts[i];
    for (int32_t i = 0; i < n_hit; ++i) {
        const int32_t e = order[i];
        c->order.splice(c->order.end(), c->order, c->pos[e]);
        slot[i] = c->slot_of[e];
        victim[i] = -1;
    }
    c->hits += n_hit;
    c->misses += n_miss;
    for (int32_t i = n_hit; i < n; ++i) {
        const int32_t e = order[i];
        const int32_t v = c->order.front(); // least recently used resident
        c->order.pop_front();
        const int32_t s = c->slot_of[v];
        c->slot_of[v] = -1;
        c->slot_of[e] = s;
        c->expert_in[s] = e;
        c->pos[e] = c->order.insert(c->order.end(), e);
        slot[i] = s;
        victim[i] = v;
    }
    return HQQ_OK;
}

int hqq_lru_plan_guess(hqq_lru *c, const int32_t *experts, int32_t n, const int32_t *keep, int32_t n_keep,
                       int32_t *order, int32_t *slot, int32_t *victim, int32_t *count)
{
    if (!c || !experts || !order || !slot || !victim || !count || (n_keep > 0 && !keep))
        return HQQ_E_NULL;
    if (n < 0 || n_keep < 0)
        return HQQ_E_CACHE;
    for (int32_t i = 0; i < n; ++i) {
        if (experts[i] < 0 || experts[i] >= c->n_experts)
            return HQQ_E_CACHE;
        for (int32_t k = 0; k < i; ++k)
            if (experts[k] == experts[i])
                return HQQ_E_CACHE; // duplicates
    }
    auto kept = [&](int32_t e) {
        for (int32_t k = 0; k < n_keep; ++k)
            if (keep[k] == e)
                return true;
        for (int32_t k = 0; k < n; ++k) // a guess does not evict another expert of the same guess either
            if (experts[k] == e)
                return true;
        return false;
    };
    int32_t w = 0;
    for (int32_t i = 0; i < n; ++i) {
        const int32_t e = experts[i];
        if (c->slot_of[e] >= 0)
            continue;
        auto it = c->order.begin(); // least recently used first
        while (it != c->order.end() && kept(*it))
            ++it;
        if (it == c->order.end())
            continue; // nothing it may evict: the guess is dropped
        const int32_t v = *it;
        c->order.erase(it);
        const int32_t s = c->slot_of[v];
        c->slot_of[v] = -1;
        c->slot_of[e] = s;
        c->expert_in[s] = e;
        c->pos[e] = c->order.insert(c->order.end(), e);
        order[w] = e, slot[w] = s, victim[w] = v;
        ++w;
    }
    *count = w;
    return HQQ_OK;
}

int64_t hqq_lru_hits(const hqq_lru *c) { return c ? c->hits : 0; }
int64_t hqq_lru_misses(const hqq_lru *c) { return c ? c->misses : 0; }
int hqq_lru_slot_of(const hqq_lru *c, int32_t e)
{
    if (!c || e < 0 || e >= c->n_experts)
        return -1;
    return c->slot_of[e];
}

} // extern "C"
