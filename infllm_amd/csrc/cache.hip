// Residency policy of the device unit cache, one object per batch row
// (inf_llm/attention/context_manager.py:246-265 values, 495-515 eviction).  Host code only: it sits between the
// arrival of a block's top-k ids and the launch of the fetch, i.e. on the critical chain of the stream, and an
// interpreter takes an order of magnitude longer over it.
//
// The reference keeps a dict unit -> value and evicts in ascending value, first-inserted first on ties (a stable
// sort over the dict's insertion order), never a unit of the current selection.  Here the residents sit in a vector
// in insertion order (an evicted unit that comes back goes to the end, as in the dict), and the eviction is a stable
// sort of that vector by value.  Values are doubles: the lru / fifo clocks are small integers, the lru-s scores are
// the reference's Python floats (same operations, same order).
#include <algorithm>
#include <vector>

#include "common.h"

namespace {

struct Resident {
    int32_t unit, slot;
    double value;
};

struct UnitCache {
    int capacity, strategy;
    double decay;
    int64_t clock = 0;
    std::vector<Resident> res;          // in insertion order
    std::vector<int32_t> free_slots;    // used from the back
    std::vector<int32_t> order;         // scratch
    Resident *find(int32_t unit) {
        for (auto &r : res)
            if (r.unit == unit) return &r;
        return nullptr;
    }
};

}  // namespace

extern "C" void *infllm_cache_create(int32_t capacity, int32_t strategy, double score_decay) {
    if (capacity < 1 || strategy < INFLLM_CACHE_LRU || strategy > INFLLM_CACHE_LRU_S) {
        infllm_fail(-1, "cache_create: capacity %d / strategy %d", capacity, strategy);
        return nullptr;
    }
    UnitCache *c = new UnitCache();
    c->capacity = capacity;
    c->strategy = strategy;
    c->decay = score_decay;
    for (int s = capacity - 1; s >= 0; --s) c->free_slots.push_back(s);     // slot 0 is handed out first
    return c;
}

extern "C" int infllm_cache_destroy(void *cache) {
    delete (UnitCache *)cache;
    return 0;
}

extern "C" int infllm_cache_touch(void *cache, const int32_t *selected, int32_t n_sel, int32_t *slots, int32_t *miss_units,
                                  int32_t *miss_slots, int32_t *evicted, int32_t *n_evicted) {
    return infllm_cache_touch_hinted(cache, selected, n_sel, slots, miss_units, miss_slots, evicted, n_evicted, nullptr, nullptr, 0);
}

extern "C" int infllm_cache_touch_hinted(void *cache, const int32_t *selected, int32_t n_sel, int32_t *slots, int32_t *miss_units,
                                         int32_t *miss_slots, int32_t *evicted, int32_t *n_evicted, const int32_t *hint_units,
                                         const int32_t *hint_slots, int32_t n_hints) {
    INFLLM_REQUIRE(cache && n_sel >= 0 && (n_sel == 0 || (selected && slots && miss_units && miss_slots)), "cache_touch: bad arguments");
    INFLLM_REQUIRE(n_hints >= 0 && (n_hints == 0 || (hint_units && hint_slots)), "cache_touch: bad hint list");
    UnitCache &c = *(UnitCache *)cache;
    INFLLM_REQUIRE(n_sel <= c.capacity, "cache_touch: %d selected units exceed max_cached_block %d", n_sel, c.capacity);
    int n_miss = 0;
    for (int i = 0; i < n_sel; ++i) {
        INFLLM_REQUIRE(selected[i] >= 0, "cache_touch: negative unit id");
        for (int j = 0; j < i; ++j) INFLLM_REQUIRE(selected[j] != selected[i], "cache_touch: unit %d selected twice", selected[i]);
        if (!c.find(selected[i])) miss_units[n_miss++] = selected[i];
    }
    // ---- eviction: ascending (value, insertion), skipping the selection
    const int surplus = (int)c.res.size() - c.capacity + n_miss;
    int n_ev = 0;
    if (surplus > 0) {
        c.order.resize(c.res.size());
        for (size_t i = 0; i < c.res.size(); ++i) c.order[i] = (int32_t)i;
        std::stable_sort(c.order.begin(), c.order.end(), [&](int32_t a, int32_t b) { return c.res[a].value < c.res[b].value; });
        std::vector<char> gone(c.res.size(), 0);
        for (int32_t idx : c.order) {
            if (n_ev >= surplus) break;
            bool chosen = false;
            for (int i = 0; i < n_sel && !chosen; ++i) chosen = selected[i] == c.res[idx].unit;
            if (chosen) continue;
            gone[idx] = 1;
            if (evicted) evicted[n_ev] = c.res[idx].unit;
            ++n_ev;
        }
        // the reference frees the slots in eviction order
        n_ev = 0;
        for (int32_t idx : c.order) {
            if (!gone[idx]) continue;
            c.free_slots.push_back(c.res[idx].slot);
            ++n_ev;
        }
        size_t w = 0;
        for (size_t i = 0; i < c.res.size(); ++i)
            if (!gone[i]) c.res[w++] = c.res[i];
        c.res.resize(w);
    }
    if (n_evicted) *n_evicted = n_ev;
    INFLLM_REQUIRE((int)c.res.size() + n_miss <= c.capacity, "cache_touch: unit cache overflow");
    // ---- values of the selection; new residents go to the end of the insertion order, in selection order
    if (c.strategy != INFLLM_CACHE_LRU_S) ++c.clock;
    int m = 0;
    for (int i = 0; i < n_sel; ++i) {
        Resident *r = c.find(selected[i]);
        const double v = c.strategy == INFLLM_CACHE_LRU_S ? 0.0 : (double)c.clock;
        if (r) {
            if (c.strategy != INFLLM_CACHE_FIFO) r->value = v;          // fifo keeps the clock of the first load
        } else {
            Resident nr{selected[i], -1, v};
            c.res.push_back(nr);
        }
    }
    // a missed unit with a hint takes the hinted slot when that is free now ...
    for (int i = 0; i < n_miss && n_hints > 0; ++i)
        for (int h = 0; h < n_hints; ++h) {
            if (hint_units[h] != miss_units[i]) continue;
            auto it = std::find(c.free_slots.begin(), c.free_slots.end(), hint_slots[h]);
            if (it != c.free_slots.end()) {
                c.find(miss_units[i])->slot = *it;
                c.free_slots.erase(it);
            }
            break;
        }
    // ... the others take slots in the order of the miss list (= selection order), after the evictions freed theirs
    for (int i = 0; i < n_miss; ++i) {
        Resident *r = c.find(miss_units[i]);
        if (r->slot < 0) {
            r->slot = c.free_slots.back();
            c.free_slots.pop_back();
        }
        miss_slots[m++] = r->slot;
    }
    for (int i = 0; i < n_sel; ++i) slots[i] = c.find(selected[i])->slot;
    return n_miss;
}

extern "C" int infllm_cache_add_scores(void *cache, const int32_t *units, const double *scores, int32_t n) {
    INFLLM_REQUIRE(cache && n >= 0 && (n == 0 || (units && scores)), "cache_add_scores: bad arguments");
    UnitCache &c = *(UnitCache *)cache;
    for (auto &r : c.res) r.value = r.value * c.decay;
    for (int i = 0; i < n; ++i) {
        Resident *r = c.find(units[i]);
        INFLLM_REQUIRE(r, "cache_add_scores: unit %d is not resident", units[i]);
        r->value += scores[i];
    }
    return 0;
}

extern "C" int infllm_cache_residents(void *cache, int32_t *units, double *values, int32_t *slots, int32_t capacity) {
    INFLLM_REQUIRE(cache && capacity >= 0, "cache_residents: bad arguments");
    UnitCache &c = *(UnitCache *)cache;
    const int n = (int)c.res.size();
    for (int i = 0; i < n && i < capacity; ++i) {
        if (units) units[i] = c.res[i].unit;
        if (values) values[i] = c.res[i].value;
        if (slots) slots[i] = c.res[i].slot;
    }
    return n;
}

extern "C" void *infllm_cache_clone(const void *src) {
    if (!src) {
        infllm_fail(-1, "cache_clone: null cache");
        return nullptr;
    }
    return new UnitCache(*(const UnitCache *)src);
}

extern "C" int infllm_cache_copy(void *dst, const void *src) {
    INFLLM_REQUIRE(dst && src, "cache_copy: null cache");
    UnitCache &d = *(UnitCache *)dst;
    const UnitCache &s = *(const UnitCache *)src;
    INFLLM_REQUIRE(d.capacity == s.capacity && d.strategy == s.strategy, "cache_copy: caches of different capacity or strategy");
    d.decay = s.decay;
    d.clock = s.clock;
    d.res = s.res;
    d.free_slots = s.free_slots;
    return 0;
}

extern "C" int infllm_cache_slot_of(void *cache, int32_t unit) {
    if (!cache) return -1;
    Resident *r = ((UnitCache *)cache)->find(unit);
    return r ? r->slot : -1;
}
