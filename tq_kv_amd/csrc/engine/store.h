// The cache's storage: keys and values for each cached run of the order, fixed-size state beside
// them, a slot for each live sequence.
//
// Runs of the order with the same need form a group.  A group of pages has storage of its own,
//     keys:   [runs in group, pages, key page...]      values: [runs in group, pages, value page...]
// (what a page looks like inside is the mixer's business: its need names the two shapes), and per
// slot the list of pages that hold the slot's positions.  A group with a window gives pages back
// as soon as every position in them has left the window.  Mixers with a fixed-size state get one
// row per slot, zeroed when the slot is taken.  The bookkeeping (free slots, lengths, page lists)
// is tqe_cache_t's (host_engine.cpp); this class owns the memory.
//
// The reference keeps one growing tensor pair per layer and one sequence
// (src/models/turbo_generic.rs:1606-1618) and resets by position (src/engine.rs:322-324).
#pragma once
#include "parts.h"

namespace tq {

struct PageGroup {
    CacheNeed need;
    std::vector<int> runs;
    int n_pages = 0;
    OwnedPtr keys, values;
};

struct StateGroup {
    CacheNeed need;
    std::vector<int> runs;
    OwnedPtr state;              // [runs, slots, shape...]
};

class CacheStore {
public:
    // needs: for each run of the order its need.  cache_of: for each run -1, or the run whose cache it reads.
    // max_tokens: positions that live sequences may hold together, each counted up to whole pages.
    CacheStore(const std::vector<CacheNeed>& needs, const std::vector<int>& cache_of, long long max_tokens, int max_slots, int dtype);
    ~CacheStore();
    CacheStore(const CacheStore&) = delete;
    CacheStore& operator=(const CacheStore&) = delete;

    bool holds_pages = false;           // false: no run keeps keys and values, max_tokens bounds nothing
    int n_pages = 0, max_slots = 0;
    std::vector<PageGroup> page_groups;
    std::vector<StateGroup> state_groups;
    tqe_cache_t* book = nullptr;

    int acquire(hipStream_t stream);    // a free slot with length 0 and zeroed state
    void release(int slot);
    int length(int slot) const;
    void reserve(int n, const int32_t* slots, const int32_t* n_new);        // all or nothing
    void commit(int n, const int32_t* slots, const int32_t* n_new);
    const CacheEntry& entry(int run) const { return entries_.at((size_t)run); }
    Json describe() const;

private:
    std::vector<CacheEntry> entries_;
};

}  // namespace tq
