// The engine's bookkeeping on the host, behind a C boundary in the manner of the
// reference's (tq-kv/include/tq_kv.h:27-84, tq-kv/src/ffi.rs:89-108): opaque handles made
// and freed by the library, plain C types, int32 status (0 ok, negative error) and a
// message for the last error.  No GPU code here: this file is compiled with the host
// compiler alone and works on a machine without a GPU.
//
// tqe_cache_t owns what the cache must never lose: which slots are free, how many
// positions every sequence holds, and for every group of cached runs which pages of the
// group's pool each slot holds (a group with a window gives pages back as soon as all
// their positions have left the window).  The storage itself (the tensors of keys,
// values and states) belongs to the caller and is indexed by the slot and page numbers
// handed out here.
//
// tqe_plan_step turns one step's batch (sequences that bring unequal numbers of new
// tokens) into the packed int32 array that the kernels read: tokens, per-token sequence
// and position, per-sequence slot, start, count and offsets, the wanted rows, the rows the
// last run has to compute, and one page table per group for the step's sequences.
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <exception>
#include <set>
#include <utility>
#include <new>
#include <vector>

#include "tq_engine.h"

namespace {

thread_local char g_error[4096] = "";
thread_local int g_status = 0;

int fail(int code, const char* fmt, ...) {
    g_status = code;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

// A pool of n numbered things, each free or held; hands out the lowest numbers first and
// reuses what came back last.
struct Pool {
    std::vector<int32_t> free;
    std::vector<uint8_t> held;
    int n = 0;
    void init(int count) {
        n = count;
        free.resize(count);
        for (int i = 0; i < count; ++i) free[i] = count - 1 - i;
        held.assign(count, 0);
    }
    int n_free() const { return (int)free.size(); }
    int take() {
        const int i = free.back();
        free.pop_back();
        held[i] = 1;
        return i;
    }
    bool give_back(int i) {
        if (i < 0 || i >= n || !held[i]) return false;
        held[i] = 0;
        free.push_back(i);
        return true;
    }
    // every item is on the free list once or held, never both
    bool consistent(const char* what, char* msg, size_t cap) const {
        std::vector<uint8_t> seen(n, 0);
        for (int i : free) {
            if (i < 0 || i >= n || seen[i]) { snprintf(msg, cap, "%s %d is on the free list twice", what, i); return false; }
            seen[i] = 1;
            if (held[i]) { snprintf(msg, cap, "%s %d is both free and held", what, i); return false; }
        }
        for (int i = 0; i < n; ++i)
            if (!seen[i] && !held[i]) { snprintf(msg, cap, "%s %d is lost", what, i); return false; }
        return true;
    }
};

// The pages of a group.  Pages lie in memory in the order of their numbers, and where a sequence's
// pages lie decides how fast the decoding attention reads them: it reads the same page of every
// sequence at the same time, and runs of pages a power of two apart (equally long prompts: 32 pages
// of a 7B cache are 2 MB) meet the same memory channels again and again.  Measured at 128
// sequences of 33 pages: 104 us for such runs, 97 us for runs one page further apart, 99 us for
// pages anywhere (which cost the rest of the step more than runs do).  So the pool always hands out
// the free page with the lowest number, whatever came back when (runs of neighbours, the same layout
// for every batch on an idle cache), and after a run the caller passes over one or two pages so
// that the next run starts an odd number of pages on: those stay free, but come last.
struct PagePool {
    std::set<std::pair<int32_t, int32_t>> free;        // (0 or 1: passed over, number)
    std::vector<uint8_t> held, late;
    int n = 0;
    void init(int count) {
        n = count;
        free.clear();
        for (int i = 0; i < count; ++i) free.insert(free.end(), std::make_pair(0, i));
        held.assign(count, 0);
        late.assign(count, 0);
    }
    int n_free() const { return (int)free.size(); }
    // what was passed over counts as new again
    void fold_late() {
        std::vector<int32_t> all;
        for (const auto& e : free) all.push_back(e.second);
        std::sort(all.begin(), all.end());
        free.clear();
        for (int32_t j : all) free.insert(free.end(), std::make_pair(0, j));
        late.assign(n, 0);
    }
    int take() {
        if (free.begin()->first != 0) fold_late();                      // no other page is left
        const int i = free.begin()->second;
        free.erase(free.begin());
        held[i] = 1;
        late[i] = 0;
        return i;
    }
    bool give_back(int i) {
        if (i < 0 || i >= n || !held[i]) return false;
        held[i] = 0;
        free.insert(std::make_pair(0, i));
        // Pages that were passed over stay last only while runs are being laid out above them: once no
        // held page lies above the lowest of them (an engine that is never wholly idle still comes
        // here as its oldest sequences end), they are ordinary free pages again.
        if (!free.empty() && free.rbegin()->first != 0) {
            const int lowest_late = free.lower_bound(std::make_pair(1, 0))->second;
            bool held_above = false;
            for (int j = lowest_late + 1; j < n && !held_above; ++j) held_above = held[j] != 0;
            if (!held_above) fold_late();
        }
        return true;
    }
    void pass_over(int k) {
        for (; k > 0 && !free.empty() && free.begin()->first == 0; --k) {
            const int i = free.begin()->second;
            free.erase(free.begin());
            late[i] = 1;
            free.insert(std::make_pair(1, i));
        }
    }
    bool consistent(const char* what, char* msg, size_t cap) const {
        std::vector<uint8_t> seen(n, 0);
        for (const auto& e : free) {
            const int i = e.second;
            if (i < 0 || i >= n || seen[i]) { snprintf(msg, cap, "%s %d is on the free list twice", what, i); return false; }
            seen[i] = 1;
            if (held[i]) { snprintf(msg, cap, "%s %d is both free and held", what, i); return false; }
            if (e.first != late[i]) { snprintf(msg, cap, "%s %d is filed in the wrong place", what, i); return false; }
        }
        for (int i = 0; i < n; ++i)
            if (!seen[i] && !held[i]) { snprintf(msg, cap, "%s %d is lost", what, i); return false; }
        return true;
    }
};

struct Group {
    PagePool pool;
    int window = 0;                                   // 0: every position stays
    std::vector<std::vector<int32_t>> pages;          // per slot: page of positions 64 i .. , -1 where given back
    std::vector<uint8_t> known;                       // per slot: whether the slot has a list at all
};

int pages_for(long long positions) { return (int)((positions + TQE_PAGE - 1) / TQE_PAGE); }

}  // namespace

// the calling thread's last message, for the engine's other files
void tqe_set_error(int code, const char* msg) {
    g_status = code;
    snprintf(g_error, sizeof(g_error), "%s", msg ? msg : "");
}

// No C++ exception crosses the boundary: every entry point that can allocate is a function-try-block
// that turns a failed allocation or a length error into a status and a message.

struct tqe_cache {
    int max_slots = 0;
    Pool slots;
    std::vector<int32_t> lengths;
    std::vector<Group> groups;
};

extern "C" {

const char* tqe_last_error(void) { return g_error; }
int tqe_last_status(void) { return g_status; }
int tqe_abi_version(void) { return 2; }

tqe_cache_t* tqe_cache_new(int max_slots, int n_groups, const int32_t* pages_per_group, const int32_t* window_per_group) try {
    if (max_slots < 1 || n_groups < 0 || n_groups > TQE_MAX_GROUPS || (n_groups > 0 && (!pages_per_group || !window_per_group))) {
        fail(TQE_ERR_ARGUMENT, "tqe_cache_new: bad arguments (slots %d, groups %d)", max_slots, n_groups);
        return nullptr;
    }
    tqe_cache_t* c = new (std::nothrow) tqe_cache();
    if (!c) { fail(TQE_ERR_ARGUMENT, "tqe_cache_new: out of memory"); return nullptr; }
    c->max_slots = max_slots;
    c->slots.init(max_slots);
    c->lengths.assign(max_slots, 0);
    c->groups.resize(n_groups);
    for (int g = 0; g < n_groups; ++g) {
        if (pages_per_group[g] < 0 || window_per_group[g] < 0) {
            fail(TQE_ERR_ARGUMENT, "tqe_cache_new: group %d with %d pages and window %d", g, pages_per_group[g], window_per_group[g]);
            delete c;
            return nullptr;
        }
        c->groups[g].pool.init(pages_per_group[g]);
        c->groups[g].window = window_per_group[g];
        c->groups[g].pages.resize(max_slots);
        c->groups[g].known.assign(max_slots, 0);
    }
    return c;
} catch (const std::exception& e) {
    fail(TQE_ERR_ARGUMENT, "tqe_cache_new: %s", e.what());
    return nullptr;
} catch (...) {
    fail(TQE_ERR_ARGUMENT, "tqe_cache_new: unknown failure");
    return nullptr;
}

void tqe_cache_free(tqe_cache_t* c) { delete c; }

int tqe_cache_acquire(tqe_cache_t* c, int32_t* slot_out) try {
    if (!c || !slot_out) return fail(TQE_ERR_ARGUMENT, "tqe_cache_acquire: null pointer");
    if (c->slots.n_free() < 1) return fail(TQE_ERR_FULL, "need 1 slot(s), 0 free of %d", c->max_slots);
    const int s = c->slots.take();
    c->lengths[s] = 0;
    *slot_out = s;
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_acquire: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_acquire: unknown failure");
}

int tqe_cache_release(tqe_cache_t* c, int slot) try {
    if (!c) return fail(TQE_ERR_ARGUMENT, "tqe_cache_release: null pointer");
    if (!c->slots.give_back(slot)) return fail(TQE_ERR_STATE, "slot %d given back but not held", slot);
    for (Group& g : c->groups) {
        for (int32_t p : g.pages[slot])
            if (p >= 0) g.pool.give_back(p);
        g.pages[slot].clear();
        g.known[slot] = 0;
    }
    c->lengths[slot] = 0;
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_release: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_release: unknown failure");
}

int tqe_cache_length(const tqe_cache_t* c, int slot) {
    if (!c || slot < 0 || slot >= c->max_slots) return fail(TQE_ERR_ARGUMENT, "tqe_cache_length: no slot %d", slot);
    return c->lengths[slot];
}

int tqe_cache_is_held(const tqe_cache_t* c, int slot) {
    return c && slot >= 0 && slot < c->max_slots && c->slots.held[slot];
}

int tqe_cache_counts(const tqe_cache_t* c, int group, int32_t* n_free, int32_t* n_total) {
    if (!c || group < -1 || group >= (int)c->groups.size()) return fail(TQE_ERR_ARGUMENT, "tqe_cache_counts: no group %d", group);
    if (n_free) *n_free = group < 0 ? c->slots.n_free() : c->groups[group].pool.n_free();
    if (n_total) *n_total = group < 0 ? c->slots.n : c->groups[group].pool.n;
    return TQE_OK;
}

int tqe_cache_reserve(tqe_cache_t* c, int n, const int32_t* slots, const int32_t* n_new) try {
    if (!c || (n > 0 && (!slots || !n_new))) return fail(TQE_ERR_ARGUMENT, "tqe_cache_reserve: null pointer");
    if (n < 0) return fail(TQE_ERR_ARGUMENT, "tqe_cache_reserve: %d sequences", n);
    for (int i = 0; i < n; ++i) {
        if (slots[i] < 0 || slots[i] >= c->max_slots || !c->slots.held[slots[i]]) return fail(TQE_ERR_STATE, "slot %d is not held", slots[i]);
        if (n_new[i] < 0) return fail(TQE_ERR_ARGUMENT, "tqe_cache_reserve: %d new positions for slot %d", n_new[i], slots[i]);
    }
    for (const Group& g : c->groups) {
        long long want = 0;
        for (int i = 0; i < n; ++i) {
            const int need = pages_for((long long)c->lengths[slots[i]] + n_new[i]) - (int)g.pages[slots[i]].size();
            if (need > 0) want += need;
        }
        if (want > g.pool.n_free())
            return fail(TQE_ERR_FULL, "step needs %lld more pages of %d positions, %d free of %d", want, TQE_PAGE, g.pool.n_free(), g.pool.n);
    }
    for (Group& g : c->groups)
        for (int i = 0; i < n; ++i) {
            std::vector<int32_t>& have = g.pages[slots[i]];
            const int need = pages_for((long long)c->lengths[slots[i]] + n_new[i]);
            g.known[slots[i]] = 1;
            int took = 0;
            for (; (int)have.size() < need; ++took) have.push_back(g.pool.take());
            // the next run starts an odd number of pages on (see PagePool)
            if (took > 1) g.pool.pass_over(took % 2 == 0 ? 1 : 2);
        }
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_reserve: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_reserve: unknown failure");
}

int tqe_cache_commit(tqe_cache_t* c, int n, const int32_t* slots, const int32_t* n_new) try {
    if (!c || (n > 0 && (!slots || !n_new))) return fail(TQE_ERR_ARGUMENT, "tqe_cache_commit: null pointer");
    if (n < 0) return fail(TQE_ERR_ARGUMENT, "tqe_cache_commit: %d sequences", n);
    // all of them or none: every slot is looked at before any length changes
    for (int i = 0; i < n; ++i) {
        const int s = slots[i];
        if (s < 0 || s >= c->max_slots || !c->slots.held[s]) return fail(TQE_ERR_STATE, "slot %d is not held", s);
        if (n_new[i] < 0) return fail(TQE_ERR_ARGUMENT, "tqe_cache_commit: %d new positions for slot %d", n_new[i], s);
        if ((long long)c->lengths[s] + n_new[i] > 0x7fffffffLL) return fail(TQE_ERR_ARGUMENT, "tqe_cache_commit: slot %d would hold too many positions", s);
        for (const Group& g : c->groups)
            if (pages_for((long long)c->lengths[s] + n_new[i]) > (int)g.pages[s].size())
                return fail(TQE_ERR_STATE, "slot %d commits %d positions that were not reserved", s, n_new[i]);
    }
    for (int i = 0; i < n; ++i) {
        const int s = slots[i];
        c->lengths[s] += n_new[i];
        for (Group& g : c->groups) {
            if (g.window <= 0) continue;
            // pages whose positions are all out of the window of the next query go back
            std::vector<int32_t>& have = g.pages[s];
            const int first_needed = std::max(0, c->lengths[s] + 1 - g.window);
            const int dead = std::min(first_needed / TQE_PAGE, (int)have.size());
            for (int k = 0; k < dead; ++k)
                if (have[k] >= 0) { g.pool.give_back(have[k]); have[k] = -1; }
        }
    }
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_commit: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_commit: unknown failure");
}

int tqe_cache_trim(tqe_cache_t* c, int n, const int32_t* slots) try {
    if (!c || (n > 0 && !slots)) return fail(TQE_ERR_ARGUMENT, "tqe_cache_trim: null pointer");
    for (int i = 0; i < n; ++i)
        if (slots[i] < 0 || slots[i] >= c->max_slots || !c->slots.held[slots[i]]) return fail(TQE_ERR_STATE, "slot %d is not held", slots[i]);
    for (Group& g : c->groups)
        for (int i = 0; i < n; ++i) {
            std::vector<int32_t>& have = g.pages[slots[i]];
            const size_t keep = (size_t)pages_for(c->lengths[slots[i]]);
            while (have.size() > keep) {
                if (have.back() >= 0) g.pool.give_back(have.back());
                have.pop_back();
            }
        }
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_trim: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_trim: unknown failure");
}

int tqe_cache_pages(const tqe_cache_t* c, int group, int slot, int32_t* out, int cap) try {
    if (!c || group < 0 || group >= (int)c->groups.size() || slot < 0 || slot >= c->max_slots)
        return fail(TQE_ERR_ARGUMENT, "tqe_cache_pages: no group %d or slot %d", group, slot);
    const Group& g = c->groups[group];
    if (!g.known[slot]) return TQE_NO_LIST;                    // (distinct from an empty list)
    const std::vector<int32_t>& have = g.pages[slot];
    if (out)
        for (int i = 0; i < (int)have.size() && i < cap; ++i) out[i] = have[i];
    return (int)have.size();
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_pages: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_pages: unknown failure");
}

int tqe_cache_check(const tqe_cache_t* c) try {
    if (!c) return fail(TQE_ERR_ARGUMENT, "tqe_cache_check: null pointer");
    char msg[256];
    if (!c->slots.consistent("slot", msg, sizeof(msg))) return fail(TQE_ERR_STATE, "%s", msg);
    for (const Group& g : c->groups) {
        if (!g.pool.consistent("page", msg, sizeof(msg))) return fail(TQE_ERR_STATE, "%s", msg);
        std::vector<uint8_t> seen(g.pool.n, 0);
        int held = 0;
        for (int s = 0; s < c->max_slots; ++s) {
            if (!g.pages[s].empty() && !c->slots.held[s]) return fail(TQE_ERR_STATE, "free slot %d still holds pages", s);
            for (int32_t p : g.pages[s]) {
                if (p < 0) continue;
                if (p >= g.pool.n || seen[p]) return fail(TQE_ERR_STATE, "a page is held by two sequences");
                seen[p] = 1;
                ++held;
            }
        }
        if (held != g.pool.n - g.pool.n_free())
            return fail(TQE_ERR_STATE, "%d pages held by sequences, pool says %d", held, g.pool.n - g.pool.n_free());
    }
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_check: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_cache_check: unknown failure");
}

// ---- the step's arrays ------------------------------------------------------------------------
int tqe_check_step(const tqe_cache_t* c, int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens,
                   int vocab_size, int max_positions) try {
    if (!c) return fail(TQE_ERR_ARGUMENT, "tqe_check_step: null pointer");
    if (n_seqs < 1 || !slots || !n_new) return fail(TQE_ERR_STEP, "a step needs at least one sequence");
    std::vector<uint8_t> seen(c->max_slots, 0);
    size_t at = 0;
    for (int i = 0; i < n_seqs; ++i) {
        const int s = slots[i];
        if (s < 0 || s >= c->max_slots || !c->slots.held[s]) return fail(TQE_ERR_STATE, "slot %d is not held", s);
        if (seen[s]) return fail(TQE_ERR_STEP, "slot %d appears twice in one step", s);
        seen[s] = 1;
        if (n_new[i] < 1) return fail(TQE_ERR_STEP, "Empty prompt");
        if (tokens)
            for (int t = 0; t < n_new[i]; ++t, ++at)
                if (tokens[at] < 0 || tokens[at] >= vocab_size)
                    return fail(TQE_ERR_STEP, "token id %d is outside the vocabulary of %d", tokens[at], vocab_size);
        if ((long long)c->lengths[s] + n_new[i] > max_positions)
            return fail(TQE_ERR_STEP, "sequence would reach %lld positions, the model has %d", (long long)c->lengths[s] + n_new[i], max_positions);
    }
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_check_step: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_check_step: unknown failure");
}


int tqe_plan_step(const tqe_cache_t* c, int n_seqs, const int32_t* slots, const int32_t* starts, const int32_t* n_new,
                  const int32_t* tokens, const int32_t* want_counts, const int32_t* want_idx, int width_step,
                  int32_t* out, int out_cap, int32_t* meta) try {
    if (n_seqs < 1 || !slots || !n_new || !want_counts || !meta) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: bad arguments");
    if (!c && !starts) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: without a cache the sequences' starts must be given");
    const int n_groups = c ? (int)c->groups.size() : 0;
    long long n_tokens = 0, n_want = 0;
    int max_new = 0;
    bool all_decode = true;
    for (int i = 0; i < n_seqs; ++i) {
        if (n_new[i] < 1) return fail(TQE_ERR_ARGUMENT, "sequence %d of the step brings no token", i);
        if (c && (slots[i] < 0 || slots[i] >= c->max_slots)) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: no slot %d", slots[i]);
        if (want_counts[i] < 0) return fail(TQE_ERR_ARGUMENT, "sequence %d of the step wants %d places", i, want_counts[i]);
        n_tokens += n_new[i];
        n_want += want_counts[i];
        max_new = std::max(max_new, n_new[i]);
        all_decode = all_decode && n_new[i] == 1;
    }
    if (n_tokens > 0x3fffffff) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: %lld tokens in one step", n_tokens);
    if (n_want > 0 && !want_idx) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: wanted places without their list");
    // the wanted rows, and those of them the last run computes: each once, in order
    std::vector<int32_t> cu(n_seqs + 1, 0), want_rows((size_t)n_want);
    for (int i = 0; i < n_seqs; ++i) cu[i + 1] = cu[i] + n_new[i];
    {
        size_t k = 0;
        for (int i = 0; i < n_seqs; ++i)
            for (int j = 0; j < want_counts[i]; ++j, ++k) {
                const int at = want_idx[k];
                if (at < 0 || at >= n_new[i])
                    return fail(TQE_ERR_RANGE, "wanted place %d is outside the %d tokens of sequence %d", at, n_new[i], i);
                want_rows[k] = cu[i] + at;
            }
    }
    std::vector<int32_t> last_rows(want_rows);
    std::sort(last_rows.begin(), last_rows.end());
    last_rows.erase(std::unique(last_rows.begin(), last_rows.end()), last_rows.end());
    const int n_last = (int)last_rows.size();
    const bool prune_last = !all_decode && n_last < n_tokens;
    const int n_last_kept = prune_last ? n_last : 0;
    // page table widths
    std::vector<int> width(n_groups, 1);
    for (int g = 0; g < n_groups; ++g) {
        int wmax = 1;
        for (int i = 0; i < n_seqs; ++i) wmax = std::max(wmax, (int)c->groups[g].pages[slots[i]].size());
        if (width_step > 1) wmax = (wmax + width_step - 1) / width_step * width_step;
        width[g] = wmax;
    }
    // layout: every array starts at a multiple of 4 values
    const long long sizes[12] = {n_tokens, n_tokens, n_tokens, n_seqs, n_seqs, n_seqs, n_seqs + 1, n_want,
                                 n_last_kept, prune_last ? n_want : 0, n_last_kept, n_last_kept};
    long long total = 0;
    int32_t* offsets = meta + TQE_META_OFFSETS;
    for (int a = 0; a < 12; ++a) {
        offsets[a] = (int32_t)total;
        total += (sizes[a] + 3) / 4 * 4;
    }
    for (int g = 0; g < n_groups; ++g) {
        offsets[12 + g] = (int32_t)total;
        total += ((long long)n_seqs * width[g] + 3) / 4 * 4;
    }
    if (total < 4) total = 4;
    if (total > 0x7fffffff) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: the step's arrays are too large");
    int max_end = 0;
    for (int i = 0; i < n_seqs; ++i) max_end = std::max(max_end, (starts ? starts[i] : c->lengths[slots[i]]) + n_new[i]);
    meta[TQE_META_TOTAL] = (int32_t)total;
    meta[TQE_META_TOKENS] = (int32_t)n_tokens;
    meta[TQE_META_WANT] = (int32_t)n_want;
    meta[TQE_META_LAST] = n_last;
    meta[TQE_META_ALL_DECODE] = all_decode ? 1 : 0;
    meta[TQE_META_PRUNE_LAST] = prune_last ? 1 : 0;
    meta[TQE_META_MAX_NEW] = max_new;
    meta[TQE_META_MAX_END] = max_end;
    meta[TQE_META_GROUPS] = n_groups;
    for (int g = 0; g < n_groups; ++g) meta[TQE_META_OFFSETS + 12 + TQE_MAX_GROUPS + g] = width[g];
    if (!out) return TQE_OK;                                   // sizes only
    if (out_cap < total) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: %lld values do not fit the %d given", total, out_cap);
    if (!tokens) return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: no tokens");
    memset(out, 0, sizeof(int32_t) * (size_t)total);
    int32_t* o_tokens = out + offsets[0];
    int32_t* o_tok_seq = out + offsets[1];
    int32_t* o_tok_pos = out + offsets[2];
    int32_t* o_slot = out + offsets[3];
    int32_t* o_start = out + offsets[4];
    int32_t* o_new = out + offsets[5];
    int32_t* o_cu = out + offsets[6];
    int32_t* o_want = out + offsets[7];
    memcpy(o_tokens, tokens, sizeof(int32_t) * (size_t)n_tokens);
    for (int i = 0; i < n_seqs; ++i) {
        const int start = starts ? starts[i] : c->lengths[slots[i]];
        o_slot[i] = slots[i];
        o_start[i] = start;
        o_new[i] = n_new[i];
        o_cu[i] = cu[i];
        for (int t = 0; t < n_new[i]; ++t) {
            o_tok_seq[cu[i] + t] = i;
            o_tok_pos[cu[i] + t] = start + t;
        }
    }
    o_cu[n_seqs] = cu[n_seqs];
    for (long long k = 0; k < n_want; ++k) o_want[k] = want_rows[(size_t)k];
    if (prune_last) {
        int32_t* o_last = out + offsets[8];
        int32_t* o_in_last = out + offsets[9];
        int32_t* o_last_seq = out + offsets[10];
        int32_t* o_last_pos = out + offsets[11];
        for (int k = 0; k < n_last; ++k) {
            o_last[k] = last_rows[k];
            o_last_seq[k] = o_tok_seq[last_rows[k]];
            o_last_pos[k] = o_tok_pos[last_rows[k]];
        }
        for (long long k = 0; k < n_want; ++k)
            o_in_last[k] = (int32_t)(std::lower_bound(last_rows.begin(), last_rows.end(), want_rows[(size_t)k]) - last_rows.begin());
    }
    for (int g = 0; g < n_groups; ++g) {
        int32_t* table = out + offsets[12 + g];
        for (long long k = 0; k < (long long)n_seqs * width[g]; ++k) table[k] = -1;
        for (int i = 0; i < n_seqs; ++i) {
            const std::vector<int32_t>& have = c->groups[g].pages[slots[i]];
            for (size_t k = 0; k < have.size(); ++k) table[(size_t)i * width[g] + k] = have[k];
        }
    }
    return TQE_OK;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_plan_step: unknown failure");
}

}  // extern "C"

// ---- the generation loop's decisions ------------------------------------------------------------
struct tqe_batch {
    int max_new;
    std::vector<int32_t> stop;          // sorted
    std::vector<int32_t> emitted;
    std::vector<uint8_t> ended;
};

int tqe_plan_batches(int n, const int32_t* prompt_lens, int max_new, long long max_tokens, int max_batch, int holds_pages,
                     int32_t* batch_of) try {
    if (n < 0 || (n > 0 && (!prompt_lens || !batch_of)) || max_batch < 1) return fail(TQE_ERR_ARGUMENT, "tqe_plan_batches: bad arguments");
    int batch = 0, in_batch = 0;
    long long used = 0;
    for (int i = 0; i < n; ++i) {
        long long need = 0;
        if (holds_pages) need = (long long)pages_for((long long)prompt_lens[i] + std::max(0, max_new - 1)) * TQE_PAGE;
        if (need > max_tokens) return fail(TQE_ERR_FULL, "request %d needs %lld cache positions, the engine has %lld", i, need, max_tokens);
        if (in_batch > 0 && (in_batch >= max_batch || used + need > max_tokens)) {
            ++batch;
            in_batch = 0;
            used = 0;
        }
        batch_of[i] = batch;
        ++in_batch;
        used += need;
    }
    return n > 0 ? batch + 1 : 0;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_plan_batches: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_plan_batches: unknown failure");
}

int tqe_prompt_steps(int n, const int32_t* lens, int max_step_tokens, int32_t* pieces, int capacity) try {
    if (n < 0 || (n > 0 && !lens) || max_step_tokens < 1 || capacity < 0 || (capacity > 0 && !pieces))
        return fail(TQE_ERR_ARGUMENT, "tqe_prompt_steps: bad arguments");
    int count = 0, step = 0, room = max_step_tokens;
    for (int i = 0; i < n; ++i) {
        int begin = 0;
        while (begin < lens[i]) {
            const int take = std::min(lens[i] - begin, room);
            if (count < capacity) {
                int32_t* p = pieces + (size_t)count * 4;
                p[0] = i; p[1] = begin; p[2] = begin + take; p[3] = step;
            }
            ++count;
            begin += take;
            room -= take;
            if (room == 0) {
                ++step;
                room = max_step_tokens;
            }
        }
    }
    return count;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_prompt_steps: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_prompt_steps: unknown failure");
}

tqe_batch_t* tqe_batch_new(int n_requests, int max_new, const int32_t* stop_ids, int n_stop_ids) try {
    if (n_requests < 0 || n_stop_ids < 0 || (n_stop_ids > 0 && !stop_ids)) {
        fail(TQE_ERR_ARGUMENT, "tqe_batch_new: bad arguments");
        return nullptr;
    }
    tqe_batch_t* b = new (std::nothrow) tqe_batch_t();
    if (!b) {
        fail(TQE_ERR_ARGUMENT, "tqe_batch_new: out of memory");
        return nullptr;
    }
    b->max_new = max_new;
    for (int i = 0; i < n_stop_ids; ++i)
        if (stop_ids[i] >= 0) b->stop.push_back(stop_ids[i]);       // no token has a negative id: such an entry stops nothing
    std::sort(b->stop.begin(), b->stop.end());
    b->emitted.assign(n_requests, 0);
    b->ended.assign(n_requests, 0);
    return b;
} catch (const std::exception& e) {
    fail(TQE_ERR_ARGUMENT, "tqe_batch_new: %s", e.what());
    return nullptr;
} catch (...) {
    fail(TQE_ERR_ARGUMENT, "tqe_batch_new: unknown failure");
    return nullptr;
}

void tqe_batch_free(tqe_batch_t* b) { delete b; }

int tqe_batch_accept(tqe_batch_t* b, int row, int token) try {
    if (!b || row < 0 || row >= (int)b->emitted.size()) return fail(TQE_ERR_ARGUMENT, "tqe_batch_accept: no request %d", row);
    if (b->ended[row]) return TQE_TOKEN_DROPPED;
    if (b->emitted[row] >= b->max_new || std::binary_search(b->stop.begin(), b->stop.end(), (int32_t)token)) {
        b->ended[row] = 1;
        return TQE_TOKEN_STOP;
    }
    if (++b->emitted[row] >= b->max_new) {
        b->ended[row] = 1;
        return TQE_TOKEN_LAST;
    }
    return TQE_TOKEN_FEED;
} catch (const std::exception& e) {
    return fail(TQE_ERR_ARGUMENT, "tqe_batch_accept: %s", e.what());
} catch (...) {
    return fail(TQE_ERR_ARGUMENT, "tqe_batch_accept: unknown failure");
}

int tqe_batch_goes_on(const tqe_batch_t* b, int row) {
    return b && row >= 0 && row < (int)b->emitted.size() && !b->ended[row] && b->emitted[row] + 1 < b->max_new;
}

int tqe_batch_emitted(const tqe_batch_t* b, int row) {
    if (!b || row < 0 || row >= (int)b->emitted.size()) return fail(TQE_ERR_ARGUMENT, "tqe_batch_emitted: no request %d", row);
    return b->emitted[row];
}

int tqe_batch_ended(const tqe_batch_t* b, int row) {
    return b && row >= 0 && row < (int)b->emitted.size() && b->ended[row];
}
