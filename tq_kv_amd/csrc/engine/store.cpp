#include "store.h"

namespace tq {

static void check_status(int status) {
    if (status != TQE_OK) throw Error(status, tqe_last_error());
}

CacheStore::CacheStore(const std::vector<CacheNeed>& needs, const std::vector<int>& cache_of, long long max_tokens, int max_slots_, int dtype) {
    if (needs.size() != cache_of.size()) raise(TQE_ERR_ARGUMENT, "cache: %zu needs for %zu runs", needs.size(), cache_of.size());
    const size_t n_runs = needs.size();
    // pages bound the cache only where some run keeps keys and values: a model whose runs all keep
    // fixed-size state (or nothing) is bounded by its slots alone
    for (size_t r = 0; r < n_runs; ++r) holds_pages = holds_pages || (needs[r].kind == CacheNeed::Pages && cache_of[r] < 0);
    if (holds_pages && max_tokens < TQE_PAGE) raise(TQE_ERR_ARGUMENT, "max_tokens must be at least %d, got %lld", TQE_PAGE, max_tokens);
    if (max_tokens / TQE_PAGE > 0x3fffffff) raise(TQE_ERR_ARGUMENT, "max_tokens %lld is too large", max_tokens);
    n_pages = holds_pages ? (int)(max_tokens / TQE_PAGE) : 0;
    max_slots = holds_pages ? std::max(1, std::min(max_slots_, n_pages)) : std::max(1, max_slots_);

    struct Place { bool pages; size_t group; int index; };
    std::vector<Place> place(n_runs, Place{false, 0, -1});
    for (size_t r = 0; r < n_runs; ++r) {
        const CacheNeed& need = needs[r];
        if (need.kind == CacheNeed::None || cache_of[r] >= 0) continue;
        if (need.kind == CacheNeed::Pages) {
            size_t g = 0;
            for (; g < page_groups.size(); ++g)
                if (page_groups[g].need == need) break;
            if (g == page_groups.size()) { page_groups.emplace_back(); page_groups[g].need = need; page_groups[g].n_pages = n_pages; }
            place[r] = Place{true, g, (int)page_groups[g].runs.size()};
            page_groups[g].runs.push_back((int)r);
        } else {
            size_t g = 0;
            for (; g < state_groups.size(); ++g)
                if (state_groups[g].need == need) break;
            if (g == state_groups.size()) { state_groups.emplace_back(); state_groups[g].need = need; }
            place[r] = Place{false, g, (int)state_groups[g].runs.size()};
            state_groups[g].runs.push_back((int)r);
        }
    }
    if ((int)page_groups.size() > TQE_MAX_GROUPS)
        raise(TQE_ERR_ARGUMENT, "%zu groups of cached runs, the engine's bookkeeping takes %d", page_groups.size(), TQE_MAX_GROUPS);
    for (PageGroup& g : page_groups) {
        std::vector<int64_t> kd = {(int64_t)g.runs.size(), n_pages}, vd = kd;
        kd.insert(kd.end(), g.need.key_page.begin(), g.need.key_page.end());
        vd.insert(vd.end(), g.need.value_page.begin(), g.need.value_page.end());
        g.keys = make_owned(dtype, kd);
        g.values = make_owned(dtype, vd);
        zero_device(g.keys->t.data, g.keys->t.bytes(), nullptr);
        zero_device(g.values->t.data, g.values->t.bytes(), nullptr);
    }
    for (StateGroup& g : state_groups) {
        std::vector<int64_t> d = {(int64_t)g.runs.size(), max_slots};
        d.insert(d.end(), g.need.state_shape.begin(), g.need.state_shape.end());
        g.state = make_owned(g.need.state_dtype, d);
        zero_device(g.state->t.data, g.state->t.bytes(), nullptr);
    }
    stream_synchronize(nullptr);

    std::vector<int32_t> pages, windows;
    for (const PageGroup& g : page_groups) { pages.push_back(g.n_pages); windows.push_back(g.need.window); }
    book = tqe_cache_new(max_slots, (int)page_groups.size(), pages.data(), windows.data());
    if (!book) throw Error(TQE_ERR_ARGUMENT, tqe_last_error());

    // what each run sees
    entries_.assign(n_runs, CacheEntry());
    for (size_t r = 0; r < n_runs; ++r) {
        const CacheNeed& need = needs[r];
        if (need.kind == CacheNeed::None) continue;
        const int src = cache_of[r];
        const size_t owner = src < 0 ? r : (size_t)src;
        if (owner >= n_runs || place[owner].index < 0) {
            tqe_cache_free(book);
            book = nullptr;
            raise(TQE_ERR_ARGUMENT, "run %zu reads the cache of run %zu, which keeps none", r, owner);
        }
        if (src >= 0 && !(needs[owner] == need)) {
            tqe_cache_free(book);
            book = nullptr;
            raise(TQE_ERR_ARGUMENT, "run %zu needs another cache than run %zu keeps", r, owner);
        }
        CacheEntry& e = entries_[r];
        e.kind = need.kind;
        e.writes = src < 0;
        const Place& p = place[owner];
        if (p.pages) {
            const PageGroup& g = page_groups[p.group];
            e.group = (int)p.group;
            e.window = need.window;
            e.keys = g.keys->t.slice(p.index, p.index + 1);
            e.values = g.values->t.slice(p.index, p.index + 1);
            // drop the leading dimension of one run
            for (Tensor* t : {&e.keys, &e.values}) {
                for (int i = 0; i + 1 < t->ndim; ++i) t->shape[i] = t->shape[i + 1];
                --t->ndim;
            }
        } else {
            const StateGroup& g = state_groups[p.group];
            e.state = g.state->t.slice(p.index, p.index + 1);
            for (int i = 0; i + 1 < e.state.ndim; ++i) e.state.shape[i] = e.state.shape[i + 1];
            --e.state.ndim;
        }
    }
}

CacheStore::~CacheStore() {
    if (book) tqe_cache_free(book);
}

int CacheStore::acquire(hipStream_t stream) {
    int32_t slot = -1;
    check_status(tqe_cache_acquire(book, &slot));
    for (StateGroup& g : state_groups) {
        const Tensor& t = g.state->t;
        const size_t row = t.bytes() / (size_t)(t.shape[0] * t.shape[1]);
        for (int64_t r = 0; r < t.shape[0]; ++r) zero_device((char*)t.data + ((size_t)r * t.shape[1] + (size_t)slot) * row, row, stream);
    }
    return slot;
}

void CacheStore::release(int slot) { check_status(tqe_cache_release(book, slot)); }

int CacheStore::length(int slot) const {
    const int n = tqe_cache_length(book, slot);
    if (n < 0) throw Error(n, tqe_last_error());
    return n;
}

void CacheStore::reserve(int n, const int32_t* slots, const int32_t* n_new) { check_status(tqe_cache_reserve(book, n, slots, n_new)); }
void CacheStore::commit(int n, const int32_t* slots, const int32_t* n_new) { check_status(tqe_cache_commit(book, n, slots, n_new)); }

static Json tensor_json(const Tensor& t) {
    Json j = Json::object();
    j.set("data", (long long)(uintptr_t)t.data);
    j.set("dtype", dtype_name(t.dtype));
    Json shape = Json::array();
    for (int i = 0; i < t.ndim; ++i) shape.push(Json((long long)t.shape[i]));
    j.set("shape", shape);
    return j;
}

Json CacheStore::describe() const {
    Json j = Json::object();
    j.set("holds_pages", holds_pages);
    j.set("n_pages", n_pages);
    j.set("max_slots", max_slots);
    Json pg = Json::array();
    for (const PageGroup& g : page_groups) {
        Json o = Json::object();
        o.set("need", g.need.to_json());
        Json runs = Json::array();
        for (int r : g.runs) runs.push(Json(r));
        o.set("runs", runs);
        o.set("n_pages", g.n_pages);
        o.set("keys", tensor_json(g.keys->t));
        o.set("values", tensor_json(g.values->t));
        pg.push(o);
    }
    j.set("page_groups", pg);
    Json sg = Json::array();
    for (const StateGroup& g : state_groups) {
        Json o = Json::object();
        o.set("need", g.need.to_json());
        Json runs = Json::array();
        for (int r : g.runs) runs.push(Json(r));
        o.set("runs", runs);
        o.set("state", tensor_json(g.state->t));
        sg.push(o);
    }
    j.set("state_groups", sg);
    return j;
}

}  // namespace tq
