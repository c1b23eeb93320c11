#include "step.h"

#include <algorithm>
#include <numeric>

#include "parts.h"

namespace tq {

StepContext::StepContext() { memset(meta_, 0, sizeof(meta_)); }
StepContext::~StepContext() {}

void StepContext::carve(StepArrays& out, const int32_t* base, const int32_t* meta) {
    const int32_t* off = meta + TQE_META_OFFSETS;
    out.tokens = base + off[0];
    out.tok_seq = base + off[1];
    out.tok_pos = base + off[2];
    out.seq_slot = base + off[3];
    out.seq_start = base + off[4];
    out.seq_new = base + off[5];
    out.cu = base + off[6];
    out.want_rows = base + off[7];
    out.last_rows = base + off[8];
    out.want_in_last = base + off[9];
    out.last_seq = base + off[10];
    out.last_pos = base + off[11];
}

void StepContext::plan(const tqe_cache* cache, int n, const int32_t* slots, const int32_t* starts, const int32_t* n_new,
                       const int32_t* tokens, const int32_t* want_counts, const int32_t* want_idx, int width_step) {
    int status = tqe_plan_step(cache, n, slots, starts, n_new, tokens, want_counts, want_idx, width_step, nullptr, 0, meta_);
    if (status != TQE_OK) throw Error(status, tqe_last_error());
    packed.assign((size_t)meta_[TQE_META_TOTAL], 0);
    status = tqe_plan_step(cache, n, slots, starts, n_new, tokens, want_counts, want_idx, width_step, packed.data(), (int)packed.size(), meta_);
    if (status != TQE_OK) throw Error(status, tqe_last_error());
    n_seqs = n;
    n_tokens = meta_[TQE_META_TOKENS];
    n_want = meta_[TQE_META_WANT];
    n_last = meta_[TQE_META_LAST];
    all_decode = meta_[TQE_META_ALL_DECODE] != 0;
    prune_last = meta_[TQE_META_PRUNE_LAST] != 0;
    max_new = meta_[TQE_META_MAX_NEW];
    max_end = meta_[TQE_META_MAX_END];
    flat_count = packed.size();
    lens.assign(n_new, n_new + n);
    carve(host, packed.data(), meta_);
    const int n_groups = meta_[TQE_META_GROUPS];
    tables.assign((size_t)n_groups, Table());
    for (int g = 0; g < n_groups; ++g) {
        tables[(size_t)g].host = packed.data() + meta_[TQE_META_OFFSETS + 12 + g];
        tables[(size_t)g].width = meta_[TQE_META_OFFSETS + 12 + TQE_MAX_GROUPS + g];
    }
    tiles_.clear();
    memo.clear();
}

void StepContext::upload(int32_t* into) {
    flat = into ? into : (int32_t*)ws->alloc(flat_count * sizeof(int32_t));
    staging->upload(flat, packed.data(), flat_count * sizeof(int32_t), stream);
    carve(dev, flat, meta_);
    for (size_t g = 0; g < tables.size(); ++g) tables[g].dev = flat + meta_[TQE_META_OFFSETS + 12 + g];
}

StepShape StepContext::shape() const {
    StepShape s;
    s.n_tokens = n_tokens;
    s.n_seqs = n_seqs;
    s.n_want = n_want;
    for (const Table& t : tables) s.widths.push_back(t.width);
    return s;
}

Tiles StepContext::upload_tiles(std::vector<int32_t>& seq, std::vector<int32_t>& tok0, std::vector<int32_t>& count,
                                const std::vector<long long>& reach) {
    const size_t n = seq.size();
    std::vector<size_t> order(n);
    std::iota(order.begin(), order.end(), (size_t)0);
    // longest first: a tile's work grows with its last position
    std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return reach[a] > reach[b]; });
    std::vector<int32_t> host(3 * n);
    for (size_t i = 0; i < n; ++i) {
        host[i] = seq[order[i]];
        host[n + i] = tok0[order[i]];
        host[2 * n + i] = count[order[i]];
    }
    Tiles t;
    t.n = (int)n;
    if (n == 0) return t;
    if (capturing) raise(TQE_ERR_STATE, "a part asked for query tiles while its step was being captured as a graph (it is not graph_safe)");
    int32_t* dev_mem = (int32_t*)ws->alloc_for_step(host.size() * sizeof(int32_t));     // later layers read them too
    staging->upload(dev_mem, host.data(), host.size() * sizeof(int32_t), stream);
    t.seq = dev_mem;
    t.tok0 = dev_mem + n;
    t.count = dev_mem + 2 * n;
    return t;
}

Tiles StepContext::query_tiles(int tile) {
    const auto key = std::make_pair(0, tile);
    auto it = tiles_.find(key);
    if (it != tiles_.end()) return it->second;
    std::vector<int32_t> seq, tok0, count;
    std::vector<long long> reach;
    for (int i = 0; i < n_seqs; ++i)
        for (int a = 0; a < lens[(size_t)i]; a += tile) {
            const int c = std::min(tile, lens[(size_t)i] - a);
            seq.push_back(i);
            tok0.push_back(host.cu[i] + a);
            count.push_back(c);
            reach.push_back((long long)host.tok_pos[host.cu[i] + a] + c);
        }
    return tiles_[key] = upload_tiles(seq, tok0, count, reach);
}

Tiles StepContext::last_tiles(int tile) {
    const auto key = std::make_pair(1, tile);
    auto it = tiles_.find(key);
    if (it != tiles_.end()) return it->second;
    std::vector<int32_t> seq, tok0, count;
    std::vector<long long> reach;
    int k = 0;
    while (prune_last && k < n_last) {
        int j = k + 1;
        while (j < n_last && j - k < tile && host.last_rows[j] == host.last_rows[j - 1] + 1 && host.last_seq[j] == host.last_seq[k]) ++j;
        seq.push_back(host.last_seq[k]);
        tok0.push_back(k);
        count.push_back(j - k);
        reach.push_back((long long)host.last_pos[k] + (j - k));
        k = j;
    }
    return tiles_[key] = upload_tiles(seq, tok0, count, reach);
}

}  // namespace tq
