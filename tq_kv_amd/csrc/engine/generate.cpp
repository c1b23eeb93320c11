#include "generate.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <map>

#include "kernels.h"

namespace tq {

void GenerationParams::validate() const {
    if (max_tokens < 0) raise(TQE_ERR_ARGUMENT, "max_tokens must not be negative, got %d", max_tokens);
    if (top_k < 0) raise(TQE_ERR_ARGUMENT, "top_k must not be negative, got %d", top_k);
    if (!(top_p > 0.0f)) raise(TQE_ERR_ARGUMENT, "top_p must be positive, got %g", (double)top_p);
    if (!(repeat_penalty > 0.0f)) raise(TQE_ERR_ARGUMENT, "repeat_penalty must be positive, got %g", (double)repeat_penalty);
}

// Integer mixing (three rounds of the splitmix64 finaliser, one each for seed, request and step), top
// 24 bits taken as a float32 in [0, 1).
static uint64_t mix64(uint64_t x) {
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

float draw_uniform(uint64_t seed, uint64_t request, uint64_t step) {
    const uint64_t golden = 0x9E3779B97F4A7C15ull;
    uint64_t x = mix64(seed + golden);
    x = mix64((x ^ request) + golden);
    x = mix64((x ^ step) + golden);
    return (float)((double)(x >> 40) / (double)(1 << 24));
}

// ---- the engine as the loop sees it ---------------------------------------------------------------
const float* EngineForLoop::step(const std::vector<StepItem>& items, const int32_t* device_tokens) {
    const size_t n = items.size();
    std::vector<int32_t> slots(n), n_new(n), want_counts(n), want_idx, tokens;
    for (size_t i = 0; i < n; ++i) {
        slots[i] = items[i].slot;
        n_new[i] = items[i].n_tokens;
        want_counts[i] = items[i].want_last ? 1 : 0;
        if (items[i].want_last) want_idx.push_back(items[i].n_tokens - 1);
        if (!device_tokens) tokens.insert(tokens.end(), items[i].tokens, items[i].tokens + items[i].n_tokens);
    }
    // the loop is done with a step's logits before it starts the next one: they stay in the engine's memory
    return e_.step((int)n, slots.data(), n_new.data(), device_tokens ? nullptr : tokens.data(), want_counts.data(), want_idx.data(), device_tokens,
                   nullptr, stream_);
}

// ---- the device sampler -----------------------------------------------------------------------------
class DeviceDraw : public Draw {
public:
    DeviceDraw(const int32_t* device, const int32_t* host, int n, hipEvent_t event) : device_(device), host_(host), n_(n), event_(event) {}
    std::vector<int32_t> read() override {
        if (!null_device()) hip_check(hipEventSynchronize(event_), "waiting for a draw");
        return std::vector<int32_t>(host_, host_ + n_);
    }
    const int32_t* device_;
    const int32_t* host_;
    int n_;
    hipEvent_t event_;
};

DeviceSampler::DeviceSampler(const GenerationParams& params, const std::vector<int>& request_ids, int vocab, hipStream_t stream)
    : p_(params), request_ids_(request_ids), steps_(request_ids.size(), 0), vocab_(vocab), stream_(stream), staging_(2 * READ_AHEAD) {
    const size_t n = std::max<size_t>(1, request_ids.size());
    use_penalty_ = p_.repeat_penalty != 1.0f;
    if (use_penalty_) {
        hist_cap_ = std::max(1, p_.max_tokens + 1);
        hist_.allocate(n * (size_t)hist_cap_ * sizeof(int32_t));
        hist_times_.allocate(hist_.bytes());
        hist_len_.allocate(n * sizeof(int32_t));
        zero_device(hist_.data(), hist_.bytes(), stream);
        zero_device(hist_times_.data(), hist_times_.bytes(), stream);
        zero_device(hist_len_.data(), hist_len_.bytes(), stream);
    }
    for (int i = 0; i < RING; ++i) {
        out_[i].allocate(n * sizeof(int32_t));
        row_req_[i].allocate(n * sizeof(int32_t));
        uniforms_[i].allocate(n * sizeof(float));
        pick_idx_[i].allocate(n * sizeof(int32_t));
        picked_[i].allocate(n * sizeof(int32_t));
    }
    for (hipEvent_t& e : events_) e = nullptr;
    null_ = null_device();
    if (null_) {
        landing_ = calloc(READ_AHEAD * n, sizeof(int32_t));
    } else {
        hip_check(hipHostMalloc(&landing_, READ_AHEAD * n * sizeof(int32_t), hipHostMallocDefault), "allocating pinned memory");
        for (hipEvent_t& e : events_) hip_check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "creating an event");
    }
}

DeviceSampler::~DeviceSampler() {
    if (null_) { free(landing_); return; }
    (void)hipStreamSynchronize(stream_);
    for (hipEvent_t e : events_)
        if (e) (void)hipEventDestroy(e);
    if (landing_) (void)hipHostFree(landing_);
}

std::unique_ptr<Draw> DeviceSampler::draw(const float* logits_c, const std::vector<int>& rows) {
    float* logits = const_cast<float*>(logits_c);           // changed in place by the penalty
    const int n = (int)rows.size();
    const size_t cap = std::max<size_t>(1, request_ids_.size());
    if ((size_t)n > cap) raise(TQE_ERR_ARGUMENT, "a draw of %d rows for a batch of %zu requests", n, request_ids_.size());
    for (int r : rows)
        if (r < 0 || (size_t)r >= request_ids_.size()) raise(TQE_ERR_ARGUMENT, "a draw names request %d of a batch of %zu", r, request_ids_.size());
    const int turn = draw_turn_;
    draw_turn_ = (draw_turn_ + 1) % RING;
    int32_t* out = (int32_t*)out_[turn].data();
    int32_t* small = (int32_t*)row_req_[turn].data();
    const int32_t* row_req = nullptr;
    if (use_penalty_) {
        std::vector<int32_t> rr(rows.begin(), rows.end());
        staging_.upload(small, rr.data(), rr.size() * sizeof(int32_t), stream_);
        row_req = small;
        K::repeat_penalty(logits, n, vocab_, row_req, (const int32_t*)hist_.data(), (const int32_t*)hist_times_.data(), hist_cap_,
                          (const int32_t*)hist_len_.data(), (int)request_ids_.size(), p_.repeat_penalty, stream_);
    }
    if (p_.greedy()) {
        const size_t need = (size_t)K::argmax_scratch_floats.raw(n, vocab_) * sizeof(float);
        if (need > scratch_bytes_) { stream_synchronize(stream_); scratch_.allocate(need); scratch_bytes_ = need; }
        K::argmax(logits, n, vocab_, out, (float*)scratch_.data(), stream_);
    } else {
        std::vector<float> u((size_t)n);
        for (int i = 0; i < n; ++i) u[(size_t)i] = draw_uniform(p_.seed, (uint64_t)request_ids_[(size_t)rows[(size_t)i]], steps_[(size_t)rows[(size_t)i]]);
        float* u_dev = (float*)uniforms_[turn].data();
        staging_.upload(u_dev, u.data(), u.size() * sizeof(float), stream_);
        const size_t need = K::sample_scratch_bytes.raw(n, vocab_, p_.top_k, p_.top_p);
        if (need > scratch_bytes_) { stream_synchronize(stream_); scratch_.allocate(need); scratch_bytes_ = need; }
        K::sample(logits, n, vocab_, p_.temperature, p_.top_k, p_.top_p, u_dev, out, scratch_.data(), stream_);
    }
    for (int r : rows) ++steps_[(size_t)r];
    if (use_penalty_)
        K::append_history(out, row_req, (int32_t*)hist_.data(), (int32_t*)hist_times_.data(), hist_cap_, (int32_t*)hist_len_.data(), n, stream_);
    int32_t* host = (int32_t*)landing_ + (size_t)turn_ * cap;
    hipEvent_t event = events_[turn_];
    turn_ = (turn_ + 1) % READ_AHEAD;
    if (null_device()) memcpy(host, out, (size_t)n * sizeof(int32_t));
    else {
        hip_check(hipMemcpyAsync(host, out, (size_t)n * sizeof(int32_t), hipMemcpyDeviceToHost, stream_), "copying a draw to the host");
        hip_check(hipEventRecord(event, stream_), "recording an event");
    }
    return std::unique_ptr<Draw>(new DeviceDraw(out, host, n, event));
}

const int32_t* DeviceSampler::pick(Draw& d, const std::vector<int>& places) {
    DeviceDraw& draw = static_cast<DeviceDraw&>(d);
    bool identity = (int)places.size() == draw.n_;
    for (size_t i = 0; identity && i < places.size(); ++i) identity = places[i] == (int)i;
    if (identity) return draw.device_;
    for (int p : places)
        if (p < 0 || p >= draw.n_) raise(TQE_ERR_ARGUMENT, "place %d of a draw of %d tokens", p, draw.n_);
    std::vector<int32_t> idx(places.begin(), places.end());
    int32_t* idx_dev = (int32_t*)pick_idx_[pick_turn_].data();
    int32_t* out = (int32_t*)picked_[pick_turn_].data();
    pick_turn_ = (pick_turn_ + 1) % RING;
    staging_.upload(idx_dev, idx.data(), idx.size() * sizeof(int32_t), stream_);
    K::gather_rows(draw.device_, idx_dev, (int)idx.size(), (long long)sizeof(int32_t), out, stream_);
    return out;
}

std::vector<int32_t> DeviceSampler::sample(const float* logits, const std::vector<int>& rows) { return draw(logits, rows)->read(); }

// ---- the loop ------------------------------------------------------------------------------------
namespace {

struct Known : Draw {
    std::vector<int32_t> tokens;
    explicit Known(std::vector<int32_t> t) : tokens(std::move(t)) {}
    std::vector<int32_t> read() override { return tokens; }
};

struct BatchGuard {
    tqe_batch_t* b;
    ~BatchGuard() { if (b) tqe_batch_free(b); }
};

void run_batch(LoopEngine& engine, const std::vector<std::vector<int32_t>>& prompts, const std::vector<int>& batch, const GenerationParams& params,
               const std::vector<int32_t>& eos, std::vector<std::vector<int32_t>>& emitted, const OnTokens& on_tokens, LoopSampler& sampler,
               int max_step_tokens) {
    // One batch from its prompts to its last token.
    //
    // Running ahead: if the engine takes a step's tokens from the device and the sampler can start
    // a draw without waiting for it, the step after a draw is started before the draw has been
    // read, for every request that goes on unless its unread token is a stop token; the host then
    // reads the draw while the device works.  A request that did stop has run one step for
    // nothing: its row of the next draw is dropped, and its slot goes back as it would have.
    // What is emitted is the same either way.
    std::map<int, int> slots;               // request -> slot
    const bool ahead = engine.takes_device_tokens() && sampler.runs_ahead();
    struct CloseAll {
        LoopEngine& e;
        std::map<int, int>& s;
        ~CloseAll() {
            for (auto& kv : s) {
                try { e.close(kv.second); } catch (...) {}
            }
        }
    } close_all{engine, slots};

    for (int r : batch) slots[r] = engine.open();
    std::vector<int32_t> lens;
    for (int r : batch) lens.push_back((int32_t)prompts[(size_t)r].size());
    int n_pieces = tqe_prompt_steps((int)lens.size(), lens.data(), max_step_tokens, nullptr, 0);
    if (n_pieces < 0) throw Error(n_pieces, tqe_last_error());
    std::vector<int32_t> pieces((size_t)std::max(n_pieces, 1) * 4);
    n_pieces = tqe_prompt_steps((int)lens.size(), lens.data(), max_step_tokens, pieces.data(), std::max(n_pieces, 1));
    if (n_pieces < 0) throw Error(n_pieces, tqe_last_error());
    std::map<int, int32_t> drawn;           // index in the batch -> its first token
    for (int at = 0; at < n_pieces;) {
        const int step = pieces[(size_t)at * 4 + 3];
        std::vector<StepItem> items;
        std::vector<int> ends;
        for (; at < n_pieces && pieces[(size_t)at * 4 + 3] == step; ++at) {
            const int b = pieces[(size_t)at * 4], begin = pieces[(size_t)at * 4 + 1], end = pieces[(size_t)at * 4 + 2];
            const std::vector<int32_t>& prompt = prompts[(size_t)batch[(size_t)b]];
            const bool last = end == (int)prompt.size();
            items.push_back(StepItem{slots[batch[(size_t)b]], prompt.data() + begin, end - begin, last});
            if (last) ends.push_back(b);
        }
        const float* logits = engine.step(items, nullptr);
        if (!ends.empty()) {
            const std::vector<int32_t> toks = sampler.sample(logits, ends);
            if (toks.size() != ends.size()) raise(TQE_ERR_STATE, "the sampler gave %zu tokens for %zu rows", toks.size(), ends.size());
            for (size_t i = 0; i < ends.size(); ++i) drawn[ends[i]] = toks[i];
        }
    }
    std::vector<int> rows;                  // indices into `batch` whose token is in `draw`
    std::vector<int32_t> first;
    for (size_t b = 0; b < batch.size(); ++b) { rows.push_back((int)b); first.push_back(drawn.at((int)b)); }
    std::unique_ptr<Draw> draw(new Known(first));
    bool draw_known = true;
    BatchGuard progress{tqe_batch_new((int)batch.size(), params.max_tokens, eos.empty() ? nullptr : eos.data(), (int)eos.size())};
    if (!progress.b) throw Error(TQE_ERR_ARGUMENT, tqe_last_error());
    int32_t zero = 0;
    while (!rows.empty()) {
        // the step after this draw, for those that go on if their unread token is no stop token
        std::vector<int> next_rows;
        std::unique_ptr<Draw> next_draw;
        if (ahead && !draw_known) {
            for (int b : rows)
                if (tqe_batch_goes_on(progress.b, b)) next_rows.push_back(b);
            if (!next_rows.empty()) {
                std::vector<int> places;
                for (int b : next_rows) places.push_back((int)(std::find(rows.begin(), rows.end(), b) - rows.begin()));
                const int32_t* tokens = sampler.pick(*draw, places);
                std::vector<StepItem> items;
                for (int b : next_rows) items.push_back(StepItem{slots[batch[(size_t)b]], &zero, 1, true});
                const float* logits = engine.step(items, tokens);
                next_draw = sampler.draw(logits, next_rows);
            }
        }
        std::vector<std::pair<int, int32_t>> feed;
        std::vector<int32_t> pair_req, pair_tok;
        const std::vector<int32_t> toks = draw->read();
        if (toks.size() != rows.size()) raise(TQE_ERR_STATE, "a draw gave %zu tokens for %zu rows", toks.size(), rows.size());
        for (size_t i = 0; i < rows.size(); ++i) {
            const int b = rows[i];
            const int32_t tok = toks[i];
            const int what = tqe_batch_accept(progress.b, b, tok);
            if (what < 0) throw Error(what, tqe_last_error());
            if (what == TQE_TOKEN_DROPPED) continue;               // it ended while a step with it was under way
            const int r = batch[(size_t)b];
            if (what == TQE_TOKEN_STOP) {                           // stop tokens are not emitted (src/engine.rs:381)
                const int slot = slots[r];
                slots.erase(r);
                engine.close(slot);
                continue;
            }
            emitted[(size_t)r].push_back(tok);
            pair_req.push_back(r);
            pair_tok.push_back(tok);
            if (what == TQE_TOKEN_LAST) {                           // nothing more to draw for it
                const int slot = slots[r];
                slots.erase(r);
                engine.close(slot);
                continue;
            }
            feed.push_back({b, tok});
        }
        if (on_tokens && !pair_req.empty()) on_tokens((int)pair_req.size(), pair_req.data(), pair_tok.data());
        if (next_draw) {
            rows = next_rows;
            draw = std::move(next_draw);
            draw_known = false;
            continue;
        }
        rows.clear();
        for (auto& f : feed) rows.push_back(f.first);
        if (rows.empty()) break;
        std::vector<StepItem> items;
        for (auto& f : feed) items.push_back(StepItem{slots[batch[(size_t)f.first]], &f.second, 1, true});
        const float* logits = engine.step(items, nullptr);
        if (ahead) {
            draw = sampler.draw(logits, rows);
            draw_known = false;
        } else {
            draw.reset(new Known(sampler.sample(logits, rows)));
            draw_known = true;
        }
    }
}

}  // namespace

std::vector<std::vector<int32_t>> generate(LoopEngine& engine, const std::vector<std::vector<int32_t>>& prompts, const GenerationParams& params,
                                           const std::vector<int32_t>& eos, const OnTokens& on_tokens, int max_batch,
                                           const SamplerFactory& make_sampler, int max_step_tokens) {
    params.validate();
    for (size_t i = 0; i < prompts.size(); ++i) {
        if (prompts[i].empty()) {
            if (prompts.size() == 1) raise(TQE_ERR_GENERATION, "Empty prompt");
            raise(TQE_ERR_GENERATION, "Empty prompt (request %zu)", i);
        }
        if ((long long)prompts[i].size() + std::max(0, params.max_tokens - 1) > engine.max_positions())
            raise(TQE_ERR_GENERATION, "request %zu: %zu prompt tokens and %d new ones exceed the model's %lld positions", i, prompts[i].size(),
                  params.max_tokens, engine.max_positions());
    }
    std::vector<std::vector<int32_t>> emitted(prompts.size());
    if (prompts.empty()) return emitted;
    max_batch = std::max(1, std::min(max_batch, engine.max_slots()));
    std::vector<int32_t> lens, batch_of(prompts.size());
    for (const auto& p : prompts) lens.push_back((int32_t)p.size());
    const int n_batches = tqe_plan_batches((int)lens.size(), lens.data(), params.max_tokens, engine.max_tokens(), max_batch,
                                           engine.holds_pages() ? 1 : 0, batch_of.data());
    if (n_batches == TQE_ERR_FULL) throw Error(TQE_ERR_GENERATION, tqe_last_error());
    if (n_batches < 0) throw Error(n_batches, tqe_last_error());
    for (int b = 0; b < n_batches; ++b) {
        std::vector<int> batch;
        for (size_t i = 0; i < prompts.size(); ++i)
            if (batch_of[i] == b) batch.push_back((int)i);
        std::unique_ptr<LoopSampler> sampler = make_sampler(params, batch);
        run_batch(engine, prompts, batch, params, eos, emitted, on_tokens, *sampler, std::max(1, max_step_tokens));
    }
    return emitted;
}

}  // namespace tq
