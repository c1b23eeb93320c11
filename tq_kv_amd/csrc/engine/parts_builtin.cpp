// The built-in kinds: RMSNorm, rotary positions (and none), grouped-query softmax attention,
// the gated-SiLU feed-forward, and the pre-norm block arrangement.
#include <math.h>

#include <mutex>

#include "kernels.h"
#include "linear.h"
#include "parts.h"
#include "step.h"
#include "trace.h"

namespace tq {

// ---- registry ----------------------------------------------------------------------------------
namespace {
const char* const CATEGORIES[] = {"norm", "position", "mixer", "feed_forward", "block"};
std::map<std::string, std::map<std::string, Factory>>& registry() {
    static std::map<std::string, std::map<std::string, Factory>> r;
    return r;
}
std::mutex g_registry_mutex;

std::string joined(const std::vector<std::string>& v) {
    std::string s;
    for (size_t i = 0; i < v.size(); ++i) s += (i ? ", " : "") + v[i];
    return s;
}
}  // namespace

void register_kind(const std::string& category, const std::string& kind, Factory factory) {
    bool known = false;
    for (const char* c : CATEGORIES) known = known || category == c;
    if (!known) raise(TQE_ERR_ARGUMENT, "unknown part category '%s' (known: norm, position, mixer, feed_forward, block)", category.c_str());
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    registry()[category][kind] = std::move(factory);
}

std::vector<std::string> known_kinds(const std::string& category) {
    register_builtin_parts();
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    std::vector<std::string> out;
    for (const auto& e : registry()[category]) out.push_back(e.first);
    return out;
}

std::shared_ptr<Part> build_part(const std::string& category, const PartSpec& spec, BuildEnv& env) {
    register_builtin_parts();
    Factory f;
    {
        std::lock_guard<std::mutex> lock(g_registry_mutex);
        auto& kinds = registry()[category];
        auto it = kinds.find(spec.kind);
        if (it != kinds.end()) f = it->second;
    }
    if (!f) raise(TQE_ERR_ARGUMENT, "unknown %s kind '%s' (known: %s)", category.c_str(), spec.kind.c_str(), joined(known_kinds(category)).c_str());
    std::shared_ptr<Part> p = f(spec, env);
    p->category = category;
    p->kind = spec.kind;
    return p;
}

Json Part::describe() const {
    Json j = Json::object();
    j.set("category", category);
    j.set("kind", kind);
    j.set("graph_safe", graph_safe);
    Json ts = Json::object();
    for (const auto& t : tensors()) ts.set(t.first, t.second.to_json());
    j.set("tensors", ts);
    return j;
}

bool Norm::lazy(const Stream& stream, LazyNorm& out) const {
    if (stream.pending.kind != Pending::Nothing || stream.xw_for != this) return false;
    out.xw = stream.xw_buffer;
    out.ss = stream.ss_buffer;
    out.n_ss = stream.n_ss;
    out.eps = fold_eps();
    return true;
}

static OwnedPtr take(Loaded& tensors, const char* name) {
    auto it = tensors.find(name);
    if (it == tensors.end() || !it->second) raise(TQE_ERR_WEIGHTS, "a part was not given its tensor '%s'", name);
    return it->second;
}

// ---- RMSNorm -----------------------------------------------------------------------------------
// As the reference computes it (src/models/turbo_generic.rs:41-51): x / sqrt(mean(x^2) + eps) *
// weight in float32, cast last; the weight is used as it is stored (no 1 + w).
class RMSNorm : public Norm {
public:
    RMSNorm(const PartSpec& spec, BuildEnv& env) : act_dtype_(env.act_dtype) {
        KeyReader r(spec.params, "rms_norm", TQE_ERR_ARGUMENT);
        size_ = r.integer("size", 1);
        eps_ = (float)r.number("eps");
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        TensorSpec t;
        t.shape = {size_};
        t.init = "one_plus_normal";
        return {{"weight", t}};
    }
    void load(Loaded& tensors, hipStream_t) override { weight_ = take(tensors, "weight"); }
    OwnedPtr held(const std::string& name) const override { return name == "weight" ? weight_ : nullptr; }
    const char* trace_name() const override { return "rms-norm"; }          // the reference's span, src/models/turbo_generic.rs:36
    int64_t size() const override { return size_; }

    void forward(StepContext& c, const Tensor& x, Tensor& out) override {
        k_add_rmsnorm(c, nullptr, Pending::of(x), weight_->t, eps_, nullptr, out.shape[0], x.shape[0], out, false);
    }
    void add_norm(StepContext& c, Tensor& h, const Pending& delta, Tensor& out) override {
        k_add_rmsnorm(c, (float*)h.data, delta, weight_->t, eps_, nullptr, out.shape[0], h.shape[0], out, delta.kind != Pending::Nothing);
    }
    void gather_add_norm(StepContext& c, const Tensor& h, const Pending& delta, const int32_t* rows, int64_t n_rows, Tensor& out) override {
        k_add_rmsnorm(c, (float*)h.data, delta, weight_->t, eps_, rows, n_rows, h.shape[0], out, false);
    }
    bool takes_partial_sums() const override { return true; }
    bool foldable() const override { return weight_ && weight_->t.dtype == BF16; }
    const Tensor* fold_weight() const override { return &weight_->t; }
    float fold_eps() const override { return eps_; }

private:
    int64_t size_;
    float eps_;
    int act_dtype_;
    OwnedPtr weight_;
};

// ---- positions ---------------------------------------------------------------------------------
// Rotary tables as the reference builds them (src/models/turbo_generic.rs:1654-1670): theta_j =
// 1 / base^(2j/d) with base rounded to float32 and the power taken in float32, angle = position *
// theta_j in float32, cos and sin of it.  Layouts: halves (:417-427, what Qwen2 uses) and pairs
// (:430-443); rot_dim < head_dim rotates the first rot_dim elements only (:752-761).
class Rotary : public Position {
public:
    Rotary(const PartSpec& spec, BuildEnv&) {
        KeyReader r(spec.params, "rotary", TQE_ERR_ARGUMENT);
        theta_ = r.number("theta");
        rot_dim_ = (int)r.integer("rot_dim");
        max_positions = r.integer("max_positions", 1);
        const std::string style = r.string_or("style", "halves");
        if (style == "halves") style_ = STYLE_HALVES;
        else if (style == "pairs") style_ = STYLE_PAIRS;
        else raise(TQE_ERR_ARGUMENT, "rotary: unknown style '%s' (known: halves, pairs)", style.c_str());
        if (rot_dim_ <= 0 || rot_dim_ % 2) raise(TQE_ERR_ARGUMENT, "rotary: rot_dim must be even and positive, got %d", rot_dim_);
        graph_safe = true;
        // The tables are computed on the host in float32, so that they are the same numbers
        // whatever device the model runs on.
        const int half = rot_dim_ / 2;
        std::vector<float> cos_h((size_t)max_positions * half), sin_h(cos_h.size());
        const float base = (float)theta_;
        std::vector<float> inv((size_t)half);
        for (int j = 0; j < half; ++j) inv[(size_t)j] = 1.0f / powf(base, (float)(2 * j) / (float)rot_dim_);
        for (int64_t p = 0; p < max_positions; ++p)
            for (int j = 0; j < half; ++j) {
                const float angle = (float)p * inv[(size_t)j];
                cos_h[(size_t)p * half + j] = cosf(angle);
                sin_h[(size_t)p * half + j] = sinf(angle);
            }
        cos_ = make_owned(F32, {max_positions, half});
        sin_ = make_owned(F32, {max_positions, half});
        copy_to_device(cos_->t.data, cos_h.data(), cos_h.size() * 4, nullptr);
        copy_to_device(sin_->t.data, sin_h.data(), sin_h.size() * 4, nullptr);
        stream_synchronize(nullptr);
    }
    Tables tables() const override {
        Tables t;
        t.cos = cos_->t;
        t.sin = sin_->t;
        t.rot_dim = rot_dim_;
        t.style = style_;
        return t;
    }
    OwnedPtr held(const std::string& name) const override { return name == "cos" ? cos_ : name == "sin" ? sin_ : nullptr; }

private:
    double theta_;
    int rot_dim_, style_;
    OwnedPtr cos_, sin_;
};

// No change of q and k (a mixer that needs no positions, or learns them elsewhere).
class NoPosition : public Position {
public:
    NoPosition(const PartSpec& spec, BuildEnv&) {
        KeyReader r(spec.params, "position none", TQE_ERR_ARGUMENT);
        max_positions = r.integer_or("max_positions", (long long)1 << 30, 1);
        graph_safe = true;
    }
};

// ---- attention -----------------------------------------------------------------------------------
// Grouped-query softmax attention over the cache.  Order of work as in the reference
// (src/models/turbo_generic.rs:770-833, 1604-1635): q, k, v projections (+ bias), head split,
// position encoding of q and k, keys and values into the cache, scores q.k/sqrt(d), mask, softmax,
// p.v, merge heads, output projection without bias.  Query head h reads kv head h // (heads //
// kv_heads) (:195-204).  The three projections are one product with the weights stacked.
//
// params: hidden, n_heads, n_kv_heads, head_dim, qkv_bias, out_bias, window (null or positions a
// query sees, itself included), scale (null: 1/sqrt(head_dim)), position (a part spec); optional
// prompt_tile: queries per tile of the prompt kernel (16, 32, 64 or 128).
//
// Its pages: keys [kv heads, page, head_dim]; values [kv heads, head_dim, page], transposed inside
// a page and the page's positions in the order the matrix cores take them (the kernels' own
// layout, which is why the mixer names the shapes and the cache only multiplies them out).
class Attention : public Mixer {
public:
    static const int DECODE_KERNEL_ROWS = 32;       // up to so many rows of a prompt step go through the decoding kernel

    Attention(const PartSpec& spec, BuildEnv& env) : act_dtype_(env.act_dtype) {
        KeyReader r(spec.params, "attention", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        n_heads_ = (int)r.integer("n_heads", 1);
        n_kv_heads_ = (int)r.integer("n_kv_heads", 1);
        head_dim_ = (int)r.integer("head_dim", 1);
        qkv_bias_ = r.boolean_or("qkv_bias", false);
        out_bias_ = r.boolean_or("out_bias", false);
        window_ = r.has("window") ? (int)r.integer("window") : 0;
        if (n_heads_ % n_kv_heads_) raise(TQE_ERR_ARGUMENT, "attention: %d heads are not a multiple of %d kv heads", n_heads_, n_kv_heads_);
        if (r.has("window") && window_ < 1) raise(TQE_ERR_ARGUMENT, "attention: window must be at least 1, got %d", window_);
        scale_ = r.has("scale") ? (float)r.number("scale") : (float)(1.0 / sqrt((double)head_dim_));
        prompt_tile_ = r.has("prompt_tile") ? (int)r.integer("prompt_tile") : 0;
        if (r.has("prompt_tile") && prompt_tile_ != 16 && prompt_tile_ != 32 && prompt_tile_ != 64 && prompt_tile_ != 128)
            raise(TQE_ERR_ARGUMENT, "attention: prompt_tile must be 16, 32, 64 or 128, got %d", prompt_tile_);
        // what no attention kernel takes is refused here, before any weight is read
        const int max_d = K::attention_max_head_dim.raw();
        if (head_dim_ > max_d)
            raise(TQE_ERR_CONFIG, "attention: head_dim %d is more than the attention kernels take (%d)", head_dim_, max_d);
        if (n_heads_ > 65535) raise(TQE_ERR_CONFIG, "attention: %d heads are more than the attention kernels take (65535)", n_heads_);
        const PartSpec pos = PartSpec::from_json(spec.params["position"], "attention: position");
        const std::string key = "position:" + pos.key();
        auto it = env.shared.find(key);
        if (it == env.shared.end()) it = env.shared.emplace(key, build_part("position", pos, env)).first;
        position_ = std::dynamic_pointer_cast<Position>(it->second);
        if (!position_) raise(TQE_ERR_ARGUMENT, "attention: part kind '%s' is no position", pos.kind.c_str());
        graph_safe = !position_->has_apply() || position_->graph_safe;
        takes_rows = true;
    }

    TensorSpecs tensors() const override {
        const int64_t q = (int64_t)n_heads_ * head_dim_, kv = (int64_t)n_kv_heads_ * head_dim_;
        auto w = [](int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; };
        auto b = [](int64_t a) { TensorSpec t; t.shape = {a}; return t; };
        TensorSpecs t = {{"q_proj.weight", w(q, hidden_)}, {"k_proj.weight", w(kv, hidden_)}, {"v_proj.weight", w(kv, hidden_)},
                         {"o_proj.weight", w(hidden_, q)}};
        if (qkv_bias_) { t.push_back({"q_proj.bias", b(q)}); t.push_back({"k_proj.bias", b(kv)}); t.push_back({"v_proj.bias", b(kv)}); }
        if (out_bias_) t.push_back({"o_proj.bias", b(hidden_)});
        return t;
    }

    // several loaded tensors stacked along their first dimension: float32 if any of them is
    static OwnedPtr stacked(const std::vector<OwnedPtr>& parts, hipStream_t stream) {
        int dtype = parts[0]->t.dtype;
        int64_t rows = 0;
        for (const OwnedPtr& p : parts) {
            if (p->t.dtype == F32) dtype = F32;
            rows += p->t.shape[0];
        }
        std::vector<int64_t> dims = {rows};
        if (parts[0]->t.ndim == 2) dims.push_back(parts[0]->t.shape[1]);
        OwnedPtr out = make_owned(dtype, dims);
        int64_t at = 0;
        for (const OwnedPtr& p : parts) {
            Tensor dst = out->t.slice(at, at + p->t.shape[0]);
            if (p->t.dtype == dtype) copy_on_device(dst.data, p->t.data, p->t.bytes(), stream);
            else if (null_device()) raise(TQE_ERR_WEIGHTS, "stacked tensors of different types cannot be converted without a GPU");
            else K::convert(p->t.data, p->t.dtype, dst.data, dtype, (long long)p->t.numel(), stream);
            at += p->t.shape[0];
        }
        stream_synchronize(stream);
        return out;
    }

    void load(Loaded& t, hipStream_t stream) override {
        OwnedPtr qkv = stacked({take(t, "q_proj.weight"), take(t, "k_proj.weight"), take(t, "v_proj.weight")}, stream);
        if (qkv_bias_) b_qkv_ = stacked({take(t, "q_proj.bias"), take(t, "k_proj.bias"), take(t, "v_proj.bias")}, stream);
        if (out_bias_) b_o_ = take(t, "o_proj.bias");
        w_qkv_ = make_weight(qkv, 1, false, stream);
        w_o_ = make_weight(take(t, "o_proj.weight"), 1, b_o_ != nullptr, stream);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == "qkv.weight") return w_qkv_.rows;
        if (name == "qkv.weight.packed") return w_qkv_.packed;
        if (name == "qkv.bias") return b_qkv_;
        if (name == "o_proj.weight") return w_o_.rows;
        if (name == "o_proj.weight.packed") return w_o_.packed;
        return nullptr;
    }
    const char* trace_name() const override { return "attn"; }             // the reference's span, src/models/turbo_generic.rs:1920
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({(int64_t)(n_heads_ + 2 * n_kv_heads_) * head_dim_, hidden_});
        out.push_back({hidden_, (int64_t)n_heads_ * head_dim_});
    }

    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = CacheNeed::Pages;
        n.key_page = {n_kv_heads_, TQE_PAGE, head_dim_};
        n.value_page = {n_kv_heads_, head_dim_, TQE_PAGE};
        n.window = window_;
        return n;
    }

    // The folded q/k/v kernel takes decoding steps (row m is sequence m) of rotary positions in the
    // halves layout over the whole head.
    bool fused_qkv_ok(const StepContext& c) const {
        if (!(c.all_decode && fusable(c.n_tokens, w_qkv_) && head_dim_ % 32 == 0)) return false;
        if (position_->has_apply()) return false;
        const Position::Tables tb = position_->tables();
        if (tb.style != STYLE_HALVES || tb.rot_dim != head_dim_) return false;
        return !b_qkv_ || b_qkv_->t.dtype == BF16;
    }
    bool folds_norm(const StepContext& c) const override { return fused_qkv_ok(c) && !reads_other_cache; }
    bool adds_to_stream(const StepContext& c) const override {
        return !b_o_ && (fusable(c.n_tokens, w_o_, true) || leaves_sums(c.n_tokens, w_o_));
    }

    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool last_rows) override {
        if (entry.kind != CacheNeed::Pages) raise(TQE_ERR_STATE, "attention was given no pages of the cache");
        const int64_t n = x.rows();
        const int dtype = x.lazy ? BF16 : x.x.dtype;
        const StepContext::Table& table = c.tables.at((size_t)entry.group);
        Tensor q = c.alloc(dtype, {n, n_heads_, head_dim_});
        const int n_pages = (int)entry.keys.shape[0];
        if (x.lazy || (c.fuse_small && entry.writes && fused_qkv_ok(c))) {
            if (x.lazy && !entry.writes) raise(TQE_ERR_STATE, "a run that reads another run's cache cannot take a folded norm");
            const Position::Tables tb = position_->tables();
            const Tensor& xin = x.lazy ? x.norm.xw : x.x;
            int packed = 0;
            const void* wp = w_qkv_.packed ? (packed = 1, w_qkv_.packed->t.data) : w_qkv_.rows->t.data;
            K::fused_qkv(xin.data, x.lazy ? (const float*)x.norm.ss.data : nullptr, x.lazy ? x.norm.n_ss : 0, x.lazy ? x.norm.eps : 0.f, wp, packed,
                         b_qkv_ ? b_qkv_->t.data : nullptr, (const float*)tb.cos.data, (const float*)tb.sin.data, (int)tb.cos.shape[0], c.dev.tok_pos,
                         table.dev, table.width, entry.keys.data, entry.values.data, n_pages, q.data, (int)n, n_heads_, n_kv_heads_, head_dim_,
                         (int)hidden_, c.stream);
        } else {
            qkv(c, x.x, entry, table, q);
        }
        const int64_t qd = (int64_t)n_heads_ * head_dim_;
        if (last_rows) {
            if (c.n_last == 0) return Tensor(nullptr, dtype, {0, hidden_});
            Tensor ql = c.alloc(dtype, {c.n_last, n_heads_, head_dim_});
            k_gather_rows(c, q, c.dev.last_rows, c.n_last, ql);
            Tensor y = c.alloc(dtype, {c.n_last, qd});
            attend_rows(c, ql, entry, table, y);
            return linear(c, y, w_o_, b_o_ ? &b_o_->t : nullptr, dtype).t;
        }
        Tensor y = c.alloc(dtype, {n, qd});
        attend(c, q, entry, table, y);
        if (stream) {
            add_product(c, *stream, y, w_o_);
            return Tensor();
        }
        return linear(c, y, w_o_, b_o_ ? &b_o_->t : nullptr, dtype).t;
    }

private:
    // queries per tile of the prompt kernel for this step
    int tile_for(StepContext& c) const {
        if (prompt_tile_) return prompt_tile_;
        const std::string key = format("prompt_tile:%d:%d:%d", n_heads_, n_kv_heads_, head_dim_);
        auto it = c.memo.find(key);
        if (it == c.memo.end()) it = c.memo.emplace(key, K::attention_prefill_tile.raw(c.n_tokens, n_heads_, n_kv_heads_, head_dim_)).first;
        return it->second;
    }

    // product, then bias, position encoding and cache write in their own kernel
    void qkv(StepContext& c, const Tensor& x, const CacheEntry& entry, const StepContext::Table& table, Tensor& q) {
        const bool own = position_->has_apply();
        const int64_t n = x.shape[0];
        const int total = (n_heads_ + 2 * n_kv_heads_) * head_dim_;
        const int n_pages = (int)entry.keys.shape[0];
        Position::Tables tb;
        bool sums_ok = false;
        if (!own) {
            tb = position_->tables();
            sums_ok = x.dtype == BF16 && K::rope_store_takes_sums.raw(BF16, b_qkv_ ? 1 : 0, b_qkv_ ? b_qkv_->t.dtype : 0, tb.rot_dim, tb.style, head_dim_) != 0;
        }
        Product p = linear(c, x, w_qkv_, nullptr, x.dtype, sums_ok);        // may come as its sums over pieces of K
        const void* bias = nullptr;
        int bias_dt = 0;
        if (own) {
            // a position encoding of its own: bias first, then it changes q and k in place
            if (b_qkv_) K::add_bias(p.t.data, p.t.dtype, b_qkv_->t.data, b_qkv_->t.dtype, (int)n, total, c.stream);
            Tensor qv(p.t.data, p.t.dtype, {n, n_heads_, head_dim_});
            Tensor kv((char*)p.t.data + (size_t)n_heads_ * head_dim_ * dtype_size(p.t.dtype), p.t.dtype, {n, n_kv_heads_, head_dim_});
            position_->apply(c, qv, kv, total);
        } else if (b_qkv_) {
            bias = b_qkv_->t.data;
            bias_dt = b_qkv_->t.dtype;
        }
        const float* cos = tb.style != STYLE_NONE ? (const float*)tb.cos.data : nullptr;
        const float* sin = tb.style != STYLE_NONE ? (const float*)tb.sin.data : nullptr;
        const int max_pos = tb.style != STYLE_NONE ? (int)tb.cos.shape[0] : 0;
        const bool write = entry.writes;
        if (p.is_sums)
            K::rope_store_sums((const float*)p.sums.sums.data, (int)p.sums.sums.shape[0], bias, bias_dt, cos, sin, tb.rot_dim, tb.style, max_pos,
                               c.dev.tok_seq, c.dev.tok_pos, write ? table.dev : nullptr, write ? table.width : 0, write ? c.n_seqs : 0,
                               write ? entry.keys.data : nullptr, write ? entry.values.data : nullptr, write ? n_pages : 0, q.data, (int)n, n_heads_,
                               n_kv_heads_, head_dim_, write ? 1 : 0, c.stream);
        else
            K::rope_store(p.t.data, p.t.dtype, bias, bias_dt, cos, sin, tb.rot_dim, tb.style, max_pos, c.dev.tok_seq, c.dev.tok_pos,
                          write ? table.dev : nullptr, write ? table.width : 0, write ? c.n_seqs : 0, write ? entry.keys.data : nullptr,
                          write ? entry.values.data : nullptr, write ? n_pages : 0, q.data, (int)n, n_heads_, n_kv_heads_, head_dim_, write ? 1 : 0,
                          c.stream);
    }

    void decode_kernel(StepContext& c, const Tensor& q, const CacheEntry& entry, const int32_t* tok_pos, const int32_t* table, int width,
                       Tensor& out) {
        const int n = (int)q.shape[0];
        const int q_blocks = (n_heads_ / n_kv_heads_ + 15) / 16;
        const int groups = std::max(1, n * n_kv_heads_ * q_blocks);
        const int target_blocks = 256;
        // partitions take the live pages in turn, four waves each: no more than a quarter of the pages there can be
        // (more partitions than one block per compute unit, so that no wave has a second page to bring in, measured
        // slower: 14.6 against 13.8 us for 8 sequences of 2100 positions at the 7B sizes; 64 sequences in 2 and 4
        // partitions 60.6 and 65.9 against 56.4 us, 128 sequences 118 and 133 against 114).  Nor fewer, larger blocks
        // that need no merge: one block of eight waves per (sequence, kv head) took 37 us for the 8 sequences, since a
        // compute unit alone pulls about 30 GB/s whatever its waves ask for.
        // (no more blocks than compute units: with 288 blocks 32 units get two, and 12 sequences took 19.5 us against
        // 16.1 with 240 blocks, 24 sequences 32.2 against 27.0, 48 sequences 48.9 + merge against 40.8 without)
        int n_parts = std::max(1, std::min((width + 3) / 4, target_blocks / groups));
        // few sequences: a partition per page of the table, which the kernel gives a block of one wave each (faster up to
        // four sequences of 2100 positions at the 7B sizes, slower from eight on)
        if (width > 1 && (long long)groups * width <= 640) n_parts = width;
        Tensor part_out, part_ml;
        if (n_parts > 1) {
            part_out = c.alloc(F32, {n, n_heads_, n_parts, head_dim_});
            part_ml = c.alloc(F32, {n, n_heads_, n_parts, 2});
        }
        K::attention_decode(q.data, entry.keys.data, entry.values.data, tok_pos, table, width, n, (int)entry.keys.shape[0], window_, scale_, n_parts,
                            part_out.data, part_ml.data, out.data, n_heads_, n_kv_heads_, head_dim_, c.stream);
    }

    // Softmax attention of q over the cache entry: picks the kernel for the step.  float32, or a
    // head size the MFMA kernels do not take: the plain kernel, one wave per (token, head).
    // bfloat16 and one token per sequence: the partitioned decoding kernel; bfloat16 otherwise: the
    // tiled prompt kernel.
    void attend(StepContext& c, const Tensor& q, const CacheEntry& entry, const StepContext::Table& table, Tensor& out) {
        const int n = (int)q.shape[0], n_pages = (int)entry.keys.shape[0];
        if (q.dtype == BF16 && c.all_decode && policy().decode_mfma && K::attention_decode_supported.raw(head_dim_))
            return decode_kernel(c, q, entry, c.dev.tok_pos, table.dev, table.width, out);
        // (not for steps of one token per sequence: tiles of one query are what the plain kernel does anyway,
        // and such a step may be replayed from a graph, which cannot carry the tiles' upload)
        if (q.dtype == BF16 && !c.all_decode && policy().prefill_mfma && K::attention_prefill_supported.raw(head_dim_)) {
            const int tile = tile_for(c);
            const Tiles t = c.query_tiles(tile);
            K::attention_prefill(q.data, entry.keys.data, entry.values.data, c.dev.tok_pos, table.dev, table.width, c.n_seqs, n_pages, t.seq, t.tok0,
                                 t.count, t.n, tile, c.dev.seq_start, c.dev.seq_new, window_, scale_, out.data, n, n_heads_, n_kv_heads_, head_dim_,
                                 c.stream);
            return;
        }
        K::attention(q.data, entry.keys.data, entry.values.data, q.dtype, c.dev.tok_seq, c.dev.tok_pos, table.dev, table.width, c.n_seqs, n_pages,
                     window_, scale_, out.data, n, n_heads_, n_kv_heads_, head_dim_, c.stream);
    }

    // The same for the step's last_rows alone (q holds their queries): the cache already holds the
    // keys and values of all the step's tokens.
    void attend_rows(StepContext& c, const Tensor& q, const CacheEntry& entry, const StepContext::Table& table, Tensor& out) {
        const int n = (int)q.shape[0], n_pages = (int)entry.keys.shape[0];
        if (q.dtype == BF16 && policy().decode_mfma && K::attention_decode_supported.raw(head_dim_) && c.n_last <= DECODE_KERNEL_ROWS) {
            // few rows: the decoding kernel shares a row's keys out over many blocks, where the prompt
            // kernel would walk them in one; a row is a sequence of its own to it
            Tensor rows_table = c.alloc(I32, {n, table.width});
            Tensor whole((void*)table.dev, I32, {c.n_seqs, table.width});
            k_gather_rows(c, whole, c.dev.last_seq, n, rows_table);
            return decode_kernel(c, q, entry, c.dev.last_pos, (const int32_t*)rows_table.data, table.width, out);
        }
        if (q.dtype == BF16 && policy().prefill_mfma && K::attention_prefill_supported.raw(head_dim_)) {
            const int tile = tile_for(c);
            const Tiles t = c.last_tiles(tile);
            K::attention_prefill(q.data, entry.keys.data, entry.values.data, c.dev.last_pos, table.dev, table.width, c.n_seqs, n_pages, t.seq, t.tok0,
                                 t.count, t.n, tile, c.dev.seq_start, c.dev.seq_new, window_, scale_, out.data, n, n_heads_, n_kv_heads_, head_dim_,
                                 c.stream);
            return;
        }
        K::attention(q.data, entry.keys.data, entry.values.data, q.dtype, c.dev.last_seq, c.dev.last_pos, table.dev, table.width, c.n_seqs, n_pages,
                     window_, scale_, out.data, n, n_heads_, n_kv_heads_, head_dim_, c.stream);
    }

    int act_dtype_;
    int64_t hidden_;
    int n_heads_, n_kv_heads_, head_dim_, window_, prompt_tile_;
    bool qkv_bias_, out_bias_;
    float scale_;
    std::shared_ptr<Position> position_;
    Weight w_qkv_, w_o_;
    OwnedPtr b_qkv_, b_o_;
};

// ---- gated SiLU ----------------------------------------------------------------------------------
// "SwiGLU" as the reference's Mlp (src/models/turbo_generic.rs:98-111): down(silu(gate(x)) * up(x)),
// no biases.  Gate and up are one product with the weights stacked.  params: hidden, inter.
class GatedSiLU : public FeedForward {
public:
    GatedSiLU(const PartSpec& spec, BuildEnv&) {
        KeyReader r(spec.params, "gated_silu", TQE_ERR_ARGUMENT);
        hidden_ = r.integer("hidden", 1);
        inter_ = r.integer("inter", 1);
        graph_safe = true;
    }
    TensorSpecs tensors() const override {
        auto w = [](int64_t a, int64_t b) { TensorSpec t; t.shape = {a, b}; return t; };
        return {{"gate_proj.weight", w(inter_, hidden_)}, {"up_proj.weight", w(inter_, hidden_)}, {"down_proj.weight", w(hidden_, inter_)}};
    }
    void load(Loaded& t, hipStream_t stream) override {
        OwnedPtr gu = Attention::stacked({take(t, "gate_proj.weight"), take(t, "up_proj.weight")}, stream);
        w_gate_up_ = make_weight(gu, 2, false, stream);
        w_down_ = make_weight(take(t, "down_proj.weight"), 1, false, stream);
    }
    OwnedPtr held(const std::string& name) const override {
        if (name == "gate_up.weight") return w_gate_up_.rows;
        if (name == "gate_up.weight.packed") return w_gate_up_.packed;
        if (name == "down_proj.weight") return w_down_.rows;
        if (name == "down_proj.weight.packed") return w_down_.packed;
        return nullptr;
    }
    const char* trace_name() const override { return "attn-mlp"; }         // the reference's span, src/models/turbo_generic.rs:1922
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        out.push_back({2 * inter_, hidden_});
        out.push_back({hidden_, inter_});
    }

    bool folds_norm(const StepContext& c) const override { return fusable(c.n_tokens, w_gate_up_); }
    bool adds_to_stream(const StepContext& c) const override {
        return (fusable(c.n_tokens, w_down_, true) && fusable(c.n_tokens, w_gate_up_)) || leaves_sums(c.n_tokens, w_down_);
    }

    Tensor forward(StepContext& c, const Activation& x, Stream* stream) override {
        if (stream && !x.lazy && x.x.shape[0] > skinny_max_rows()) {
            add_product(c, *stream, gated_silu_linear(c, x.x, w_gate_up_), w_down_);
            return Tensor();
        }
        if (x.lazy || stream) {
            const Tensor& xin = x.lazy ? x.norm.xw : x.x;
            Tensor act = c.alloc(BF16, {xin.shape[0], inter_});
            int packed = 0;
            const void* wp = w_gate_up_.packed ? (packed = 1, w_gate_up_.packed->t.data) : w_gate_up_.rows->t.data;
            K::fused_gated(xin.data, x.lazy ? (const float*)x.norm.ss.data : nullptr, x.lazy ? x.norm.n_ss : 0, x.lazy ? x.norm.eps : 0.f, wp, packed,
                           act.data, (int)xin.shape[0], (int)(2 * inter_), (int)hidden_, c.stream);
            if (!stream) return linear(c, act, w_down_, nullptr, BF16).t;
            add_product(c, *stream, act, w_down_);
            return Tensor();
        }
        return linear(c, gated_silu_linear(c, x.x, w_gate_up_), w_down_, nullptr, x.x.dtype).t;
    }

private:
    int64_t hidden_, inter_;
    Weight w_gate_up_, w_down_;
};

// ---- the pre-norm block ----------------------------------------------------------------------------
// The reference's decoder layer (src/models/turbo_generic.rs:1959-1981): x = x + mixer(norm(x));
// x = x + ff(norm(x)), with optional norms on the mixer's and the feed-forward's outputs
// (:1965-1968, :1976-1979).
//
// The residual stream is float32.  A part's output is left pending on the stream and added inside
// the next norm's kernel (for mid-sized steps a part's last product may even leave its sums over
// pieces of K pending: the norm's kernel adds those up too).  In small decoding steps the
// framework's parts go further: a product that consumes a norm computes it itself (LazyNorm) and a
// part's last product adds its result to the stream in its epilogue, so that the norm kernels
// disappear; parts that do not offer this are simply given tensors.
//
// params: mixer, feed_forward, mixer_norm, ff_norm (part specs); optional post_mixer_norm,
// post_ff_norm; names: part -> tensor-name prefix inside the layer (e.g. {"mixer": "self_attn."}).
class PreNormBlock : public Block {
public:
    PreNormBlock(const PartSpec& spec, BuildEnv& env) {
        const Json& names = spec.params["names"];
        auto one = [&](const char* role, const char* category, bool optional) -> std::shared_ptr<Part> {
            const Json& p = spec.params[role];
            if (p.is_null()) {
                if (optional) return nullptr;
                raise(TQE_ERR_ARGUMENT, "pre_norm block: no '%s' given", role);
            }
            std::shared_ptr<Part> part = build_part(category, PartSpec::from_json(p, role), env);
            if (!names[role].is_string()) raise(TQE_ERR_ARGUMENT, "pre_norm block: no tensor-name prefix for '%s'", role);
            roles_.push_back({role, names[role].as_string(), part});
            return part;
        };
        mixer_ = std::dynamic_pointer_cast<Mixer>(one("mixer", "mixer", false));
        feed_forward_ = std::dynamic_pointer_cast<FeedForward>(one("feed_forward", "feed_forward", false));
        mixer_norm_ = std::dynamic_pointer_cast<Norm>(one("mixer_norm", "norm", false));
        ff_norm_ = std::dynamic_pointer_cast<Norm>(one("ff_norm", "norm", false));
        post_mixer_norm_ = std::dynamic_pointer_cast<Norm>(one("post_mixer_norm", "norm", true));
        post_ff_norm_ = std::dynamic_pointer_cast<Norm>(one("post_ff_norm", "norm", true));
        if (!mixer_ || !feed_forward_ || !mixer_norm_ || !ff_norm_) raise(TQE_ERR_ARGUMENT, "pre_norm block: a part is of the wrong category");
        graph_safe = true;
        for (const Role& r : roles_) graph_safe = graph_safe && r.part->graph_safe;
    }
    TensorSpecs tensors() const override {
        TensorSpecs out;
        for (const Role& r : roles_)
            for (const auto& t : r.part->tensors()) out.push_back({r.prefix + t.first, t.second});
        return out;
    }
    void load(Loaded& tensors, hipStream_t stream) override {
        for (const Role& r : roles_) {
            Loaded own;
            for (const auto& t : r.part->tensors()) own[t.first] = take(tensors, (r.prefix + t.first).c_str());
            r.part->load(own, stream);
        }
    }
    OwnedPtr held(const std::string& name) const override {
        for (const Role& r : roles_)
            if (name.compare(0, r.prefix.size(), r.prefix) == 0)
                if (OwnedPtr p = r.part->held(name.substr(r.prefix.size()))) return p;
        return nullptr;
    }
    Json describe() const override {
        Json j = Part::describe();
        Json parts = Json::object();
        for (const Role& r : roles_) parts.set(r.role, r.part->describe());
        j.set("parts", parts);
        return j;
    }
    void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const override {
        for (const Role& r : roles_) r.part->product_shapes(out);
    }
    CacheNeed cache_need() const override { return mixer_->cache_need(); }
    Norm* first_norm() override { return mixer_norm_.get(); }
    Mixer* mixer() override { return mixer_.get(); }

    Stream* forward(StepContext& c, Stream* stream, const CacheEntry& entry, Norm* next_norm, bool last) override {
        if (last && c.prune_last && policy().prune_last && mixer_->takes_rows) return forward_last_rows(c, stream, entry);
        Activation x = normed(c, *mixer_norm_, *stream, mixer_->folds_norm(c));
        {
            Span span(mixer_->trace_name());
            const bool adds = (c.fuse_small || c.fuse_mid) && !post_mixer_norm_ && mixer_->adds_to_stream(c);
            if (adds) stream->next_norm = ff_norm_.get();
            settle(c, *stream, mixer_->forward(c, x, entry, adds ? stream : nullptr, false), post_mixer_norm_.get());
        }
        x = normed(c, *ff_norm_, *stream, feed_forward_->folds_norm(c));
        {
            Span span(feed_forward_->trace_name());
            const bool adds = (c.fuse_small || c.fuse_mid) && !post_ff_norm_ && feed_forward_->adds_to_stream(c);
            if (adds) stream->next_norm = next_norm;
            settle(c, *stream, feed_forward_->forward(c, x, adds ? stream : nullptr), post_ff_norm_.get());
        }
        return stream;
    }

private:
    struct Role { std::string role, prefix; std::shared_ptr<Part> part; };

    // the part's input: the norm of the stream, computed now, or left to the part
    Activation normed(StepContext& c, Norm& norm, Stream& stream, bool part_folds) {
        Activation a;
        if (c.fuse_small && part_folds && norm.lazy(stream, a.norm)) {
            a.lazy = true;
            return a;
        }
        Span span(norm.trace_name());
        a.x = c.alloc(c.act_dtype, {stream.h.shape[0], stream.h.shape[1]});
        norm.add_norm(c, stream.h, stream.pending, a.x);
        stream.pending = Pending();
        stream.invalidate();
        return a;
    }
    // a part's output that it did not add to the stream itself is left pending for the next norm's kernel
    void settle(StepContext& c, Stream& stream, Tensor out, Norm* post_norm) {
        if (!out.defined()) return;
        if (post_norm) {
            Tensor y = c.alloc(out.dtype, {out.shape[0], out.shape[1]});
            post_norm->forward(c, out, y);
            out = y;
        }
        stream.pending = Pending::of(out);
        stream.invalidate();
    }

    Stream* forward_last_rows(StepContext& c, Stream* stream, const CacheEntry& entry) {
        Activation x;
        {
            Span span(mixer_norm_->trace_name());
            x.x = c.alloc(c.act_dtype, {stream->h.shape[0], stream->h.shape[1]});
            mixer_norm_->add_norm(c, stream->h, stream->pending, x.x);
        }
        Tensor y;
        {
            Span span(mixer_->trace_name());
            y = mixer_->forward(c, x, entry, nullptr, true);        // keys and values of all tokens, output of the rows
        }
        c.sub_stream.reset(new Stream());
        Stream* sub = c.sub_stream.get();
        sub->of_last_rows = true;
        sub->h = c.alloc(F32, {c.n_last, stream->h.shape[1]});
        if (c.n_last == 0) return sub;
        k_gather_rows(c, stream->h, c.dev.last_rows, c.n_last, sub->h);
        settle(c, *sub, y, post_mixer_norm_.get());
        {
            Span span(ff_norm_->trace_name());
            x.x = c.alloc(c.act_dtype, {c.n_last, stream->h.shape[1]});
            ff_norm_->add_norm(c, sub->h, sub->pending, x.x);
            sub->pending = Pending();
        }
        Tensor out;
        {
            Span span(feed_forward_->trace_name());
            out = feed_forward_->forward(c, x, nullptr);
        }
        settle(c, *sub, out, post_ff_norm_.get());
        return sub;
    }

    std::vector<Role> roles_;
    std::shared_ptr<Mixer> mixer_;
    std::shared_ptr<FeedForward> feed_forward_;
    std::shared_ptr<Norm> mixer_norm_, ff_norm_, post_mixer_norm_, post_ff_norm_;
};

void register_builtin_parts() {
    static std::once_flag once;
    std::call_once(once, [] {
        register_kind("norm", "rms_norm", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<RMSNorm>(s, e); });
        register_kind("position", "rotary", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<Rotary>(s, e); });
        register_kind("position", "none", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<NoPosition>(s, e); });
        register_kind("mixer", "attention", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<Attention>(s, e); });
        register_kind("feed_forward", "gated_silu", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<GatedSiLU>(s, e); });
        register_kind("block", "pre_norm", [](const PartSpec& s, BuildEnv& e) { return std::make_shared<PreNormBlock>(s, e); });
    });
}

}  // namespace tq
