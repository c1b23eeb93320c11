#include "model.h"

#include <algorithm>

#include "kernels.h"
#include "trace.h"

namespace tq {

Model::Model(const ModelSpec& s, int dtype_, bool on_gpu_) : spec(s), dtype(dtype_), on_gpu(on_gpu_) {
    if (dtype != F32 && dtype != BF16) raise(TQE_ERR_ARGUMENT, "dtype must be bfloat16 or float32");
    env_.act_dtype = dtype;
    env_.null_device = !on_gpu;
    stop_token_ids = spec.eos_token_ids;
    for (const LayerSpec& layer : spec.layers) blocks_.push_back(build<Block>("block", layer.block, env_));
    final_norm_ = build<Norm>("norm", spec.final_norm, env_);
    if (spec.stream_position.defined()) {
        stream_position_ = build<Position>("position", spec.stream_position, env_);
        if (!stream_position_->acts_on_stream())
            raise(TQE_ERR_ARGUMENT, "position kind '%s' cannot act on the stream (it has no add_to_stream)", spec.stream_position.kind.c_str());
    }
    for (size_t i = 0; i < spec.order.size(); ++i) {
        const Run& run = spec.order[i];
        if (run.layer < 0 || run.layer >= (int)blocks_.size())
            raise(TQE_ERR_ARGUMENT, "run %zu names layer %d, the model has %zu", i, run.layer, blocks_.size());
        if (run.cache_of != -1 && (run.cache_of < 0 || run.cache_of >= (int)i))
            raise(TQE_ERR_ARGUMENT, "run %zu reads the cache of run %d, which is not an earlier run", i, run.cache_of == INT32_MIN ? -1 : run.cache_of);
        needs.push_back(blocks_[(size_t)run.layer]->cache_need());
        cache_of.push_back(run.cache_of);
        if (run.cache_of >= 0)
            if (Mixer* m = blocks_[(size_t)run.layer]->mixer()) m->reads_other_cache = true;
    }
    // a step can be captured as a graph if every part's forward launches the same kernels whatever
    // the step's data are
    graph_safe = final_norm_->graph_safe && (!stream_position_ || stream_position_->graph_safe);
    for (const auto& b : blocks_) graph_safe = graph_safe && b->graph_safe;
}

TensorSpecs Model::tensor_specs() const {
    TensorSpecs out;
    TensorSpec table;
    table.shape = {spec.vocab_size, spec.hidden_size};
    out.push_back({spec.embedding_name, table});
    for (size_t l = 0; l < blocks_.size(); ++l)
        for (const auto& t : blocks_[l]->tensors()) out.push_back({spec.layers[l].prefix + t.first, t.second});
    for (const auto& t : final_norm_->tensors()) out.push_back({spec.final_norm_prefix + t.first, t.second});
    if (!spec.head_name.empty()) out.push_back({spec.head_name, table});
    if (stream_position_)
        for (const auto& t : stream_position_->tensors()) out.push_back({spec.stream_position_prefix + t.first, t.second});
    if (!spec.head_bias_name.empty()) {
        TensorSpec b;
        b.shape = {spec.vocab_size};
        out.push_back({spec.head_bias_name, b});
    }
    return out;
}

static OwnedPtr need(Loaded& tensors, const std::string& name) {
    auto it = tensors.find(name);
    if (it == tensors.end() || !it->second) raise(TQE_ERR_WEIGHTS, "Missing tensor: %s", name.c_str());
    return it->second;
}

void Model::load(Loaded& tensors, hipStream_t stream) {
    embedding_ = need(tensors, spec.embedding_name);
    for (size_t l = 0; l < blocks_.size(); ++l) {
        Loaded own;
        for (const auto& t : blocks_[l]->tensors()) own[t.first] = need(tensors, spec.layers[l].prefix + t.first);
        blocks_[l]->load(own, stream);
    }
    {
        Loaded own;
        for (const auto& t : final_norm_->tensors()) own[t.first] = need(tensors, spec.final_norm_prefix + t.first);
        final_norm_->load(own, stream);
    }
    if (stream_position_) {
        Loaded own;
        for (const auto& t : stream_position_->tensors()) own[t.first] = need(tensors, spec.stream_position_prefix + t.first);
        stream_position_->load(own, stream);
    }
    if (!spec.head_bias_name.empty()) {
        OwnedPtr b = need(tensors, spec.head_bias_name);
        if (b->t.dtype == F32) head_bias_ = b;
        else {
            head_bias_ = make_owned(F32, {b->t.shape[0]});
            if (on_gpu) K::convert(b->t.data, b->t.dtype, head_bias_->t.data, F32, (long long)b->t.numel(), stream);
            stream_synchronize(stream);
        }
    }
    // a tied head's rows are the embedding: they stay whatever the policy says
    head_ = make_weight(spec.head_name.empty() ? embedding_ : need(tensors, spec.head_name), 1, spec.head_name.empty(), stream);
    stream_synchronize(stream);
    loaded = true;
}

OwnedPtr Model::held(const std::string& name) const {
    if (name == spec.embedding_name) return embedding_;
    if (!spec.head_name.empty() && name == spec.head_name) return head_.rows;
    if (name == "head.packed") return head_.packed;
    if (!spec.head_bias_name.empty() && name == spec.head_bias_name) return head_bias_;
    for (size_t l = 0; l < blocks_.size(); ++l) {
        const std::string& prefix = spec.layers[l].prefix;
        if (name.compare(0, prefix.size(), prefix) == 0)
            if (OwnedPtr p = blocks_[l]->held(name.substr(prefix.size()))) return p;
    }
    if (name.compare(0, spec.final_norm_prefix.size(), spec.final_norm_prefix) == 0)
        if (OwnedPtr p = final_norm_->held(name.substr(spec.final_norm_prefix.size()))) return p;
    if (stream_position_ && name.compare(0, spec.stream_position_prefix.size(), spec.stream_position_prefix) == 0)
        if (OwnedPtr p = stream_position_->held(name.substr(spec.stream_position_prefix.size()))) return p;
    return nullptr;
}

// whether anything the stream holds lies in this arena of the workspace
static bool lives_in(const Workspace& ws, const Stream& s, int arena) {
    for (const void* p : {s.h.data, s.pending.t.data, s.pending.s.sums.data, s.xw_buffer.data, s.ss_buffer.data})
        if (p && ws.arena_of(p) == arena) return true;
    return false;
}

Tensor Model::forward(StepContext& c, const CacheStore& cache, float* out) {
    if (!loaded) raise(TQE_ERR_STATE, "the model has no weights yet");
    Span span("model");                     // the reference's span, src/models/turbo_generic.rs:1932
    const ModelSpec& s = spec;
    Tensor h = c.alloc(F32, {c.n_tokens, s.hidden_size});
    // which kind of step this is for the products' folding is parts/linear's to say
    classify_step(c, s.hidden_size);
    // the norm that reads the stream first in every run, and after the last one
    std::vector<Norm*> firsts;
    for (const Run& run : s.order) firsts.push_back(blocks_[(size_t)run.layer]->first_norm());
    firsts.push_back(final_norm_.get());
    const float scale = s.has_embedding_scale ? (float)s.embedding_scale : 1.0f;
    Stream stream;
    stream.h = h;
    const Tensor& table = embedding_->t;
    if (c.fuse_small) {
        stream.xw_buffer = c.alloc(BF16, {c.n_tokens, s.hidden_size});
        stream.ss_buffer = c.alloc(F32, {(s.hidden_size + 15) / 16, 16});        // the most pieces a product gives
        const Norm* norm = firsts[0]->foldable() ? firsts[0] : nullptr;
        K::embed(table.data, table.dtype, c.dev.tokens, c.n_tokens, (int)s.hidden_size, (int)s.vocab_size, scale, (float*)h.data,
                 stream.xw_buffer.data, norm ? norm->fold_weight()->data : nullptr, (float*)stream.ss_buffer.data, c.stream);
        stream.xw_for = norm;
        stream.n_ss = 1;
    } else {
        K::embed(table.data, table.dtype, c.dev.tokens, c.n_tokens, (int)s.hidden_size, (int)s.vocab_size, scale, (float*)h.data, nullptr, nullptr,
                 nullptr, c.stream);
    }
    if (stream_position_) {
        stream_position_->add_to_stream(c, h);
        stream.invalidate();            // what the gather prepared for the first norm is of the stream before this
    }
    Stream* cur = &stream;
    for (size_t i = 0; i < s.order.size(); ++i) {
        // The layers take their temporaries from two arenas in turn.  What a layer leaves for the next one (an update
        // of the stream that is still pending) is read by that next layer, so the arena of the layer before the last
        // holds nothing that is still needed: unless a block handed on what it was given, which is looked for.
        const int arena = 1 + (int)(i & 1);
        if (!lives_in(*c.ws, *cur, arena)) c.ws->rewind(arena);
        c.ws->use(arena);
        cur = blocks_[(size_t)s.order[i].layer]->forward(c, cur, cache.entry((int)i), firsts[i + 1], i + 1 == s.order.size());
    }
    c.ws->use(Workspace::STEP);
    if (c.n_want == 0) return Tensor(nullptr, F32, {0, s.vocab_size});
    Span out_span("output");                // src/models/turbo_generic.rs:1933
    Tensor logits = head_logits(c, *cur, out);
    if (head_bias_ || s.has_logit_scale || s.has_logit_cap)
        K::finish_logits((float*)logits.data, c.n_want, (int)s.vocab_size, head_bias_ ? (const float*)head_bias_->t.data : nullptr,
                         s.has_logit_scale ? (float)s.logit_scale : 1.0f, s.has_logit_cap ? (float)s.logit_cap : 0.0f, c.stream);
    return logits;
}

Tensor Model::head_logits(StepContext& c, Stream& stream, float* out) {
    const ModelSpec& s = spec;
    const int64_t n_rows = c.n_want;
    Tensor logits(out, F32, {n_rows, s.vocab_size});
    if (!out) logits = c.alloc(F32, {n_rows, s.vocab_size});
    // the last block may have gone on with the wanted rows alone, numbered among themselves
    const int32_t* want_rows = stream.of_last_rows ? c.dev.want_in_last : c.dev.want_rows;
    LazyNorm lazy;
    if (c.fuse_small && final_norm_->lazy(stream, lazy) && n_rows <= skinny_max_rows() && fusable(n_rows, head_)) {
        int packed = 0;
        const void* wp = head_.packed ? (packed = 1, head_.packed->t.data) : head_.rows->t.data;
        K::fused_store(lazy.xw.data, want_rows, (const float*)lazy.ss.data, lazy.n_ss, lazy.eps, wp, packed, logits.data, F32, (int)n_rows,
                       (int)head_.n, (int)head_.k, c.stream);
        return logits;
    }
    Tensor x = c.alloc(c.act_dtype, {n_rows, s.hidden_size});
    final_norm_->gather_add_norm(c, stream.h, stream.pending, want_rows, n_rows, x);
    linear(c, x, head_, nullptr, F32, false, &logits);
    return logits;
}

void Model::tune_library(int64_t rows, hipStream_t stream) {
    if (dtype != BF16 || !on_gpu || !policy().library) return;
    const int64_t own_rows = policy().mid && policy().packed ? mid_max_rows() : skinny_max_rows();
    if (rows <= own_rows) return;
    std::vector<std::pair<int64_t, int64_t>> shapes;
    for (const auto& b : blocks_) b->product_shapes(shapes);
    std::sort(shapes.begin(), shapes.end());
    shapes.erase(std::unique(shapes.begin(), shapes.end()), shapes.end());
    for (const auto& nk : shapes) library_tune(rows, nk.first, nk.second, BF16, stream);
}

Json Model::describe() const {
    Json j = Json::object();
    j.set("spec", spec.to_json());
    j.set("config", config);
    j.set("dtype", dtype_name(dtype));
    j.set("on_gpu", on_gpu);
    j.set("graph_safe", graph_safe);
    j.set("loaded", loaded);
    Json stop = Json::array();
    for (int32_t t : stop_token_ids) stop.push(Json((int)t));
    j.set("stop_token_ids", stop);
    Json ns = Json::array();
    for (const CacheNeed& n : needs) ns.push(n.to_json());
    j.set("needs", ns);
    Json co = Json::array();
    for (int cidx : cache_of) co.push(cidx >= 0 ? Json(cidx) : Json());
    j.set("cache_of", co);
    Json ts = Json::object();
    for (const auto& t : tensor_specs()) ts.set(t.first, t.second.to_json());
    j.set("tensors", ts);
    return j;
}

}  // namespace tq
