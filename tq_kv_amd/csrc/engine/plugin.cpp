#include "plugin.h"

namespace tq {

tqe_tensor_t to_c(const Tensor& t, int64_t row_stride) {
    tqe_tensor_t c;
    memset(&c, 0, sizeof(c));
    c.data = t.data;
    c.dtype = t.dtype;
    c.ndim = t.ndim;
    for (int i = 0; i < t.ndim && i < 6; ++i) c.shape[i] = t.shape[i];
    c.row_stride = row_stride;
    return c;
}

Tensor from_c(const tqe_tensor_t& c) {
    Tensor t;
    if (c.ndim < 0 || c.ndim > 6) raise(TQE_ERR_ARGUMENT, "a tensor of %d dimensions", c.ndim);
    if (c.dtype != F32 && c.dtype != BF16 && c.dtype != I32) raise(TQE_ERR_ARGUMENT, "a tensor of unknown dtype code %d", c.dtype);
    t.data = c.data;
    t.dtype = c.dtype;
    t.ndim = c.data ? c.ndim : 0;
    for (int i = 0; i < t.ndim; ++i) {
        if (c.shape[i] < 0) raise(TQE_ERR_ARGUMENT, "a tensor with a negative size");
        t.shape[i] = c.shape[i];
    }
    return t;
}

void fill_step_view(const StepContext& c, tqe_step_view_t& v) {
    memset(&v, 0, sizeof(v));
    v.n_seqs = c.n_seqs;
    v.n_tokens = c.n_tokens;
    v.n_want = c.n_want;
    v.n_last = c.n_last;
    v.all_decode = c.all_decode;
    v.prune_last = c.prune_last;
    v.max_new = c.max_new;
    v.max_end = c.max_end;
    v.act_dtype = c.act_dtype;
    v.n_groups = (int32_t)c.tables.size();
    const int32_t* const h[12] = {c.host.tokens, c.host.tok_seq, c.host.tok_pos, c.host.seq_slot, c.host.seq_start, c.host.seq_new, c.host.cu,
                                  c.host.want_rows, c.host.last_rows, c.host.want_in_last, c.host.last_seq, c.host.last_pos};
    const int32_t* const d[12] = {c.dev.tokens, c.dev.tok_seq, c.dev.tok_pos, c.dev.seq_slot, c.dev.seq_start, c.dev.seq_new, c.dev.cu,
                                  c.dev.want_rows, c.dev.last_rows, c.dev.want_in_last, c.dev.last_seq, c.dev.last_pos};
    const int kept = c.prune_last ? c.n_last : 0;
    const int32_t sizes[12] = {c.n_tokens, c.n_tokens, c.n_tokens, c.n_seqs, c.n_seqs, c.n_seqs, c.n_seqs + 1, c.n_want,
                               kept, c.prune_last ? c.n_want : 0, kept, kept};
    for (int i = 0; i < 12; ++i) { v.host[i] = h[i]; v.dev[i] = d[i]; v.sizes[i] = sizes[i]; }
    for (size_t g = 0; g < c.tables.size() && g < TQE_MAX_GROUPS; ++g) {
        v.table_host[g] = c.tables[g].host;
        v.table_dev[g] = c.tables[g].dev;
        v.table_width[g] = c.tables[g].width;
    }
    v.entry_group = -1;
    v.entry_writes = 1;
    v.stream = (void*)c.stream;
}

namespace {

// one instance of a caller's kind
struct Instance {
    tqe_part_callbacks_t cb;
    void* user = nullptr;
    void* handle = nullptr;
    Json info;
    std::string kind;
    std::vector<OwnedPtr> keep;             // the tensors handed to it

    ~Instance() {
        if (handle && cb.destroy) cb.destroy(user, handle);
    }
    [[noreturn]] void fail(const char* what) const {
        const char* msg = cb.last_error ? cb.last_error(user) : nullptr;
        throw Error(TQE_ERR_PART, format("part '%s': %s: %s", kind.c_str(), what, msg && *msg ? msg : "failed"));
    }
    void create(const char* category, const PartSpec& spec, const BuildEnv& env) {
        kind = spec.kind;
        if (!cb.create || !cb.describe || !cb.call) raise(TQE_ERR_ARGUMENT, "part kind '%s' was registered without create, describe or call", kind.c_str());
        const std::string params = spec.params.dump();
        if (cb.create(user, category, kind.c_str(), params.c_str(), env.act_dtype, env.null_device ? 0 : 1, &handle) != 0 || !handle) {
            handle = nullptr;
            fail("building it");
        }
        const char* text = cb.describe(user, handle);
        if (!text) fail("describing itself");
        try {
            info = Json::parse(text);
        } catch (const JsonError& e) {
            raise(TQE_ERR_PART, "part '%s' describes itself in invalid JSON: %s", kind.c_str(), e.what());
        }
    }
    TensorSpecs tensors() const {
        TensorSpecs out;
        if (info["tensors"].is_object())
            for (const Json::Member& m : info["tensors"].members()) out.push_back({m.first, TensorSpec::from_json(m.second)});
        return out;
    }
    void load(Loaded& tensors) {
        std::vector<std::string> names;
        std::vector<const char*> name_ptrs;
        std::vector<tqe_tensor_t> views;
        for (const auto& t : this->tensors()) {
            auto it = tensors.find(t.first);
            if (it == tensors.end() || !it->second) raise(TQE_ERR_WEIGHTS, "part '%s' was not given its tensor '%s'", kind.c_str(), t.first.c_str());
            keep.push_back(it->second);
            names.push_back(t.first);
            views.push_back(to_c(it->second->t));
        }
        for (const std::string& n : names) name_ptrs.push_back(n.c_str());
        if (cb.load && cb.load(user, handle, (int)names.size(), name_ptrs.data(), views.data()) != 0) fail("taking its tensors");
    }
    void call(const char* method, StepContext* c, std::vector<tqe_tensor_t>& args, const CacheEntry* entry = nullptr, bool last_rows = false) {
        tqe_step_view_t view;
        if (c) {
            if (c->capturing) raise(TQE_ERR_STATE, "part '%s' cannot run inside a captured graph", kind.c_str());
            fill_step_view(*c, view);
            if (entry) {
                view.entry_group = entry->group;
                view.entry_writes = entry->writes ? 1 : 0;
                view.entry_window = entry->window;
            }
            view.last_rows_only = last_rows ? 1 : 0;
        }
        if (cb.call(user, handle, method, c ? &view : nullptr, (int)args.size(), args.data()) != 0) fail(method);
    }
    OwnedPtr held(const std::string& name) const {
        const TensorSpecs ts = tensors();
        for (size_t i = 0; i < ts.size() && i < keep.size(); ++i)
            if (ts[i].first == name) return keep[i];
        return nullptr;
    }
};

tqe_tensor_t absent() {
    tqe_tensor_t t;
    memset(&t, 0, sizeof(t));
    return t;
}

tqe_tensor_t pending_arg(StepContext& c, const Pending& delta) {
    if (delta.kind == Pending::Nothing) return absent();
    if (delta.kind == Pending::Sums) raise(TQE_ERR_STATE, "a caller's norm was handed a product's unfinished sums");
    (void)c;
    return to_c(delta.t);
}

#define TQ_PLUGIN_COMMON                                                                                       \
    Instance inst;                                                                                             \
    TensorSpecs tensors() const override { return inst.tensors(); }                                            \
    void load(Loaded& t, hipStream_t s) override { stream_synchronize(s); inst.load(t); }                      \
    OwnedPtr held(const std::string& name) const override { return inst.held(name); }                          \
    const char* trace_name() const override { return trace_.c_str(); }                                         \
    std::string trace_;                                                                                        \
    void init(const char* category, const PartSpec& spec, BuildEnv& env, const tqe_part_callbacks_t& cb, void* user) { \
        inst.cb = cb;                                                                                          \
        inst.user = user;                                                                                      \
        inst.create(category, spec, env);                                                                      \
        graph_safe = false;                                                                                    \
        trace_ = inst.info["trace_name"].is_string() ? inst.info["trace_name"].as_string() : "part";           \
    }

class PluginNorm : public Norm {
public:
    TQ_PLUGIN_COMMON
    int64_t size_ = 0;
    int64_t size() const override { return size_; }
    void forward(StepContext& c, const Tensor& x, Tensor& out) override {
        std::vector<tqe_tensor_t> a = {to_c(x), to_c(out)};
        inst.call("forward", &c, a);
    }
    void add_norm(StepContext& c, Tensor& h, const Pending& delta, Tensor& out) override {
        std::vector<tqe_tensor_t> a = {to_c(h), pending_arg(c, delta), to_c(out)};
        inst.call("add_norm", &c, a);
    }
    void gather_add_norm(StepContext& c, const Tensor& h, const Pending& delta, const int32_t* rows, int64_t n_rows, Tensor& out) override {
        Tensor r((void*)rows, I32, {n_rows});
        std::vector<tqe_tensor_t> a = {to_c(h), pending_arg(c, delta), to_c(r), to_c(out)};
        inst.call("gather_add_norm", &c, a);
    }
};

class PluginPosition : public Position {
public:
    TQ_PLUGIN_COMMON
    bool has_apply_ = false, on_stream_ = false;
    bool has_apply() const override { return has_apply_; }
    bool acts_on_stream() const override { return on_stream_; }
    void apply(StepContext& c, Tensor& q, Tensor& k, int64_t row_stride) override {
        std::vector<tqe_tensor_t> a = {to_c(q, row_stride), to_c(k, row_stride)};
        inst.call("apply", &c, a);
    }
    void add_to_stream(StepContext& c, Tensor& h) override {
        std::vector<tqe_tensor_t> a = {to_c(h)};
        inst.call("add_to_stream", &c, a);
    }
};

class PluginMixer : public Mixer {
public:
    TQ_PLUGIN_COMMON
    CacheNeed need_;
    int64_t hidden_out_ = 0;
    CacheNeed cache_need() const override { return need_; }
    Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream*, bool last_rows) override {
        if (x.lazy) raise(TQE_ERR_STATE, "a caller's mixer was handed a folded norm");
        Tensor out = c.alloc(x.x.dtype, {last_rows ? c.n_last : x.x.shape[0], x.x.shape[1]});
        std::vector<tqe_tensor_t> a = {to_c(x.x), to_c(out)};
        if (entry.kind == CacheNeed::Pages) { a.push_back(to_c(entry.keys)); a.push_back(to_c(entry.values)); }
        else if (entry.kind == CacheNeed::State) a.push_back(to_c(entry.state));
        inst.call("forward", &c, a, &entry, last_rows);
        return out;
    }
};

class PluginFeedForward : public FeedForward {
public:
    TQ_PLUGIN_COMMON
    Tensor forward(StepContext& c, const Activation& x, Stream*) override {
        if (x.lazy) raise(TQE_ERR_STATE, "a caller's feed-forward was handed a folded norm");
        Tensor out = c.alloc(x.x.dtype, {x.x.shape[0], x.x.shape[1]});
        std::vector<tqe_tensor_t> a = {to_c(x.x), to_c(out)};
        inst.call("forward", &c, a);
        return out;
    }
};

}  // namespace

void register_plugin_kind(const std::string& category, const std::string& kind, const tqe_part_callbacks_t& cb, void* user) {
    if (category == "norm") {
        register_kind(category, kind, [cb, user](const PartSpec& s, BuildEnv& e) {
            auto p = std::make_shared<PluginNorm>();
            p->init("norm", s, e, cb, user);
            p->size_ = s.params["size"].is_int() ? s.params["size"].as_int() : 0;
            return p;
        });
    } else if (category == "position") {
        register_kind(category, kind, [cb, user](const PartSpec& s, BuildEnv& e) {
            auto p = std::make_shared<PluginPosition>();
            p->init("position", s, e, cb, user);
            p->has_apply_ = p->inst.info["has_apply"].is_bool() && p->inst.info["has_apply"].as_bool();
            p->on_stream_ = p->inst.info["acts_on_stream"].is_bool() && p->inst.info["acts_on_stream"].as_bool();
            if (p->inst.info["max_positions"].is_int()) p->max_positions = p->inst.info["max_positions"].as_int();
            return p;
        });
    } else if (category == "mixer") {
        register_kind(category, kind, [cb, user](const PartSpec& s, BuildEnv& e) {
            auto p = std::make_shared<PluginMixer>();
            p->init("mixer", s, e, cb, user);
            p->need_ = CacheNeed::from_json(p->inst.info["cache_need"]);
            p->takes_rows = p->inst.info["takes_rows"].is_bool() && p->inst.info["takes_rows"].as_bool();
            return p;
        });
    } else if (category == "feed_forward") {
        register_kind(category, kind, [cb, user](const PartSpec& s, BuildEnv& e) {
            auto p = std::make_shared<PluginFeedForward>();
            p->init("feed_forward", s, e, cb, user);
            return p;
        });
    } else {
        raise(TQE_ERR_ARGUMENT, "parts of category '%s' cannot be registered through the C boundary (norm, position, mixer, feed_forward can)",
              category.c_str());
    }
}

}  // namespace tq
