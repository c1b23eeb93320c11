// The parts a layer is put together from, and the registry of their kinds.
//
// A part is built from a PartSpec (kind + parameters) and a BuildEnv.  It names its tensors,
// takes them when they are loaded, and computes.  No part knows which model it is in: sizes
// and constants come in as parameters only.
//
// Categories and what each offers beyond tensors() and load():
//   norm          forward(x) -> y; add_norm(h, delta) -> y (h += delta in place, then norm of h);
//                 gather_add_norm(h, delta, rows) -> y for chosen rows only
//   position      the way a mixer turns positions into a change of q and k: tables() (cos,
//                 sin, rot_dim, style) for the fused kernel, or apply(q, k) for a position
//                 encoding of its own; or add_to_stream(h) for one that acts on the stream
//   mixer         cache_need(); forward(x, cache entry) -> y, x and y [tokens, hidden]
//   feed_forward  forward(x) -> y
//   block         the arrangement: forward(stream, cache entry, next norm, last) -> stream
//
// Optional, never needed for a part to work: a mixer with takes_rows computes, in the last run
// of the order, its output for the step's last_rows alone; a norm that is foldable lets the
// product after it do the division in small decoding steps (LazyNorm); a mixer or feed-forward
// that folds_norm takes such a norm as its input, and one that adds_to_stream adds its output
// to the stream itself.
//
// A kind is either built in (C++ classes in parts_builtin.cpp) or registered by the caller
// through the C boundary with a table of callbacks (plugin.cpp): such a part gets tensors as
// pointers with shapes and the step's arrays, and computes however it likes on the stream it
// is given.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "core.h"
#include "spec.h"

namespace tq {

struct StepContext;
class Norm;

// memory that a part (or the model) owns, with its shape
struct Owned {
    Buffer mem;
    Tensor t;
};
using OwnedPtr = std::shared_ptr<Owned>;
OwnedPtr make_owned(int dtype, std::initializer_list<int64_t> dims);
OwnedPtr make_owned(int dtype, const std::vector<int64_t>& dims);

// the loaded tensors of one part, by the names of its tensors()
using Loaded = std::map<std::string, OwnedPtr>;

// ---- the residual stream ---------------------------------------------------------------------
// A product [rows, n] that has not been added up: float32 [pieces, rows, n] over pieces of its
// K; dtype: what the finished product would be rounded to.
struct PartialSums {
    Tensor sums;
    int dtype = BF16;
    int64_t rows() const { return sums.shape[1]; }
    int64_t cols() const { return sums.shape[2]; }
};

// An update of the stream that has not been added yet: nothing, a tensor of the activation
// dtype, or a product's partial sums (only for a norm that takes those).
struct Pending {
    enum Kind { Nothing, Plain, Sums };
    Kind kind = Nothing;
    Tensor t;
    PartialSums s;
    static Pending of(const Tensor& t) { Pending p; p.kind = t.defined() ? Plain : Nothing; p.t = t; return p; }
    static Pending of(const PartialSums& s) { Pending p; p.kind = Sums; p.s = s; return p; }
};

// An RMSNorm of the stream that has not been computed: xw is the stream times the norm's weight,
// ss the rows' sums of squares in n_ss pieces; the product that takes it divides its result by
// the rows' rms.
struct LazyNorm {
    Tensor xw, ss;
    int n_ss = 0;
    float eps = 0.f;
};

// What a mixer or feed-forward gets as input: the (normed) step [tokens, hidden], or a LazyNorm of it.
struct Activation {
    Tensor x;
    bool lazy = false;
    LazyNorm norm;
    int64_t rows() const { return lazy ? norm.xw.shape[0] : x.shape[0]; }
};

// The residual stream of a step.  h: float32 [tokens, hidden].  In small decoding steps the
// kernels that add to h also prepare the next norm: xw is bfloat16(h * weight of norm xw_for)
// and ss the rows' sums of squares in n_ss pieces (valid only while nothing is pending).
// next_norm is set by whoever runs a part, to the norm that will read the stream after it.
struct Stream {
    Tensor h;
    Pending pending;
    Tensor xw_buffer, ss_buffer;
    const Norm* xw_for = nullptr;
    int n_ss = 0;
    Norm* next_norm = nullptr;
    bool of_last_rows = false;
    void invalidate() { xw_for = nullptr; }
};

// ---- building --------------------------------------------------------------------------------
class Part;
class Position;

struct BuildEnv {
    int act_dtype = BF16;
    bool null_device = false;
    std::map<std::string, std::shared_ptr<Part>> shared;       // parts without weights (position tables) shared between layers
};

class Part {
public:
    virtual ~Part() {}
    std::string category, kind;
    // True if forward() launches the same kernels with the same arguments whatever the step's
    // data are (it reads positions, tables and slots on the device only), so that a step can be
    // captured once as a graph and replayed.
    bool graph_safe = false;
    virtual TensorSpecs tensors() const { return {}; }
    virtual void load(Loaded& tensors, hipStream_t stream) { (void)tensors; (void)stream; }
    virtual const char* trace_name() const { return "part"; }
    // a tensor the part holds, by the name it was loaded under or a name of the part's own
    // ("qkv.weight"): for inspection
    virtual OwnedPtr held(const std::string& name) const { (void)name; return nullptr; }
    virtual Json describe() const;
    // the matrix products the part runs through linear(): (n, k) of each weight (what the library can be tuned for)
    virtual void product_shapes(std::vector<std::pair<int64_t, int64_t>>& out) const { (void)out; }
};

class Norm : public Part {
public:
    virtual void forward(StepContext& c, const Tensor& x, Tensor& out) = 0;
    // h [T, size] float32, delta an update or nothing: h += delta in place; out = norm(h), activation dtype
    virtual void add_norm(StepContext& c, Tensor& h, const Pending& delta, Tensor& out) = 0;
    // out = norm(h[rows] + delta[rows]) for the int32 row indices (on the device); h is left as it is
    virtual void gather_add_norm(StepContext& c, const Tensor& h, const Pending& delta, const int32_t* rows, int64_t n_rows, Tensor& out) = 0;
    virtual bool takes_partial_sums() const { return false; }
    // whether the kernels that add to the stream can prepare this norm, and with what
    virtual bool foldable() const { return false; }
    virtual const Tensor* fold_weight() const { return nullptr; }
    virtual float fold_eps() const { return 0.f; }
    bool lazy(const Stream& stream, LazyNorm& out) const;
    virtual int64_t size() const = 0;
};

enum RotaryStyle { STYLE_NONE = 0, STYLE_HALVES = 1, STYLE_PAIRS = 2 };

class Position : public Part {
public:
    int64_t max_positions = (int64_t)1 << 30;
    struct Tables { Tensor cos, sin; int rot_dim = 0; int style = STYLE_NONE; };
    virtual bool has_apply() const { return false; }
    virtual Tables tables() const { return Tables(); }
    // a position encoding of its own changes q [T, heads, d] and k [T, kv heads, d] in place (rows of
    // q and k are `row_stride` values apart)
    virtual void apply(StepContext& c, Tensor& q, Tensor& k, int64_t row_stride) { (void)c; (void)q; (void)k; (void)row_stride; }
    virtual bool acts_on_stream() const { return false; }
    virtual void add_to_stream(StepContext& c, Tensor& h) { (void)c; (void)h; }
};

// What a mixer sees of the cache for one run of the order.
struct CacheEntry {
    int kind = CacheNeed::None;
    int group = -1;                 // pages: which group's page table the step carries for it
    Tensor keys, values;            // pages: [pages, key_page...], [pages, value_page...]
    Tensor state;                   // state: [slots, shape...]; row `slot` is a sequence's
    bool writes = true;             // false: reads another run's cache
    int window = 0;
};

class Mixer : public Part {
public:
    bool takes_rows = false;            // forward(..., last_rows) computes the step's last_rows only
    bool reads_other_cache = false;     // set when a run of this layer reads another run's cache
    virtual CacheNeed cache_need() const { return CacheNeed(); }
    virtual bool folds_norm(const StepContext& c) const { (void)c; return false; }
    virtual bool adds_to_stream(const StepContext& c) const { (void)c; return false; }
    // x: the (normed) step.  stream: add the output to it instead of returning it (then the
    // result is undefined()).  last_rows: keys and values of all tokens go to the cache as always,
    // but the output is computed for the step's last_rows alone.
    virtual Tensor forward(StepContext& c, const Activation& x, const CacheEntry& entry, Stream* stream, bool last_rows) = 0;
};

class FeedForward : public Part {
public:
    virtual bool folds_norm(const StepContext& c) const { (void)c; return false; }
    virtual bool adds_to_stream(const StepContext& c) const { (void)c; return false; }
    virtual Tensor forward(StepContext& c, const Activation& x, Stream* stream) = 0;
};

class Block : public Part {
public:
    virtual CacheNeed cache_need() const = 0;
    virtual Norm* first_norm() = 0;
    virtual Mixer* mixer() { return nullptr; }
    // next_norm: the norm that reads the stream after this block.  last: nothing but the head
    // reads the stream after it.  Returns the stream to go on with.
    virtual Stream* forward(StepContext& c, Stream* stream, const CacheEntry& entry, Norm* next_norm, bool last) = 0;
};

// ---- the registry ------------------------------------------------------------------------------
using Factory = std::function<std::shared_ptr<Part>(const PartSpec&, BuildEnv&)>;
void register_kind(const std::string& category, const std::string& kind, Factory factory);
std::vector<std::string> known_kinds(const std::string& category);
std::shared_ptr<Part> build_part(const std::string& category, const PartSpec& spec, BuildEnv& env);
template <typename T> std::shared_ptr<T> build(const char* category, const PartSpec& spec, BuildEnv& env) {
    std::shared_ptr<T> p = std::dynamic_pointer_cast<T>(build_part(category, spec, env));
    if (!p) raise(TQE_ERR_ARGUMENT, "part kind '%s' is no %s", spec.kind.c_str(), category);
    return p;
}
void register_builtin_parts();          // idempotent

}  // namespace tq
