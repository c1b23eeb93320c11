// Data that describes a model: which parts, with which sizes, run in which order.  Nothing
// here computes.  An architecture turns its typed configuration into a ModelSpec; the loader,
// the random-weights writer, the cache and the engine work from the ModelSpec alone and never
// ask which architecture it came from.  Every spec reads from and writes to JSON, which is how
// one made by hand (a test, another language) crosses the C boundary.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "core.h"
#include "json.h"

namespace tq {

// One named tensor of a part.  init: how the random-weights mode fills it: "normal" (N(0, std)),
// "one_plus_normal" (1 + N(0, std)), "zeros", or a kind registered with register_init.
// dtype: "float" follows the run's weight dtype; "int32" is an integer table.
struct TensorSpec {
    std::vector<int64_t> shape;
    std::string init = "normal";
    double std_dev = 0.02;
    std::string dtype = "float";
    int64_t numel() const { int64_t n = 1; for (int64_t s : shape) n *= s; return n; }
    Json to_json() const;
    static TensorSpec from_json(const Json& j);
};
// name -> spec, in the order a part lists them
using TensorSpecs = std::vector<std::pair<std::string, TensorSpec>>;

// A part by kind and parameters; parameters may hold further part specs
// ({"kind": ..., "params": {...}}).
struct PartSpec {
    std::string kind;
    Json params = Json::object();
    bool defined() const { return !kind.empty(); }
    Json to_json() const;
    static PartSpec from_json(const Json& j, const char* what);
    std::string key() const { return kind + ":" + params.dump(); }
};

// What a mixer keeps per sequence.  Pages: keys and values for every position, in pages of
// TQE_PAGE positions whose layout is the mixer's own: key_page and value_page are the shapes
// of one page (window > 0: only the last `window` positions are ever read).  State: a
// fixed-size row per sequence, zero at the start.
struct CacheNeed {
    enum Kind { None = 0, Pages = 1, State = 2 };
    int kind = None;
    std::vector<int64_t> key_page, value_page;
    int window = 0;
    std::vector<int64_t> state_shape;
    int state_dtype = F32;
    bool operator==(const CacheNeed& o) const {
        return kind == o.kind && key_page == o.key_page && value_page == o.value_page && window == o.window &&
               state_shape == o.state_shape && state_dtype == o.state_dtype;
    }
    Json to_json() const;
    static CacheNeed from_json(const Json& j);
};

struct LayerSpec {
    std::string prefix;          // where the layer's tensors live
    PartSpec block;              // the arrangement, which names its mixer, feed-forward and norms
};

// One entry of the run order: run layer `layer`; cache_of >= 0 names an earlier entry whose
// cache this run reads instead of keeping its own.
struct Run {
    int layer = 0;
    int cache_of = -1;
};

struct ModelSpec {
    std::string architecture;
    int64_t vocab_size = 0, hidden_size = 0, max_positions = 0;
    std::string embedding_name;
    std::vector<LayerSpec> layers;
    std::vector<Run> order;
    PartSpec final_norm;
    std::string final_norm_prefix;
    std::string head_name;                 // empty: the head is the embedding matrix (tied)
    std::vector<int32_t> eos_token_ids;
    // What an architecture may do around the blocks; all off for the reference's decoder.
    bool has_embedding_scale = false; double embedding_scale = 1.0;
    PartSpec stream_position;              // a position part that acts on the stream after the gather
    std::string stream_position_prefix;
    std::string head_bias_name;
    bool has_logit_scale = false; double logit_scale = 1.0;
    bool has_logit_cap = false; double logit_cap = 0.0;

    Json to_json() const;
    static ModelSpec from_json(const Json& j);
};

// ---- typed reading of JSON objects (config.json keys, part parameters) -----------------------
// Says which key is missing or of the wrong type; `where` names the file or the part.
class KeyReader {
public:
    KeyReader(const Json& raw, std::string where, int error_code = TQE_ERR_CONFIG);
    bool has(const char* key) const;                         // present and not null
    long long integer(const char* key, long long minimum = INT64_MIN) const;
    long long integer_or(const char* key, long long fallback, long long minimum = INT64_MIN) const;
    double number(const char* key, bool positive = false) const;
    double number_or(const char* key, double fallback, bool positive = false) const;
    bool boolean_or(const char* key, bool fallback) const;
    std::string string_or(const char* key, const std::string& fallback) const;
    std::string string(const char* key) const;
    std::vector<int32_t> token_ids(const char* key) const;   // an id or a list of ids; absent -> none
    const Json& raw() const { return raw_; }
    const std::string& where() const { return where_; }
private:
    const Json& raw_;
    std::string where_;
    int code_;
    const Json* get(const char* key, bool required) const;
};

}  // namespace tq
