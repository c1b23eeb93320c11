#include "spec.h"

#include <math.h>

namespace tq {

static Json shape_json(const std::vector<int64_t>& shape) {
    Json a = Json::array();
    for (int64_t s : shape) a.push(Json((long long)s));
    return a;
}

static std::vector<int64_t> shape_from(const Json& j, const char* what) {
    if (!j.is_array()) raise(TQE_ERR_ARGUMENT, "%s: expected a list of sizes", what);
    std::vector<int64_t> out;
    for (const Json& v : j.items()) {
        if (!v.is_int() || v.as_int() < 0) raise(TQE_ERR_ARGUMENT, "%s: sizes must be non-negative integers", what);
        out.push_back(v.as_int());
    }
    return out;
}

Json TensorSpec::to_json() const {
    Json j = Json::object();
    j.set("shape", shape_json(shape));
    j.set("init", init);
    j.set("std", std_dev);
    j.set("dtype", dtype);
    return j;
}

TensorSpec TensorSpec::from_json(const Json& j) {
    TensorSpec t;
    t.shape = shape_from(j["shape"], "tensor spec");
    if (j["init"].is_string()) t.init = j["init"].as_string();
    if (j["std"].is_number()) t.std_dev = j["std"].as_number();
    if (j["dtype"].is_string()) t.dtype = j["dtype"].as_string();
    if (t.dtype != "float" && t.dtype != "int32") raise(TQE_ERR_ARGUMENT, "tensor spec: dtype must be \"float\" or \"int32\", got \"%s\"", t.dtype.c_str());
    return t;
}

Json PartSpec::to_json() const {
    Json j = Json::object();
    j.set("kind", kind);
    j.set("params", params);
    return j;
}

PartSpec PartSpec::from_json(const Json& j, const char* what) {
    if (!j.is_object() || !j["kind"].is_string()) raise(TQE_ERR_ARGUMENT, "%s: expected a part {\"kind\": ..., \"params\": {...}}", what);
    PartSpec p;
    p.kind = j["kind"].as_string();
    if (j["params"].is_object()) p.params = j["params"];
    else if (!j["params"].is_null()) raise(TQE_ERR_ARGUMENT, "%s: the parameters of part '%s' must be an object", what, p.kind.c_str());
    return p;
}

Json CacheNeed::to_json() const {
    if (kind == None) return Json();
    Json j = Json::object();
    if (kind == Pages) {
        j.set("kind", "pages");
        j.set("key_page", shape_json(key_page));
        j.set("value_page", shape_json(value_page));
        j.set("window", window > 0 ? Json(window) : Json());
    } else {
        j.set("kind", "state");
        j.set("shape", shape_json(state_shape));
        j.set("dtype", dtype_name(state_dtype));
    }
    return j;
}

CacheNeed CacheNeed::from_json(const Json& j) {
    CacheNeed n;
    if (j.is_null()) return n;
    const std::string kind = j["kind"].is_string() ? j["kind"].as_string() : "";
    if (kind == "pages") {
        n.kind = Pages;
        n.key_page = shape_from(j["key_page"], "cache need");
        n.value_page = shape_from(j["value_page"], "cache need");
        if (j["window"].is_int()) n.window = (int)j["window"].as_int();
        if (n.window < 0) raise(TQE_ERR_ARGUMENT, "cache need: window %d", n.window);
    } else if (kind == "state") {
        n.kind = State;
        n.state_shape = shape_from(j["shape"], "cache need");
        const std::string dt = j["dtype"].is_string() ? j["dtype"].as_string() : "float32";
        if (dt == "float32") n.state_dtype = F32;
        else if (dt == "bfloat16") n.state_dtype = BF16;
        else if (dt == "int32") n.state_dtype = I32;
        else raise(TQE_ERR_ARGUMENT, "state of kind '%s' (known: bfloat16, float32, int32)", dt.c_str());
    } else {
        raise(TQE_ERR_ARGUMENT, "cache need: unknown kind '%s' (known: pages, state)", kind.c_str());
    }
    return n;
}

Json ModelSpec::to_json() const {
    Json j = Json::object();
    j.set("architecture", architecture);
    j.set("vocab_size", (long long)vocab_size);
    j.set("hidden_size", (long long)hidden_size);
    j.set("max_positions", (long long)max_positions);
    j.set("embedding_name", embedding_name);
    Json ls = Json::array();
    for (const LayerSpec& l : layers) {
        Json o = Json::object();
        o.set("prefix", l.prefix);
        o.set("block", l.block.to_json());
        ls.push(o);
    }
    j.set("layers", ls);
    Json rs = Json::array();
    for (const Run& r : order) {
        Json o = Json::object();
        o.set("layer", r.layer);
        o.set("cache_of", r.cache_of >= 0 ? Json(r.cache_of) : Json());
        rs.push(o);
    }
    j.set("order", rs);
    j.set("final_norm", final_norm.to_json());
    j.set("final_norm_prefix", final_norm_prefix);
    j.set("head_name", head_name.empty() ? Json() : Json(head_name));
    Json eos = Json::array();
    for (int32_t t : eos_token_ids) eos.push(Json((int)t));
    j.set("eos_token_ids", eos);
    j.set("embedding_scale", has_embedding_scale ? Json(embedding_scale) : Json());
    j.set("stream_position", stream_position.defined() ? stream_position.to_json() : Json());
    j.set("stream_position_prefix", stream_position_prefix);
    j.set("head_bias_name", head_bias_name.empty() ? Json() : Json(head_bias_name));
    j.set("logit_scale", has_logit_scale ? Json(logit_scale) : Json());
    j.set("logit_cap", has_logit_cap ? Json(logit_cap) : Json());
    return j;
}

ModelSpec ModelSpec::from_json(const Json& j) {
    if (!j.is_object()) raise(TQE_ERR_ARGUMENT, "model spec: expected a JSON object");
    KeyReader r(j, "model spec", TQE_ERR_ARGUMENT);
    ModelSpec s;
    s.architecture = r.string_or("architecture", "");
    s.vocab_size = r.integer("vocab_size", 1);
    s.hidden_size = r.integer("hidden_size", 1);
    s.max_positions = r.integer("max_positions", 1);
    s.embedding_name = r.string("embedding_name");
    if (!j["layers"].is_array()) raise(TQE_ERR_ARGUMENT, "model spec: 'layers' must be a list");
    for (const Json& l : j["layers"].items()) {
        LayerSpec ls;
        ls.prefix = l["prefix"].is_string() ? l["prefix"].as_string() : "";
        ls.block = PartSpec::from_json(l["block"], "layer");
        s.layers.push_back(ls);
    }
    if (!j["order"].is_array()) raise(TQE_ERR_ARGUMENT, "model spec: 'order' must be a list");
    for (const Json& o : j["order"].items()) {
        Run run;
        if (!o["layer"].is_int()) raise(TQE_ERR_ARGUMENT, "model spec: a run names no layer");
        run.layer = (int)o["layer"].as_int();
        run.cache_of = o["cache_of"].is_int() ? (int)o["cache_of"].as_int() : -1;
        if (o["cache_of"].is_int() && run.cache_of < 0) run.cache_of = INT32_MIN;        // named, and wrong: refused by the model
        s.order.push_back(run);
    }
    s.final_norm = PartSpec::from_json(j["final_norm"], "final norm");
    s.final_norm_prefix = r.string_or("final_norm_prefix", "");
    s.head_name = r.string_or("head_name", "");
    s.eos_token_ids = r.token_ids("eos_token_ids");
    if (r.has("embedding_scale")) { s.has_embedding_scale = true; s.embedding_scale = r.number("embedding_scale"); }
    if (r.has("stream_position")) s.stream_position = PartSpec::from_json(j["stream_position"], "stream position");
    s.stream_position_prefix = r.string_or("stream_position_prefix", "");
    s.head_bias_name = r.string_or("head_bias_name", "");
    if (r.has("logit_scale")) { s.has_logit_scale = true; s.logit_scale = r.number("logit_scale"); }
    if (r.has("logit_cap")) { s.has_logit_cap = true; s.logit_cap = r.number("logit_cap"); }
    return s;
}

// ---- KeyReader -------------------------------------------------------------------------------
KeyReader::KeyReader(const Json& raw, std::string where, int error_code) : raw_(raw), where_(std::move(where)), code_(error_code) {
    if (!raw.is_object()) raise(code_, "%s: expected a JSON object at the top level", where_.c_str());
}

const Json* KeyReader::get(const char* key, bool required) const {
    const Json* v = raw_.find(key);
    if (!v || v->is_null()) {
        if (required) raise(code_, "%s: missing required key '%s'", where_.c_str(), key);
        return nullptr;
    }
    return v;
}

bool KeyReader::has(const char* key) const { return get(key, false) != nullptr; }

static long long as_integer(const Json& v, const std::string& where, const char* key, int code) {
    if (v.is_int()) return v.as_int();
    if (v.kind() == Json::Float && v.as_number() == floor(v.as_number()) && fabs(v.as_number()) < 9e15) return (long long)v.as_number();
    raise(code, "%s: key '%s' must be an integer, got %s", where.c_str(), key, v.dump().c_str());
}

long long KeyReader::integer(const char* key, long long minimum) const {
    const long long v = as_integer(*get(key, true), where_, key, code_);
    if (v < minimum) raise(code_, "%s: key '%s' must be >= %lld, got %lld", where_.c_str(), key, minimum, v);
    return v;
}

long long KeyReader::integer_or(const char* key, long long fallback, long long minimum) const {
    const Json* j = get(key, false);
    if (!j) return fallback;
    const long long v = as_integer(*j, where_, key, code_);
    if (v < minimum) raise(code_, "%s: key '%s' must be >= %lld, got %lld", where_.c_str(), key, minimum, v);
    return v;
}

double KeyReader::number(const char* key, bool positive) const {
    const Json& v = *get(key, true);
    if (!v.is_number()) raise(code_, "%s: key '%s' must be a number, got %s", where_.c_str(), key, v.dump().c_str());
    if (positive && !(v.as_number() > 0.0)) raise(code_, "%s: key '%s' must be > 0, got %s", where_.c_str(), key, v.dump().c_str());
    return v.as_number();
}

double KeyReader::number_or(const char* key, double fallback, bool positive) const {
    return get(key, false) ? number(key, positive) : fallback;
}

bool KeyReader::boolean_or(const char* key, bool fallback) const {
    const Json* v = get(key, false);
    if (!v) return fallback;
    if (!v->is_bool()) raise(code_, "%s: key '%s' must be true or false, got %s", where_.c_str(), key, v->dump().c_str());
    return v->as_bool();
}

std::string KeyReader::string(const char* key) const {
    const Json& v = *get(key, true);
    if (!v.is_string()) raise(code_, "%s: key '%s' must be a string, got %s", where_.c_str(), key, v.dump().c_str());
    return v.as_string();
}

std::string KeyReader::string_or(const char* key, const std::string& fallback) const {
    return get(key, false) ? string(key) : fallback;
}

std::vector<int32_t> KeyReader::token_ids(const char* key) const {
    std::vector<int32_t> out;
    const Json* v = get(key, false);
    if (!v) return out;
    auto one = [&](const Json& t) {
        if (!t.is_int() || t.as_int() < 0 || t.as_int() > INT32_MAX)
            raise(code_, "%s: key '%s' must hold token ids, got %s", where_.c_str(), key, v->dump().c_str());
        out.push_back((int32_t)t.as_int());
    };
    if (v->is_array())
        for (const Json& t : v->items()) one(t);
    else
        one(*v);
    return out;
}

}  // namespace tq
