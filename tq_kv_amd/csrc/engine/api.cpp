// The C boundary of the engine (csrc/tq_engine.h): every entry point turns its arguments into
// calls on the classes of this folder and every C++ exception into a status and a message.
#include <mutex>

#include "config.h"
#include "engine.h"
#include "generate.h"
#include "kernels.h"
#include "plugin.h"
#include "trace.h"
#include "weights.h"

using namespace tq;

void tqe_set_error(int code, const char* msg);          // host_engine.cpp: the calling thread's last status and message

namespace {

thread_local std::string g_detail, g_warning, g_text;

int set_error(int code, const std::string& msg, const std::string& detail = "") {
    tqe_set_error(code, msg.c_str());
    g_detail = detail;
    return code;
}

// runs f; returns its status, or the status of what it threw
template <typename F> int guarded(F f) {
    try {
        g_detail.clear();
        g_warning.clear();
        f();
        return TQE_OK;
    } catch (const Error& e) {
        return set_error(e.code, e.what(), e.detail);
    } catch (const JsonError& e) {
        return set_error(TQE_ERR_ARGUMENT, std::string("invalid JSON: ") + e.what());
    } catch (const std::bad_alloc&) {
        return set_error(TQE_ERR_ARGUMENT, "out of memory");
    } catch (const std::exception& e) {
        return set_error(TQE_ERR_ARGUMENT, e.what());
    } catch (...) {
        return set_error(TQE_ERR_ARGUMENT, "unknown failure");
    }
}

template <typename T, typename F> T* guarded_new(F f) {
    T* out = nullptr;
    guarded([&] { out = f(); });
    return out;
}

template <typename F> const char* guarded_text(F f) {
    bool ok = false;
    std::string text;
    guarded([&] { text = f(); ok = true; });
    if (!ok) return nullptr;
    g_text = std::move(text);
    return g_text.c_str();
}

void need(const void* p, const char* what) {
    if (!p) raise(TQE_ERR_ARGUMENT, "%s: null pointer", what);
}

int run_dtype(int code) {
    if (code != TQE_F32 && code != TQE_BF16) raise(TQE_ERR_ARGUMENT, "dtype must be bfloat16 (%d) or float32 (%d), got %d", TQE_BF16, TQE_F32, code);
    return code;
}

Json ids_json(const std::vector<int32_t>& ids) {
    Json a = Json::array();
    for (int32_t i : ids) a.push(Json((int)i));
    return a;
}

Json names_json(const std::vector<std::string>& names) {
    Json a = Json::array();
    for (const std::string& n : names) a.push(n);
    return a;
}

// a tensor of the caller's copied into memory of the current device
OwnedPtr copy_in(const tqe_tensor_t& c, bool on_device, hipStream_t stream) {
    const Tensor t = from_c(c);
    if (!t.data && t.numel() != 0) raise(TQE_ERR_ARGUMENT, "a tensor without data");
    std::vector<int64_t> dims(t.shape, t.shape + c.ndim);
    OwnedPtr o = make_owned(t.dtype, dims);
    if (o->t.bytes()) {
        if (on_device) copy_on_device(o->t.data, t.data, o->t.bytes(), stream);
        else copy_to_device(o->t.data, t.data, o->t.bytes(), stream);
        stream_synchronize(stream);
    }
    return o;
}

GenerationParams params_from(const tqe_generation_params_t* p) {
    GenerationParams g;
    if (p) {
        g.max_tokens = p->max_tokens;
        g.temperature = p->temperature;
        g.top_p = p->top_p;
        g.top_k = p->top_k;
        g.repeat_penalty = p->repeat_penalty;
        g.seed = p->seed;
    }
    g.validate();
    return g;
}

}  // namespace

struct tqe_model {
    std::shared_ptr<Model> m;
    Loaded pending;                     // tensors set one by one, until tqe_model_finish
    std::string text;
};
struct tqe_folder {
    std::unique_ptr<Folder> f;
    std::string text;
};
struct tqe_part {
    BuildEnv env;
    std::shared_ptr<Part> p;
    Loaded pending;
    bool on_gpu = true;
    std::string text;
};
struct tqe_store {
    std::unique_ptr<CacheStore> s;
    bool on_gpu = true;
    std::string text;
};
struct tqe_stepctx {
    StepContext c;
    Workspace ws;
    Staging staging;
    bool on_gpu = true;
};
struct tqe_engine {
    std::unique_ptr<Engine> e;
    std::shared_ptr<Model> model;
    std::string text;
};
struct tqe_sampler {
    std::unique_ptr<DeviceSampler> s;
    int vocab = 0;
};

extern "C" {

const char* tqe_last_error_detail(void) { return g_detail.c_str(); }
const char* tqe_last_warning(void) { return g_warning.c_str(); }
int tqe_page_size(void) { return TQE_PAGE; }

int tqe_set_kernel_library(const char* path) {
    return guarded([&] { need(path, "tqe_set_kernel_library"); set_kernel_library(path); });
}
void tqe_set_kernel_builder(tqe_kernel_builder_t builder) { set_kernel_builder(builder); }
const char* tqe_kernel_library(void) {
    return guarded_text([] { return kernel_library_path(); });
}
int tqe_policy_set(const char* name, int value) {
    return guarded([&] {
        need(name, "tqe_policy_set");
        int* field = policy_field(name);
        if (!field) raise(TQE_ERR_ARGUMENT, "unknown switch '%s'", name);
        *field = value ? 1 : 0;
    });
}
int tqe_policy_get(const char* name) {
    int* field = name ? policy_field(name) : nullptr;
    return field ? *field : -1;
}
int tqe_trace_enable(int on) { return trace_enable(on != 0) ? 1 : 0; }
int tqe_trace_enabled(void) { return trace_enabled() ? 1 : 0; }
void tqe_trace_sink(int (*push)(const char*), int (*pop)(void)) { trace_set_sink(push, pop); }
static thread_local std::vector<Span*> g_spans;
void tqe_trace_push(const char* name) { g_spans.push_back(new Span(name ? name : "")); }
void tqe_trace_pop(void) {
    if (g_spans.empty()) return;
    delete g_spans.back();
    g_spans.pop_back();
}

// ---- configuration -------------------------------------------------------------------------------
const char* tqe_known_architectures(void) {
    return guarded_text([] { return names_json(known_architectures()).dump(); });
}
const char* tqe_known_parts(const char* category) {
    return guarded_text([&] { need(category, "tqe_known_parts"); return names_json(known_kinds(category)).dump(); });
}
static Json parse_config_text(const char* config_json) {
    need(config_json, "config");
    try {
        return Json::parse(config_json);
    } catch (const JsonError& e) {
        raise(TQE_ERR_CONFIG, "Invalid config.json: %s", e.what());
    }
}
const char* tqe_config_parse(const char* config_json) {
    return guarded_text([&] {
        const Json raw = parse_config_text(config_json);
        const Architecture& a = architecture_for(raw);
        Json out = Json::object();
        out.set("architecture", a.name);
        out.set("config", a.typed_config(raw, "config.json"));
        return out.dump();
    });
}
const char* tqe_config_spec(const char* config_json) {
    return guarded_text([&] {
        const Json raw = parse_config_text(config_json);
        const Architecture& a = architecture_for(raw);
        return a.build_spec(a.typed_config(raw, "config.json")).to_json().dump();
    });
}
const char* tqe_read_config(const char* model_dir) {
    return guarded_text([&] { need(model_dir, "tqe_read_config"); return read_config_json(model_dir).dump(); });
}
const char* tqe_stop_token_ids(const char* model_dir) {
    return guarded_text([&] {
        need(model_dir, "tqe_stop_token_ids");
        std::vector<int32_t> config_ids;
        struct stat_probe { };
        FILE* f = fopen((std::string(model_dir) + "/config.json").c_str(), "rb");
        if (f) {
            fclose(f);
            const Json raw = read_config_json(model_dir);
            if (raw.is_object()) config_ids = KeyReader(raw, "config.json").token_ids("eos_token_id");
        }
        return ids_json(folder_stop_token_ids(model_dir, config_ids)).dump();
    });
}

// ---- parts and init kinds of the caller's -----------------------------------------------------------
int tqe_register_part(const char* category, const char* kind, const tqe_part_callbacks_t* callbacks, void* user) {
    return guarded([&] {
        need(category, "tqe_register_part");
        need(kind, "tqe_register_part");
        need(callbacks, "tqe_register_part");
        register_builtin_parts();
        register_plugin_kind(category, kind, *callbacks, user);
    });
}
int tqe_register_init(const char* kind, tqe_init_fill fill, void* user) {
    return guarded([&] {
        need(kind, "tqe_register_init");
        need((const void*)fill, "tqe_register_init");
        const std::string k = kind;
        register_init(k, [fill, user, k](const std::string& name, const TensorSpec& spec, uint64_t seed, int64_t begin, int64_t count, float* out) {
            const std::string spec_json = spec.to_json().dump();
            if (fill(user, name.c_str(), spec_json.c_str(), seed, begin, count, out) != 0)
                raise(TQE_ERR_PART, "the caller's init '%s' failed on tensor %s", k.c_str(), name.c_str());
        });
    });
}

// ---- models ----------------------------------------------------------------------------------------
static tqe_model_t* model_from_config(const Json& raw, int dtype, int on_gpu) {
    const Architecture& a = architecture_for(raw);
    const Json typed = a.typed_config(raw, "config.json");
    std::unique_ptr<tqe_model_t> h(new tqe_model_t());
    h->m = std::make_shared<Model>(a.build_spec(typed), run_dtype(dtype), on_gpu != 0);
    Json config = Json::object();
    config.set("architecture", a.name);
    config.set("config", typed);
    h->m->config = config;
    return h.release();
}

tqe_model_t* tqe_model_load(const char* model_dir, int dtype, int on_gpu, int strict) {
    return guarded_new<tqe_model_t>([&] {
        need(model_dir, "tqe_model_load");
        DeviceScope scope(on_gpu != 0);
        std::unique_ptr<tqe_model_t> h(model_from_config(read_config_json(model_dir), dtype, on_gpu));
        h->m->stop_token_ids = folder_stop_token_ids(model_dir, h->m->spec.eos_token_ids);
        std::string warning;
        load_folder(*h->m, model_dir, strict != 0, &warning, nullptr);
        g_warning = warning;
        return h.release();
    });
}

tqe_model_t* tqe_model_random(const char* config_json, uint64_t seed, int dtype, int on_gpu) {
    return guarded_new<tqe_model_t>([&] {
        DeviceScope scope(on_gpu != 0);
        std::unique_ptr<tqe_model_t> h(model_from_config(parse_config_text(config_json), dtype, on_gpu));
        random_weights(*h->m, seed, nullptr);
        return h.release();
    });
}

tqe_model_t* tqe_model_new(const char* config_json, int dtype, int on_gpu) {
    return guarded_new<tqe_model_t>([&] {
        DeviceScope scope(on_gpu != 0);
        return model_from_config(parse_config_text(config_json), dtype, on_gpu);
    });
}

tqe_model_t* tqe_model_from_spec(const char* spec_json, int dtype, int on_gpu) {
    return guarded_new<tqe_model_t>([&] {
        need(spec_json, "tqe_model_from_spec");
        DeviceScope scope(on_gpu != 0);
        std::unique_ptr<tqe_model_t> h(new tqe_model_t());
        h->m = std::make_shared<Model>(ModelSpec::from_json(Json::parse(spec_json)), run_dtype(dtype), on_gpu != 0);
        return h.release();
    });
}

int tqe_model_set_tensor(tqe_model_t* model, const char* name, const tqe_tensor_t* tensor, int on_device, void* stream) {
    return guarded([&] {
        need(model, "tqe_model_set_tensor");
        need(name, "tqe_model_set_tensor");
        need(tensor, "tqe_model_set_tensor");
        DeviceScope scope(model->m->on_gpu);
        model->pending[name] = copy_in(*tensor, on_device != 0, (hipStream_t)stream);
    });
}

// names, shapes and kinds of tensors given one by one, as the loader checks a folder's
static void check_pending(const Loaded& pending, const TensorSpecs& wanted, bool strict, std::string* warning) {
    std::map<std::string, StoredTensor> stored;
    for (const auto& p : pending) {
        StoredTensor st;
        st.name = p.first;
        st.dtype = p.second->t.dtype == F32 ? "F32" : p.second->t.dtype == BF16 ? "BF16" : "I32";
        st.shape.assign(p.second->t.shape, p.second->t.shape + p.second->t.ndim);
        stored[p.first] = st;
    }
    check_weights(stored, wanted, strict, warning);
}

int tqe_model_finish(tqe_model_t* model, int strict, void* stream) {
    return guarded([&] {
        need(model, "tqe_model_finish");
        DeviceScope scope(model->m->on_gpu);
        std::string warning;
        check_pending(model->pending, model->m->tensor_specs(), strict != 0, &warning);
        g_warning = warning;
        Loaded loaded;
        loaded.swap(model->pending);
        model->m->load(loaded, (hipStream_t)stream);
    });
}

int tqe_model_randomize(tqe_model_t* model, uint64_t seed, void* stream) {
    return guarded([&] {
        need(model, "tqe_model_randomize");
        DeviceScope scope(model->m->on_gpu);
        random_weights(*model->m, seed, (hipStream_t)stream);
    });
}

int tqe_model_tune_library(tqe_model_t* model, int rows, void* stream) {
    return guarded([&] {
        need(model, "tqe_model_tune_library");
        DeviceScope scope(model->m->on_gpu);
        model->m->tune_library(rows, (hipStream_t)stream);
    });
}

const char* tqe_model_describe(const tqe_model_t* model) {
    if (!model) { set_error(TQE_ERR_ARGUMENT, "tqe_model_describe: null pointer"); return nullptr; }
    tqe_model_t* m = const_cast<tqe_model_t*>(model);
    const int status = guarded([&] { m->text = m->m->describe().dump(); });
    return status == TQE_OK ? m->text.c_str() : nullptr;
}

int tqe_model_tensor(const tqe_model_t* model, const char* name, tqe_tensor_t* out) {
    return guarded([&] {
        need(model, "tqe_model_tensor");
        need(name, "tqe_model_tensor");
        need(out, "tqe_model_tensor");
        OwnedPtr p = model->m->held(name);
        if (!p) raise(TQE_ERR_ARGUMENT, "the model holds no tensor '%s' (tensors folded into others are gone)", name);
        *out = to_c(p->t);
    });
}

int tqe_model_set_stop_tokens(tqe_model_t* model, int n, const int32_t* ids) {
    return guarded([&] {
        need(model, "tqe_model_set_stop_tokens");
        if (n < 0 || (n > 0 && !ids)) raise(TQE_ERR_ARGUMENT, "tqe_model_set_stop_tokens: bad arguments");
        model->m->stop_token_ids.assign(ids, ids + n);
    });
}

void tqe_model_free(tqe_model_t* model) {
    if (!model) return;
    guarded([&] { DeviceScope scope(model->m && model->m->on_gpu); delete model; });
}

int tqe_write_random_folder(const char* folder, const char* config_json, uint64_t seed, int store_dtype) {
    return guarded([&] {
        need(folder, "tqe_write_random_folder");
        DeviceScope scope(false);
        const Json raw = parse_config_text(config_json);
        const Architecture& a = architecture_for(raw);
        Model model(a.build_spec(a.typed_config(raw, "config.json")), F32, false);
        write_random_folder(folder, config_json, model.tensor_specs(), seed, store_dtype);
    });
}

int tqe_random_stream(uint64_t seed, const char* tensor_name, int64_t begin, int64_t count, float* out) {
    return guarded([&] {
        need(tensor_name, "tqe_random_stream");
        if (count < 0 || begin < 0 || (count > 0 && !out)) raise(TQE_ERR_ARGUMENT, "tqe_random_stream: bad arguments");
        standard_normal_host(tensor_key(seed, tensor_name), begin, count, out);
    });
}

int tqe_random_stream_of_key(uint64_t key, int64_t begin, int64_t count, float* out) {
    return guarded([&] {
        if (count < 0 || begin < 0 || (count > 0 && !out)) raise(TQE_ERR_ARGUMENT, "tqe_random_stream_of_key: bad arguments");
        standard_normal_host(key, begin, count, out);
    });
}

uint64_t tqe_tensor_key(uint64_t seed, const char* tensor_name) { return tensor_name ? tensor_key(seed, tensor_name) : 0; }

// ---- safetensors ------------------------------------------------------------------------------------
tqe_folder_t* tqe_folder_open(const char* model_dir) {
    return guarded_new<tqe_folder_t>([&] {
        need(model_dir, "tqe_folder_open");
        std::unique_ptr<tqe_folder_t> h(new tqe_folder_t());
        h->f = open_folder(model_dir);
        return h.release();
    });
}
void tqe_folder_free(tqe_folder_t* folder) { delete folder; }
const char* tqe_folder_describe(const tqe_folder_t* folder) {
    if (!folder) { set_error(TQE_ERR_ARGUMENT, "tqe_folder_describe: null pointer"); return nullptr; }
    tqe_folder_t* f = const_cast<tqe_folder_t*>(folder);
    const int status = guarded([&] {
        Json out = Json::object();
        for (const auto& t : f->f->tensors) {
            Json info = Json::object();
            info.set("dtype", t.second.dtype);
            Json shape = Json::array();
            for (int64_t s : t.second.shape) shape.push(Json((long long)s));
            info.set("shape", shape);
            info.set("data", (long long)(uintptr_t)t.second.data);
            info.set("bytes", (long long)t.second.bytes);
            out.append(t.first, info);
        }
        f->text = out.dump();
    });
    return status == TQE_OK ? f->text.c_str() : nullptr;
}
int tqe_check_weights(const tqe_folder_t* folder, const char* wanted_json, int strict) {
    return guarded([&] {
        need(folder, "tqe_check_weights");
        need(wanted_json, "tqe_check_weights");
        const Json wanted = Json::parse(wanted_json);
        TensorSpecs specs;
        if (!wanted.is_object()) raise(TQE_ERR_ARGUMENT, "tqe_check_weights: the wanted tensors must be an object");
        for (const Json::Member& m : wanted.members()) specs.push_back({m.first, TensorSpec::from_json(m.second)});
        std::string warning;
        check_weights(folder->f->tensors, specs, strict != 0, &warning);
        g_warning = warning;
    });
}
int tqe_write_safetensors(const char* path, const char* tensors_json, const void* const* data, const char* metadata_json) {
    return guarded([&] {
        need(path, "tqe_write_safetensors");
        need(tensors_json, "tqe_write_safetensors");
        const Json list = Json::parse(tensors_json);
        if (!list.is_object()) raise(TQE_ERR_ARGUMENT, "tqe_write_safetensors: the tensors must be an object");
        std::vector<TensorToWrite> out;
        size_t i = 0;
        for (const Json::Member& m : list.members()) {
            TensorToWrite t;
            t.name = m.first;
            t.dtype = m.second["dtype"].as_string();
            size_t n = 1;
            for (const Json& s : m.second["shape"].items()) { t.shape.push_back(s.as_int()); n *= (size_t)s.as_int(); }
            const size_t item = (t.dtype == "F64" || t.dtype == "I64") ? 8 : (t.dtype == "F32" || t.dtype == "I32") ? 4
                                : (t.dtype == "BF16" || t.dtype == "F16" || t.dtype == "I16") ? 2 : 1;
            t.bytes = n * item;
            const void* src = data ? data[i] : nullptr;
            if (t.bytes && !src) raise(TQE_ERR_ARGUMENT, "tqe_write_safetensors: tensor %s has no data", t.name.c_str());
            const size_t bytes = t.bytes;
            t.write = [src, bytes](FILE* f) { if (bytes) fwrite(src, 1, bytes, f); };
            out.push_back(std::move(t));
            ++i;
        }
        write_safetensors(path, out, metadata_json ? Json::parse(metadata_json) : Json());
    });
}

// ---- single parts, a cache and a step of one's own ------------------------------------------------------
tqe_part_t* tqe_part_new(const char* category, const char* spec_json, int act_dtype, int on_gpu) {
    return guarded_new<tqe_part_t>([&] {
        need(category, "tqe_part_new");
        need(spec_json, "tqe_part_new");
        DeviceScope scope(on_gpu != 0);
        std::unique_ptr<tqe_part_t> h(new tqe_part_t());
        h->on_gpu = on_gpu != 0;
        h->env.act_dtype = run_dtype(act_dtype);
        h->env.null_device = !h->on_gpu;
        h->p = build_part(category, PartSpec::from_json(Json::parse(spec_json), category), h->env);
        return h.release();
    });
}
void tqe_part_free(tqe_part_t* part) {
    if (!part) return;
    guarded([&] { DeviceScope scope(part->on_gpu); delete part; });
}
const char* tqe_part_describe(const tqe_part_t* part) {
    if (!part) { set_error(TQE_ERR_ARGUMENT, "tqe_part_describe: null pointer"); return nullptr; }
    tqe_part_t* p = const_cast<tqe_part_t*>(part);
    const int status = guarded([&] {
        Json j = p->p->describe();
        if (Mixer* m = dynamic_cast<Mixer*>(p->p.get())) j.set("cache_need", m->cache_need().to_json());
        if (Block* b = dynamic_cast<Block*>(p->p.get())) j.set("cache_need", b->cache_need().to_json());
        if (Position* pos = dynamic_cast<Position*>(p->p.get())) {
            j.set("max_positions", (long long)pos->max_positions);
            j.set("has_apply", pos->has_apply());
            j.set("acts_on_stream", pos->acts_on_stream());
            const Position::Tables t = pos->tables();
            j.set("rot_dim", t.rot_dim);
            j.set("style", t.style);
        }
        p->text = j.dump();
    });
    return status == TQE_OK ? p->text.c_str() : nullptr;
}
int tqe_part_set_tensor(tqe_part_t* part, const char* name, const tqe_tensor_t* tensor, int on_device, void* stream) {
    return guarded([&] {
        need(part, "tqe_part_set_tensor");
        need(name, "tqe_part_set_tensor");
        need(tensor, "tqe_part_set_tensor");
        DeviceScope scope(part->on_gpu);
        part->pending[name] = copy_in(*tensor, on_device != 0, (hipStream_t)stream);
    });
}
int tqe_part_finish(tqe_part_t* part, void* stream) {
    return guarded([&] {
        need(part, "tqe_part_finish");
        DeviceScope scope(part->on_gpu);
        check_pending(part->pending, part->p->tensors(), true, nullptr);
        Loaded loaded;
        loaded.swap(part->pending);
        part->p->load(loaded, (hipStream_t)stream);
        stream_synchronize((hipStream_t)stream);
    });
}
int tqe_part_tensor(const tqe_part_t* part, const char* name, tqe_tensor_t* out) {
    return guarded([&] {
        need(part, "tqe_part_tensor");
        need(name, "tqe_part_tensor");
        need(out, "tqe_part_tensor");
        OwnedPtr p = part->p->held(name);
        if (!p) raise(TQE_ERR_ARGUMENT, "the part holds no tensor '%s'", name);
        *out = to_c(p->t);
    });
}

static Tensor arg(const tqe_tensor_t* args, int n_args, int i, const char* what, int dtype, int64_t rows, int64_t cols) {
    if (i >= n_args) raise(TQE_ERR_ARGUMENT, "%s: argument %d is missing", what, i);
    Tensor t = from_c(args[i]);
    if (!t.data) raise(TQE_ERR_ARGUMENT, "%s: argument %d has no data", what, i);
    if (args[i].row_stride != 0 && args[i].row_stride != t.cols()) raise(TQE_ERR_ARGUMENT, "%s: argument %d must lie row after row", what, i);
    if (dtype >= 0 && t.dtype != dtype) raise(TQE_ERR_ARGUMENT, "%s: argument %d must be %s, got %s", what, i, dtype_name(dtype), t.describe().c_str());
    if ((rows >= 0 && t.shape[0] != rows) || (cols >= 0 && t.cols() != cols))
        raise(TQE_ERR_ARGUMENT, "%s: argument %d must be [%lld, %lld], got %s", what, i, (long long)rows, (long long)cols, t.describe().c_str());
    return t;
}

int tqe_part_call(tqe_part_t* part, const char* method, tqe_stepctx_t* step, tqe_store_t* store, int run, int n_args, const tqe_tensor_t* args,
                  void* stream) {
    return guarded([&] {
        need(part, "tqe_part_call");
        need(method, "tqe_part_call");
        if (n_args < 0 || (n_args > 0 && !args)) raise(TQE_ERR_ARGUMENT, "tqe_part_call: bad arguments");
        DeviceScope scope(part->on_gpu);
        const std::string m = method;
        const int act = part->env.act_dtype;
        // a step of its own where the caller has none: a stream, a workspace, nothing else
        std::unique_ptr<tqe_stepctx_t> own;
        if (!step) {
            own.reset(new tqe_stepctx_t());
            own->c.ws = &own->ws;
            own->c.staging = &own->staging;
            own->c.act_dtype = act;
            step = own.get();
        }
        StepContext& c = step->c;
        c.stream = (hipStream_t)stream;
        if (Norm* norm = dynamic_cast<Norm*>(part->p.get())) {
            const int64_t size = norm->size();
            auto pending = [&](int i, int64_t rows) {
                if (i >= n_args || !args[i].data) return Pending();
                return Pending::of(arg(args, n_args, i, method, act, rows, size));
            };
            if (m == "forward") {
                Tensor x = arg(args, n_args, 0, method, act, -1, size), out = arg(args, n_args, 1, method, act, x.shape[0], size);
                norm->forward(c, x, out);
            } else if (m == "add_norm") {
                Tensor h = arg(args, n_args, 0, method, F32, -1, size), out = arg(args, n_args, 2, method, act, h.shape[0], size);
                norm->add_norm(c, h, pending(1, h.shape[0]), out);
            } else if (m == "gather_add_norm") {
                Tensor h = arg(args, n_args, 0, method, F32, -1, size), rows = arg(args, n_args, 2, method, I32, -1, 1);
                Tensor out = arg(args, n_args, 3, method, act, rows.shape[0], size);
                norm->gather_add_norm(c, h, pending(1, h.shape[0]), (const int32_t*)rows.data, rows.shape[0], out);
            } else raise(TQE_ERR_ARGUMENT, "a norm has no method '%s' (forward, add_norm, gather_add_norm)", method);
        } else if (FeedForward* ff = dynamic_cast<FeedForward*>(part->p.get())) {
            if (m != "forward") raise(TQE_ERR_ARGUMENT, "a feed-forward has no method '%s' (forward)", method);
            Activation x;
            x.x = arg(args, n_args, 0, method, act, -1, -1);
            Tensor out = arg(args, n_args, 1, method, act, x.x.shape[0], -1);
            if (c.n_tokens == 0) c.n_tokens = (int)x.x.shape[0];
            Tensor y = ff->forward(c, x, nullptr);
            if (y.bytes() != out.bytes()) raise(TQE_ERR_ARGUMENT, "%s: the output is %s, the buffer given %s", method, y.describe().c_str(), out.describe().c_str());
            copy_on_device(out.data, y.data, y.bytes(), c.stream);
        } else if (Mixer* mixer = dynamic_cast<Mixer*>(part->p.get())) {
            if (m != "forward") raise(TQE_ERR_ARGUMENT, "a mixer has no method '%s' (forward)", method);
            if (own || !store) raise(TQE_ERR_ARGUMENT, "a mixer needs a step and a cache");
            Activation x;
            x.x = arg(args, n_args, 0, method, act, c.n_tokens, -1);
            Tensor out = arg(args, n_args, 1, method, act, c.n_tokens, -1);
            classify_step(c, x.x.shape[1]);
            Tensor y = mixer->forward(c, x, store->s->entry(run), nullptr, false);
            if (y.bytes() != out.bytes()) raise(TQE_ERR_ARGUMENT, "%s: the output is %s, the buffer given %s", method, y.describe().c_str(), out.describe().c_str());
            copy_on_device(out.data, y.data, y.bytes(), c.stream);
        } else {
            raise(TQE_ERR_ARGUMENT, "parts of category '%s' are not called one by one", part->p->category.c_str());
        }
        if (own) stream_synchronize(c.stream);         // its workspace goes with it
    });
}

tqe_store_t* tqe_store_new(const char* needs_json, const int32_t* cache_of, int n_runs, long long max_tokens, int max_slots, int dtype, int on_gpu) {
    return guarded_new<tqe_store_t>([&] {
        need(needs_json, "tqe_store_new");
        DeviceScope scope(on_gpu != 0);
        const Json needs = Json::parse(needs_json);
        if (!needs.is_array() || (int)needs.items().size() != n_runs || (n_runs > 0 && !cache_of))
            raise(TQE_ERR_ARGUMENT, "tqe_store_new: %d runs need a list of %d needs and their cache_of", n_runs, n_runs);
        std::vector<CacheNeed> ns;
        for (const Json& n : needs.items()) ns.push_back(CacheNeed::from_json(n));
        std::unique_ptr<tqe_store_t> h(new tqe_store_t());
        h->on_gpu = on_gpu != 0;
        h->s.reset(new CacheStore(ns, std::vector<int>(cache_of, cache_of + n_runs), max_tokens, max_slots, run_dtype(dtype)));
        return h.release();
    });
}
void tqe_store_free(tqe_store_t* store) {
    if (!store) return;
    guarded([&] { DeviceScope scope(store->on_gpu); delete store; });
}
tqe_cache_t* tqe_store_cache(tqe_store_t* store) { return store ? store->s->book : nullptr; }
const char* tqe_store_describe(const tqe_store_t* store) {
    if (!store) { set_error(TQE_ERR_ARGUMENT, "tqe_store_describe: null pointer"); return nullptr; }
    tqe_store_t* s = const_cast<tqe_store_t*>(store);
    const int status = guarded([&] { s->text = s->s->describe().dump(); });
    return status == TQE_OK ? s->text.c_str() : nullptr;
}
int tqe_store_acquire(tqe_store_t* store, int32_t* slot_out, void* stream) {
    return guarded([&] {
        need(store, "tqe_store_acquire");
        need(slot_out, "tqe_store_acquire");
        DeviceScope scope(store->on_gpu);
        *slot_out = store->s->acquire((hipStream_t)stream);
    });
}

tqe_stepctx_t* tqe_stepctx_new(tqe_store_t* store, int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens,
                               const int32_t* want_counts, const int32_t* want_idx, int act_dtype, void* stream) {
    return guarded_new<tqe_stepctx_t>([&] {
        need(store, "tqe_stepctx_new");
        DeviceScope scope(store->on_gpu);
        std::unique_ptr<tqe_stepctx_t> h(new tqe_stepctx_t());
        h->on_gpu = store->on_gpu;
        h->c.stream = (hipStream_t)stream;
        h->c.ws = &h->ws;
        h->c.staging = &h->staging;
        h->c.act_dtype = run_dtype(act_dtype);
        h->c.plan(store->s->book, n_seqs, slots, nullptr, n_new, tokens, want_counts, want_idx, 1);
        h->c.upload();
        return h.release();
    });
}
void tqe_stepctx_free(tqe_stepctx_t* step) {
    if (!step) return;
    guarded([&] {
        DeviceScope scope(step->on_gpu);
        stream_synchronize(step->c.stream);
        delete step;
    });
}
int tqe_stepctx_view(tqe_stepctx_t* step, tqe_step_view_t* out) {
    return guarded([&] {
        need(step, "tqe_stepctx_view");
        need(out, "tqe_stepctx_view");
        fill_step_view(step->c, *out);
    });
}

// ---- the engine ----------------------------------------------------------------------------------------
tqe_engine_t* tqe_engine_new(tqe_model_t* model, long long max_tokens, int max_slots, int use_graphs) {
    return guarded_new<tqe_engine_t>([&] {
        need(model, "tqe_engine_new");
        DeviceScope scope(model->m->on_gpu);
        std::unique_ptr<tqe_engine_t> h(new tqe_engine_t());
        h->model = model->m;
        h->e.reset(new Engine(model->m, max_tokens, max_slots, use_graphs != 0));
        return h.release();
    });
}
void tqe_engine_free(tqe_engine_t* engine) {
    if (!engine) return;
    guarded([&] { DeviceScope scope(engine->model->on_gpu); delete engine; });
}
int tqe_engine_open(tqe_engine_t* engine, int32_t* slot_out, void* stream) {
    return guarded([&] {
        need(engine, "tqe_engine_open");
        need(slot_out, "tqe_engine_open");
        DeviceScope scope(engine->model->on_gpu);
        *slot_out = engine->e->open((hipStream_t)stream);
    });
}
int tqe_engine_close(tqe_engine_t* engine, int slot) {
    return guarded([&] { need(engine, "tqe_engine_close"); engine->e->close(slot); });
}
tqe_cache_t* tqe_engine_cache(tqe_engine_t* engine) { return engine ? engine->e->cache->book : nullptr; }
const char* tqe_engine_describe(const tqe_engine_t* engine) {
    if (!engine) { set_error(TQE_ERR_ARGUMENT, "tqe_engine_describe: null pointer"); return nullptr; }
    tqe_engine_t* e = const_cast<tqe_engine_t*>(engine);
    const int status = guarded([&] {
        Json j = e->e->cache->describe();
        j.set("max_tokens", (long long)e->e->max_tokens);
        j.set("use_graphs", e->e->use_graphs);
        j.set("n_graphs", e->e->n_graphs());
        j.set("vocab_size", (long long)e->model->spec.vocab_size);
        j.set("max_positions", (long long)e->model->spec.max_positions);
        e->text = j.dump();
    });
    return status == TQE_OK ? e->text.c_str() : nullptr;
}

int tqe_step(tqe_engine_t* engine, int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens, const int32_t* want_counts,
             const int32_t* want_idx, const int32_t* device_tokens, float* logits_out, int logits_on_host, const float** logits_kept, void* stream) {
    return guarded([&] {
        need(engine, "tqe_step");
        DeviceScope scope(engine->model->on_gpu);
        hipStream_t s = (hipStream_t)stream;
        const float* where = engine->e->step(n_seqs, slots, n_new, tokens, want_counts, want_idx, device_tokens,
                                             logits_on_host ? nullptr : logits_out, s);
        if (logits_on_host && logits_out) {
            long long n_want = 0;
            for (int i = 0; i < n_seqs; ++i) n_want += want_counts[i];
            copy_to_host(logits_out, where, (size_t)n_want * (size_t)engine->model->spec.vocab_size * sizeof(float), s);
        }
        if (logits_kept) *logits_kept = where;
    });
}

// ---- sampling and the loop ---------------------------------------------------------------------------------
void tqe_generation_defaults(tqe_generation_params_t* p) {
    if (!p) return;
    const GenerationParams g;
    p->max_tokens = g.max_tokens;
    p->temperature = g.temperature;
    p->top_p = g.top_p;
    p->top_k = g.top_k;
    p->repeat_penalty = g.repeat_penalty;
    p->seed = g.seed;
}
float tqe_draw_uniform(uint64_t seed, uint64_t request, uint64_t step) { return draw_uniform(seed, request, step); }

static std::vector<std::vector<int32_t>> prompts_from(int n_prompts, const int32_t* prompt_lens, const int32_t* tokens) {
    if (n_prompts < 0 || (n_prompts > 0 && (!prompt_lens || !tokens))) raise(TQE_ERR_ARGUMENT, "the prompts are missing");
    std::vector<std::vector<int32_t>> prompts;
    size_t at = 0;
    for (int i = 0; i < n_prompts; ++i) {
        if (prompt_lens[i] < 0) raise(TQE_ERR_ARGUMENT, "prompt %d has %d tokens", i, prompt_lens[i]);
        prompts.emplace_back(tokens + at, tokens + at + prompt_lens[i]);
        at += (size_t)prompt_lens[i];
    }
    return prompts;
}

static void emit(const std::vector<std::vector<int32_t>>& emitted, int max_tokens, int32_t* out_tokens, int32_t* out_counts) {
    for (size_t i = 0; i < emitted.size(); ++i) {
        if (out_counts) out_counts[i] = (int32_t)emitted[i].size();
        if (out_tokens)
            for (size_t k = 0; k < emitted[i].size() && (int)k < max_tokens; ++k) out_tokens[i * (size_t)max_tokens + k] = emitted[i][k];
    }
}

int tqe_generate(tqe_engine_t* engine, int n_prompts, const int32_t* prompt_lens, const int32_t* tokens, const tqe_generation_params_t* params,
                 const int32_t* stop_ids, int n_stop_ids, int max_batch, int max_step_tokens, tqe_on_tokens on_tokens, void* user,
                 int32_t* out_tokens, int32_t* out_counts, void* stream) {
    return guarded([&] {
        need(engine, "tqe_generate");
        DeviceScope scope(engine->model->on_gpu);
        hipStream_t s = (hipStream_t)stream;
        const GenerationParams p = params_from(params);
        const std::vector<std::vector<int32_t>> prompts = prompts_from(n_prompts, prompt_lens, tokens);
        std::vector<int32_t> eos = n_stop_ids < 0 ? engine->model->stop_token_ids : std::vector<int32_t>(stop_ids, stop_ids + (stop_ids ? n_stop_ids : 0));
        EngineForLoop loop(*engine->e, s);
        const int vocab = (int)engine->model->spec.vocab_size;
        OnTokens cb;
        if (on_tokens) cb = [on_tokens, user](int n, const int32_t* r, const int32_t* t) { on_tokens(user, n, r, t); };
        const auto emitted = generate(loop, prompts, p, eos, cb, max_batch > 0 ? max_batch : 64,
                                      [&](const GenerationParams& gp, const std::vector<int>& ids) {
                                          return std::unique_ptr<LoopSampler>(new DeviceSampler(gp, ids, vocab, s));
                                      },
                                      max_step_tokens > 0 ? max_step_tokens : 8192);
        emit(emitted, p.max_tokens, out_tokens, out_counts);
    });
}

namespace {
struct CallbackEngine : LoopEngine {
    const tqe_loop_callbacks_t& cb;
    void* user;
    CallbackEngine(const tqe_loop_callbacks_t& c, void* u) : cb(c), user(u) {}
    [[noreturn]] void fail(int status, const char* what) {
        const char* msg = cb.last_error ? cb.last_error(user) : nullptr;
        throw Error(status, msg && *msg ? msg : what);
    }
    int open() override {
        int32_t slot = -1;
        const int st = cb.open(user, &slot);
        if (st != 0) fail(st, "the caller's engine could not open a sequence");
        return slot;
    }
    void close(int slot) override {
        const int st = cb.close(user, slot);
        if (st != 0) fail(st, "the caller's engine could not close a sequence");
    }
    // the tokens of a step that runs ahead: a draw of the caller's sampler and places in it
    int pending_draw = -1;
    std::vector<int32_t> pending_places;
    int32_t pending_marker = 0;
    bool takes_device_tokens() const override { return cb.draw && cb.read && cb.step_ahead; }
    const float* step(const std::vector<StepItem>& items, const int32_t* device_tokens) override {
        if (device_tokens) {
            if (device_tokens != &pending_marker || pending_places.size() != items.size())
                throw Error(TQE_ERR_STATE, "a step that runs ahead without the draw it feeds on");
            std::vector<int32_t> ahead_slots;
            for (const StepItem& it : items) ahead_slots.push_back(it.slot);
            const int st = cb.step_ahead(user, (int)items.size(), ahead_slots.data(), pending_draw, pending_places.data());
            if (st != 0) fail(st, "the caller's engine failed in a step");
            return nullptr;
        }
        std::vector<int32_t> slots, n_new, tokens, want;
        for (const StepItem& it : items) {
            slots.push_back(it.slot);
            n_new.push_back(it.n_tokens);
            tokens.insert(tokens.end(), it.tokens, it.tokens + it.n_tokens);
            want.push_back(it.want_last ? 1 : 0);
        }
        const int st = cb.step(user, (int)items.size(), slots.data(), n_new.data(), tokens.data(), want.data());
        if (st != 0) fail(st, "the caller's engine failed in a step");
        return nullptr;
    }
    long long max_tokens() const override { return cb.max_tokens; }
    long long max_positions() const override { return cb.max_positions; }
    int max_slots() const override { return cb.max_slots; }
    bool holds_pages() const override { return cb.holds_pages != 0; }
};
struct CallbackDraw : Draw {
    CallbackEngine& e;
    int id, n;
    CallbackDraw(CallbackEngine& eng, int id_, int n_) : e(eng), id(id_), n(n_) {}
    std::vector<int32_t> read() override {
        std::vector<int32_t> out((size_t)n, 0);
        const int st = e.cb.read(e.user, id, n, out.data());
        if (st != 0) e.fail(st, "the caller's sampler could not read a draw");
        return out;
    }
};
struct CallbackSampler : LoopSampler {
    CallbackEngine& e;
    explicit CallbackSampler(CallbackEngine& eng) : e(eng) {}
    bool runs_ahead() const override { return e.takes_device_tokens(); }
    std::unique_ptr<Draw> draw(const float*, const std::vector<int>& rows) override {
        std::vector<int32_t> r(rows.begin(), rows.end());
        int32_t id = -1;
        const int st = e.cb.draw(e.user, (int)rows.size(), r.data(), &id);
        if (st != 0) e.fail(st, "the caller's sampler could not start a draw");
        return std::unique_ptr<Draw>(new CallbackDraw(e, id, (int)rows.size()));
    }
    const int32_t* pick(Draw& d, const std::vector<int>& places) override {
        e.pending_draw = static_cast<CallbackDraw&>(d).id;
        e.pending_places.assign(places.begin(), places.end());
        return &e.pending_marker;
    }
    std::vector<int32_t> sample(const float*, const std::vector<int>& rows) override {
        std::vector<int32_t> r(rows.begin(), rows.end()), out(rows.size(), 0);
        const int st = e.cb.sample(e.user, (int)rows.size(), r.data(), out.data());
        if (st != 0) e.fail(st, "the caller's sampler failed");
        return out;
    }
};
}  // namespace

int tqe_generate_with(const tqe_loop_callbacks_t* callbacks, void* user, int n_prompts, const int32_t* prompt_lens, const int32_t* tokens,
                      const tqe_generation_params_t* params, const int32_t* stop_ids, int n_stop_ids, int max_batch, int max_step_tokens,
                      tqe_on_tokens on_tokens, void* on_tokens_user, int32_t* out_tokens, int32_t* out_counts) {
    return guarded([&] {
        need(callbacks, "tqe_generate_with");
        if (!callbacks->open || !callbacks->close || !callbacks->step || !callbacks->sample)
            raise(TQE_ERR_ARGUMENT, "tqe_generate_with: open, close, step and sample are needed");
        const GenerationParams p = params_from(params);
        const auto prompts = prompts_from(n_prompts, prompt_lens, tokens);
        std::vector<int32_t> eos(stop_ids, stop_ids + (stop_ids && n_stop_ids > 0 ? n_stop_ids : 0));
        CallbackEngine loop(*callbacks, user);
        OnTokens cb;
        if (on_tokens) cb = [on_tokens, on_tokens_user](int n, const int32_t* r, const int32_t* t) { on_tokens(on_tokens_user, n, r, t); };
        const auto emitted = generate(loop, prompts, p, eos, cb, max_batch > 0 ? max_batch : 64,
                                      [&](const GenerationParams&, const std::vector<int>& ids) {
                                          if (callbacks->new_batch) {
                                              std::vector<int32_t> r(ids.begin(), ids.end());
                                              const int st = callbacks->new_batch(user, (int)r.size(), r.data());
                                              if (st != 0) loop.fail(st, "the caller's sampler could not start a batch");
                                          }
                                          return std::unique_ptr<LoopSampler>(new CallbackSampler(loop));
                                      },
                                      max_step_tokens > 0 ? max_step_tokens : 8192);
        emit(emitted, p.max_tokens, out_tokens, out_counts);
    });
}

tqe_sampler_t* tqe_sampler_new(const tqe_generation_params_t* params, int n_requests, const int32_t* request_ids, int vocab, void* stream) {
    return guarded_new<tqe_sampler_t>([&] {
        if (n_requests < 0 || (n_requests > 0 && !request_ids) || vocab < 1) raise(TQE_ERR_ARGUMENT, "tqe_sampler_new: bad arguments");
        std::unique_ptr<tqe_sampler_t> h(new tqe_sampler_t());
        h->vocab = vocab;
        h->s.reset(new DeviceSampler(params_from(params), std::vector<int>(request_ids, request_ids + n_requests), vocab, (hipStream_t)stream));
        return h.release();
    });
}
void tqe_sampler_free(tqe_sampler_t* sampler) { delete sampler; }
int tqe_sampler_sample(tqe_sampler_t* sampler, float* logits, int n_rows, const int32_t* rows, int32_t* tokens_out) {
    return guarded([&] {
        need(sampler, "tqe_sampler_sample");
        need(logits, "tqe_sampler_sample");
        need(tokens_out, "tqe_sampler_sample");
        if (n_rows < 0 || (n_rows > 0 && !rows)) raise(TQE_ERR_ARGUMENT, "tqe_sampler_sample: bad arguments");
        const std::vector<int32_t> toks = sampler->s->sample(logits, std::vector<int>(rows, rows + n_rows));
        std::copy(toks.begin(), toks.end(), tokens_out);
    });
}

}  // extern "C"
