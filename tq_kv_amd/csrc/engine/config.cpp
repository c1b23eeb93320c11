#include "config.h"

#include <errno.h>
#include <sys/stat.h>

#include <algorithm>
#include <map>
#include <mutex>

namespace tq {

namespace {
std::vector<Architecture>& architectures() {
    static std::vector<Architecture> a;
    return a;
}
std::once_flag g_builtin_once;
void ensure_builtin() { std::call_once(g_builtin_once, [] { register_qwen2(); }); }
std::string joined(const std::vector<std::string>& v) {
    std::string s;
    for (size_t i = 0; i < v.size(); ++i) s += (i ? ", " : "") + v[i];
    return s;
}
}  // namespace

void register_architecture(const Architecture& a) {
    for (Architecture& have : architectures())
        if (have.name == a.name) { have = a; return; }
    architectures().push_back(a);
}

std::vector<std::string> known_architectures() {
    ensure_builtin();
    std::vector<std::string> out;
    for (const Architecture& a : architectures()) out.push_back(a.name);
    std::sort(out.begin(), out.end());
    return out;
}

const Architecture& architecture_for(const Json& raw) {
    ensure_builtin();
    if (!raw.is_object()) raise(TQE_ERR_CONFIG, "config.json: expected a JSON object at the top level");
    const Json& archs = raw["architectures"];
    if (archs.is_array() && !archs.items().empty()) {
        const std::string name = archs.items()[0].is_string() ? archs.items()[0].as_string() : archs.items()[0].dump();
        for (const Architecture& a : architectures())
            if (a.name == name) return a;
        raise(TQE_ERR_CONFIG, "Unknown architecture '%s'. Known architectures: %s", name.c_str(), joined(known_architectures()).c_str());
    }
    const Json& mt = raw["model_type"];
    if (mt.is_string())
        for (const Architecture& a : architectures())
            for (const std::string& t : a.model_types)
                if (t == mt.as_string()) return a;
    raise(TQE_ERR_CONFIG, "config.json names no known architecture (architectures=%s, model_type=%s). Known architectures: %s", archs.dump().c_str(),
          mt.dump().c_str(), joined(known_architectures()).c_str());
}

std::string read_text_file(const std::string& path, const char* what, int error_code) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) raise(error_code, "Cannot read %s: %s: %s", what, path.c_str(), strerror(errno));
    std::string text;
    char buf[1 << 16];
    size_t n;
    while ((n = fread(buf, 1, sizeof(buf), f)) > 0) text.append(buf, n);
    const bool bad = ferror(f) != 0;
    fclose(f);
    if (bad) raise(error_code, "Cannot read %s: %s", what, path.c_str());
    return text;
}

Json read_config_json(const std::string& model_dir) {
    const std::string text = read_text_file(model_dir + "/config.json", "config.json", TQE_ERR_CONFIG);
    try {
        return Json::parse(text);
    } catch (const JsonError& e) {
        raise(TQE_ERR_CONFIG, "Invalid config.json: %s", e.what());
    }
}

static bool exists(const std::string& path) {
    struct stat st;
    return stat(path.c_str(), &st) == 0;
}

std::vector<int32_t> generation_config_stop_ids(const std::string& model_dir) {
    const std::string path = model_dir + "/generation_config.json";
    if (!exists(path)) return {};
    Json raw;
    try {
        raw = Json::parse(read_text_file(path, "generation_config.json", TQE_ERR_CONFIG));
    } catch (const JsonError& e) {
        raise(TQE_ERR_CONFIG, "Invalid generation_config.json: %s", e.what());
    }
    return KeyReader(raw, "generation_config.json").token_ids("eos_token_id");
}

// src/engine.rs:301-308
static const char* const STOP_STRINGS[] = {"<|eot_id|>", "<|im_end|>", "<|endoftext|>", "<|end|>", "<end_of_turn>", "</s>"};

std::vector<int32_t> tokenizer_stop_ids(const std::string& model_dir) {
    const std::string path = model_dir + "/tokenizer.json";
    if (!exists(path)) return {};
    Json raw;
    try {
        raw = Json::parse(read_text_file(path, "tokenizer.json", TQE_ERR_CONFIG));
    } catch (const JsonError& e) {
        raise(TQE_ERR_CONFIG, "Invalid tokenizer.json: %s", e.what());
    }
    std::map<std::string, long long> ids;
    if (raw.is_object()) {
        const Json& vocab = raw["model"]["vocab"];
        if (vocab.is_object())
            for (const Json::Member& m : vocab.members())
                for (const char* s : STOP_STRINGS)
                    if (m.first == s && m.second.is_int()) ids[s] = m.second.as_int();
        if (raw["added_tokens"].is_array())
            for (const Json& tok : raw["added_tokens"].items())
                if (tok.is_object() && tok["content"].is_string() && tok["id"].is_int())
                    for (const char* s : STOP_STRINGS)
                        if (tok["content"].as_string() == s) ids[s] = tok["id"].as_int();
    }
    std::vector<int32_t> out;
    for (const char* s : STOP_STRINGS) {
        auto it = ids.find(s);
        if (it != ids.end() && it->second >= 0 && it->second <= INT32_MAX) out.push_back((int32_t)it->second);
    }
    return out;
}

std::vector<int32_t> folder_stop_token_ids(const std::string& model_dir, const std::vector<int32_t>& config_ids) {
    std::vector<int32_t> out;
    auto add = [&](const std::vector<int32_t>& ids) {
        for (int32_t i : ids)
            if (std::find(out.begin(), out.end(), i) == out.end()) out.push_back(i);
    };
    add(config_ids);
    add(generation_config_stop_ids(model_dir));
    add(tokenizer_stop_ids(model_dir));
    return out;
}

}  // namespace tq
