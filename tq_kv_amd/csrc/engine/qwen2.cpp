// Qwen2ForCausalLM: the dense decoder the reference runs through src/models/turbo_generic.rs
// (grouped-query attention with q/k/v bias and no output bias, gated-SiLU feed-forward, RMSNorm
// before mixer and feed-forward, rotary positions in the halves layout, tied or untied head).
//
// This file holds what is particular to the architecture: which config.json keys it reads and how
// they become a ModelSpec with the HF tensor names the reference loads by (:2075-2126).  Nothing
// here computes.
#include "config.h"

namespace tq {
namespace {

// Keys as the reference reads them (src/models/turbo_generic.rs:2013-2030), plus those it takes
// from tensor shapes or presence (vocab_size, intermediate_size, tie_word_embeddings) and the
// sliding-window keys.  Sizes have no defaults here; num_key_value_heads and head_dim default as
// the reference's do (:2014, :2020-2022).
Json qwen2_typed(const Json& raw, const std::string& where) {
    KeyReader r(raw, where);
    const long long nh = r.integer("num_attention_heads", 1);
    const long long hidden = r.integer("hidden_size", 1);
    const long long nkv = r.integer_or("num_key_value_heads", nh, 1);
    long long head_dim;
    if (r.has("head_dim")) head_dim = r.integer("head_dim", 1);
    else {
        if (hidden % nh)
            raise(TQE_ERR_CONFIG, "%s: hidden_size %lld is not a multiple of num_attention_heads %lld and no head_dim is given", where.c_str(), hidden, nh);
        head_dim = hidden / nh;
    }
    if (nh % nkv) raise(TQE_ERR_CONFIG, "%s: num_attention_heads %lld is not a multiple of num_key_value_heads %lld", where.c_str(), nh, nkv);
    if (head_dim % 2) raise(TQE_ERR_CONFIG, "%s: head_dim %lld must be even for rotary positions", where.c_str(), head_dim);
    const std::string act = r.string_or("hidden_act", "silu");
    if (act != "silu") raise(TQE_ERR_CONFIG, "%s: hidden_act '%s' is not supported (only 'silu')", where.c_str(), act.c_str());
    if (!raw["rope_scaling"].is_null()) raise(TQE_ERR_CONFIG, "%s: rope_scaling is not supported (must be null or absent)", where.c_str());
    const long long layers = r.integer("num_hidden_layers", 1);
    const bool use_window = r.boolean_or("use_sliding_window", false);
    Json c = Json::object();
    c.set("vocab_size", r.integer("vocab_size", 1));
    c.set("hidden_size", hidden);
    c.set("intermediate_size", r.integer("intermediate_size", 1));
    c.set("num_hidden_layers", layers);
    c.set("num_attention_heads", nh);
    c.set("num_key_value_heads", nkv);
    c.set("head_dim", head_dim);
    c.set("rms_norm_eps", r.number("rms_norm_eps", true));
    c.set("rope_theta", r.number("rope_theta", true));
    c.set("max_position_embeddings", r.integer("max_position_embeddings", 1));
    c.set("tie_word_embeddings", r.boolean_or("tie_word_embeddings", false));
    c.set("use_sliding_window", use_window);
    c.set("sliding_window", use_window ? Json(r.integer("sliding_window", 1)) : Json());
    c.set("max_window_layers", use_window ? Json(r.integer("max_window_layers", 0)) : Json());
    Json eos = Json::array();
    for (int32_t t : r.token_ids("eos_token_id")) eos.push(Json((int)t));
    c.set("eos_token_ids", eos);
    return c;
}

// Layer l is windowed iff use_sliding_window and l >= max_window_layers; a windowed query at
// position i sees the sliding_window keys i-W < j <= i.
Json layer_window(const Json& c, long long layer) {
    if (c["use_sliding_window"].as_bool() && layer >= c["max_window_layers"].as_int()) return c["sliding_window"];
    return Json();
}

PartSpec part(const char* kind, std::initializer_list<std::pair<const char*, Json>> params) {
    PartSpec p;
    p.kind = kind;
    for (const auto& kv : params) p.params.set(kv.first, kv.second);
    return p;
}

ModelSpec qwen2_spec(const Json& c) {
    const long long hidden = c["hidden_size"].as_int(), head_dim = c["head_dim"].as_int(), layers = c["num_hidden_layers"].as_int();
    const PartSpec position = part("rotary", {{"theta", c["rope_theta"]}, {"rot_dim", head_dim}, {"max_positions", c["max_position_embeddings"]},
                                              {"style", "halves"}});
    const PartSpec norm = part("rms_norm", {{"size", hidden}, {"eps", c["rms_norm_eps"]}});
    const PartSpec feed_forward = part("gated_silu", {{"hidden", hidden}, {"inter", c["intermediate_size"]}});
    Json names = Json::object();
    names.set("mixer", "self_attn.");
    names.set("feed_forward", "mlp.");
    names.set("mixer_norm", "input_layernorm.");
    names.set("ff_norm", "post_attention_layernorm.");
    ModelSpec s;
    s.architecture = "Qwen2ForCausalLM";
    s.vocab_size = c["vocab_size"].as_int();
    s.hidden_size = hidden;
    s.max_positions = c["max_position_embeddings"].as_int();
    s.embedding_name = "model.embed_tokens.weight";
    for (long long l = 0; l < layers; ++l) {
        const PartSpec mixer = part("attention", {{"hidden", hidden}, {"n_heads", c["num_attention_heads"]}, {"n_kv_heads", c["num_key_value_heads"]},
                                                  {"head_dim", head_dim}, {"qkv_bias", true}, {"out_bias", false}, {"window", layer_window(c, l)},
                                                  {"scale", Json()}, {"position", position.to_json()}});
        LayerSpec layer;
        layer.prefix = format("model.layers.%lld.", l);
        layer.block = part("pre_norm", {{"mixer", mixer.to_json()}, {"feed_forward", feed_forward.to_json()}, {"mixer_norm", norm.to_json()},
                                        {"ff_norm", norm.to_json()}, {"names", names}});
        s.layers.push_back(layer);
        Run run;
        run.layer = (int)l;
        s.order.push_back(run);
    }
    s.final_norm = norm;
    s.final_norm_prefix = "model.norm.";
    s.head_name = c["tie_word_embeddings"].as_bool() ? "" : "lm_head.weight";
    for (const Json& t : c["eos_token_ids"].items()) s.eos_token_ids.push_back((int32_t)t.as_int());
    return s;
}

}  // namespace

void register_qwen2() {
    Architecture a;
    a.name = "Qwen2ForCausalLM";
    a.model_types = {"qwen2"};
    a.typed_config = qwen2_typed;
    a.build_spec = qwen2_spec;
    register_architecture(a);
}

}  // namespace tq
