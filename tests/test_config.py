"""Configuration: typed keys of config.json, the architecture registry, the catalog."""
import json

import pytest

from helpers import TINY_A, TINY_B
from tq_kv_amd.architectures.qwen2 import Qwen2Config, build_spec
from tq_kv_amd.config import ConfigError, catalog, config_from_dict, known_architectures, load_config


def test_reads_every_key():
    name, cfg = config_from_dict(TINY_B)
    assert name == "Qwen2ForCausalLM"
    assert (cfg.vocab_size, cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (320, 96, 224, 3)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (3, 1, 32)
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 1e6 and cfg.max_position_embeddings == 96
    assert cfg.tie_word_embeddings is False
    assert [cfg.layer_window(l) for l in range(3)] == [None, 12, 12]
    assert config_from_dict(cfg.to_dict())[1] == cfg


def test_defaults_as_the_reference():
    raw = dict(TINY_A)
    del raw["num_key_value_heads"], raw["head_dim"]
    cfg = config_from_dict(raw)[1]
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 16       # kv heads = heads, head_dim = hidden / heads


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "rms_norm_eps", "rope_theta", "max_position_embeddings"])
def test_missing_key_is_named(key):
    raw = dict(TINY_A)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(raw)


def test_wrong_types_and_combinations():
    for key, bad in [("hidden_size", "64"), ("rms_norm_eps", "tiny"), ("tie_word_embeddings", 1), ("num_hidden_layers", 0),
                     ("num_attention_heads", 2.5)]:
        with pytest.raises(ConfigError, match=key):
            config_from_dict(dict(TINY_A, **{key: bad}))
    with pytest.raises(ConfigError, match="multiple"):
        config_from_dict(dict(TINY_A, num_key_value_heads=3))
    with pytest.raises(ConfigError, match="hidden_act"):
        config_from_dict(dict(TINY_A, hidden_act="gelu"))
    with pytest.raises(ConfigError, match="rope_scaling"):
        config_from_dict(dict(TINY_A, rope_scaling={"type": "yarn"}))
    with pytest.raises(ConfigError, match="sliding_window"):
        config_from_dict(dict(TINY_A, use_sliding_window=True, max_window_layers=1))
    with pytest.raises(ConfigError, match="head_dim"):
        raw = dict(TINY_A, hidden_size=66)
        del raw["head_dim"]
        config_from_dict(raw)


def test_what_no_kernel_takes_is_refused_before_any_weight_is_read(tmp_path):
    """A head size beyond what the attention kernels take is a fine config.json as far as the architecture goes; the
    model refuses it when its parts are built (from the kernel library's own word on its limit), not at the first step."""
    from tq_kv_amd import Model
    raw = dict(TINY_A, head_dim=320)
    assert config_from_dict(raw)[1].head_dim == 320
    with pytest.raises(ConfigError, match="head_dim 320 is more than the attention kernels take"):
        Model.from_config_dict(raw, "float32", "cpu")
    (tmp_path / "config.json").write_text(json.dumps(raw))          # a folder without weights: the refusal comes first
    with pytest.raises(ConfigError, match="head_dim 320"):
        Model.from_dir(str(tmp_path), dtype="bfloat16", device="cpu")
    assert Model.from_config_dict(dict(TINY_A, head_dim=256), "float32", "cpu").config.head_dim == 256


def test_unknown_architecture_lists_the_known():
    with pytest.raises(ConfigError, match="Qwen2ForCausalLM"):
        config_from_dict(dict(TINY_A, architectures=["LlamaForCausalLM"]))
    raw = dict(TINY_A)
    del raw["architectures"]
    assert config_from_dict(raw)[0] == "Qwen2ForCausalLM"          # model_type alone is enough
    del raw["model_type"]
    with pytest.raises(ConfigError, match="Known architectures"):
        config_from_dict(raw)
    assert "Qwen2ForCausalLM" in known_architectures()


def test_config_json_errors(tmp_path):
    with pytest.raises(ConfigError, match="Cannot read config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="Invalid config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert load_config(str(tmp_path))[1].hidden_size == 64


def test_eos_ids():
    assert config_from_dict(dict(TINY_A, eos_token_id=7))[1].eos_token_ids == (7,)
    assert config_from_dict(dict(TINY_A, eos_token_id=[7, 9]))[1].eos_token_ids == (7, 9)
    with pytest.raises(ConfigError):
        config_from_dict(dict(TINY_A, eos_token_id="</s>"))


def test_spec_is_data_from_the_config():
    cfg = config_from_dict(TINY_B)[1]
    spec = build_spec(cfg)
    assert [r.layer for r in spec.order] == [0, 1, 2] and all(r.cache_of is None for r in spec.order)
    assert spec.head_name == "lm_head.weight" and build_spec(config_from_dict(TINY_A)[1]).head_name is None
    mixer = spec.layers[2].block.params["mixer"]
    assert mixer.kind == "attention" and mixer.params["window"] == 12 and mixer.params["n_kv_heads"] == 1
    assert spec.layers[0].block.params["mixer"].params["window"] is None
    assert mixer.params["position"].params == {"theta": 1e6, "rot_dim": 32, "max_positions": 96, "style": "halves"}
    assert spec.layers[1].block.params["mixer_norm"].params == {"size": 96, "eps": 1e-5}


def test_catalog_find():
    # exact "name:tag", then the name alone (first entry), as src/catalog.rs:88-103
    assert catalog.find("tiny:b")["hidden_size"] == 96
    assert catalog.find("tiny")["hidden_size"] == 64
    assert catalog.find("qwen2.5:7b")["num_hidden_layers"] == 28
    assert catalog.find("qwen2.5:70b") is None and catalog.find("nothing") is None
    for name, tag in catalog.entries():
        config_from_dict(catalog.find("%s:%s" % (name, tag)))
    assert catalog.find("tiny:a") == TINY_A and catalog.find("tiny:b") == TINY_B


# ---- stop tokens of a model folder (src/engine.rs:301-316) ---------------------------------------
def _folder_with(tmp_path, config_eos=None, generation=None, tokenizer=None):
    raw = dict(TINY_A)
    if config_eos is not None:
        raw["eos_token_id"] = config_eos
    (tmp_path / "config.json").write_text(json.dumps(raw))
    if generation is not None:
        (tmp_path / "generation_config.json").write_text(json.dumps(generation))
    if tokenizer is not None:
        (tmp_path / "tokenizer.json").write_text(json.dumps(tokenizer))
    return str(tmp_path)


def test_stop_tokens_are_the_union_of_every_place_that_names_them(tmp_path):
    from tq_kv_amd.config.generation import stop_token_ids
    folder = _folder_with(
        tmp_path, config_eos=7, generation={"eos_token_id": [9, 7], "temperature": 0.7},
        tokenizer={"added_tokens": [{"id": 9, "content": "<|im_end|>"}, {"id": 11, "content": "<|endoftext|>"},
                                    {"id": 12, "content": "<|im_start|>"}],
                   "model": {"vocab": {"</s>": 2, "a": 3}}})
    cfg = load_config(folder)[1]
    assert cfg.eos_token_ids == (7,)
    # config.json first, then generation_config.json, then the reference's stop strings; each once
    assert stop_token_ids(folder, cfg.eos_token_ids) == (7, 9, 11, 2)


def test_stop_tokens_of_each_place_alone(tmp_path):
    from tq_kv_amd.config.generation import stop_token_ids
    a, b, c, d = [tmp_path / n for n in "abcd"]
    for p in (a, b, c, d):
        p.mkdir()
    assert stop_token_ids(_folder_with(a)) == ()                       # random weights: none, no fallback id
    assert stop_token_ids(_folder_with(b, generation={"eos_token_id": 5})) == (5,)
    assert stop_token_ids(_folder_with(c, generation={"max_new_tokens": 3})) == ()
    with pytest.raises(ConfigError, match="generation_config.json.*eos_token_id"):
        stop_token_ids(_folder_with(d, generation={"eos_token_id": "x"}))
    (d / "generation_config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="Invalid generation_config.json"):
        stop_token_ids(str(d))


def test_a_loaded_model_carries_its_folders_stop_tokens(tmp_path):
    from tq_kv_amd import Model
    folder = Model.write_random_folder(str(tmp_path / "m"), dict(TINY_A, eos_token_id=3), seed=0)
    with open(tmp_path / "m" / "generation_config.json", "w") as f:
        json.dump({"eos_token_id": [3, 200]}, f)
    model = Model.from_dir(folder, dtype="float32", device="cpu")
    assert model.spec.eos_token_ids == (3,) and model.stop_token_ids == (3, 200)
