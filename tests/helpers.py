"""Shared by the tests: the two tiny configurations, model folders with random
weights in a temporary place, reading them back for the plain implementation."""
import json
import os

import torch

TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "vocab_size": 256, "hidden_size": 64, "intermediate_size": 160, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16, "rms_norm_eps": 1e-6,
    "rope_theta": 10000.0, "max_position_embeddings": 128, "tie_word_embeddings": True,
    "use_sliding_window": False,
}
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "vocab_size": 320, "hidden_size": 96, "intermediate_size": 224, "num_hidden_layers": 3,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32, "rms_norm_eps": 1e-5,
    "rope_theta": 1000000.0, "max_position_embeddings": 96, "tie_word_embeddings": False,
    "use_sliding_window": True, "sliding_window": 12, "max_window_layers": 1,
}
# A third one for long sequences: several pages per sequence, a window that crosses pages,
# head size 48 (a multiple of 16 that is no power of two), 6 heads in 2 groups.
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "vocab_size": 509, "hidden_size": 144, "intermediate_size": 200, "num_hidden_layers": 4,
    "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 48, "rms_norm_eps": 3e-6,
    "rope_theta": 50000.0, "max_position_embeddings": 640, "tie_word_embeddings": False,
    "use_sliding_window": True, "sliding_window": 100, "max_window_layers": 2,
}
# A fourth one with the head size of the large models (128) in three groups of two heads, at a width that is no power of two.
TINY_D = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "vocab_size": 411, "hidden_size": 160, "intermediate_size": 288, "num_hidden_layers": 2,
    "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 128, "rms_norm_eps": 2e-6,
    "rope_theta": 300000.0, "max_position_embeddings": 256, "tie_word_embeddings": True,
    "use_sliding_window": False,
}
CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3)}


def make_folder(tmp, cfg, seed, store_dtype=torch.bfloat16):
    """A model folder with random weights, written by the framework's random-weights mode."""
    from tq_kv_amd import Model
    folder = os.path.join(str(tmp), "model_seed%d_%s" % (seed, str(store_dtype).split(".")[-1]))
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        Model.write_random_folder(folder, cfg, seed=seed, store_dtype=store_dtype)
    return folder


def read_folder(folder):
    """(config dict, name -> float32 tensor) read with the safetensors package, not with the
    framework's own reader."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    weights = {k: v.to(torch.float32) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, weights


def random_tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
