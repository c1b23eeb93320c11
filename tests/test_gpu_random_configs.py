"""Configurations drawn at random (seeded): head counts and groups, head sizes in steps of 16,
widths and vocabularies that are no power of two, windows, tied and untied heads.  For each, a
batch of unequal prompts in one step, then decoding steps in which the shorter requests end
earlier, against the plain implementation; in float32 and in bfloat16 (weights sharpened so that
attention picks keys out)."""
import random

import pytest
import torch

import gpu_common as G
import helpers
import plain_qwen2 as plain
from tq_kv_amd import Engine, Model
from tq_kv_amd.weights import random_tensors

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = random.Random(seed)
    n_kv = rng.choice([1, 1, 2, 3, 4])
    n_rep = rng.choice([1, 2, 3, 5, 7, 8])
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    hidden = rng.choice([32, 64, 96, 160]) if rng.random() < 0.7 else rng.choice([40, 72, 104, 136])
    window = rng.choice([None, None, 5, 40, 70])
    layers = rng.choice([1, 2, 3])
    cfg = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
        "vocab_size": rng.randrange(90, 700), "hidden_size": hidden, "intermediate_size": 8 * rng.randrange(5, 40),
        "num_hidden_layers": layers, "num_attention_heads": n_kv * n_rep, "num_key_value_heads": n_kv, "head_dim": d,
        "rms_norm_eps": rng.choice([1e-6, 1e-5, 3e-6]), "rope_theta": rng.choice([1e4, 5e4, 1e6]),
        "max_position_embeddings": 256, "tie_word_embeddings": rng.random() < 0.5,
        "use_sliding_window": window is not None,
    }
    if window is not None:
        cfg.update(sliding_window=window, max_window_layers=rng.randrange(0, layers + 1))
    return cfg, rng


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(40))
def test_a_random_configuration_equals_the_plain_implementation(seed, dtype):
    cfg, rng = draw_config(seed)
    specs = Model.from_config_dict(cfg, "float32", "cpu").tensor_specs()
    tensors = random_tensors(specs, 100 + seed, torch.bfloat16, "cuda")
    # sharper attention: a key that is missed or wrongly seen then moves the logits
    tensors = {k: (v.float() * 4.0).to(v.dtype) if ("q_proj.weight" in k or "k_proj.weight" in k) else v for k, v in tensors.items()}
    model = Model.from_config_dict(cfg, dtype, "cuda")
    model.load({k: v.to(model.dtype) for k, v in tensors.items()})
    eng = Engine(model, max_tokens=64 * 16)
    lens = [rng.choice([1, 2, 9, 33, 64, 65, 100, 130]) for _ in range(rng.choice([2, 3, 5]))]
    n_decode = [rng.randrange(0, 5) for _ in lens]
    reqs = [helpers.random_tokens(n + k, cfg["vocab_size"], 1000 * seed + i) for i, (n, k) in enumerate(zip(lens, n_decode))]
    w = {k: v.float().cpu() for k, v in tensors.items()}
    refs = [plain.forward(w, cfg, r) for r in reqs]
    slots = [eng.open() for _ in reqs]
    out = eng.step([(s, r[:n], [0, n - 1]) for s, r, n in zip(slots, reqs, lens)])
    for i, n in enumerate(lens):
        G.close(out[2 * i], refs[i][0], dtype, "seed %d request %d first place" % (seed, i))
        G.close(out[2 * i + 1], refs[i][n - 1], dtype, "seed %d request %d end of prompt %d" % (seed, i, n))
    pos = list(lens)
    live = [i for i in range(len(reqs)) if pos[i] < len(reqs[i])]
    for i in range(len(reqs)):
        if i not in live:
            eng.close(slots[i])
    while live:
        out = eng.step([(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
        for j, i in enumerate(live):
            G.close(out[j], refs[i][pos[i]], dtype, "seed %d request %d place %d (%s)" % (seed, i, pos[i], cfg))
            pos[i] += 1
        for i in live:
            if pos[i] == len(reqs[i]):
                eng.close(slots[i])
        live = [i for i in live if pos[i] < len(reqs[i])]
    eng.cache.check()
    assert all(not eng.cache.slots.is_held(s) for s in slots)
