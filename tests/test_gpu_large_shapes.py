"""The layer sizes of the three large shapes (Qwen2.5-7B, 1.5B, 32B) with two layers each:
the float32 path against the plain implementation (7B sizes), and the bfloat16 path against
the float32 path at spot-checked positions, prompt and decoding, in a batch of unequal
lengths.  Sizes here are what the small configurations cannot show: 28/40/12 heads in groups
of 7/5/6, widths and vocabularies that are no power of two, rows of 18944 and 27648."""
import pytest
import torch

import helpers
import plain_qwen2 as plain
from tq_kv_amd import Engine, Model
from tq_kv_amd.config import catalog
from tq_kv_amd.weights import random_tensors

pytestmark = pytest.mark.gpu


def two_layer(shape):
    raw = dict(catalog.find(shape))
    raw["num_hidden_layers"] = 2
    return raw


def build(raw, dtype, tensors):
    model = Model.from_config_dict(raw, dtype, "cuda")
    want = torch.float32 if dtype == "float32" else torch.bfloat16
    return model.load({k: v.to(want) for k, v in tensors.items()})


def tensors_for(raw, seed):
    specs = Model.from_config_dict(raw, "float32", "cpu").tensor_specs()
    return random_tensors(specs, seed, torch.bfloat16, "cuda")


@pytest.mark.parametrize("shape", ["qwen2.5:7b", "qwen2.5:1.5b", "qwen2.5:32b"])
def test_bfloat16_tracks_float32_at_large_sizes(shape):
    raw = two_layer(shape)
    tensors = tensors_for(raw, 3)
    lens = [300, 70, 1]
    prompts = [helpers.random_tokens(n, raw["vocab_size"], 50 + i) for i, n in enumerate(lens)]
    nxt = [7, 11, 13]
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine(build(raw, dtype, tensors), max_tokens=1024)
        slots = [eng.open() for _ in prompts]
        a = eng.step([(s, p, [len(p) - 1, 0] if len(p) > 1 else [0]) for s, p in zip(slots, prompts)])
        b = eng.step([(s, [t], [0]) for s, t in zip(slots, nxt)])
        outs[dtype] = torch.cat([a, b]).cpu()
        for s in slots:
            eng.close(s)
        del eng
        torch.cuda.empty_cache()
    scale = outs["float32"].abs().max().item()
    assert 0.05 < scale < 50
    torch.testing.assert_close(outs["bfloat16"], outs["float32"], atol=0.03 * max(1.0, scale), rtol=0.03)


@pytest.mark.parametrize("shape,n_seqs", [("qwen2.5:7b", 20), ("qwen2.5:32b", 40)])
def test_bfloat16_tracks_float32_in_steps_of_17_to_64_rows_at_large_sizes(shape, n_seqs):
    """The kernels for 17 to 64 rows at the real widths (sums over pieces of K finished by the norm
    and the rotation kernels, the head product with float32 output): a short prompt step of 24
    tokens, then two decoding steps of n_seqs rows."""
    raw = two_layer(shape)
    tensors = tensors_for(raw, 5)
    first = [helpers.random_tokens(1 + i % 3, raw["vocab_size"], 80 + i) for i in range(n_seqs)]
    nxt = [[(17 * i + 3) % raw["vocab_size"], (29 * i + 5) % raw["vocab_size"]] for i in range(n_seqs)]
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine(build(raw, dtype, tensors), max_tokens=64 * n_seqs)
        slots = [eng.open() for _ in first]
        got = [eng.step([(s, p, [len(p) - 1]) for s, p in zip(slots[:12], first[:12])])]          # 24 tokens, 12 wanted
        eng.step([(s, p, []) for s, p in zip(slots[12:], first[12:])])
        for step in range(2):
            got.append(eng.step([(s, [t[step]], [0]) for s, t in zip(slots, nxt)]))
        outs[dtype] = torch.cat(got).cpu()
        for s in slots:
            eng.close(s)
        del eng
        torch.cuda.empty_cache()
    scale = outs["float32"].abs().max().item()
    assert 0.05 < scale < 50
    torch.testing.assert_close(outs["bfloat16"], outs["float32"], atol=0.03 * max(1.0, scale), rtol=0.03)


def test_float32_path_equals_plain_at_7b_sizes():
    raw = two_layer("qwen2.5:7b")
    tensors = tensors_for(raw, 4)
    prompt = helpers.random_tokens(40, raw["vocab_size"], 60)
    eng = Engine(build(raw, "float32", tensors), max_tokens=256)
    s = eng.open()
    got = [eng.step([(s, prompt[:33], [0, 32])])]
    for t in range(33, 40):
        got.append(eng.step([(s, [prompt[t]], [0])]))
    eng.close(s)
    got = torch.cat(got).cpu()
    cfg = dict(raw)
    want = plain.forward({k: v.float().cpu() for k, v in tensors.items()}, cfg, prompt)[[0] + list(range(32, 40))]
    torch.testing.assert_close(got, want, atol=2e-5 * max(1.0, want.abs().max().item()), rtol=2e-5)


def test_generation_through_graphs_and_running_ahead_equals_plain_stepping_at_7b_sizes():
    # the generation loop (captured graphs, next step started from the device's tokens before the
    # draw is read) against steps given one by one with the host's tokens and no graphs: the same
    # kernels either way, so the same tokens; sampled with the default parameters
    from tq_kv_amd import GenerationParams, generate
    from tq_kv_amd.sampling.sampler import Sampler
    raw = two_layer("qwen2.5:7b")
    model = build(raw, "bfloat16", tensors_for(raw, 5))
    prompts = [helpers.random_tokens(n, raw["vocab_size"], 70 + i) for i, n in enumerate([90, 17, 40])]
    params = GenerationParams(max_tokens=20, seed=3)
    fast = generate(Engine(model, max_tokens=1024), prompts, params)
    eng = Engine(model, max_tokens=1024, use_graphs=False)
    sampler = Sampler(params, [0, 1, 2], model.device)
    slots = [eng.open() for _ in prompts]
    toks = sampler.sample(eng.step([(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)]), [0, 1, 2])
    slow = [[t] for t in toks]
    for _ in range(19):
        toks = sampler.sample(eng.step([(s, [t], [0]) for s, t in zip(slots, toks)]), [0, 1, 2])
        for o, t in zip(slow, toks):
            o.append(t)
    assert fast == slow
