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
    tensors = sharpened(tensors_for(raw, 3))
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
    rms, worst = row_errors(outs["bfloat16"], outs["float32"])
    assert rms.max().item() < 0.07 and worst.max().item() < 0.35, (rms.max().item(), worst.max().item())


@pytest.mark.parametrize("shape", ["qwen2.5:32b", "qwen2.5:1.5b"])
def test_a_wrong_kv_head_is_noticed_at_the_large_sizes(shape):
    """What the comparison of bfloat16 with the float32 path at these sizes can see: the same model with the keys and
    values of two kv heads of layer 1 exchanged (in the weights of the bfloat16 run alone, which is what a kernel that
    maps a query head to the wrong kv head would compute) must fail it, in a prompt step and in a decoding step;
    the groups are of 5 (32B) and of 6 heads (1.5B)."""
    raw = two_layer(shape)
    tensors = sharpened(tensors_for(raw, 3))
    d, nkv = raw["head_dim"], raw["num_key_value_heads"]
    swapped = dict(tensors)
    for part in ("k_proj", "v_proj"):
        for kind in ("weight", "bias"):
            name = "model.layers.1.self_attn.%s.%s" % (part, kind)
            t = tensors[name].clone()
            a, b = slice(0, d), slice((nkv - 1) * d, nkv * d)
            t[a], t[b] = tensors[name][b], tensors[name][a]
            swapped[name] = t
    prompts = [helpers.random_tokens(n, raw["vocab_size"], 50 + i) for i, n in enumerate([300, 70])]

    def run(dtype, which):
        eng = Engine(build(raw, dtype, which), max_tokens=1024)
        slots = [eng.open() for _ in prompts]
        a = eng.step([(s, p, [len(p) - 1, len(p) // 2]) for s, p in zip(slots, prompts)])
        b = eng.step([(s, [t], [0]) for s, t in zip(slots, [7, 11])])
        for s in slots:
            eng.close(s)
        del eng
        torch.cuda.empty_cache()
        return torch.cat([a, b]).cpu()

    f32, good, bad = run("float32", tensors), run("bfloat16", tensors), run("bfloat16", swapped)
    rms, worst = row_errors(good, f32)
    assert rms.max().item() < 0.07 and worst.max().item() < 0.35, (rms.max().item(), worst.max().item())
    rms_bad, _ = row_errors(bad, f32)
    assert rms_bad.min().item() > 0.14, rms_bad                   # every row, twice the allowance and more
    print("clean rms", rms.max().item(), "with two kv heads exchanged", rms_bad.min().item())


@pytest.mark.parametrize("shape,n_seqs", [("qwen2.5:7b", 20), ("qwen2.5:32b", 40), ("qwen2.5:7b", 100), ("qwen2.5:7b", 128),
                                          ("qwen2.5:7b", 129), ("qwen2.5:1.5b", 200)])
def test_bfloat16_tracks_float32_in_steps_of_17_and_more_rows_at_large_sizes(shape, n_seqs):
    """The kernels for 17 to 128 rows at the real widths (sums over pieces of K finished by the norm
    and the rotation kernels, the head product with float32 output), and the steps beyond them (129 and
    200 rows: eager, the library's products): a short prompt step of 24 tokens, then two decoding steps
    of n_seqs rows."""
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


@pytest.mark.parametrize("shape", ["qwen2.5:7b", "qwen2.5:1.5b", "qwen2.5:32b"])
def test_float32_path_equals_plain_at_large_sizes(shape):
    raw = two_layer(shape)
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


# ---- the lengths that are benchmarked ---------------------------------------------------------------
def sharpened(tensors):
    """q and k projections doubled, so that attention picks out few keys among thousands and a
    key that is missed or wrongly seen moves the logits."""
    return {k: (v.float() * 2.0).to(v.dtype) if ("q_proj" in k or "k_proj" in k) else v for k, v in tensors.items()}


def plain_rows(tensors, cfg, tokens, rows):
    """The plain implementation's logits at chosen places (the head on all of 2100 places of a
    vocabulary of 152064 would only cost time)."""
    w = {k: v.float().cpu() for k, v in tensors.items()}
    x = w["model.embed_tokens.weight"][torch.as_tensor(tokens)]
    for layer in range(cfg["num_hidden_layers"]):
        x = plain.decoder_layer(x, w, layer, cfg)
    x = plain.rms_norm(x[rows], w["model.norm.weight"], cfg["rms_norm_eps"])
    return plain.linear(x, w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"])


def row_errors(got, want):
    """For every row the rms and the largest difference, in units of the reference's spread."""
    sigma = want.std().item()
    err = (got - want).float()
    return err.pow(2).mean(dim=1).sqrt() / sigma, err.abs().amax(dim=1) / sigma


def test_prompts_of_two_thousand_tokens_and_graphed_decoding_at_7b_sizes():
    """What bench.py times, checked: eight prompts of up to 2111 tokens in one step (33 pages a
    sequence, the prompt kernel's long tile lists), then eight decoding steps of the batch through
    captured graphs (page tables padded to 40, eight and more partitions per sequence).

    Three runs: float32; bfloat16; bfloat16 with the plain attention kernel in place of the two
    matrix-core attention kernels.  The float32 run equals the plain implementation (longest
    sequence, prompt places and decoded ones).  The two bfloat16 runs differ by the rounding of
    the probabilities alone, so they agree far more closely than bfloat16 and float32 do (whose
    difference at these sizes is rounding noise of 2 to 4 % of the logits' spread in every row):
    close enough that one foreign page among a sequence's 33 shows, which the last part asserts."""
    from tq_kv_amd import POLICY
    raw = two_layer("qwen2.5:7b")
    tensors = sharpened(tensors_for(raw, 6))
    lens = [2100, 1990, 2048, 1500, 2111, 64, 1, 700]
    prompts = [helpers.random_tokens(n, raw["vocab_size"], 150 + i) for i, n in enumerate(lens)]
    tails = [helpers.random_tokens(8, raw["vocab_size"], 170 + i) for i in range(len(lens))]
    wants = [sorted({0, n // 2, n - 1}) for n in lens]
    n_first = sum(len(w) for w in wants)

    def run(dtype, spoil=False):
        eng = Engine(build(raw, dtype, tensors), max_tokens=len(lens) * 2240)        # (the tensors of the seed at hand)
        slots = [eng.open() for _ in prompts]
        got = [eng.step([(s, p, w) for s, p, w in zip(slots, prompts, wants)])]
        if spoil:          # sequence 0's page 10 (positions 640..703) becomes sequence 2's, in every layer
            g = eng.cache.kv_groups[0]
            a, b = g.pages[slots[0]][10], g.pages[slots[2]][10]
            g.keys[:, a], g.values[:, a] = g.keys[:, b].clone(), g.values[:, b].clone()
        for step in range(8):
            got.append(eng.step([(s, [t[step]], [0]) for s, t in zip(slots, tails)]))
        n_graphs = len(eng.graphs)
        for s in slots:
            eng.close(s)
        del eng
        torch.cuda.empty_cache()
        return torch.cat(got).cpu(), n_graphs

    f32, _ = run("float32")
    bf16, n_graphs = run("bfloat16")
    assert n_graphs >= 1                                   # the one-token steps went through captured graphs
    old = dict(POLICY.items())
    POLICY.update(decode_mfma=False, prefill_mfma=False)
    try:
        bf16_plain_kernel, _ = run("bfloat16")
    finally:
        POLICY.update(old)
    rms, worst = row_errors(bf16, f32)
    assert rms.max().item() < 0.07 and worst.max().item() < 0.35, (rms.max().item(), worst.max().item())
    rms, worst = row_errors(bf16, bf16_plain_kernel)
    assert rms.max().item() < 0.02 and worst.max().item() < 0.1, (rms.max().item(), worst.max().item())
    # the float32 path itself, for the first sequence: its three prompt places and its eight decoded ones
    seq = prompts[0] + tails[0]
    rows = wants[0] + [lens[0] + i for i in range(8)]
    want = plain_rows(tensors, dict(raw), seq, rows)
    got = torch.cat([f32[:len(wants[0])]] + [f32[n_first + len(lens) * i][None] for i in range(8)])
    torch.testing.assert_close(got, want, atol=2e-5 * max(1.0, want.abs().max().item()), rtol=2e-5)
    # a foreign page is noticed, in the sequence it belongs to and nowhere else; on three sets of weights, so that the
    # distance between a clean run (under 0.02 of the spread) and a spoiled one (over 0.03) is known to hold
    decoded_0 = [n_first + len(lens) * i for i in range(8)]
    for seed in (6, 16, 26):
        if seed != 6:
            tensors = sharpened(tensors_for(raw, seed))
            POLICY.update(decode_mfma=False, prefill_mfma=False)
            try:
                bf16_plain_kernel, _ = run("bfloat16")
            finally:
                POLICY.update(old)
            clean, _ = run("bfloat16")
            rms, worst = row_errors(clean, bf16_plain_kernel)
            assert rms.max().item() < 0.02 and worst.max().item() < 0.1, (seed, rms.max().item(), worst.max().item())
        spoiled, _ = run("bfloat16", spoil=True)
        rms, _ = row_errors(spoiled, bf16_plain_kernel)
        others = [r for r in range(spoiled.shape[0]) if r not in decoded_0]
        assert rms[decoded_0].min().item() > 0.03, (seed, rms[decoded_0])
        assert rms[others].max().item() < 0.02, (seed, rms[others].max())
        print("seed", seed, "rms of the spoiled sequence's rows", rms[decoded_0], "largest of the others", rms[others].max())


def test_a_step_of_more_than_three_thousand_tokens_takes_the_wide_tiles():
    """A step of 3300 tokens (one prompt of 3200 and one of 100) runs the prompt kernel with
    tiles of 128 queries; 1.5B sizes (12 heads in groups of 6), bfloat16 against the float32 path."""
    raw = two_layer("qwen2.5:1.5b")
    tensors = sharpened(tensors_for(raw, 7))
    prompts = [helpers.random_tokens(n, raw["vocab_size"], 190 + i) for i, n in enumerate([3200, 100])]
    wants = [[0, 1599, 3199], [0, 99]]
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine(build(raw, dtype, tensors), max_tokens=3328 + 128)
        slots = [eng.open() for _ in prompts]
        a = eng.step([(s, p, w) for s, p, w in zip(slots, prompts, wants)])
        b = eng.step([(s, [5], [0]) for s in slots])
        outs[dtype] = torch.cat([a, b]).cpu()
        for s in slots:
            eng.close(s)
        del eng
        torch.cuda.empty_cache()
    rms, worst = row_errors(outs["bfloat16"], outs["float32"])
    assert rms.max().item() < 0.07 and worst.max().item() < 0.35, (rms.max().item(), worst.max().item())
    want = plain_rows(tensors, dict(raw), prompts[1] + [5], [0, 99, 100])
    got = torch.cat([outs["float32"][3:5], outs["float32"][6:7]])
    torch.testing.assert_close(got, want, atol=2e-5 * max(1.0, want.abs().max().item()), rtol=2e-5)


@pytest.mark.parametrize("shape", ["qwen2.5:7b", "qwen2.5:1.5b"])
def test_a_model_without_weight_rows_gives_the_same_results(shape):
    """POLICY["keep_rows"] off: the rows of packed weights are given back, and a product of more than
    128 rows (a prompt) gets them back from the packed copy for its own length and goes to the library
    as it would have.  So every step is equal bit for bit either way; the prompt of 300 tokens is also
    compared with the plain implementation as the other bfloat16 runs here are."""
    from tq_kv_amd import POLICY
    raw = two_layer(shape)
    tensors = sharpened(tensors_for(raw, 6))
    prompts = [helpers.random_tokens(n, raw["vocab_size"], 70 + i) for i, n in enumerate([300, 100, 20])]
    outs, held = {}, {}
    for keep in (True, False):
        torch.cuda.empty_cache()
        torch.cuda.synchronize()
        before = torch.cuda.mem_get_info()[0]         # the model's memory is the engine library's, not torch's
        old = POLICY["keep_rows"]
        POLICY["keep_rows"] = keep
        try:
            model = build(raw, "bfloat16", tensors)
        finally:
            POLICY["keep_rows"] = old
        torch.cuda.synchronize()
        held[keep] = before - torch.cuda.mem_get_info()[0]
        for name in ("self_attn.qkv.weight", "self_attn.o_proj.weight", "mlp.gate_up.weight", "mlp.down_proj.weight"):
            assert model.holds("model.layers.0." + name) == keep and model.holds("model.layers.0." + name + ".packed")
        if not raw.get("tie_word_embeddings"):
            assert model.holds("lm_head.weight") == keep
        assert model.holds("model.embed_tokens.weight") and model.holds("head.packed")
        eng = Engine(model, max_tokens=1024)
        slots = [eng.open() for _ in prompts]
        got = [eng.step([(slots[0], prompts[0], [0, 127, 128, 299])]),
               eng.step([(slots[1], prompts[1], [0, 99]), (slots[2], prompts[2], [19])]),
               eng.step([(s, [5 + i], [0]) for i, s in enumerate(slots)])]
        outs[keep] = [g.cpu() for g in got]
        for s in slots:
            eng.close(s)
        del eng, model
    for a, b in zip(outs[True], outs[False]):
        assert torch.equal(a, b)
    want = plain_rows(tensors, raw, prompts[0], [0, 127, 128, 299])
    for keep in (True, False):
        rms, worst = row_errors(outs[keep][0], want)
        assert rms.max().item() < 0.07 and worst.max().item() < 0.35, (keep, rms, worst)
    # what is given back: the rows of every packed weight (all the products' weights, and an untied head)
    rows = sum(v.numel() * 2 for k, v in tensors.items()
               if k.endswith("_proj.weight") or k == "lm_head.weight")
    assert abs((held[True] - held[False]) - rows) < 0.05 * rows + (8 << 20), (held, rows)
