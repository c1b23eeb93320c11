"""Shared by the GPU tests: model folders, engines and plain logits, each made once."""
import os
import tempfile

import torch
from safetensors.torch import load_file, save_file

import helpers
import plain_qwen2 as plain

_TMP = None
_FOLDERS = {}
_PLAIN = {}
_ENGINES = {}

# Largest allowed |engine - plain|.  The float32 path differs from the plain implementation
# only by the order of float32 additions.  The bfloat16 path rounds activations at every
# kernel boundary; its allowance is tied to the logits' own spread (their standard deviation,
# 0.16 to 0.25 for the tiny models): measured, a clean run stays below 0.06 of it on every
# configuration, while one cache page taken from another sequence moves the logits by 0.17 of
# it or more (test_a_foreign_page_in_the_cache_is_noticed asserts that such a fault fails).
TOL = {"float32": dict(atol=2e-5, rtol=2e-5), "bfloat16": dict(atol=3e-2, rtol=3e-2)}
BF16_SPREAD = 0.1        # bfloat16: atol = BF16_SPREAD * std(reference), rtol = BF16_RTOL
BF16_RTOL = 0.02


def tmp():
    global _TMP
    if _TMP is None:
        _TMP = tempfile.mkdtemp(prefix="tqkv_tests_")
    return _TMP


def folder(name, sharp=False):
    """Model folder of tiny configuration `name`.  sharp: the q and k projections are
    scaled up so that attention picks out single keys instead of averaging: a key that
    is wrongly seen, missed or read from the wrong place then changes the logits a lot.
    (Measured: with these factors one changed early token moves late logits by 0.1 to 0.2,
    several times the bfloat16 tolerance, while bfloat16 rounding itself stays near 0.01;
    larger factors let rounding alone grow past the tolerance.)"""
    key = (name, sharp)
    if key not in _FOLDERS:
        cfg, seed = helpers.CONFIGS[name]
        base = helpers.make_folder(os.path.join(tmp(), name), cfg, seed)
        if sharp:
            t = load_file(os.path.join(base, "model.safetensors"))
            for k in list(t):
                if "q_proj" in k or "k_proj" in k:
                    t[k] = (t[k].float() * 6.0).to(t[k].dtype)
                if "v_proj.weight" in k or "o_proj" in k:
                    t[k] = (t[k].float() * 2.0).to(t[k].dtype)
            out = os.path.join(tmp(), name + "_sharp")
            os.makedirs(out, exist_ok=True)
            save_file(t, os.path.join(out, "model.safetensors"))
            with open(os.path.join(base, "config.json")) as f, open(os.path.join(out, "config.json"), "w") as g:
                g.write(f.read())
            base = out
        _FOLDERS[key] = base
    return _FOLDERS[key]


def plain_model(name, sharp=False):
    key = (name, sharp)
    if key not in _PLAIN:
        _PLAIN[key] = helpers.read_folder(folder(name, sharp))
    return _PLAIN[key]


def plain_logits(name, tokens, sharp=False):
    cfg, w = plain_model(name, sharp)
    return plain.forward(w, cfg, tokens)


def engine(name, dtype, sharp=False, max_tokens=8192):
    from tq_kv_amd import Engine, Model
    key = (name, dtype, sharp, max_tokens)
    if key not in _ENGINES:
        _ENGINES[key] = Engine(Model.from_dir(folder(name, sharp), dtype=dtype), max_tokens=max_tokens)
    return _ENGINES[key]


def prompts(name, lens, seed=100):
    vocab = helpers.CONFIGS[name][0]["vocab_size"]
    return [helpers.random_tokens(n, vocab, seed + i) for i, n in enumerate(lens)]


def close(a, b, dtype, what=""):
    """a: the engine's logits, b: the reference's."""
    a, b = a.cpu().float(), b.cpu().float()
    tol = TOL[dtype]
    if dtype == "bfloat16" and b.numel() > 1:
        tol = dict(atol=BF16_SPREAD * b.std().item(), rtol=BF16_RTOL)
    torch.testing.assert_close(a, b, msg=lambda m: "%s: %s" % (what, m), **tol)


def poison_free_pages(eng):
    """Fill every page no sequence holds with NaN: nothing may read them."""
    for g in eng.cache.kv_groups:
        held = {p for pages in g.pages.values() for p in pages if p >= 0}
        free = [p for p in range(g.pool.n) if p not in held]
        if free:
            idx = torch.tensor(free, device=g.keys.device)
            g.keys[:, idx] = float("nan")
            g.values[:, idx] = float("nan")
