"""Each part alone against its plain counterpart, and the generality of the
arrangement: a run order that names a layer twice, a run that reads another run's
cache, a norm after the mixer, and toy parts that are defined here, registered, built
and stepped without a change to the framework: a mixer with state of its own, a
feed-forward with routing, a position encoding of its own."""
import pytest
import torch

import gpu_common as G
import helpers
import plain_qwen2 as plain
from tq_kv_amd import Engine, Model
from tq_kv_amd.cache import Cache
from tq_kv_amd.engine.context import StepContext
from tq_kv_amd.parts import (BuildEnv, KVNeed, LayerSpec, ModelSpec, Part, PartSpec, Run, StateNeed, TensorSpec,
                             register)
from tq_kv_amd.weights import random_tensors

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=1e-5, rtol=1e-5), "bfloat16": dict(atol=2e-2, rtol=2e-2)}


def load_random(part, dtype, seed, std=0.1):
    specs = {n: TensorSpec(s.shape, s.init, std if s.init == "normal" else 0.1) for n, s in part.tensors().items()}
    t = random_tensors(specs, seed, DT[dtype], "cpu")
    part.load({k: v.to(DEV) for k, v in t.items()})
    return {k: v.float() for k, v in t.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rms_norm_part(dtype):
    env = BuildEnv(DEV, DT[dtype])
    norm = env.build("norm", PartSpec("rms_norm", {"size": 200, "eps": 1e-4}))
    w = load_random(norm, dtype, 1)
    h = torch.randn(5, 200, device=DEV)
    d = torch.randn(5, 200, device=DEV).to(DT[dtype])
    want_h = h + d.float()
    got = norm.add_norm(h, d)
    assert torch.equal(h, want_h) and got.dtype == DT[dtype]
    torch.testing.assert_close(got.float().cpu(), plain.rms_norm(want_h.cpu(), w["weight"], 1e-4), **TOL[dtype])
    torch.testing.assert_close(norm.forward(d).float().cpu(), plain.rms_norm(d.float().cpu(), w["weight"], 1e-4), **TOL[dtype])
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    got = norm.gather_add_norm(h, d, rows)
    torch.testing.assert_close(got.float().cpu(), plain.rms_norm((want_h + d.float()).cpu()[[4, 1]], w["weight"], 1e-4), **TOL[dtype])


def test_rotary_part_tables():
    env = BuildEnv(DEV, torch.float32)
    rot = env.build("position", PartSpec("rotary", {"theta": 1e6, "rot_dim": 48, "max_positions": 300, "style": "halves"}))
    cos, sin, rot_dim, _ = rot.tables()
    c, s = plain.rope_tables(48, 1e6, 300)
    # the engine takes the float32 power, cosine and sine from the C library (as the reference's Rust does), the plain
    # implementation from torch: where the two round theta_j differently by one unit in the last place, the angle at
    # position p differs by p * 6e-8 * theta_j, which is all that this allowance covers (a wrong base, pairing or
    # position would be off by far more)
    assert rot_dim == 48 and cos.shape == c.shape
    torch.testing.assert_close(cos.cpu(), c, atol=300 * 6e-8 + 2e-7, rtol=0)
    torch.testing.assert_close(sin.cpu(), s, atol=300 * 6e-8 + 2e-7, rtol=0)
    assert torch.equal(cos[0].cpu(), torch.ones(24)) and torch.equal(sin[0].cpu(), torch.zeros(24))
    torch.testing.assert_close(cos[:, 0].cpu(), c[:, 0], atol=2e-7, rtol=0)         # theta_0 = 1: the angle is the position itself
    with pytest.raises(ValueError):
        env.build("position", PartSpec("rotary", {"theta": 1e4, "rot_dim": 7, "max_positions": 8}))


def step_ctx(cache, items):
    """items: [(slot, tokens)]; reserves, builds the context; the caller commits."""
    sizes = [(s, len(t)) for s, t in items]
    cache.reserve(sizes)
    ctx = StepContext([(s, cache.length(s), t) for s, t in items], [[] for _ in items], cache, DEV)
    return ctx, sizes


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,d,window", [(6, 2, 48, None), (3, 1, 32, 20), (4, 4, 16, 70)])
def test_attention_part(dtype, nh, nkv, d, window):
    hidden = 88
    env = BuildEnv(DEV, DT[dtype])
    pos = PartSpec("rotary", {"theta": 1e4, "rot_dim": d, "max_positions": 256, "style": "halves"})
    att = env.build("mixer", PartSpec("attention", {"hidden": hidden, "n_heads": nh, "n_kv_heads": nkv, "head_dim": d,
                                                    "qkv_bias": True, "window": window, "position": pos}))
    assert att.cache_need() == KVNeed(nkv, d, window)
    w = load_random(att, dtype, 2)
    cfg = {"num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": d, "rope_theta": 1e4}
    cache = Cache([att.cache_need()], [None], 64 * 16, 4, DT[dtype], DEV)
    xs = [torch.randn(n, hidden).to(DT[dtype]) for n in (150, 40)]     # outputs of size about 1
    slots = [cache.acquire(), cache.acquire()]
    # sequence 0 in two chunks and then single tokens, sequence 1 whole, in shared steps
    plan = [[(0, 0, 100), (1, 0, 40)], [(0, 100, 140)]] + [[(0, t, t + 1)] for t in range(140, 150)]
    got = [[], []]
    for step in plan:
        ctx, sizes = step_ctx(cache, [(slots[i], [0] * (b - a)) for i, a, b in step])
        x = torch.cat([xs[i][a:b] for i, a, b in step]).to(DEV)
        y = att.forward(x, ctx, cache.entry(0))
        cache.commit(sizes)
        off = 0
        for i, a, b in step:
            got[i].append(y[off:off + b - a])
            off += b - a
    for i in range(2):
        want = plain.attention(xs[i].float(), w, "", cfg, window)
        torch.testing.assert_close(torch.cat(got[i]).float().cpu(), want, **TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_part(dtype):
    env = BuildEnv(DEV, DT[dtype])
    ff = env.build("feed_forward", PartSpec("gated_silu", {"hidden": 72, "inter": 200}))
    w = load_random(ff, dtype, 3)
    x = torch.randn(9, 72).to(DT[dtype])
    torch.testing.assert_close(ff.forward(x.to(DEV), None).float().cpu(), plain.swiglu_mlp(x.float(), w, ""), **TOL[dtype])


def tiny_spec(cfg, order=None, post_norms=False, mixers=None, ffs=None, position=None):
    """A ModelSpec put together by hand from the parts (what an architecture file does)."""
    h, d = cfg["hidden_size"], cfg["head_dim"]
    norm = PartSpec("rms_norm", {"size": h, "eps": cfg["rms_norm_eps"]})
    pos = position or PartSpec("rotary", {"theta": cfg["rope_theta"], "rot_dim": d,
                                          "max_positions": cfg["max_position_embeddings"], "style": "halves"})
    layers = []
    for l in range(cfg["num_hidden_layers"]):
        mixer = (mixers or {}).get(l) or PartSpec("attention", {
            "hidden": h, "n_heads": cfg["num_attention_heads"], "n_kv_heads": cfg["num_key_value_heads"], "head_dim": d,
            "qkv_bias": True, "window": plain.layer_window(cfg, l), "position": pos})
        names = {"mixer": "self_attn.", "feed_forward": "mlp.", "mixer_norm": "input_layernorm.",
                 "ff_norm": "post_attention_layernorm."}
        ff = (ffs or {}).get(l) or PartSpec("gated_silu", {"hidden": h, "inter": cfg["intermediate_size"]})
        params = {"mixer": mixer, "feed_forward": ff, "mixer_norm": norm, "ff_norm": norm, "names": names}
        if post_norms:
            params.update({"post_mixer_norm": norm, "post_ff_norm": norm})
            names.update({"post_mixer_norm": "post_mixer_norm.", "post_ff_norm": "post_ff_norm."})
        layers.append(LayerSpec("model.layers.%d." % l, PartSpec("pre_norm", params)))
    return ModelSpec(architecture="test", vocab_size=cfg["vocab_size"], hidden_size=h,
                     max_positions=cfg["max_position_embeddings"], embedding_name="model.embed_tokens.weight",
                     layers=layers, order=order or [Run(l) for l in range(len(layers))], final_norm=norm,
                     final_norm_prefix="model.norm.", head_name="lm_head.weight")


def run_all(model, prompt, cut):
    eng = Engine(model, max_tokens=1024)
    s = eng.open()
    outs = [eng.step([(s, prompt[:cut], list(range(cut)))])]
    for t in range(cut, len(prompt)):
        outs.append(eng.step([(s, [prompt[t]], [0])]))
    eng.close(s)
    eng.cache.check()
    return torch.cat(outs).cpu()


def test_block_is_the_plain_decoder_layer_and_a_layer_may_run_twice():
    cfg = dict(helpers.TINY_B)
    _, w = G.plain_model("B", True)
    prompt = helpers.random_tokens(40, cfg["vocab_size"], 1)
    # order 0, 1, 2, 1: layer 1 runs twice, each run with a cache of its own
    model = Model(tiny_spec(cfg, order=[Run(0), Run(1), Run(2), Run(1)]), "float32", DEV)
    assert len(model.needs) == 4
    model.load({k: v.to(DEV) for k, v in w.items()})
    # the same thing for the plain implementation: a four-layer model whose layer 3 is layer 1
    # (both windowed, as l >= max_window_layers)
    w4 = dict(w)
    for k, v in w.items():
        if k.startswith("model.layers.1."):
            w4[k.replace("layers.1.", "layers.3.")] = v
    want = plain.forward(w4, dict(cfg, num_hidden_layers=4), prompt)
    torch.testing.assert_close(run_all(model, prompt, 25), want, atol=2e-5, rtol=2e-5)


def test_a_run_reads_another_runs_cache():
    cfg = dict(helpers.TINY_A)
    _, w = G.plain_model("A", True)
    prompt = helpers.random_tokens(30, cfg["vocab_size"], 2)
    model = Model(tiny_spec(cfg, order=[Run(0), Run(1, cache_of=0)]), "float32", DEV)
    model.load({k: v.to(DEV) for k, v in w.items() if k != "lm_head.weight"} | {"lm_head.weight": w["model.embed_tokens.weight"].to(DEV)})
    assert len(model.needs) == 2 and Engine(model, max_tokens=256).cache.kv_groups[0].runs == [0]
    # plain: layer 1 attends with its own queries over layer 0's rotated keys and values
    nh, nkv, d, eps = 4, 2, 16, cfg["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][prompt]
    t = len(prompt)
    cos, sin = plain.rope_tables(d, cfg["rope_theta"], t)
    p0, p1 = "model.layers.0.", "model.layers.1."
    h = plain.rms_norm(x, w[p0 + "input_layernorm.weight"], eps)
    k0 = plain.rope_half(plain.linear(h, w[p0 + "self_attn.k_proj.weight"], w[p0 + "self_attn.k_proj.bias"]).reshape(t, nkv, d).transpose(0, 1), cos, sin)
    v0 = plain.linear(h, w[p0 + "self_attn.v_proj.weight"], w[p0 + "self_attn.v_proj.bias"]).reshape(t, nkv, d).transpose(0, 1)
    x = plain.decoder_layer(x, w, 0, cfg)
    h = plain.rms_norm(x, w[p1 + "input_layernorm.weight"], eps)
    q1 = plain.rope_half(plain.linear(h, w[p1 + "self_attn.q_proj.weight"], w[p1 + "self_attn.q_proj.bias"]).reshape(t, nh, d).transpose(0, 1), cos, sin)
    y = plain.attention_core(q1, k0, v0, plain.visibility(t)).transpose(0, 1).reshape(t, nh * d)
    x = x + plain.linear(y, w[p1 + "self_attn.o_proj.weight"])
    x = x + plain.swiglu_mlp(plain.rms_norm(x, w[p1 + "post_attention_layernorm.weight"], eps), w, p1 + "mlp.")
    want = plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["model.embed_tokens.weight"])
    torch.testing.assert_close(run_all(model, prompt, 17), want, atol=2e-5, rtol=2e-5)


def test_norms_after_mixer_and_feed_forward():
    # the optional norms of src/models/turbo_generic.rs:1965-1968, 1976-1979
    cfg = dict(helpers.TINY_A, num_hidden_layers=1)
    model = Model(tiny_spec(cfg, post_norms=True), "float32", DEV)
    specs = {n: TensorSpec(s.shape, s.init, 0.2 if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    w = random_tensors(specs, 5, torch.float32, "cpu")
    model.load({k: v.to(DEV) for k, v in w.items()})
    prompt = helpers.random_tokens(12, cfg["vocab_size"], 3)
    p, eps = "model.layers.0.", cfg["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][prompt]
    a = plain.attention(plain.rms_norm(x, w[p + "input_layernorm.weight"], eps), w, p + "self_attn.", cfg, None)
    x = x + plain.rms_norm(a, w[p + "post_mixer_norm.weight"], eps)
    f = plain.swiglu_mlp(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p + "mlp.")
    x = x + plain.rms_norm(f, w[p + "post_ff_norm.weight"], eps)
    want = plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])
    torch.testing.assert_close(run_all(model, prompt, 7), want, atol=2e-5, rtol=2e-5)


# ---- a toy mixer with state of its own -------------------------------------------------------
@register("mixer", "toy_decay")
class ToyDecay(Part):
    """y_t = W s_t with s_t = decay * s_{t-1} + x_t: a recurrence with a fixed-size state per
    sequence, kept in the cache's state rows.  Plain torch on the device; it exists to show
    that the framework's interfaces carry a mixer that is not attention."""

    def __init__(self, params, env):
        self.hidden, self.decay = params["hidden"], params["decay"]

    def tensors(self):
        return {"mix.weight": TensorSpec((self.hidden, self.hidden))}

    def load(self, tensors):
        self.w = tensors["mix.weight"]

    def cache_need(self):
        return StateNeed((self.hidden,))

    def forward(self, x, ctx, entry):
        out = torch.empty_like(x)
        for b in range(ctx.n_seqs):
            a, e = int(ctx.host.cu[b]), int(ctx.host.cu[b + 1])
            s = entry.state[int(ctx.host.seq_slot[b])]
            # all states of the piece at once: s_t = decay^(t+1) s_before + sum_j decay^(t-j) x_j
            t = torch.arange(e - a, device=x.device, dtype=torch.float32)
            powers = torch.tril(self.decay ** (t[:, None] - t[None, :]).clamp(min=0))
            states = powers @ x[a:e].float() + (self.decay ** (t + 1))[:, None] * s[None, :]
            out[a:e] = (states @ self.w.float().t()).to(x.dtype)
            s.copy_(states[-1])
        return out


def test_toy_mixer_with_state_is_registered_built_and_stepped():
    cfg = dict(helpers.TINY_A, num_hidden_layers=3)
    toy = PartSpec("toy_decay", {"hidden": cfg["hidden_size"], "decay": 0.5})
    model = Model(tiny_spec(cfg, mixers={1: toy}), "float32", DEV)       # attention, toy, attention
    assert model.needs[1] == StateNeed((64,)) and isinstance(model.needs[0], KVNeed)
    assert "model.layers.1.self_attn.mix.weight" in model.tensor_specs()
    specs = {n: TensorSpec(s.shape, s.init, 0.2 if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    w = random_tensors(specs, 6, torch.float32, "cpu")
    model.load({k: v.to(DEV) for k, v in w.items()})
    eng = Engine(model, max_tokens=1024)
    assert len(eng.cache.state_groups) == 1 and len(eng.cache.kv_groups) == 1

    def plain_forward(tokens):
        x = w["model.embed_tokens.weight"][tokens]
        eps = cfg["rms_norm_eps"]
        for l in range(3):
            p = "model.layers.%d." % l
            h = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
            if l == 1:
                s, ys = torch.zeros(64), []
                for t in range(len(tokens)):
                    s = 0.5 * s + h[t]
                    ys.append(w[p + "self_attn.mix.weight"] @ s)
                x = x + torch.stack(ys)
            else:
                x = x + plain.attention(h, w, p + "self_attn.", cfg, None)
            x = x + plain.swiglu_mlp(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p + "mlp.")
        return plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])

    a, b = helpers.random_tokens(20, 256, 4), helpers.random_tokens(9, 256, 5)
    for round_ in range(2):                      # twice: the second time on used slots, whose state must be zero again
        sa, sb = eng.open(), eng.open()
        out = eng.step([(sa, a[:12], list(range(12))), (sb, b[:4], list(range(4)))])
        got_a, got_b = [out[:12]], [out[12:]]
        for t in range(5):
            out = eng.step([(sa, [a[12 + t]], [0]), (sb, [b[4 + t]], [0])])
            got_a.append(out[:1]), got_b.append(out[1:])
        eng.close(sb)
        for t in range(17, 20):
            got_a.append(eng.step([(sa, [a[t]], [0])]))
        eng.close(sa)
        torch.testing.assert_close(torch.cat(got_a).cpu(), plain_forward(a), atol=2e-5, rtol=2e-5)
        torch.testing.assert_close(torch.cat(got_b).cpu(), plain_forward(b), atol=2e-5, rtol=2e-5)
    eng.cache.check()


@register("mixer", "toy_half_values")
class ToyHalfValues(Part):
    """Causal softmax attention of one head whose values are half as wide as its keys, kept in pages of its own layout
    (keys [page, width], values [page, width / 2], positions in order): the need names the two page shapes and the cache
    multiplies them out; the mixer writes and reads its pages itself through the step's page table.  No position
    encoding, no window."""

    def __init__(self, params, env):
        self.hidden, self.width = params["hidden"], params["width"]

    def tensors(self):
        h, w = self.hidden, self.width
        return {"q.weight": TensorSpec((w, h)), "k.weight": TensorSpec((w, h)), "v.weight": TensorSpec((w // 2, h)),
                "o.weight": TensorSpec((h, w // 2))}

    def load(self, tensors):
        self.w = {k: v.float() for k, v in tensors.items()}

    def cache_need(self):
        from tq_kv_amd.cache import PAGE
        return KVNeed(key_page=(PAGE, self.width), value_page=(PAGE, self.width // 2))

    def forward(self, x, ctx, entry):
        from tq_kv_amd.cache import PAGE
        xf = x.float()
        q, k, v = (xf @ self.w[n + ".weight"].t() for n in "qkv")
        table = ctx.page_table(entry.group)
        out = torch.empty_like(xf)
        for b in range(ctx.n_seqs):
            a, e, start = int(ctx.host.cu[b]), int(ctx.host.cu[b + 1]), int(ctx.host.seq_start[b])
            pos = torch.arange(start, start + e - a, device=x.device)
            pages = table[b].long()[pos // PAGE]
            assert (pages >= 0).all()
            entry.keys[pages, pos % PAGE] = k[a:e].to(entry.keys.dtype)
            entry.values[pages, pos % PAGE] = v[a:e].to(entry.values.dtype)
            past = torch.arange(start + e - a, device=x.device)
            keys = entry.keys[table[b].long()[past // PAGE], past % PAGE].float()
            values = entry.values[table[b].long()[past // PAGE], past % PAGE].float()
            scores = (q[a:e] @ keys.t()) / self.width ** 0.5
            scores = scores.masked_fill(past[None, :] > pos[:, None], float("-inf"))
            out[a:e] = (torch.softmax(scores, -1) @ values) @ self.w["o.weight"].t()
        return out.to(x.dtype)


def test_a_toy_mixer_whose_values_are_half_as_wide_as_its_keys_brings_its_own_pages():
    cfg = dict(helpers.TINY_A, num_hidden_layers=3)
    h = cfg["hidden_size"]
    toy = PartSpec("toy_half_values", {"hidden": h, "width": 24})
    model = Model(tiny_spec(cfg, mixers={1: toy}), "float32", DEV)       # attention, toy, attention
    from tq_kv_amd.cache import PAGE
    assert model.needs[1] == KVNeed(key_page=(PAGE, 24), value_page=(PAGE, 12)) and model.needs[0] == KVNeed(2, 16)
    specs = {n: TensorSpec(s.shape, s.init, 0.2 if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    w = random_tensors(specs, 16, torch.float32, "cpu")
    model.load({k: v.to(DEV) for k, v in w.items()})
    eng = Engine(model, max_tokens=1024)
    groups = eng.cache.kv_groups
    assert len(groups) == 2 and groups[0].runs == [0, 2] and groups[1].runs == [1]
    assert tuple(groups[1].keys.shape) == (1, 16, PAGE, 24) and tuple(groups[1].values.shape) == (1, 16, PAGE, 12)

    def plain_forward(tokens):
        x = w["model.embed_tokens.weight"][tokens]
        eps, t = cfg["rms_norm_eps"], len(tokens)
        for l in range(3):
            p = "model.layers.%d." % l
            hn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
            if l == 1:
                q, k, v = (hn @ w[p + "self_attn.%s.weight" % n].t() for n in "qkv")
                scores = (q @ k.t()) / 24 ** 0.5
                scores = scores.masked_fill(~plain.visibility(t), float("-inf"))
                x = x + (torch.softmax(scores, -1) @ v) @ w[p + "self_attn.o.weight"].t()
            else:
                x = x + plain.attention(hn, w, p + "self_attn.", cfg, None)
            x = x + plain.swiglu_mlp(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p + "mlp.")
        return plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])

    a, b = helpers.random_tokens(100, 256, 4), helpers.random_tokens(9, 256, 5)
    for round_ in range(2):                      # the second time on pages that were used before
        sa, sb = eng.open(), eng.open()
        out = eng.step([(sa, a[:70], list(range(70))), (sb, b[:4], list(range(4)))])       # sequence a crosses a page
        got_a, got_b = [out[:70]], [out[70:]]
        for t in range(5):
            out = eng.step([(sa, [a[70 + t]], [0]), (sb, [b[4 + t]], [0])])
            got_a.append(out[:1]), got_b.append(out[1:])
        eng.close(sb)
        got_a.append(eng.step([(sa, a[75:], list(range(25)))]))
        eng.close(sa)
        torch.testing.assert_close(torch.cat(got_a).cpu(), plain_forward(a), atol=2e-5, rtol=2e-5)
        torch.testing.assert_close(torch.cat(got_b).cpu(), plain_forward(b), atol=2e-5, rtol=2e-5)
    eng.cache.check()
    assert all(g.pool.n_held == 0 for g in groups)


@register("feed_forward", "toy_fuse")
class ToyFuse(Part):
    """A feed-forward that fails when told to: y = x otherwise."""
    blow = [False]

    def __init__(self, params, env):
        pass

    def forward(self, x, ctx):
        if self.blow[0]:
            raise RuntimeError("the toy blew")
        return x


def test_a_step_that_fails_in_the_model_leaves_nothing_behind():
    """A part fails in the middle of a step: the caller sees the part's own exception, the sequences keep the lengths they
    had, the pages reserved for the step are free again, and the next step is as if nothing had happened."""
    cfg = dict(helpers.TINY_A)
    model = Model(tiny_spec(cfg, ffs={1: PartSpec("toy_fuse", {})}), "float32", DEV)
    specs = {n: TensorSpec(s.shape, s.init, 0.2 if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    model.load({k: v.to(DEV) for k, v in random_tensors(specs, 17, torch.float32, "cpu").items()})
    eng = Engine(model, max_tokens=1024)
    prompt = helpers.random_tokens(120, 256, 9)
    s = eng.open()
    first = eng.step([(s, prompt[:10], [9])])
    held = [g.pool.n_held for g in eng.cache.kv_groups]
    ToyFuse.blow[0] = True
    try:
        with pytest.raises(RuntimeError, match="the toy blew"):
            eng.step([(s, prompt[10:], [0])])           # would have taken another page
    finally:
        ToyFuse.blow[0] = False
    eng.cache.check()
    assert eng.length(s) == 10 and [g.pool.n_held for g in eng.cache.kv_groups] == held
    again = eng.step([(s, prompt[10:], [109])])
    eng.close(s)
    s2 = eng.open()
    whole = eng.step([(s2, prompt, [9, 119])])
    eng.close(s2)
    torch.testing.assert_close(torch.cat([first, again]).cpu(), whole.cpu(), atol=2e-5, rtol=2e-5)
    eng.cache.check()


# ---- a toy feed-forward with routing ----------------------------------------------------------
@register("feed_forward", "toy_routed")
class ToyRouted(Part):
    """Every token goes to the one expert (a square matrix) whose router score is largest,
    scaled by the softmax weight of that score.  Router scores and softmax in float32."""

    def __init__(self, params, env):
        self.hidden, self.experts = params["hidden"], params["experts"]

    def tensors(self):
        t = {"router.weight": TensorSpec((self.experts, self.hidden))}
        for e in range(self.experts):
            t["experts.%d.weight" % e] = TensorSpec((self.hidden, self.hidden))
        return t

    def load(self, tensors):
        self.router = tensors["router.weight"]
        self.w = [tensors["experts.%d.weight" % e] for e in range(self.experts)]

    def forward(self, x, ctx):
        scores = torch.softmax(x.float() @ self.router.float().t(), -1)
        best = scores.argmax(-1)
        out = torch.zeros_like(x)
        for e in range(self.experts):
            rows = (best == e).nonzero()[:, 0]
            if rows.numel():
                out[rows] = ((x[rows].float() @ self.w[e].float().t()) * scores[rows, e, None]).to(x.dtype)
        return out


# ---- a toy position encoding ------------------------------------------------------------------
@register("position", "toy_ramp")
class ToyRamp(Part):
    """Not a rotation and not relative: q and k of position p are scaled by 1 + slope * p in
    their first half and by 1 - slope * p in their second.  It has `apply`, no tables."""

    def __init__(self, params, env):
        self.slope = params["slope"]
        self.max_positions = params["max_positions"]

    def apply(self, q, k, ctx):
        pos = ctx.dev.tok_pos.to(torch.float32)[:, None, None] * self.slope
        for t in (q, k):
            half = t.shape[-1] // 2
            t[..., :half] = (t[..., :half].float() * (1 + pos)).to(t.dtype)
            t[..., half:] = (t[..., half:].float() * (1 - pos)).to(t.dtype)


def toy_model_and_plain(dtype):
    """Layer 0: attention with the toy position encoding, the model's feed-forward; layer 1: the toy
    mixer with state, the toy routed feed-forward.  Returns model, weights, plain forward."""
    cfg = dict(helpers.TINY_A, num_hidden_layers=2)
    h, nh, nkv, d, eps = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    slope = 0.01
    spec = tiny_spec(cfg, mixers={1: PartSpec("toy_decay", {"hidden": h, "decay": 0.5})},
                     ffs={1: PartSpec("toy_routed", {"hidden": h, "experts": 3})},
                     position=PartSpec("toy_ramp", {"slope": slope, "max_positions": cfg["max_position_embeddings"]}))
    model = Model(spec, dtype, DEV)
    specs = {n: TensorSpec(s.shape, s.init, 0.08 if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    w = random_tensors(specs, 8, DT[dtype], "cpu")
    model.load({k: v.to(DEV) for k, v in w.items()})
    w = {k: v.float() for k, v in w.items()}

    def plain_forward(tokens):
        t = len(tokens)
        x = w["model.embed_tokens.weight"][tokens]
        p = "model.layers.0."
        hn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
        ramp = torch.arange(t, dtype=torch.float32)[None, :, None] * slope
        scale = torch.cat([(1 + ramp).expand(1, t, d // 2), (1 - ramp).expand(1, t, d // 2)], -1)
        q = plain.linear(hn, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]).reshape(t, nh, d).transpose(0, 1) * scale
        k = plain.linear(hn, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"]).reshape(t, nkv, d).transpose(0, 1) * scale
        v = plain.linear(hn, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).reshape(t, nkv, d).transpose(0, 1)
        y = plain.attention_core(q, k, v, plain.visibility(t)).transpose(0, 1).reshape(t, nh * d)
        x = x + plain.linear(y, w[p + "self_attn.o_proj.weight"])
        x = x + plain.swiglu_mlp(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p + "mlp.")
        p = "model.layers.1."
        hn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
        s, ys = torch.zeros(h), []
        for i in range(t):
            s = 0.5 * s + hn[i]
            ys.append(w[p + "self_attn.mix.weight"] @ s)
        x = x + torch.stack(ys)
        hn = plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        scores = torch.softmax(hn @ w[p + "mlp.router.weight"].t(), -1)
        best = scores.argmax(-1)
        x = x + torch.stack([(w[p + "mlp.experts.%d.weight" % int(best[i])] @ hn[i]) * scores[i, best[i]] for i in range(t)])
        return plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])
    return model, w, plain_forward


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_feed_forward_with_routing_and_toy_position_encoding(dtype):
    # in bfloat16 the small decoding steps fold norms and residual sums into the framework's own
    # products; parts that know nothing of that (all the toys) sit between them and get plain tensors
    model, w, plain_forward = toy_model_and_plain(dtype)
    assert not model.graph_safe                      # the toys launch kernels that depend on the step's data
    eng = Engine(model, max_tokens=1024)
    a, b = helpers.random_tokens(24, 256, 6), helpers.random_tokens(11, 256, 7)
    sa, sb = eng.open(), eng.open()
    out = eng.step([(sa, a[:10], list(range(10))), (sb, b[:3], list(range(3)))])
    got_a, got_b = [out[:10]], [out[10:]]
    for t in range(8):
        out = eng.step([(sa, [a[10 + t]], [0]), (sb, [b[3 + t]], [0])])
        got_a.append(out[:1]), got_b.append(out[1:])
    eng.close(sb)
    for t in range(18, 24):
        got_a.append(eng.step([(sa, [a[t]], [0])]))
    eng.close(sa)
    eng.cache.check()
    tol = dict(atol=2e-5, rtol=2e-5) if dtype == "float32" else G.TOL["bfloat16"]
    got_a, got_b, want_a, want_b = torch.cat(got_a).cpu(), torch.cat(got_b).cpu(), plain_forward(a), plain_forward(b)
    if dtype == "bfloat16":
        # a token whose two best router scores are nearly equal may go to the other expert in bfloat16
        close = (got_a - want_a).abs().max(-1).values < tol["atol"]
        assert close.float().mean() > 0.8
        got_a, want_a = got_a[close], want_a[close]
        close = (got_b - want_b).abs().max(-1).values < tol["atol"]
        assert close.float().mean() > 0.8
        got_b, want_b = got_b[close], want_b[close]
    torch.testing.assert_close(got_a, want_a, **tol)
    torch.testing.assert_close(got_b, want_b, **tol)


# ---- a toy norm: none of the folding hooks ---------------------------------------------------
@register("norm", "toy_centered")
class ToyCentered(Part):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * weight: a norm with another formula and without
    `lazy`, `foldable` or `takes_partial_sums`.  The framework's products around it must hand it
    finished tensors whatever the size of the step."""
    graph_safe = True

    def __init__(self, params, env):
        self.size, self.eps, self.env = params["size"], params["eps"], env

    def tensors(self):
        return {"weight": TensorSpec((self.size,), init="one_plus_normal")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def _norm(self, x):
        x = x.float()
        x = x - x.mean(-1, keepdim=True)
        return (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight.float()).to(self.env.act_dtype)

    def forward(self, x):
        return self._norm(x)

    def add_norm(self, h, delta):
        if delta is not None:
            assert isinstance(delta, torch.Tensor)          # never a product's unfinished sums
            h += delta.float()
        return self._norm(h)

    def gather_add_norm(self, h, delta, rows):
        x = h[rows.long()]
        if delta is not None:
            assert isinstance(delta, torch.Tensor)
            x = x + delta[rows.long()].float()
        return self._norm(x)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_between_the_frameworks_products_in_steps_of_every_size(dtype):
    cfg = dict(helpers.TINY_B)
    spec = tiny_spec(cfg)
    toy = PartSpec("toy_centered", {"size": cfg["hidden_size"], "eps": 1e-5})
    for layer in spec.layers:
        layer.block.params["mixer_norm"] = layer.block.params["ff_norm"] = toy
    import dataclasses
    model = Model(dataclasses.replace(spec, final_norm=toy), dtype, DEV)
    # weights small enough that the logits stay near 1: the bfloat16 tolerance is an absolute one (measured at
    # 0.08: logits up to 2.6 and rounding errors up to 0.038 whichever kernels run, the library's included)
    specs = {n: TensorSpec(s.shape, s.init, 0.04 if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    w = random_tensors(specs, 9, DT[dtype], "cpu")
    model.load({k: v.to(DEV) for k, v in w.items()})
    w = {k: v.float() for k, v in w.items()}

    def norm(x, weight):
        x = x - x.mean(-1, keepdim=True)
        return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * weight

    def plain_forward(tokens):
        x = w["model.embed_tokens.weight"][tokens]
        for l in range(cfg["num_hidden_layers"]):
            p = "model.layers.%d." % l
            x = x + plain.attention(norm(x, w[p + "input_layernorm.weight"]), w, p + "self_attn.", cfg, plain.layer_window(cfg, l))
            x = x + plain.swiglu_mlp(norm(x, w[p + "post_attention_layernorm.weight"]), w, p + "mlp.")
        return plain.linear(norm(x, w["model.norm.weight"]), w["lm_head.weight"])

    eng = Engine(model, max_tokens=4096)
    # 24 sequences: a prompt step of 24 x 3 = 72 tokens (the library's products), then steps of 24
    # rows (the products for 17 to 64 rows), then, as sequences end, of 8 rows (the few-row products)
    reqs = [helpers.random_tokens(8 if i < 8 else 6, cfg["vocab_size"], 50 + i) for i in range(24)]
    slots = [eng.open() for _ in reqs]
    got = [[eng_out] for eng_out in eng.step([(s, r[:3], [0, 1, 2]) for s, r in zip(slots, reqs)]).split(3)]
    for t in range(3, 8):
        live = [i for i, r in enumerate(reqs) if t < len(r)]
        out = eng.step([(slots[i], [reqs[i][t]], [0]) for i in live])
        for j, i in enumerate(live):
            got[i].append(out[j:j + 1])
    for s in slots:
        eng.close(s)
    eng.cache.check()
    tol = dict(atol=2e-5, rtol=2e-5) if dtype == "float32" else G.TOL["bfloat16"]
    for i, r in enumerate(reqs):
        torch.testing.assert_close(torch.cat(got[i]).cpu(), plain_forward(r), msg=lambda m: "request %d: %s" % (i, m), **tol)


# ---- what an architecture may do around the blocks -----------------------------------------------
@register("position", "toy_learned")
class ToyLearned(Part):
    """Learned absolute positions: the stream of the token at position p gets row p of a table
    added.  It acts on the stream after the gather (add_to_stream), not on q and k."""
    graph_safe = True

    def __init__(self, params, env):
        self.hidden, self.max_positions = params["hidden"], params["max_positions"]

    def tensors(self):
        return {"weight": TensorSpec((self.max_positions, self.hidden))}

    def load(self, tensors):
        self.table = tensors["weight"].float()

    def add_to_stream(self, h, ctx):
        h += self.table.index_select(0, ctx.dev.tok_pos.long())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_scale_positions_on_the_stream_head_bias_and_logit_scale_and_cap(dtype):
    """The model spec's optional fields, none of which the reference's decoder uses: the stream
    starts as embedding * scale plus a learned position row, the logits get a bias, a scale and
    a soft cap.  Prompt step, then small decoding steps (whose gather would otherwise prepare the
    first norm), through captured graphs."""
    import dataclasses
    cfg = dict(helpers.TINY_A)
    h = cfg["hidden_size"]
    spec = dataclasses.replace(
        tiny_spec(cfg, position=PartSpec("none", {})), embedding_scale=float(h) ** 0.5,
        stream_position=PartSpec("toy_learned", {"hidden": h, "max_positions": cfg["max_position_embeddings"]}),
        stream_position_prefix="model.positions.", head_bias_name="lm_head.bias", logit_scale=0.5, logit_cap=0.75)
    model = Model(spec, dtype, DEV)
    assert {"model.positions.weight", "lm_head.bias"} <= set(model.tensor_specs()) and not model.graph_safe
    std = {"model.positions.weight": 0.5, "lm_head.bias": 1.0, "model.embed_tokens.weight": 0.1}
    specs = {n: TensorSpec(s.shape, s.init, std.get(n, 0.08) if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    w = random_tensors(specs, 12, DT[dtype], "cpu")
    model.load({k: v.to(DEV) for k, v in w.items()})
    bare = Model(dataclasses.replace(spec, stream_position=None), dtype, DEV)
    assert bare.graph_safe
    bare.load({k: v.to(DEV) for k, v in w.items() if k != "model.positions.weight"})
    w = {k: v.float() for k, v in w.items()}
    eps = cfg["rms_norm_eps"]
    with_positions = [True]

    def plain_forward(tokens):
        t = len(tokens)
        x = w["model.embed_tokens.weight"][tokens] * (float(h) ** 0.5)
        if with_positions[0]:
            x = x + w["model.positions.weight"][:t]
        nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
        for l in range(cfg["num_hidden_layers"]):
            p = "model.layers.%d." % l
            hn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
            q, k, v = (plain.linear(hn, w[p + "self_attn.%s_proj.weight" % n], w[p + "self_attn.%s_proj.bias" % n])
                       .reshape(t, heads, d).transpose(0, 1) for n, heads in (("q", nh), ("k", nkv), ("v", nkv)))
            y = plain.attention_core(q, k, v, plain.visibility(t)).transpose(0, 1).reshape(t, nh * d)     # no rotation
            x = x + plain.linear(y, w[p + "self_attn.o_proj.weight"])
            x = x + plain.swiglu_mlp(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p + "mlp.")
        logits = (plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"]) + w["lm_head.bias"]) * 0.5
        return 0.75 * torch.tanh(logits / 0.75)

    a, b = helpers.random_tokens(30, 256, 14), helpers.random_tokens(12, 256, 15)
    for round_ in range(4):                               # with positions twice, then without twice: the last round replays the graphs of the third
        with_positions[0] = round_ < 2
        if round_ in (0, 2):
            eng = Engine(model if with_positions[0] else bare, max_tokens=1024)
        sa, sb = eng.open(), eng.open()
        out = eng.step([(sa, a[:20], list(range(20))), (sb, b[:5], list(range(5)))])
        got_a, got_b = [out[:20]], [out[20:]]
        for t in range(7):
            out = eng.step([(sa, [a[20 + t]], [0]), (sb, [b[5 + t]], [0])])
            got_a.append(out[:1].clone()), got_b.append(out[1:].clone())
        eng.close(sb)
        for t in range(27, 30):
            got_a.append(eng.step([(sa, [a[t]], [0])]))
        eng.close(sa)
        want_a, want_b = plain_forward(a), plain_forward(b)
        assert want_a.abs().max() > 0.55 and want_a.abs().max() < 0.75         # the cap bites, and holds
        tol = dict(atol=2e-5, rtol=2e-5) if dtype == "float32" else dict(atol=0.1 * want_a.std().item(), rtol=0.02)
        torch.testing.assert_close(torch.cat(got_a).cpu(), want_a, **tol)
        torch.testing.assert_close(torch.cat(got_b).cpu(), want_b, **tol)
        assert (len(eng.graphs) >= 1) == (round_ >= 2)
    with pytest.raises(ValueError, match="cannot act on the stream"):
        Model(dataclasses.replace(spec, stream_position=PartSpec("none", {})), dtype, DEV)


def test_a_model_of_state_alone_is_not_bounded_by_cache_positions():
    """Every run keeps a fixed-size state and none keeps keys: the cache holds no pages, so
    max_tokens bounds nothing and the generation loop plans by slots alone.  300 requests of 500
    tokens through an engine made with max_tokens=64."""
    from tq_kv_amd import GenerationParams, generate
    cfg = dict(helpers.TINY_A, num_hidden_layers=2, max_position_embeddings=600)
    toy = PartSpec("toy_decay", {"hidden": cfg["hidden_size"], "decay": 0.5})
    model = Model(tiny_spec(cfg, mixers={0: toy, 1: toy}), "float32", DEV)
    specs = {n: TensorSpec(s.shape, s.init, 0.2 if s.init == "normal" else 0.1) for n, s in model.tensor_specs().items()}
    model.load({k: v.to(DEV) for k, v in random_tensors(specs, 13, torch.float32, "cpu").items()})
    eng = Engine(model, max_tokens=64, max_slots=64)
    assert not eng.holds_pages and eng.cache.kv_groups == [] and eng.max_slots == 64
    prompts = [helpers.random_tokens(500, 256, 1000 + i % 7) for i in range(300)]
    out = generate(eng, prompts, GenerationParams(max_tokens=2, temperature=0.0, repeat_penalty=1.0), max_batch=64)
    assert len(out) == 300 and all(len(o) == 2 for o in out)
    for i in range(7, 300):
        assert out[i] == out[i % 7]                       # equal prompts, equal tokens, whatever the batch and the slot
    assert len({tuple(o) for o in out[:7]}) > 1
    eng.cache.check()
    assert eng.cache.slots.n_held == 0
