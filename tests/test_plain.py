"""Pins the plain implementation by what fixes it beside the reference's text:
library routines it must reduce to, closed-form special cases, invariants.  Each check
is chosen so that a plausible misreading (wrong pairing or sign of the rotation, a norm
in the wrong place, the wrong kv head, an off-by-one window) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen2 as plain
from helpers import TINY_A, TINY_B


def rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def tiny_weights(cfg, seed=0, std=0.05):
    """Random weights with the reference's tensor names (src/models/turbo_generic.rs:2075-2126)."""
    h, nh, nkv, d, i, v = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
                           cfg["head_dim"], cfg["intermediate_size"], cfg["vocab_size"])
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * std
    w = {"model.embed_tokens.weight": r(v, h), "model.norm.weight": 1 + r(h)}
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = r(v, h)
    for l in range(cfg["num_hidden_layers"]):
        p = "model.layers.%d." % l
        w.update({p + "self_attn.q_proj.weight": r(nh * d, h), p + "self_attn.q_proj.bias": r(nh * d),
                  p + "self_attn.k_proj.weight": r(nkv * d, h), p + "self_attn.k_proj.bias": r(nkv * d),
                  p + "self_attn.v_proj.weight": r(nkv * d, h), p + "self_attn.v_proj.bias": r(nkv * d),
                  p + "self_attn.o_proj.weight": r(h, nh * d),
                  p + "mlp.gate_proj.weight": r(i, h), p + "mlp.up_proj.weight": r(i, h), p + "mlp.down_proj.weight": r(h, i),
                  p + "input_layernorm.weight": 1 + r(h), p + "post_attention_layernorm.weight": 1 + r(h)})
    return w


# ---- RMSNorm ------------------------------------------------------------------------
def test_rms_norm_is_the_library_routine():
    x, w = rand(5, 96, seed=1, scale=3.0), 1 + rand(96, seed=2, scale=0.1)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), rtol=1e-6, atol=1e-6)


def test_rms_norm_unit_rms_and_scale_invariance():
    x = rand(4, 64, seed=3, scale=2.0)
    y = plain.rms_norm(x, torch.ones(64), 0.0)
    torch.testing.assert_close((y * y).mean(-1).sqrt(), torch.ones(4), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(plain.rms_norm(7.5 * x, torch.ones(64), 0.0), y, rtol=1e-5, atol=1e-6)
    # eps is added to the mean of squares, under the root: with x = 0 the result is 0, and a
    # large eps shrinks the output by sqrt(mean + eps)
    x1 = torch.full((1, 4), 2.0)
    assert torch.allclose(plain.rms_norm(x1, torch.ones(4), 12.0), torch.full((1, 4), 2.0 / 4.0))


def test_rms_norm_weight_is_used_as_stored():
    x = rand(2, 8, seed=4)
    assert torch.allclose(plain.rms_norm(x, torch.zeros(8), 1e-6), torch.zeros(2, 8))   # not 1 + w


# ---- linear ------------------------------------------------------------------------
def test_linear_is_the_library_routine():
    x, w, b = rand(3, 10, seed=5), rand(7, 10, seed=6), rand(7, seed=7)
    torch.testing.assert_close(plain.linear(x, w, b), F.linear(x, w, b))
    torch.testing.assert_close(plain.linear(x, torch.eye(10)), x)


# ---- rotation ------------------------------------------------------------------------
def test_rope_tables_closed_form():
    cos, sin = plain.rope_tables(8, 10000.0, 6)
    assert cos.shape == (6, 4)
    for p in range(6):
        for j in range(4):
            ang = p * 10000.0 ** (-(2 * j) / 8)
            assert abs(cos[p, j].item() - math.cos(ang)) < 1e-5 and abs(sin[p, j].item() - math.sin(ang)) < 1e-5
    assert cos[3, 0].item() == pytest.approx(math.cos(3.0), abs=1e-6)       # theta_0 = 1


def test_rope_position_zero_is_identity_and_norm_is_kept():
    x = rand(2, 5, 16, seed=8)
    cos, sin = plain.rope_tables(16, 10000.0, 5)
    y = plain.rope_half(x, cos, sin)
    torch.testing.assert_close(y[:, 0], x[:, 0])
    # each pair (j, j + d/2) keeps its length
    torch.testing.assert_close(y[..., :8] ** 2 + y[..., 8:] ** 2, x[..., :8] ** 2 + x[..., 8:] ** 2, rtol=1e-5, atol=1e-6)


def test_rope_pairs_halves_with_the_right_sign():
    # a unit vector on element 0 at position p turns into cos(p) on element 0 and +sin(p) on
    # element d/2 (pairs of neighbours, or the other sign, put it elsewhere)
    d, p = 8, 3
    x = torch.zeros(1, p + 1, d)
    x[0, p, 0] = 1.0
    cos, sin = plain.rope_tables(d, 10000.0, p + 1)
    y = plain.rope_half(x, cos, sin)[0, p]
    want = torch.zeros(d)
    want[0], want[d // 2] = math.cos(p), math.sin(p)
    torch.testing.assert_close(y, want, rtol=1e-6, atol=1e-6)


def test_rope_is_a_complex_multiplication():
    d, t = 12, 7
    x = rand(1, t, d, seed=9)
    cos, sin = plain.rope_tables(d, 500.0, t)
    y = plain.rope_half(x, cos, sin)[0]
    z = torch.complex(x[0, :, :d // 2], x[0, :, d // 2:]) * torch.complex(cos, sin)
    torch.testing.assert_close(torch.cat([z.real, z.imag], -1), y, rtol=1e-5, atol=1e-6)


def test_rope_scores_depend_on_distance_only():
    d = 16
    q, k = rand(1, 1, d, seed=10), rand(1, 1, d, seed=11)
    cos, sin = plain.rope_tables(d, 10000.0, 40)

    def score(m, n):
        qm = plain.rope_half(q, cos[m:m + 1], sin[m:m + 1])
        kn = plain.rope_half(k, cos[n:n + 1], sin[n:n + 1])
        return (qm * kn).sum().item()
    assert score(9, 4) == pytest.approx(score(30, 25), abs=1e-4)
    assert score(9, 4) != pytest.approx(score(9, 5), abs=1e-4)


# ---- grouped heads ----------------------------------------------------------------------
@pytest.mark.parametrize("nh,nkv", [(64, 8), (32, 32), (6, 2), (3, 1)])
def test_gqa_map(nh, nkv):
    # query head h reads kv head h // (nh // nkv): the reference's own test covers 64/8 and
    # 32/32 (src/diagnostics.rs:398-410)
    n_rep = nh // nkv
    x = torch.arange(nkv, dtype=torch.float32)[:, None, None].expand(nkv, 2, 4)
    y = plain.repeat_kv(x, n_rep)
    assert y.shape == (nh, 2, 4)
    for h in range(nh):
        assert y[h, 0, 0].item() == h // n_rep
    torch.testing.assert_close(y, x.repeat_interleave(n_rep, dim=0))


# ---- attention ---------------------------------------------------------------------------
def test_softmax_is_the_library_routine():
    x = rand(3, 9, seed=12, scale=4.0)
    torch.testing.assert_close(plain.softmax_last(x), torch.softmax(x, -1))
    torch.testing.assert_close(plain.softmax_last(x).sum(-1), torch.ones(3))


def test_attention_core_is_sdpa_with_an_explicit_mask():
    nh, nkv, t, d = 6, 2, 11, 16
    q, k, v = rand(nh, t, d, seed=13), rand(nkv, t, d, seed=14), rand(nkv, t, d, seed=15)
    for window in (None, 4):
        vis = plain.visibility(t, window)
        want = F.scaled_dot_product_attention(q[None], k.repeat_interleave(3, 0)[None], v.repeat_interleave(3, 0)[None],
                                              attn_mask=vis)[0]
        torch.testing.assert_close(plain.attention_core(q, k, v, vis), want, rtol=1e-5, atol=1e-6)


def test_attention_one_head_no_mask_is_plain_sdpa():
    q, k, v = rand(1, 5, 8, seed=16), rand(1, 5, 8, seed=17), rand(1, 5, 8, seed=18)
    full = torch.ones(5, 5, dtype=torch.bool)
    torch.testing.assert_close(plain.attention_core(q, k, v, full), F.scaled_dot_product_attention(q, k, v),
                               rtol=1e-5, atol=1e-6)


def test_visibility_edges():
    vis = plain.visibility(6, 3)
    assert vis[5].tolist() == [False, False, False, True, True, True]     # W keys, itself included
    assert vis[1].tolist() == [True, True, False, False, False, False]
    assert torch.equal(plain.visibility(6, 6), plain.visibility(6, None))  # window >= T is causal
    assert torch.equal(plain.visibility(6, 1), torch.eye(6, dtype=torch.bool))


def test_attention_single_key_returns_its_value():
    q, k, v = rand(2, 4, 8, seed=19), rand(1, 4, 8, seed=20), rand(1, 4, 8, seed=21)
    y = plain.attention_core(q, k, v, plain.visibility(4, 1))              # window 1: own position only
    torch.testing.assert_close(y, v.expand(2, 4, 8))
    y = plain.attention_core(q, k, v, plain.visibility(4, None))
    torch.testing.assert_close(y[:, 0], v[:, 0].expand(2, 8))              # first query sees one key


def test_score_scale_is_one_over_sqrt_d():
    # two keys, q.k0 = d, q.k1 = 0: weights are softmax([sqrt(d), 0])
    d = 16
    q = torch.ones(1, 2, d)
    k = torch.zeros(1, 2, d)
    k[0, 0] = 1.0
    v = torch.tensor([[[1.0], [0.0]]]).expand(1, 2, 1).contiguous()
    y = plain.attention_core(q, k, v, torch.ones(2, 2, dtype=torch.bool))
    assert y[0, 0, 0].item() == pytest.approx(1 / (1 + math.exp(-math.sqrt(d))), abs=1e-6)


# ---- feed-forward ---------------------------------------------------------------------------
def test_swiglu():
    g = rand(4, 10, seed=22, scale=3.0)
    torch.testing.assert_close(plain.silu(g), F.silu(g), rtol=1e-6, atol=1e-6)
    assert plain.silu(torch.zeros(1)).item() == 0.0
    x = rand(3, 8, seed=23)
    w = {"gate_proj.weight": rand(5, 8, seed=24), "up_proj.weight": rand(5, 8, seed=25), "down_proj.weight": rand(8, 5, seed=26)}
    want = F.linear(F.silu(F.linear(x, w["gate_proj.weight"])) * F.linear(x, w["up_proj.weight"]), w["down_proj.weight"])
    torch.testing.assert_close(plain.swiglu_mlp(x, w, ""), want, rtol=1e-5, atol=1e-6)


def test_silu_acts_on_the_gate_projection_not_on_up():
    # src/models/turbo_generic.rs:105-111: down(silu(gate(x)) * up(x)).  A gate that is large and
    # negative everywhere closes the feed-forward whatever up gives; with the roles swapped
    # (silu on up, times gate) the same weights would give something huge instead.
    x = rand(4, 8, seed=27).abs() + 0.5
    w = {"gate_proj.weight": -10.0 * torch.ones(6, 8), "up_proj.weight": rand(6, 8, seed=28),
         "down_proj.weight": rand(8, 6, seed=29)}
    assert plain.swiglu_mlp(x, w, "").abs().max().item() < 1e-10
    swapped = F.linear(F.silu(F.linear(x, w["up_proj.weight"])) * F.linear(x, w["gate_proj.weight"]), w["down_proj.weight"])
    assert swapped.abs().max().item() > 1.0
    # and the other way round: a wide-open gate passes up(x) times gate(x)
    w["gate_proj.weight"] = 10.0 * torch.ones(6, 8)
    g, u = F.linear(x, w["gate_proj.weight"]), F.linear(x, w["up_proj.weight"])
    torch.testing.assert_close(plain.swiglu_mlp(x, w, ""), F.linear(g * u, w["down_proj.weight"]), rtol=1e-5, atol=1e-5)


# ---- the whole model -----------------------------------------------------------------------
def test_norms_sit_before_mixer_and_feed_forward():
    # with o_proj and down_proj zero every layer adds nothing: logits = head(norm(embedding)).
    # A norm after the residual sum instead of before the part would change the stream.
    cfg = dict(TINY_B)
    w = tiny_weights(cfg, seed=3)
    for l in range(cfg["num_hidden_layers"]):
        w["model.layers.%d.self_attn.o_proj.weight" % l].zero_()
        w["model.layers.%d.mlp.down_proj.weight" % l].zero_()
    toks = [5, 9, 200, 31]
    e = w["model.embed_tokens.weight"][toks]
    want = plain.linear(plain.rms_norm(e, w["model.norm.weight"], cfg["rms_norm_eps"]), w["lm_head.weight"])
    torch.testing.assert_close(plain.forward(w, cfg, toks), want, rtol=1e-5, atol=1e-6)


def test_each_norm_weight_acts_at_its_own_site():
    # src/models/turbo_generic.rs:1959-1981: input_layernorm feeds the mixer, post_attention_layernorm
    # the feed-forward.  One layer, one token (attention over a single key returns its value), norm
    # weights that are distinct constants: the logits show which weight sat where.
    cfg = dict(TINY_A, num_hidden_layers=1)
    w = tiny_weights(cfg, seed=31, std=0.3)
    p = "model.layers.0."
    a, b = 3.0, 0.25
    w[p + "input_layernorm.weight"] = torch.full((cfg["hidden_size"],), a)
    w[p + "post_attention_layernorm.weight"] = torch.full((cfg["hidden_size"],), b)
    eps, tok = cfg["rms_norm_eps"], [17]
    x0 = w["model.embed_tokens.weight"][tok]
    unit = lambda x: x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    head = lambda x: F.linear(unit(x) * w["model.norm.weight"], w["model.embed_tokens.weight"])
    n_rep = cfg["num_attention_heads"] // cfg["num_key_value_heads"]

    def mixer(scale):
        v = F.linear(unit(x0) * scale, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"])
        v = v.reshape(1, cfg["num_key_value_heads"], cfg["head_dim"]).repeat_interleave(n_rep, dim=1).reshape(1, -1)
        return F.linear(v, w[p + "self_attn.o_proj.weight"])

    def ff(x, scale):
        h = unit(x) * scale
        return F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                        w[p + "mlp.down_proj.weight"])
    x1 = x0 + mixer(a)
    want = head(x1 + ff(x1, b))
    got = plain.forward(w, cfg, tok)
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    x1s = x0 + mixer(b)
    swapped = head(x1s + ff(x1s, a))
    assert (swapped - want).abs().max().item() > 0.05              # the other placing is far away


def test_qkv_have_biases_and_the_output_projection_has_none():
    # src/models/turbo_generic.rs:2103-2105 (q, k, v biases), :2094 and :2139 (o_proj: weight only).
    # With zero projection weights every key is equal, every value is the v bias: the mixer's
    # output is o_proj(v bias repeated over the heads of its group) for every token, and nothing
    # is added after o_proj.
    cfg = dict(TINY_B)
    w = tiny_weights(cfg, seed=32)
    p = "model.layers.0.self_attn."
    for name in ("q_proj.weight", "k_proj.weight", "v_proj.weight"):
        w[p + name].zero_()
    x = rand(7, cfg["hidden_size"], seed=33)
    n_rep = cfg["num_attention_heads"] // cfg["num_key_value_heads"]
    bias = w[p + "v_proj.bias"].reshape(cfg["num_key_value_heads"], cfg["head_dim"]).repeat_interleave(n_rep, dim=0).reshape(-1)
    want = F.linear(bias, w[p + "o_proj.weight"]).expand(7, -1)
    torch.testing.assert_close(plain.attention(x, w, p, cfg, None), want, rtol=1e-5, atol=1e-6)
    assert want.abs().max().item() > 1e-3
    # without the biases the same weights would give exactly nothing
    w[p + "v_proj.bias"].zero_()
    assert plain.attention(x, w, p, cfg, None).abs().max().item() == 0.0
    # an o_proj.bias is not looked up: planting one changes nothing
    w[p + "o_proj.bias"] = torch.ones(cfg["hidden_size"])
    assert plain.attention(x, w, p, cfg, None).abs().max().item() == 0.0


def test_max_window_layers_decides_which_layers_are_windowed():
    # layer l is windowed iff l >= max_window_layers: 0, 1 and 3 of tiny B's three layers give
    # three different models at a position beyond the window, and the same model inside it
    cfg = dict(TINY_B)
    w = tiny_weights(cfg, seed=34, std=0.2)
    toks = [(7 * i + 3) % cfg["vocab_size"] for i in range(41)]
    outs = [plain.forward(w, dict(cfg, max_window_layers=m), toks) for m in (0, 1, 3)]
    for i in range(3):
        for j in range(i + 1, 3):
            assert (outs[i][40] - outs[j][40]).abs().max().item() > 1e-4
            torch.testing.assert_close(outs[i][:cfg["sliding_window"]], outs[j][:cfg["sliding_window"]])
    torch.testing.assert_close(outs[2], plain.forward(w, dict(cfg, use_sliding_window=False), toks))


def test_tied_and_untied_head():
    cfg = dict(TINY_A)
    w = tiny_weights(cfg, seed=4)
    toks = [1, 2, 3, 250, 7]
    tied = plain.forward(w, cfg, toks)
    cfg2 = dict(cfg, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    torch.testing.assert_close(plain.forward(w2, cfg2, toks), tied)
    w2["lm_head.weight"] = w2["lm_head.weight"] * 2
    torch.testing.assert_close(plain.forward(w2, cfg2, toks), 2 * tied, rtol=1e-5, atol=1e-6)


def test_causality_and_window_in_the_whole_model():
    cfg = dict(TINY_B)
    w = tiny_weights(cfg, seed=5, std=0.2)
    toks = list(range(40, 70))
    base = plain.forward(w, cfg, toks)
    changed = list(toks)
    changed[-1] = 3
    torch.testing.assert_close(plain.forward(w, cfg, changed)[:-1], base[:-1])     # the future is not seen
    # layer 0 sees everything, so an early token still matters at the end
    changed = list(toks)
    changed[0] = 3
    assert (plain.forward(w, cfg, changed)[-1] - base[-1]).abs().max() > 1e-4
    # with every layer windowed, what lies further back than layers * (window - 1) cannot matter
    cfg_all = dict(cfg, max_window_layers=0, sliding_window=4)
    base = plain.forward(w, cfg_all, toks)
    reach = cfg["num_hidden_layers"] * 3
    changed = list(toks)
    changed[len(toks) - 1 - reach - 1] = 3
    torch.testing.assert_close(plain.forward(w, cfg_all, changed)[-1], base[-1])
    changed = list(toks)
    changed[len(toks) - 1 - reach] = 3
    assert (plain.forward(w, cfg_all, changed)[-1] - base[-1]).abs().max() > 1e-7


def test_shift_of_all_positions_changes_nothing():
    # only distances between positions count
    cfg = dict(TINY_A)
    w = tiny_weights(cfg, seed=6, std=0.2)
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    torch.testing.assert_close(plain.forward(w, cfg, toks, offset=37), plain.forward(w, cfg, toks), rtol=1e-4, atol=2e-5)


def test_layer_window_rule():
    cfg = dict(TINY_B)
    assert [plain.layer_window(cfg, l) for l in range(3)] == [None, 12, 12]
    assert plain.layer_window(dict(TINY_A), 1) is None


# ---- sampling and the loop ------------------------------------------------------------------
def test_repeat_penalty_vector():
    # src/engine.rs:403-419: positive scores are divided, negative ones multiplied, once per occurrence
    l = torch.tensor([2.0, -2.0, 4.0, 1.0])
    out = plain.apply_repeat_penalty(l, [0, 1, 2, 2], 2.0)
    assert out.tolist() == [1.0, -4.0, 1.0, 1.0]


def test_greedy_and_ties():
    assert plain.greedy(torch.tensor([0.1, 0.7, 0.7, 0.2])) == 1


def test_top_k_top_p_keep():
    z = torch.log(torch.tensor([0.1, 0.4, 0.2, 0.3], dtype=torch.float64))
    assert plain.keep_top_k_top_p(z, 2, 1.0).tolist() == [False, True, False, True]
    assert plain.keep_top_k_top_p(z, 0, 0.69).tolist() == [False, True, False, True]     # 0.4 + 0.3 >= 0.69
    assert plain.keep_top_k_top_p(z, 0, 0.71).tolist() == [False, True, True, True]
    assert plain.keep_top_k_top_p(z, 3, 0.5).tolist() == [False, True, False, True]      # of 0.9: 0.4 < 0.45 <= 0.7
    z = torch.zeros(5, dtype=torch.float64)
    assert plain.keep_top_k_top_p(z, 2, 1.0).tolist() == [True, True, False, False, False]  # ties: lower ids


def test_sample_token_inverse_cdf():
    logits = torch.log(torch.tensor([0.1, 0.4, 0.2, 0.3]))
    pick = lambda u: plain.sample_token(logits, [], 1.0, 0, 1.0, 1.0, u)
    assert [pick(u) for u in (0.0, 0.09, 0.11, 0.49, 0.51, 0.69, 0.71, 0.999)] == [0, 0, 1, 1, 2, 2, 3, 3]
    assert plain.sample_token(logits, [], 0.0, 0, 1.0, 1.0, 0.9) == 1
    # a low temperature concentrates on the argmax
    assert all(plain.sample_token(logits, [], 0.01, 0, 1.0, 1.0, u) == 1 for u in (0.01, 0.5, 0.99))


def test_generate_stops_without_emitting_the_stop_token():
    cfg = dict(TINY_A)
    w = tiny_weights(cfg, seed=7, std=0.3)
    free = plain.generate_greedy(w, cfg, [1, 2, 3], 6)
    assert len(free) == 6
    stop = free[3]
    first = free.index(stop)
    assert plain.generate_greedy(w, cfg, [1, 2, 3], 6, eos_ids=(stop,)) == free[:first]
    assert plain.generate(w, cfg, [1, 2, 3], 6) == free
    assert plain.generate_greedy(w, cfg, [1, 2, 3], 0) == []
