"""Plain, slow, whole-sequence float32 implementation of the Qwen2 dense decoder.

It exists only to check the engine: one function for each part, whole sequences,
no cache, no batching, nothing imported from the product package.  Every formula
is taken from the reference's text (file:line cited at each function, paths
relative to the reference checkout).  Sliding-window masking and the tied/untied
switch are not in the reference; their meaning is written where they are used.

All functions take and return float32 CPU (or any-device) torch tensors.
"""
import math

import torch


def rms_norm(x, weight, eps):
    """src/models/turbo_generic.rs:41-51.  x32 / sqrt(mean(x32^2) + eps) * w, all in f32."""
    x32 = x.to(torch.float32)
    variance = (x32 * x32).mean(dim=-1, keepdim=True)
    rms = torch.sqrt(variance + eps)
    return (x32 / rms) * weight.to(torch.float32)


def linear(x, weight, bias=None):
    """src/models/turbo_generic.rs:779-781, 805-813.  y = x W^T (+ b); W is [out, in]."""
    y = x @ weight.t()
    if bias is not None:
        y = y + bias
    return y


def rope_tables(head_dim, theta, n_positions):
    """src/models/turbo_generic.rs:1654-1670.

    theta_j = 1 / base^(i/d) for i = 0, 2, ... in f32 (base itself rounded to f32,
    :2018), angle[p, j] = p * theta_j in f32, cos and sin of it: [n_positions, d/2].
    """
    base = torch.tensor(float(theta), dtype=torch.float32)
    i = torch.arange(0, head_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / torch.pow(base, i / float(head_dim))
    positions = torch.arange(n_positions, dtype=torch.float32)
    angle = positions[:, None] * inv_freq[None, :]
    return torch.cos(angle), torch.sin(angle)


def rope_half(x, cos, sin):
    """src/models/turbo_generic.rs:417-427.  x: [heads, T, d]; cos, sin: [T, d/2].

    out = cat(x0*cos - x1*sin, x0*sin + x1*cos) with x0, x1 the two halves of d.
    """
    half = x.shape[-1] // 2
    x0, x1 = x[..., :half], x[..., half:]
    c, s = cos[None, :, :], sin[None, :, :]
    return torch.cat([x0 * c - x1 * s, x0 * s + x1 * c], dim=-1)


def repeat_kv(x, n_rep):
    """src/models/turbo_generic.rs:195-204.  [nkv, T, d] -> [nkv*n_rep, T, d];
    query head h reads kv head h // n_rep (src/diagnostics.rs:398-410)."""
    if n_rep == 1:
        return x
    nkv, t, d = x.shape
    return x[:, None, :, :].expand(nkv, n_rep, t, d).reshape(nkv * n_rep, t, d)


def visibility(n_tokens, window=None):
    """[T, T] bool, True where query i may see key j.

    Causal part: src/models/turbo_generic.rs:1937-1948 masks j > i.  Window (not in
    the reference): with a window of W the query at i sees the W keys i-W < j <= i.
    """
    i = torch.arange(n_tokens)[:, None]
    j = torch.arange(n_tokens)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (j > i - window)
    return ok


def softmax_last(x):
    """src/models/turbo_generic.rs:56-62; tq-kv/tests/qjl_attention_context.rs:23-43."""
    m = x.max(dim=-1, keepdim=True).values
    e = torch.exp(x - m)
    return e / e.sum(dim=-1, keepdim=True)


def attention_core(q, k, v, visible):
    """src/models/turbo_generic.rs:1620-1631.  q: [nh, T, d]; k, v: [nkv, T, d].

    att = (q k^T) / sqrt(d); masked to -inf; softmax; att v.  Returns [nh, T, d].
    """
    nh, _, d = q.shape
    n_rep = nh // k.shape[0]
    k = repeat_kv(k, n_rep)
    v = repeat_kv(v, n_rep)
    att = (q @ k.transpose(-1, -2)) / math.sqrt(d)
    att = torch.where(visible[None, :, :], att, torch.full_like(att, float("-inf")))
    att = softmax_last(att)
    return att @ v


def attention(x, w, prefix, cfg, window, offset=0):
    """src/models/turbo_generic.rs:770-833 and 1604-1635 for one whole sequence.

    Projections with bias, head split, rotation of q and k at positions
    offset..offset+T-1 (the reference's index_pos, :749-750), causal (and windowed)
    softmax attention, merge heads, o_proj without bias.
    """
    t = x.shape[0]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = linear(x, w[prefix + "q_proj.weight"], w[prefix + "q_proj.bias"])
    k = linear(x, w[prefix + "k_proj.weight"], w[prefix + "k_proj.bias"])
    v = linear(x, w[prefix + "v_proj.weight"], w[prefix + "v_proj.bias"])
    q = q.reshape(t, nh, d).transpose(0, 1)
    k = k.reshape(t, nkv, d).transpose(0, 1)
    v = v.reshape(t, nkv, d).transpose(0, 1)
    cos, sin = rope_tables(d, cfg["rope_theta"], offset + t)
    cos, sin = cos[offset:], sin[offset:]
    q = rope_half(q, cos, sin)
    k = rope_half(k, cos, sin)
    y = attention_core(q, k, v, visibility(t, window))
    y = y.transpose(0, 1).reshape(t, nh * d)
    return linear(y, w[prefix + "o_proj.weight"])


def silu(x):
    """src/models/turbo_generic.rs:64-66.  x * sigmoid(x)."""
    return x / (1.0 + torch.exp(-x))


def swiglu_mlp(x, w, prefix):
    """src/models/turbo_generic.rs:105-111.  down(silu(gate(x)) * up(x)), no biases."""
    g = linear(x, w[prefix + "gate_proj.weight"])
    u = linear(x, w[prefix + "up_proj.weight"])
    return linear(silu(g) * u, w[prefix + "down_proj.weight"])


def layer_window(cfg, layer):
    """Window of a layer or None.  Not in the reference: layer l is windowed iff
    use_sliding_window and l >= max_window_layers."""
    if cfg.get("use_sliding_window", False) and layer >= cfg["max_window_layers"]:
        return cfg["sliding_window"]
    return None


def decoder_layer(x, w, layer, cfg, offset=0):
    """src/models/turbo_generic.rs:1959-1981.  x + attn(norm(x)); x + mlp(norm(x))."""
    p = "model.layers.%d." % layer
    eps = cfg["rms_norm_eps"]
    h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
    x = x + attention(h, w, p + "self_attn.", cfg, layer_window(cfg, layer), offset)
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    return x + swiglu_mlp(h, w, p + "mlp.")


def forward(weights, cfg, tokens, offset=0):
    """src/models/turbo_generic.rs:1950-1987 for one sequence, but the logits of every
    position are returned ([T, V]) instead of the last row only.

    weights: name -> tensor (any float dtype; read as f32).  cfg: dict of config.json
    keys.  Tied embeddings: lm_head is the embedding matrix (:2079-2084).  offset: the
    position of the first token (0 in every real use; tests shift it).
    """
    w = {k: v.to(torch.float32) for k, v in weights.items()}
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = w["model.embed_tokens.weight"][ids]
    for layer in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, w, layer, cfg, offset)
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return linear(x, head)


# ---------------------------------------------------------------------------
# sampling and the generation loop, plain
# ---------------------------------------------------------------------------

def apply_repeat_penalty(logits, generated, penalty):
    """src/engine.rs:403-419.  For every generated token, once per occurrence:
    l > 0 ? l / penalty : l * penalty."""
    out = logits.clone()
    for tok in generated:
        if 0 <= tok < out.numel():
            s = out[tok]
            out[tok] = s / penalty if s > 0 else s * penalty
    return out


def greedy(logits):
    """src/engine.rs:353-354 (temperature <= 0 is argmax); ties go to the lowest id."""
    m = logits.max()
    return int(torch.nonzero(logits == m)[0, 0])


def generate_greedy(weights, cfg, prompt, max_tokens, eos_ids=()):
    """src/engine.rs:364-438 with greedy sampling and no repeat penalty: the prompt
    whole, then one token at a time; a stop token ends the sequence and is not
    emitted; at most max_tokens tokens are emitted."""
    tokens = list(prompt)
    emitted = []
    nxt = greedy(forward(weights, cfg, tokens)[-1])
    while len(emitted) < max_tokens:
        if nxt in eos_ids:
            break
        emitted.append(nxt)
        tokens.append(nxt)
        nxt = greedy(forward(weights, cfg, tokens)[-1])
    return emitted


def keep_top_k_top_p(z, top_k, top_p):
    """Which tokens stay after "top-k then top-p" (src/engine.rs:356-360 names the method;
    its ties and cut are defined by this framework): the k largest z, lower ids first
    among equals; of those, every token at least as probable as the one at which the
    cumulative probability, from the largest down, first reaches top_p of their total.
    z: float64 [V] (already penalised and divided by the temperature).  Returns bool [V]."""
    v = z.numel()
    order = sorted(range(v), key=lambda i: (-float(z[i]), i))
    if 0 < top_k < v:
        order = order[:top_k]
    w = torch.exp(z - z.max())
    keep = torch.zeros(v, dtype=torch.bool)
    if top_p < 1.0:
        total = sum(float(w[i]) for i in order)
        cum, cut = 0.0, order[-1]
        for i in order:
            cum += float(w[i])
            if cum >= top_p * total:
                cut = i
                break
        order = [i for i in order if float(z[i]) >= float(z[cut])]
    keep[order] = True
    return keep


def sample_token(logits, generated, temperature, top_k, top_p, penalty, u):
    """One draw as src/engine.rs:353-373, 403-423 orders it: repeat penalty over the
    generated tokens, argmax if temperature <= 0, else top-k then top-p at the
    temperature; the draw itself (this framework's definition): the first kept token, in
    order of id, whose cumulative kept probability exceeds u times the kept total."""
    z = apply_repeat_penalty(logits.to(torch.float32), generated, penalty) if penalty != 1.0 else logits.to(torch.float32)
    if temperature <= 0:
        return greedy(z)
    z = z.to(torch.float64) / temperature
    keep = keep_top_k_top_p(z, top_k, top_p)
    w = torch.where(keep, torch.exp(z - z.max()), torch.zeros_like(z))
    cum = torch.cumsum(w, 0)
    target = u * float(cum[-1])
    hits = torch.nonzero((cum > target) & keep)
    return int(hits[0, 0]) if hits.numel() else int(torch.nonzero(keep)[-1, 0])


def draw_uniform(seed, request, step):
    """The uniform number of draw `step` of request `request`: three rounds of the
    splitmix64 finaliser over (seed, request, step), top 24 bits.  (Defined by this
    framework; the reference seeds one generator per request, src/engine.rs:362.)"""
    mask = (1 << 64) - 1

    def mix(x):
        x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & mask
        x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & mask
        return x ^ (x >> 31)
    golden = 0x9E3779B97F4A7C15
    x = mix((seed + golden) & mask)
    x = mix(((x ^ request) + golden) & mask)
    x = mix(((x ^ step) + golden) & mask)
    return (x >> 40) / float(1 << 24)


def generate(weights, cfg, prompt, max_tokens, temperature=0.0, top_k=0, top_p=1.0, penalty=1.0, seed=0,
             request=0, eos_ids=()):
    """src/engine.rs:364-438 for one request with any sampling settings."""
    tokens, emitted, step = list(prompt), [], 0
    nxt = sample_token(forward(weights, cfg, tokens)[-1], emitted, temperature, top_k, top_p, penalty,
                       draw_uniform(seed, request, step))
    while len(emitted) < max_tokens:
        if nxt in eos_ids:
            break
        emitted.append(nxt)
        tokens.append(nxt)
        if len(emitted) >= max_tokens:
            break
        step += 1
        nxt = sample_token(forward(weights, cfg, tokens)[-1], emitted, temperature, top_k, top_p, penalty,
                           draw_uniform(seed, request, step))
    return emitted
