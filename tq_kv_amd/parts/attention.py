"""The attention mixer: grouped-query softmax attention over the cache.

Order of work as in the reference (src/models/turbo_generic.rs:770-833, 1604-1635):
q, k, v projections (+ bias), head split, position encoding of q and k, keys and
values into the cache, scores q.k/sqrt(d), mask, softmax, p.v, merge heads, output
projection without bias.  Query head h reads kv head h // (heads // kv_heads)
(:195-204).  The three projections are one product with the weights stacked.
"""
import math

import torch

from .. import kernels as K
from .linear import LazyNorm, few_rows_form, fusable, leaves_sums, linear, rows_or_stand_in
from .registry import Part, register
from .spec import KVNeed, TensorSpec


@register("mixer", "attention")
class Attention(Part):
    """params: hidden, n_heads, n_kv_heads, head_dim, qkv_bias (bool), out_bias (bool),
    window (None or positions a query sees, itself included), scale (None: 1/sqrt(head_dim)),
    position (PartSpec); optional prompt_tile: queries per tile of the prompt kernel (16, 32, 64 or
    128; default: what the kernel library finds fitting for the step's size and these head counts)."""
    trace_name = "attn"                 # the reference's span, src/models/turbo_generic.rs:1920

    def __init__(self, params, env):
        self.env = env
        self.graph_safe = True
        self.hidden = int(params["hidden"])
        self.n_heads = int(params["n_heads"])
        self.n_kv_heads = int(params["n_kv_heads"])
        self.head_dim = int(params["head_dim"])
        self.qkv_bias = bool(params.get("qkv_bias", False))
        self.out_bias = bool(params.get("out_bias", False))
        self.window = params.get("window")
        if self.n_heads % self.n_kv_heads:
            raise ValueError("attention: %d heads are not a multiple of %d kv heads" % (self.n_heads, self.n_kv_heads))
        if self.window is not None and self.window < 1:
            raise ValueError("attention: window must be at least 1, got %r" % (self.window,))
        scale = params.get("scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.prompt_tile = params.get("prompt_tile")
        if self.prompt_tile is not None and self.prompt_tile not in (16, 32, 64, 128):
            raise ValueError("attention: prompt_tile must be 16, 32, 64 or 128, got %r" % (self.prompt_tile,))
        spec = params["position"]
        key = ("position", spec.kind, tuple(sorted(spec.params.items())))
        if key not in env.shared:
            env.shared[key] = env.build("position", spec)
        self.position = env.shared[key]
        self.graph_safe = not hasattr(self.position, "apply") or getattr(self.position, "graph_safe", False)
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None
        self.few_qkv = self.few_o = None    # the weights' copies for the few-row kernels
        self.reads_other_cache = False      # set when a run of this layer reads another run's cache
        self.takes_rows = True              # forward(..., last_rows=True) computes the step's last_rows only

    def tensors(self):
        q, kv = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
        t = {"q_proj.weight": TensorSpec((q, self.hidden)), "k_proj.weight": TensorSpec((kv, self.hidden)),
             "v_proj.weight": TensorSpec((kv, self.hidden)), "o_proj.weight": TensorSpec((self.hidden, q))}
        if self.qkv_bias:
            t.update({"q_proj.bias": TensorSpec((q,)), "k_proj.bias": TensorSpec((kv,)), "v_proj.bias": TensorSpec((kv,))})
        if self.out_bias:
            t["o_proj.bias"] = TensorSpec((self.hidden,))
        return t

    def load(self, tensors):
        ws = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        dtype = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.w_qkv = torch.cat([w.to(dtype) for w in ws], dim=0).contiguous()
        if self.qkv_bias:
            bs = [tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]]
            bdtype = torch.float32 if any(b.dtype == torch.float32 for b in bs) else bs[0].dtype
            self.b_qkv = torch.cat([b.to(bdtype) for b in bs], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        self.b_o = tensors.get("o_proj.bias")
        self.few_qkv = few_rows_form(self.w_qkv)
        self.few_o = few_rows_form(self.w_o)
        self.w_qkv = rows_or_stand_in(self.w_qkv, self.few_qkv)
        self.w_o = rows_or_stand_in(self.w_o, self.few_o, needed=self.b_o is not None)

    def cache_need(self):
        return KVNeed(self.n_kv_heads, self.head_dim, self.window)

    def product_weights(self):
        return [(w, None) for w in (self.w_qkv, self.w_o) if torch.is_tensor(w)]

    def _fused_qkv_ok(self, ctx):
        """The folded q/k/v kernel takes decoding steps (row m is sequence m) of rotary
        positions in the halves layout over the whole head."""
        if not (ctx.all_decode and fusable(ctx.n_tokens, self.w_qkv) and self.head_dim % 32 == 0):
            return False
        if hasattr(self.position, "apply"):
            return False
        cos, _, rot_dim, style = self.position.tables()
        if style != K.STYLE_HALVES or rot_dim != self.head_dim:
            return False
        return self.b_qkv is None or self.b_qkv.dtype == torch.bfloat16

    def folds_norm(self, ctx):
        return self._fused_qkv_ok(ctx) and not self.reads_other_cache

    def adds_to_stream(self, ctx):
        return self.b_o is None and (fusable(ctx.n_tokens, self.w_o, adds=True) or leaves_sums(ctx.n_tokens, self.w_o, self.few_o))

    def forward(self, x, ctx, entry, stream=None, last_rows=False):
        """x: the (normed) step [tokens, hidden], or a LazyNorm of it.  stream: add the output to
        it instead of returning it.  last_rows: keys and values of all tokens go to the cache as
        always, but the output is computed for ctx's last_rows alone, [n_last, hidden]."""
        lazy = isinstance(x, LazyNorm)
        n = x.xw.shape[0] if lazy else x.shape[0]
        dtype = torch.bfloat16 if lazy else x.dtype
        table = ctx.page_table(entry.group)
        q = torch.empty((n, self.n_heads, self.head_dim), dtype=dtype, device=self.w_qkv.device)
        if lazy or (ctx.fuse_small and entry.writes and self._fused_qkv_ok(ctx)):
            if lazy and not entry.writes:
                raise RuntimeError("a run that reads another run's cache cannot take a folded norm")
            cos, sin, _, _ = self.position.tables()
            K.fused_qkv(x.xw if lazy else x, self.few_qkv or self.w_qkv, self.b_qkv, cos, sin, ctx.dev.tok_pos, table,
                        entry.keys, entry.values, q, self.n_heads, self.n_kv_heads, self.head_dim,
                        norm=x.norm if lazy else None)
        else:
            self._qkv(x, ctx, entry, table, q)
        if last_rows:
            d = ctx.dev
            if ctx.n_last == 0:
                return torch.empty((0, self.hidden), dtype=dtype, device=q.device)
            y = torch.empty((ctx.n_last, self.n_heads * self.head_dim), dtype=dtype, device=q.device)
            attend_rows(q.index_select(0, d.last_rows), entry, table, ctx, self.window, self.scale, y, self.tile_for)
            return linear(y, self.w_o, self.b_o, few=self.few_o)
        y = torch.empty((n, self.n_heads * self.head_dim), dtype=dtype, device=q.device)
        attend(q, entry, table, ctx, self.window, self.scale, y, self.tile_for)
        if stream is not None:
            stream.add_product(y, self.few_o or self.w_o)
            return None
        return linear(y, self.w_o, self.b_o, few=self.few_o)

    def tile_for(self, ctx):
        """Queries per tile of the prompt kernel for this step."""
        if self.prompt_tile is not None:
            return self.prompt_tile
        if not hasattr(ctx, "_prompt_tile"):
            ctx._prompt_tile = {}
        key = (self.n_heads, self.n_kv_heads, self.head_dim)
        if key not in ctx._prompt_tile:
            ctx._prompt_tile[key] = K.attention_prefill_tile(ctx.n_tokens, *key)
        return ctx._prompt_tile[key]

    def _qkv(self, x, ctx, entry, table, q):
        """Product, then bias, position encoding and cache write in their own kernel."""
        own = hasattr(self.position, "apply")
        sums_ok = False
        if not own:
            _, _, rot_dim, style = self.position.tables()
            sums_ok = K.rope_store_takes_sums(x.dtype, self.b_qkv, rot_dim, style, self.head_dim)
        qkv = linear(x, self.w_qkv, few=self.few_qkv, leave_sums=sums_ok)      # may come as its sums over pieces of K
        if own:
            # a position encoding of its own: bias first, then it changes q and k in place
            if self.b_qkv is not None:
                qkv += self.b_qkv.to(qkv.dtype)
            qd, kd = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
            self.position.apply(qkv[:, :qd].unflatten(1, (self.n_heads, self.head_dim)),
                                qkv[:, qd:qd + kd].unflatten(1, (self.n_kv_heads, self.head_dim)), ctx)
            cos = sin = bias = None
            rot_dim, style = 0, K.STYLE_NONE
        else:
            cos, sin, rot_dim, style = self.position.tables()
            bias = self.b_qkv
        K.rope_store(qkv, bias, cos, sin, rot_dim, style, ctx.dev.tok_seq, ctx.dev.tok_pos, table,
                     entry.keys, entry.values, q, self.n_heads, self.n_kv_heads, self.head_dim,
                     write_kv=entry.writes)


# The bfloat16 attention kernels can be switched off one by one (tests compare each with
# the plain kernel); nothing else reads these.
POLICY = {"decode_mfma": True, "prefill_mfma": True}


def attend(q, entry, table, ctx, window, scale, out, tile_for=None):
    """Softmax attention of q over the cache entry: picks the kernel for the step.

    float32, or a head size the MFMA kernels do not take: the plain kernel, one wave per
    (token, head).  bfloat16 and one token per sequence: the partitioned decoding kernel;
    bfloat16 otherwise: the tiled prompt kernel."""
    head_dim = q.shape[2]
    if q.dtype == torch.bfloat16 and ctx.all_decode and POLICY["decode_mfma"] and K.attention_decode_supported(head_dim):
        return K.attention_decode(q, entry.keys, entry.values, ctx.dev.tok_pos, table, window, scale, out)
    if q.dtype == torch.bfloat16 and POLICY["prefill_mfma"] and K.attention_prefill_supported(head_dim):
        d = ctx.dev
        tile = tile_for(ctx) if tile_for is not None else 64
        tile_seq, tile_tok0, tile_count = ctx.query_tiles(tile)
        return K.attention_prefill(q, entry.keys, entry.values, d.tok_pos, table, tile_seq, tile_tok0, tile_count,
                                   d.seq_start, d.seq_new, window, scale, out, tile_queries=tile)
    return K.attention(q, entry.keys, entry.values, ctx.dev.tok_seq, ctx.dev.tok_pos, table, window, scale, out)


DECODE_KERNEL_ROWS = 32     # up to so many rows of a prompt step go through the decoding kernel


def attend_rows(q, entry, table, ctx, window, scale, out, tile_for=None):
    """The same for the step's last_rows alone (q holds their queries): the cache already holds
    the keys and values of all the step's tokens."""
    head_dim = q.shape[2]
    d = ctx.dev
    if (q.dtype == torch.bfloat16 and POLICY["decode_mfma"] and K.attention_decode_supported(head_dim)
            and ctx.n_last <= DECODE_KERNEL_ROWS):
        # few rows: the decoding kernel shares a row's keys out over many blocks, where the prompt
        # kernel would walk them in one; a row is a sequence of its own to it
        return K.attention_decode(q, entry.keys, entry.values, d.last_pos, table.index_select(0, d.last_seq), window, scale, out)
    if q.dtype == torch.bfloat16 and POLICY["prefill_mfma"] and K.attention_prefill_supported(head_dim):
        tile = tile_for(ctx) if tile_for is not None else 64
        tile_seq, tile_tok0, tile_count = ctx.last_tiles(tile)
        return K.attention_prefill(q, entry.keys, entry.values, d.last_pos, table, tile_seq, tile_tok0,
                                   tile_count, d.seq_start, d.seq_new, window, scale, out, tile_queries=tile)
    return K.attention(q, entry.keys, entry.values, d.last_seq, d.last_pos, table, window, scale, out)
