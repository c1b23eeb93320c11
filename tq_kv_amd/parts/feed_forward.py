"""Feed-forward parts.  Gated SiLU ("SwiGLU") as the reference's Mlp
(src/models/turbo_generic.rs:98-111): down(silu(gate(x)) * up(x)), no biases.  Gate and
up are one product with the weights stacked."""
import torch

from .. import kernels as K
from .linear import LazyNorm, few_rows_form, fusable, gated_silu_linear, leaves_sums, linear, rows_or_stand_in
from .registry import Part, register
from .spec import TensorSpec


@register("feed_forward", "gated_silu")
class GatedSiLU(Part):
    """params: hidden, inter."""
    graph_safe = True
    trace_name = "attn-mlp"             # the reference's span, src/models/turbo_generic.rs:1922

    def __init__(self, params, env):
        self.hidden = int(params["hidden"])
        self.inter = int(params["inter"])
        self.w_gate_up = self.w_down = None
        self.few_gate_up = self.few_down = None         # the weights' copies for the few-row kernels

    def tensors(self):
        return {"gate_proj.weight": TensorSpec((self.inter, self.hidden)),
                "up_proj.weight": TensorSpec((self.inter, self.hidden)),
                "down_proj.weight": TensorSpec((self.hidden, self.inter))}

    def load(self, tensors):
        ws = [tensors["gate_proj.weight"], tensors["up_proj.weight"]]
        dtype = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.w_gate_up = torch.cat([w.to(dtype) for w in ws], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]
        self.few_gate_up = few_rows_form(self.w_gate_up, parts=2)
        self.few_down = few_rows_form(self.w_down)
        self.w_gate_up = rows_or_stand_in(self.w_gate_up, self.few_gate_up)
        self.w_down = rows_or_stand_in(self.w_down, self.few_down)

    def product_weights(self):
        return [(w, None) for w in (self.w_gate_up, self.w_down) if torch.is_tensor(w)]

    def folds_norm(self, ctx):
        return fusable(ctx.n_tokens, self.w_gate_up)

    def adds_to_stream(self, ctx):
        return ((fusable(ctx.n_tokens, self.w_down, adds=True) and fusable(ctx.n_tokens, self.w_gate_up))
                or leaves_sums(ctx.n_tokens, self.w_down, self.few_down))

    def forward(self, x, ctx, stream=None):
        lazy = isinstance(x, LazyNorm)
        if stream is not None and not lazy and x.shape[0] > 16:
            stream.add_product(gated_silu_linear(x, self.w_gate_up, self.few_gate_up), self.few_down)
            return None
        if lazy or stream is not None:
            xin = x.xw if lazy else x
            act = torch.empty((xin.shape[0], self.inter), dtype=torch.bfloat16, device=self.w_down.device)
            K.fused_gated(xin, self.few_gate_up or self.w_gate_up, act, x.norm if lazy else None)
            if stream is None:
                return linear(act, self.w_down, few=self.few_down)
            stream.add_product(act, self.few_down or self.w_down)
            return None
        return linear(gated_silu_linear(x, self.w_gate_up, self.few_gate_up), self.w_down, few=self.few_down)
