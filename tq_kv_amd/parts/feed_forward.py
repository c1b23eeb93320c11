"""Feed-forward parts.  Gated SiLU ("SwiGLU") as the reference's Mlp
(src/models/turbo_generic.rs:98-111): down(silu(gate(x)) * up(x)), no biases.  Gate and
up are one product with the weights stacked."""
import torch

from .linear import gated_silu_linear, linear
from .registry import Part, register
from .spec import TensorSpec


@register("feed_forward", "gated_silu")
class GatedSiLU(Part):
    """params: hidden, inter."""
    graph_safe = True

    def __init__(self, params, env):
        self.hidden = int(params["hidden"])
        self.inter = int(params["inter"])
        self.w_gate_up = self.w_down = None

    def tensors(self):
        return {"gate_proj.weight": TensorSpec((self.inter, self.hidden)),
                "up_proj.weight": TensorSpec((self.inter, self.hidden)),
                "down_proj.weight": TensorSpec((self.hidden, self.inter))}

    def load(self, tensors):
        ws = [tensors["gate_proj.weight"], tensors["up_proj.weight"]]
        dtype = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.w_gate_up = torch.cat([w.to(dtype) for w in ws], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def product_weights(self):
        return [(self.w_gate_up, None), (self.w_down, None)]

    def forward(self, x, ctx):
        return linear(gated_silu_linear(x, self.w_gate_up), self.w_down)
