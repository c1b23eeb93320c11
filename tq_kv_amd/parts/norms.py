"""Norms.  RMSNorm as the reference computes it (src/models/turbo_generic.rs:41-51):
x / sqrt(mean(x^2) + eps) * weight in float32, cast last; the weight is used as it
is stored (no 1 + w)."""
import torch

from .. import kernels as K
from .registry import Part, register
from .spec import TensorSpec


@register("norm", "rms_norm")
class RMSNorm(Part):
    """params: size, eps."""
    graph_safe = True
    trace_name = "rms-norm"             # the reference's span, src/models/turbo_generic.rs:36
    takes_partial_sums = True       # add_norm and gather_add_norm take a product's kernels.PartialSums as the update

    def __init__(self, params, env):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.env = env
        self.weight = None

    def tensors(self):
        return {"weight": TensorSpec((self.size,), init="one_plus_normal")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, x):
        """x: [T, size] of the activation dtype -> its norm, same dtype."""
        out = torch.empty_like(x)
        return K.add_rmsnorm(None, x, self.weight, self.eps, out)

    @property
    def foldable(self):
        """Whether the kernels that add to the stream can prepare this norm (bfloat16 weight)."""
        return self.weight is not None and self.weight.dtype == torch.bfloat16

    def lazy(self, stream):
        """The norm of the stream, left to the product that consumes it: possible if the
        kernel that last added to the stream prepared it for this norm."""
        from .linear import LazyNorm
        if stream.pending is not None or stream.xw_for is not self:
            return None
        return LazyNorm(stream.xw_buffer, stream.ss_buffer, stream.n_ss, self.eps)

    def add_norm(self, h, delta):
        """h: [T, size] float32 residual stream, delta: update of the activation dtype or
        None.  h += delta in place; returns norm(h) in the activation dtype."""
        out = torch.empty(h.shape, dtype=self.env.act_dtype, device=h.device)
        return K.add_rmsnorm(h, delta, self.weight, self.eps, out, write_back=delta is not None)

    def gather_add_norm(self, h, delta, rows):
        """norm(h[rows] + delta[rows]) for the int32 row indices `rows`; h is left as it is."""
        out = torch.empty((rows.shape[0], self.size), dtype=self.env.act_dtype, device=h.device)
        return K.add_rmsnorm(h, delta, self.weight, self.eps, out, rows=rows)
