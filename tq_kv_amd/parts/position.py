"""Position encodings.  Rotary tables as the reference builds them
(src/models/turbo_generic.rs:1654-1670): theta_j = 1 / base^(2j/d) with base rounded
to float32 and the power taken in float32, angle = position * theta_j in float32,
cos and sin of it.  Layouts: halves (:417-427, what Qwen2 uses) and pairs (:430-443);
rot_dim < head_dim rotates the first rot_dim elements only (:752-761)."""
import torch

from .. import kernels as K
from .registry import Part, register


@register("position", "rotary")
class Rotary(Part):
    """params: theta, rot_dim, max_positions, style ("halves" | "pairs")."""

    STYLES = {"halves": K.STYLE_HALVES, "pairs": K.STYLE_PAIRS}

    def __init__(self, params, env):
        self.theta = float(params["theta"])
        self.rot_dim = int(params["rot_dim"])
        self.max_positions = int(params["max_positions"])
        if params.get("style", "halves") not in self.STYLES:
            raise ValueError("rotary: unknown style %r (known: halves, pairs)" % params.get("style"))
        self.style = self.STYLES[params.get("style", "halves")]
        if self.rot_dim <= 0 or self.rot_dim % 2:
            raise ValueError("rotary: rot_dim must be even and positive, got %d" % self.rot_dim)
        # The tables are computed on the host in float32, so that they are the same
        # numbers whatever device the model runs on.
        base = torch.tensor(self.theta, dtype=torch.float32)
        i = torch.arange(0, self.rot_dim, 2, dtype=torch.float32)
        inv_freq = 1.0 / torch.pow(base, i / float(self.rot_dim))
        angle = torch.arange(self.max_positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
        self.cos = torch.cos(angle).contiguous().to(env.device)
        self.sin = torch.sin(angle).contiguous().to(env.device)

    def tables(self):
        """(cos, sin, rot_dim, style) for the fused bias + rotation + cache-write kernel."""
        return self.cos, self.sin, self.rot_dim, self.style


@register("position", "none")
class NoPosition(Part):
    """No change of q and k (a mixer that needs no positions, or learns them elsewhere)."""

    def __init__(self, params, env):
        self.max_positions = int(params.get("max_positions", 1 << 30))

    def tables(self):
        return None, None, 0, K.STYLE_NONE
