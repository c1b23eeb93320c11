"""Block arrangements: how a layer's mixer, feed-forward and norms are put together.

"pre_norm" is the reference's decoder layer (src/models/turbo_generic.rs:1959-1981):
x = x + mixer(norm(x)); x = x + ff(norm(x)), with optional norms on the mixer's and
the feed-forward's outputs (:1965-1968, :1976-1979).

The residual stream h is float32.  A block receives h and the previous block's
update that has not been added yet, and returns its own last update the same way, so
that each addition happens inside the next norm's kernel.
"""
from .registry import Part, register


@register("block", "pre_norm")
class PreNormBlock(Part):
    """params: mixer, feed_forward, mixer_norm, ff_norm (PartSpecs); optional
    post_mixer_norm, post_ff_norm (PartSpecs); names: part -> tensor-name prefix inside
    the layer (e.g. {"mixer": "self_attn."})."""

    PARTS = (("mixer", "mixer"), ("feed_forward", "feed_forward"), ("mixer_norm", "norm"), ("ff_norm", "norm"),
             ("post_mixer_norm", "norm"), ("post_ff_norm", "norm"))

    def __init__(self, params, env):
        self.names = dict(params["names"])
        self.parts = {}
        for role, category in self.PARTS:
            spec = params.get(role)
            if spec is None:
                if role.startswith("post_"):
                    continue
                raise ValueError("pre_norm block: no '%s' given" % role)
            self.parts[role] = env.build(category, spec)
            if role not in self.names:
                raise ValueError("pre_norm block: no tensor-name prefix for '%s'" % role)
        self.mixer = self.parts["mixer"]
        self.feed_forward = self.parts["feed_forward"]
        self.mixer_norm = self.parts["mixer_norm"]
        self.ff_norm = self.parts["ff_norm"]
        self.post_mixer_norm = self.parts.get("post_mixer_norm")
        self.post_ff_norm = self.parts.get("post_ff_norm")
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.parts.values())

    def tensors(self):
        out = {}
        for role, part in self.parts.items():
            for name, spec in part.tensors().items():
                out[self.names[role] + name] = spec
        return out

    def load(self, tensors):
        for role, part in self.parts.items():
            prefix = self.names[role]
            part.load({name: tensors[prefix + name] for name in part.tensors()})

    def cache_need(self):
        return self.mixer.cache_need()

    def product_weights(self):
        return [w for part in self.parts.values() for w in part.product_weights()]

    def forward(self, h, delta, ctx, entry):
        x = self.mixer_norm.add_norm(h, delta)
        a = self.mixer.forward(x, ctx, entry)
        if self.post_mixer_norm is not None:
            a = self.post_mixer_norm.forward(a)
        x = self.ff_norm.add_norm(h, a)
        f = self.feed_forward.forward(x, ctx)
        if self.post_ff_norm is not None:
            f = self.post_ff_norm.forward(f)
        return f
