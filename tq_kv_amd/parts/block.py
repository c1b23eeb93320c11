"""Block arrangements: how a layer's mixer, feed-forward and norms are put together.

"pre_norm" is the reference's decoder layer (src/models/turbo_generic.rs:1959-1981):
x = x + mixer(norm(x)); x = x + ff(norm(x)), with optional norms on the mixer's and
the feed-forward's outputs (:1965-1968, :1976-1979).

The residual stream is float32 (parts.linear.Stream).  A part's output is left pending
on the stream and added inside the next norm's kernel (for steps of 17 to 128 tokens a
part's last product may even leave its sums over pieces of K pending: the norm's kernel
adds those up too).  In small decoding steps the
framework's parts go further: a product that consumes a norm computes it itself
(LazyNorm) and a part's last product adds its result to the stream in its epilogue, so
that the norm kernels disappear; parts that do not offer this (`folds_norm`,
`adds_to_stream`) are simply given tensors.
"""
from ..tracing import span
from .linear import POLICY
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

    def first_norm(self):
        """The norm that reads the stream first when this block runs."""
        return self.mixer_norm

    def _normed(self, norm, stream, part, ctx):
        """The part's input: the norm of the stream, computed now, or left to the part."""
        if ctx.fuse_small and hasattr(norm, "lazy") and getattr(part, "folds_norm", None) and part.folds_norm(ctx):
            lazy = norm.lazy(stream)
            if lazy is not None:
                return lazy
        with span(getattr(norm, "trace_name", "norm")):
            x = norm.add_norm(stream.h, stream.pending)
        stream.pending = None
        stream.invalidate()
        return x

    def _run(self, part, post_norm, next_norm, x, stream, ctx, *extra):
        """Run a part; its output is added to the stream by the part itself (it returns None)
        or is left pending for the next norm's kernel."""
        with span(getattr(part, "trace_name", "part")):
            if ((ctx.fuse_small or getattr(ctx, "fuse_mid", False)) and post_norm is None
                    and getattr(part, "adds_to_stream", None) and part.adds_to_stream(ctx)):
                stream.next_norm = next_norm
                out = part.forward(x, ctx, *extra, stream=stream)
            else:
                out = part.forward(x, ctx, *extra)
        if out is not None:
            if post_norm is not None:
                out = post_norm.forward(out)
            stream.pending = out
            stream.invalidate()

    def forward(self, stream, ctx, entry, next_norm=None, last=False):
        """next_norm: the norm that reads the stream after this block.  last: nothing but the
        head reads the stream after this block, so where the step wants fewer rows than it has
        tokens (ctx.prune_last) and the mixer can do so, only those rows are computed once the
        mixer has seen all tokens: the stream of those rows is returned in place of `stream`."""
        if last and ctx.prune_last and POLICY["prune_last"] and getattr(self.mixer, "takes_rows", False):
            return self._forward_last_rows(stream, ctx, entry)
        x = self._normed(self.mixer_norm, stream, self.mixer, ctx)
        self._run(self.mixer, self.post_mixer_norm, self.ff_norm, x, stream, ctx, entry)
        x = self._normed(self.ff_norm, stream, self.feed_forward, ctx)
        self._run(self.feed_forward, self.post_ff_norm, next_norm, x, stream, ctx)
        return stream

    def _forward_last_rows(self, stream, ctx, entry):
        with span(getattr(self.mixer_norm, "trace_name", "norm")):
            x = self.mixer_norm.add_norm(stream.h, stream.pending)
        with span(getattr(self.mixer, "trace_name", "part")):
            y = self.mixer.forward(x, ctx, entry, last_rows=True)      # keys and values of all tokens, output of the rows
        sub = type(stream)(stream.h.index_select(0, ctx.dev.last_rows))
        sub.of_last_rows = True
        if ctx.n_last == 0:
            return sub
        sub.pending = self.post_mixer_norm.forward(y) if self.post_mixer_norm is not None else y
        with span(getattr(self.ff_norm, "trace_name", "norm")):
            x = self.ff_norm.add_norm(sub.h, sub.pending)
        with span(getattr(self.feed_forward, "trace_name", "part")):
            out = self.feed_forward.forward(x, ctx)
        sub.pending = self.post_ff_norm.forward(out) if self.post_ff_norm is not None else out
        return sub
