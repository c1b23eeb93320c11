"""The registry of part kinds and the interface each category of part has.

A part is built from a PartSpec (kind + parameters) and a BuildEnv.  It names its
tensors, takes them when they are loaded, and computes.  No part knows which
model it is in: sizes and constants come in as parameters only.

Categories and what each must offer beyond `tensors()` and `load()`:

  norm          forward(x) -> y;  add_norm(h, delta) -> y  (h += delta in place, then
                norm of h);  gather_add_norm(h, delta, rows) -> y for chosen rows only
  position      the way a mixer turns positions into a change of q and k: either
                `tables()` (cos, sin, rot_dim, style) for the fused kernel or
                `apply(q, k, positions)` for a position encoding of its own
  mixer         cache_need() -> KVNeed | StateNeed | None;
                forward(x, ctx, cache_entry) -> y, x and y [tokens, hidden]
  feed_forward  forward(x, ctx) -> y
  block         the arrangement: forward(stream, ctx, cache_entry, next_norm, last) -> stream,
                where stream (parts.linear.Stream) holds the float32 residual stream h and
                the update not yet added to it, next_norm is the norm that reads the stream
                after this block, and last says that only the head does; first_norm() -> the
                norm this block reads the stream with

Optional, for a step that wants fewer rows than it has tokens: a mixer with `takes_rows` accepts
`last_rows=True` in the last run of the order and returns its output for ctx's last_rows alone
(its cache still takes all tokens); the block then goes on with those rows only.

Optional, for small decoding steps (ctx.fuse_small), and never needed for a part to work:
a norm with `foldable` and `lazy(stream)` lets the product after it do the division; a
mixer or feed-forward with `folds_norm(ctx)` accepts a parts.linear.LazyNorm as x, and
with `adds_to_stream(ctx)` accepts `stream=` and adds its output to the stream itself
(Stream.add_product), returning None.
"""
from typing import Callable, Dict

from .spec import PartSpec

CATEGORIES = ("norm", "position", "mixer", "feed_forward", "block")
_REGISTRY: Dict[str, Dict[str, Callable]] = {c: {} for c in CATEGORIES}


def register(category, kind):
    """Class decorator: make `kind` buildable in `category`."""
    if category not in _REGISTRY:
        raise KeyError("unknown part category '%s' (known: %s)" % (category, ", ".join(CATEGORIES)))

    def deco(cls):
        _REGISTRY[category][kind] = cls
        cls.category = category
        cls.kind = kind
        return cls
    return deco


def known(category):
    return sorted(_REGISTRY[category])


class BuildEnv:
    """What a part needs to know about the run: device, activation dtype, and a place
    where parts without weights (position tables) are shared between layers."""

    def __init__(self, device, act_dtype):
        self.device = device
        self.act_dtype = act_dtype
        self.shared = {}

    def build(self, category, spec: PartSpec):
        kinds = _REGISTRY[category]
        if spec.kind not in kinds:
            raise KeyError("unknown %s kind '%s' (known: %s)" % (category, spec.kind, ", ".join(sorted(kinds))))
        return kinds[spec.kind](dict(spec.params), self)


class Part:
    """Base of every part."""
    category = None
    kind = None
    # True if forward() launches the same kernels with the same arguments whatever the
    # step's data are (it reads positions, tables and slots on the device only), so that a
    # step can be captured once as a graph and replayed.
    graph_safe = False

    def tensors(self):
        """name (relative to the part's prefix) -> TensorSpec"""
        return {}

    def load(self, tensors):
        """Take the loaded tensors (same names as tensors())."""

    def cache_need(self):
        return None

    def product_weights(self):
        """[(weight [N, K], output dtype or None)] of the matrix products the part runs
        through parts.linear (what the library can be tuned for)."""
        return []
