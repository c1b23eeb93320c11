"""Data that describes a model: which parts, with which sizes, run in which order.

Nothing here computes.  An architecture turns its typed configuration into a ModelSpec; the
weight loader, the random-weights writer, the cache and the engine all work from the ModelSpec
alone and never ask which architecture it came from.  These classes mirror the engine library's
(csrc/engine/spec.h) and cross the C boundary as JSON.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from .. import native


@dataclass(frozen=True)
class TensorSpec:
    """One named tensor of a part.

    init: how the random-weights mode fills it: "normal" (N(0, std)), "one_plus_normal"
    (1 + N(0, std)), "zeros", or a kind registered with weights.register_init.
    dtype: "float" follows the run's weight dtype; "int32" is an integer table.
    """
    shape: Tuple[int, ...]
    init: str = "normal"
    std: float = 0.02
    dtype: str = "float"

    def to_json(self):
        return {"shape": [int(s) for s in self.shape], "init": self.init, "std": float(self.std), "dtype": self.dtype}

    @classmethod
    def from_json(cls, j):
        return cls(tuple(j["shape"]), j.get("init", "normal"), j.get("std", 0.02), j.get("dtype", "float"))


@dataclass(frozen=True)
class PartSpec:
    """A part by kind and parameters; params may hold further PartSpecs."""
    kind: str
    params: Dict = field(default_factory=dict)

    def to_json(self):
        return {"kind": self.kind, "params": {k: _plain(v) for k, v in self.params.items()}}

    @classmethod
    def from_json(cls, j):
        return cls(j["kind"], {k: _revive(v) for k, v in (j.get("params") or {}).items()})


def _plain(v):
    if isinstance(v, PartSpec):
        return v.to_json()
    if isinstance(v, dict):
        return {k: _plain(x) for k, x in v.items()}
    if isinstance(v, (list, tuple)):
        return [_plain(x) for x in v]
    return v


def _revive(v):
    if isinstance(v, dict):
        if set(v) == {"kind", "params"} and isinstance(v["kind"], str):
            return PartSpec.from_json(v)
        return {k: _revive(x) for k, x in v.items()}
    return v


@dataclass(frozen=True)
class KVNeed:
    """A mixer that keeps keys and values for every position (window: only the last `window`
    positions are ever read), in pages of native.page_size() positions whose layout is the mixer's
    own: key_page and value_page are the shapes of one page.  Given kv heads and a head size
    only, the pages are the attention kernels': keys [kv heads, page, head_dim], values [kv heads,
    value_dim or head_dim, page] (transposed inside a page)."""
    n_kv_heads: int = 0
    head_dim: int = 0
    window: Optional[int] = None
    value_dim: Optional[int] = None
    key_page: Optional[Tuple[int, ...]] = None
    value_page: Optional[Tuple[int, ...]] = None

    def pages(self):
        page = native.page_size()
        key = tuple(self.key_page) if self.key_page is not None else (self.n_kv_heads, page, self.head_dim)
        value = tuple(self.value_page) if self.value_page is not None else (self.n_kv_heads, self.value_dim or self.head_dim, page)
        return key, value

    def to_json(self):
        key, value = self.pages()
        return {"kind": "pages", "key_page": list(key), "value_page": list(value), "window": self.window}


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a fixed-size state per sequence (zero at start).  dtype: "float32",
    "bfloat16" or "int32"."""
    shape: Tuple[int, ...]
    dtype: str = "float32"

    def to_json(self):
        return {"kind": "state", "shape": [int(s) for s in self.shape], "dtype": self.dtype}


def need_from_json(j):
    """The need the engine library reports: pages in the attention kernels' layout come back as the
    KVNeed(kv heads, head size, window) that asks for them."""
    if j is None:
        return None
    if j["kind"] == "state":
        return StateNeed(tuple(j["shape"]), j.get("dtype", "float32"))
    key, value = tuple(j["key_page"]), tuple(j["value_page"])
    page = native.page_size()
    if len(key) == 3 and len(value) == 3 and key[1] == page and value[2] == page and key[0] == value[0]:
        return KVNeed(key[0], key[2], j.get("window"), None if value[1] == key[2] else value[1])
    return KVNeed(window=j.get("window"), key_page=key, value_page=value)


def need_to_json(need):
    return None if need is None else need.to_json()


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement (which names its mixer, feed-forward and norms)
    and the tensor-name prefix its parts' tensors live under."""
    prefix: str
    block: PartSpec


@dataclass(frozen=True)
class Run:
    """One entry of the run order: run layer `layer`.  `cache_of` names an earlier
    entry of the order whose cache this run reads instead of keeping its own."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding_name: str
    layers: List[LayerSpec]
    order: List[Run]
    final_norm: PartSpec
    final_norm_prefix: str
    head_name: Optional[str]      # None: the head is the embedding matrix (tied)
    eos_token_ids: Tuple[int, ...] = ()
    # What an architecture may do around the blocks; all off for the reference's decoder.
    embedding_scale: Optional[float] = None        # the stream starts as embedding * scale
    stream_position: Optional[PartSpec] = None     # a position part that acts on the stream after the
    stream_position_prefix: str = ""               #   gather (add_to_stream), and where its tensors live
    head_bias_name: Optional[str] = None           # logits += this tensor [vocab]
    logit_scale: Optional[float] = None            # logits *= scale
    logit_cap: Optional[float] = None              # logits = cap * tanh(logits / cap)

    def to_json(self):
        return {
            "architecture": self.architecture, "vocab_size": int(self.vocab_size), "hidden_size": int(self.hidden_size),
            "max_positions": int(self.max_positions), "embedding_name": self.embedding_name,
            "layers": [{"prefix": l.prefix, "block": l.block.to_json()} for l in self.layers],
            "order": [{"layer": int(r.layer), "cache_of": None if r.cache_of is None else int(r.cache_of)} for r in self.order],
            "final_norm": self.final_norm.to_json(), "final_norm_prefix": self.final_norm_prefix, "head_name": self.head_name,
            "eos_token_ids": [int(t) for t in self.eos_token_ids], "embedding_scale": self.embedding_scale,
            "stream_position": None if self.stream_position is None else self.stream_position.to_json(),
            "stream_position_prefix": self.stream_position_prefix, "head_bias_name": self.head_bias_name,
            "logit_scale": self.logit_scale, "logit_cap": self.logit_cap}

    @classmethod
    def from_json(cls, j):
        return cls(
            architecture=j["architecture"], vocab_size=j["vocab_size"], hidden_size=j["hidden_size"], max_positions=j["max_positions"],
            embedding_name=j["embedding_name"],
            layers=[LayerSpec(l["prefix"], PartSpec.from_json(l["block"])) for l in j["layers"]],
            order=[Run(r["layer"], r.get("cache_of")) for r in j["order"]],
            final_norm=PartSpec.from_json(j["final_norm"]), final_norm_prefix=j["final_norm_prefix"], head_name=j.get("head_name"),
            eos_token_ids=tuple(j.get("eos_token_ids") or ()), embedding_scale=j.get("embedding_scale"),
            stream_position=None if j.get("stream_position") is None else PartSpec.from_json(j["stream_position"]),
            stream_position_prefix=j.get("stream_position_prefix", ""), head_bias_name=j.get("head_bias_name"),
            logit_scale=j.get("logit_scale"), logit_cap=j.get("logit_cap"))
