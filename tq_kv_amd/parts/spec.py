"""Data that describes a model: which parts, with which sizes, run in which order.

Nothing here computes.  An architecture turns its typed configuration into a
ModelSpec; the weight loader, the random-weights writer, the cache and the engine
all work from the ModelSpec alone and never ask which architecture it came from.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple


@dataclass(frozen=True)
class TensorSpec:
    """One named tensor of a part.

    init: how the random-weights mode fills it: "normal" (N(0, std)),
    "one_plus_normal" (1 + N(0, std)) or "zeros".
    dtype: "float" follows the run's weight dtype; "int32" is an integer table.
    """
    shape: Tuple[int, ...]
    init: str = "normal"
    std: float = 0.02
    dtype: str = "float"


@dataclass(frozen=True)
class PartSpec:
    """A part by kind and parameters; params may hold further PartSpecs."""
    kind: str
    params: Dict = field(default_factory=dict)


@dataclass(frozen=True)
class KVNeed:
    """A mixer that keeps keys and values for every position (window: only the last
    `window` positions are ever read)."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a fixed-size state per sequence (zero at start).  dtype: "float32",
    "bfloat16" or "int32"."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


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
