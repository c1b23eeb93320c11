"""Parts that layers are put together from: norms, position encodings, mixers,
feed-forwards and block arrangements, each chosen by kind from a registry."""
from . import attention, block, feed_forward, norms, position  # noqa: F401  (registers the kinds)
from .registry import BuildEnv, Part, known, register
from .spec import KVNeed, LayerSpec, ModelSpec, PartSpec, Run, StateNeed, TensorSpec

__all__ = ["BuildEnv", "Part", "known", "register", "KVNeed", "LayerSpec", "ModelSpec", "PartSpec", "Run",
           "StateNeed", "TensorSpec"]
