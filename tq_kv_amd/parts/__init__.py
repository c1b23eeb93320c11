"""Parts that layers are put together from: norms, position encodings, mixers, feed-forwards and
block arrangements, each chosen by kind from the engine library's registry; kinds written in
Python join it through `register`."""
from .registry import BuildEnv, Part, PartHandle, known, register
from .spec import KVNeed, LayerSpec, ModelSpec, PartSpec, Run, StateNeed, TensorSpec

__all__ = ["BuildEnv", "Part", "PartHandle", "known", "register", "KVNeed", "LayerSpec", "ModelSpec", "PartSpec", "Run",
           "StateNeed", "TensorSpec"]
