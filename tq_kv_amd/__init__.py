"""tq_kv_amd: a small inference library for MI355X (gfx950) after the generation path
of onur-gokyildiz-bhi/tq-kv: from a model folder (config.json + safetensors) or a
seeded random-weights shape to generated tokens on one GPU.

    from tq_kv_amd import Model, Engine, GenerationParams, generate
    model = Model.random("tiny:a", seed=0, dtype="float32")
    engine = Engine(model, max_tokens=4096)
    out = generate(engine, [[1, 2, 3]], GenerationParams(max_tokens=8, temperature=0.0))
"""
from . import architectures  # noqa: F401  (the typed configurations as Python sees them)
from .config import ConfigError
from .engine import Engine, GenerationError, Model, StepError, generate
from .policy import POLICY
from .sampling import GenerationParams

__all__ = ["Model", "Engine", "StepError", "ConfigError", "GenerationError", "GenerationParams", "generate", "POLICY"]
__version__ = "0.1.0"
