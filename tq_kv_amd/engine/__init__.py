from ..native import GenerationError, StepError
from .engine import Engine
from .generate import generate, plan_batches
from .model import Model

__all__ = ["Engine", "StepError", "Model", "GenerationError", "generate", "plan_batches"]
