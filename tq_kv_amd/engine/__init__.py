from .engine import Engine, StepError
from .generate import GenerationError, generate, plan_batches
from .model import Model

__all__ = ["Engine", "StepError", "Model", "GenerationError", "generate", "plan_batches"]
