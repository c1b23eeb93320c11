"""Architectures: each file registers a configuration class and a ModelSpec builder."""
from ..config.registry import register_architecture
from . import qwen2

register_architecture("Qwen2ForCausalLM", qwen2.Qwen2Config, qwen2.build_spec, model_types=("qwen2",))
