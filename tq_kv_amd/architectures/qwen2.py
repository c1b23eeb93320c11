"""Qwen2ForCausalLM: the dense decoder the reference runs through src/models/turbo_generic.rs.

Which config.json keys the architecture reads and how they become a ModelSpec is
csrc/engine/qwen2.cpp's; this is the typed configuration as Python sees it.
"""
from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..config.registry import config_class, spec_from_dict


@config_class("Qwen2ForCausalLM")
@dataclass(frozen=True)
class Qwen2Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    use_sliding_window: bool
    sliding_window: Optional[int]
    max_window_layers: Optional[int]
    eos_token_ids: Tuple[int, ...] = field(default=())

    @classmethod
    def from_typed(cls, typed):
        """From what the engine library made of a config.json (every key, defaults filled in)."""
        typed = dict(typed)
        typed["eos_token_ids"] = tuple(typed.get("eos_token_ids") or ())
        return cls(**typed)

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        from ..config.registry import config_from_dict
        return config_from_dict(dict(raw, architectures=["Qwen2ForCausalLM"]), where)[1]

    def to_dict(self):
        """The config.json that reads back as this configuration."""
        d = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
             "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
             "intermediate_size": self.intermediate_size, "num_hidden_layers": self.num_hidden_layers,
             "num_attention_heads": self.num_attention_heads, "num_key_value_heads": self.num_key_value_heads,
             "head_dim": self.head_dim, "rms_norm_eps": self.rms_norm_eps, "rope_theta": self.rope_theta,
             "max_position_embeddings": self.max_position_embeddings,
             "tie_word_embeddings": self.tie_word_embeddings, "use_sliding_window": self.use_sliding_window}
        if self.use_sliding_window:
            d["sliding_window"] = self.sliding_window
            d["max_window_layers"] = self.max_window_layers
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d

    def layer_window(self, layer):
        """Layer l is windowed iff use_sliding_window and l >= max_window_layers; a windowed
        query at position i sees the sliding_window keys i-W < j <= i."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None


def build_spec(cfg: Qwen2Config):
    return spec_from_dict(cfg.to_dict())
