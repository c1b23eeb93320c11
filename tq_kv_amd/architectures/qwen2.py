"""Qwen2ForCausalLM: the dense decoder the reference runs through
src/models/turbo_generic.rs (grouped-query attention with q/k/v bias and no output
bias, gated-SiLU feed-forward, RMSNorm before mixer and feed-forward, rotary
positions in the halves layout, tied or untied head).

This file holds what is particular to the architecture: which config.json keys it
reads and how they become a ModelSpec with the HF tensor names the reference loads
by (:2075-2126).  Nothing here computes.
"""
from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..config.base import ConfigError, KeyReader
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, Run


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
    def from_dict(cls, raw, where="config.json"):
        """Keys as the reference reads them (src/models/turbo_generic.rs:2013-2030), plus
        those it takes from tensor shapes or presence (vocab_size, intermediate_size,
        tie_word_embeddings) and the sliding-window keys.  Sizes have no defaults here;
        num_key_value_heads and head_dim default as the reference's do (:2014, :2020-2022)."""
        r = KeyReader(raw, where)
        nh = r.integer("num_attention_heads", minimum=1)
        hidden = r.integer("hidden_size", minimum=1)
        nkv = r.integer("num_key_value_heads", default=nh, minimum=1)
        head_dim = r.integer("head_dim", default=None, minimum=1)
        if head_dim is None:
            if hidden % nh:
                raise ConfigError("%s: hidden_size %d is not a multiple of num_attention_heads %d and no head_dim is given"
                                  % (where, hidden, nh))
            head_dim = hidden // nh
        if nh % nkv:
            raise ConfigError("%s: num_attention_heads %d is not a multiple of num_key_value_heads %d" % (where, nh, nkv))
        if head_dim % 2:
            raise ConfigError("%s: head_dim %d must be even for rotary positions" % (where, head_dim))
        act = r.string("hidden_act", default="silu")
        if act != "silu":
            raise ConfigError("%s: hidden_act '%s' is not supported (only 'silu')" % (where, act))
        if raw.get("rope_scaling") is not None:
            raise ConfigError("%s: rope_scaling is not supported (must be null or absent)" % where)
        layers = r.integer("num_hidden_layers", minimum=1)
        use_window = r.boolean("use_sliding_window", default=False)
        window = max_window_layers = None
        if use_window:
            window = r.integer("sliding_window", minimum=1)
            max_window_layers = r.integer("max_window_layers", minimum=0)
        return cls(
            vocab_size=r.integer("vocab_size", minimum=1), hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size", minimum=1), num_hidden_layers=layers,
            num_attention_heads=nh, num_key_value_heads=nkv, head_dim=head_dim,
            rms_norm_eps=r.number("rms_norm_eps", positive=True), rope_theta=r.number("rope_theta", positive=True),
            max_position_embeddings=r.integer("max_position_embeddings", minimum=1),
            tie_word_embeddings=r.boolean("tie_word_embeddings", default=False),
            use_sliding_window=use_window, sliding_window=window, max_window_layers=max_window_layers,
            eos_token_ids=tuple(r.token_ids("eos_token_id")))

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


def build_spec(cfg: Qwen2Config) -> ModelSpec:
    position = PartSpec("rotary", {"theta": cfg.rope_theta, "rot_dim": cfg.head_dim,
                                   "max_positions": cfg.max_position_embeddings, "style": "halves"})
    norm = PartSpec("rms_norm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    feed_forward = PartSpec("gated_silu", {"hidden": cfg.hidden_size, "inter": cfg.intermediate_size})
    layers = []
    for l in range(cfg.num_hidden_layers):
        mixer = PartSpec("attention", {
            "hidden": cfg.hidden_size, "n_heads": cfg.num_attention_heads, "n_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "qkv_bias": True, "out_bias": False, "window": cfg.layer_window(l),
            "scale": None, "position": position})
        block = PartSpec("pre_norm", {
            "mixer": mixer, "feed_forward": feed_forward, "mixer_norm": norm, "ff_norm": norm,
            "names": {"mixer": "self_attn.", "feed_forward": "mlp.", "mixer_norm": "input_layernorm.",
                      "ff_norm": "post_attention_layernorm."}})
        layers.append(LayerSpec(prefix="model.layers.%d." % l, block=block))
    return ModelSpec(
        architecture="Qwen2ForCausalLM", vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
        max_positions=cfg.max_position_embeddings, embedding_name="model.embed_tokens.weight",
        layers=layers, order=[Run(l) for l in range(cfg.num_hidden_layers)],
        final_norm=norm, final_norm_prefix="model.norm.",
        head_name=None if cfg.tie_word_embeddings else "lm_head.weight",
        eos_token_ids=cfg.eos_token_ids)
