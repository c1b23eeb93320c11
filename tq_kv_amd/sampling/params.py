"""Generation parameters with the reference's names and defaults
(GenerationParams, src/engine.rs:29-49; the flags of `tq chat`, src/main.rs:56-69)."""
from dataclasses import dataclass


@dataclass
class GenerationParams:
    max_tokens: int = 512          # -n / --max-tokens
    temperature: float = 0.7       # -t / --temperature; <= 0 is greedy (src/engine.rs:353-354)
    top_p: float = 0.9             # --top-p
    top_k: int = 40                # --top-k; 0 switches it off
    repeat_penalty: float = 1.1    # --repeat-penalty; 1.0 switches it off (src/engine.rs:403)
    seed: int = 0

    def __post_init__(self):
        if self.max_tokens < 0:
            raise ValueError("max_tokens must not be negative, got %r" % (self.max_tokens,))
        if self.top_k < 0:
            raise ValueError("top_k must not be negative, got %r" % (self.top_k,))
        if not self.top_p > 0.0:
            raise ValueError("top_p must be positive, got %r" % (self.top_p,))
        if not self.repeat_penalty > 0.0:
            raise ValueError("repeat_penalty must be positive, got %r" % (self.repeat_penalty,))

    @property
    def greedy(self):
        return self.temperature <= 0.0

    def __repr__(self):
        return ("GenerationParams(max_tokens=%d, temperature=%g, top_p=%g, top_k=%d, repeat_penalty=%g, seed=%d)"
                % (self.max_tokens, self.temperature, self.top_p, self.top_k, self.repeat_penalty, self.seed))
