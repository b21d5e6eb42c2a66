"""Per-request sampling options (reference sampling_params.py:3-11)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0        # 0 = greedy (argmax); otherwise logits are divided by it
    max_tokens: int = 64            # most tokens to generate
    ignore_eos: bool = False        # keep generating past the end-of-sequence token
    seed: int | None = None         # None: the engine's seed; the noise also depends on the request and the output index

    def __post_init__(self):
        if not self.temperature >= 0:
            raise ValueError("temperature must be >= 0")
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be >= 1")
