"""Token embedding and output head (reference layers/embed_head.py:5-23)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Head, ParamSpec, Part


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, hidden_size: int):
        super().__init__()
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.add_param("weight", ParamSpec((vocab_size, hidden_size), init="matrix", dtype="compute"))

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return ops.gather_rows(self.weight, token_ids)


class LMHead(Head):
    """logits = x . W^T in float32. When tied, W is the embedding matrix itself: the same
    tensor, not a copy (reference models/qwen3.py:107-109)."""

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding | None = None):
        super().__init__()
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied_to = tied_to
        if tied_to is None:
            self.add_param("weight", ParamSpec((vocab_size, hidden_size), init="matrix", dtype="compute"))

    def matrix(self) -> torch.Tensor:
        return self.tied_to.weight if self.tied_to is not None else self.weight

    def forward(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """`out`: a float32 [rows, vocab] tensor to write the logits into (a step with a fixed layout
        keeps one)."""
        return ops.linear(x, self.matrix(), torch.float32, out=out)
