"""Rotary position encoding with half-split pairs (reference layers/rotary_embedding.py:5-25)."""
from __future__ import annotations

import torch

from .base import PositionEncoding, register_part


@register_part("position_encoding", "rotary")
class RotaryEmbedding(PositionEncoding):
    """angle[p, i] = p * theta^(-2i/D); the pair (x_i, x_{i+D/2}) is rotated by angle[p, i].

    One instance is shared by all layers that use it (reference models/qwen3.py:81). The
    angles, their cos/sin and the rotation are float32 (the reference rounds cos/sin to the
    activations' dtype, layers/rotary_embedding.py:21-22). The table is [P, D/2, 2] with
    (cos, sin) adjacent, the form the fused query/key kernel reads.
    """

    def __init__(self, head_dim: int, theta: float):
        super().__init__()
        if head_dim % 2:
            raise ValueError("rotary encoding needs an even head size")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.table = None

    def finalize(self, device, dtype, max_positions):
        if self.table is not None and self.table.shape[0] >= max_positions and self.table.device == torch.device(device):
            return
        half = self.head_dim // 2
        # same expression as the reference: 1 / theta^(2i/D), float32 throughout
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim))
        t = torch.arange(max_positions, dtype=torch.float32)
        ang = torch.outer(t, inv_freq)                      # [P, D/2]
        self.table = torch.stack((ang.cos(), ang.sin()), dim=-1).contiguous().to(device)
        assert self.table.shape == (max_positions, half, 2)

    def rotary_table(self):
        return self.table

    def apply(self, q, k, positions):
        """Unfused form for mixers that do not use the fused kernel. q: [T, Hq, D], k: [T, Hkv, D]."""
        cs = self.table[positions.long()]                   # [T, D/2, 2]
        c, s = cs[..., 0].unsqueeze(1), cs[..., 1].unsqueeze(1)
        half = self.head_dim // 2
        for x in (q, k):
            x1, x2 = x[..., :half].float(), x[..., half:].float()
            lo, hi = x1 * c - x2 * s, x2 * c + x1 * s      # both halves before either is overwritten
            x[..., :half] = lo.to(x.dtype)
            x[..., half:] = hi.to(x.dtype)
