"""Dense gated feed-forward (reference models/qwen3.py:42-51)."""
from __future__ import annotations

from ..kernels import ops
from .base import FeedForward, PendingNorm, register_part
from .linear import Linear


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)); gate and up are one packed product with gate's rows first
    (reference layers/linear.py:29-45, layers/activation.py:5-7)."""

    takes_pending_norm = True      # x goes to the packed product and nowhere else

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.add_child("gate_up", Linear(hidden_size, 2 * intermediate_size,
                                         parts={"gate": intermediate_size, "up": intermediate_size}))
        self.add_child("down", Linear(intermediate_size, hidden_size))

    def forward(self, x):
        rows = x.x.shape[-2] if isinstance(x, PendingNorm) else x.shape[0]
        if ops.gated_linear_rows(rows, self.gate_up.weight):
            # few rows (or a few hundred over a small weight): the gating in the gate/up product's epilogue (every gate formed
            # once), a plain down product
            return self.down.forward(self.gate_up.forward(x, gated=True), allow_partials=True)
        gu = self.gate_up.forward(x)
        return ops.silu_mul_linear(gu, self.down.weight, allow_partials=True)
