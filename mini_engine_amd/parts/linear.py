"""Bias-free linear maps with weights stored [out, in] (reference layers/linear.py:4-45)."""
from __future__ import annotations

from ..kernels import ops
from .base import ParamSpec, Part, PendingNorm


class Linear(Part):
    """y = x . W^T. `parts` names row blocks of W that are stored separately in a checkpoint
    (packed projections: reference layers/linear.py:13-22,37-42); the loader concatenates them."""

    def __init__(self, in_features: int, out_features: int, parts: dict | None = None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.row_blocks = dict(parts) if parts else None   # name -> rows, in storage order
        if self.row_blocks is not None and sum(self.row_blocks.values()) != out_features:
            raise ValueError("row blocks do not add up to out_features")
        self.add_param("weight", ParamSpec((out_features, in_features), init="matrix", dtype="compute"))

    def forward(self, x, out_dtype=None, allow_partials: bool = False, gated: bool = False):
        """With allow_partials the result may be float32 partial sums [P, M, N] (a product whose K
        range was split over workgroups); the consumer, a norm, adds them. x may be a `PendingNorm`:
        the norm then runs inside the product where there is a kernel for that, else in front of it.
        gated: this is a packed gate/up map (gate's rows first) and the result is silu(gate) * up,
        [M, out_features / 2] (reference layers/activation.py:5-7), from the product's own epilogue where
        there is a kernel for that, else from the activation kernel behind it."""
        if isinstance(x, PendingNorm):
            y = x.into_linear(self.weight, out_dtype, gated)
            if y is not None:
                return y
            x = x.value()
        if not gated:
            return ops.linear(x, self.weight, out_dtype, allow_partials)
        if ops.gated_linear_fuses(x, self.weight):
            return ops.gated_linear(x, self.weight)
        return ops.silu_and_mul(ops.linear(x, self.weight))
