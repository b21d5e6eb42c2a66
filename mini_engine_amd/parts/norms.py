"""RMSNorm, fused with the residual sum (reference layers/layernorm.py:5-24)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Norm, ParamSpec, register_part


@register_part("norm", "rms")
class RMSNorm(Norm):
    """y = weight * r / sqrt(mean(r^2) + eps), r = x + residual.

    The weight is a plain multiplier (reference layers/layernorm.py:16). The sum, the mean
    of squares and the scaling are float32; the residual stream is returned in float32.
    """

    accepts_partials = True

    def __init__(self, size: int, eps: float):
        super().__init__()
        self.size = size
        self.eps = eps
        self.add_param("weight", ParamSpec((size,), init="norm", dtype="float32"))
        self.out_dtype = torch.float32

    def finalize(self, device, dtype, max_positions):
        self.out_dtype = dtype

    def forward(self, x, residual, want_residual: bool = True):
        return ops.rms_norm(x, self.weight, self.eps, residual, self.out_dtype, want_residual)

    def linear_behind(self, x, residual, weight, out_dtype=None, gated: bool = False):
        if weight.dtype != self.out_dtype or not ops.norm_linear_fuses(x, weight):
            return None
        return ops.norm_linear(x, residual, self.weight, self.eps, weight, out_dtype, gated=gated)
