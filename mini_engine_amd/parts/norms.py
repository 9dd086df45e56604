"""RMSNorm, fused with the residual sum (reference layers/layernorm.py:5-24)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Norm, ParamSpec, register_part


def _around_zero(shape, generator, device):
    return torch.rand(shape, generator=generator, dtype=torch.float32, device=device) * 0.2 - 0.1


@register_part("norm", "rms")
class RMSNorm(Norm):
    """y = weight * r / sqrt(mean(r^2) + eps), r = x + residual.

    The weight is a plain multiplier (reference layers/layernorm.py:16). The sum, the mean
    of squares and the scaling are float32; the residual stream is returned in float32.
    """

    accepts_partials = True

    def __init__(self, size: int, eps: float, one_plus: bool = False):
        """`one_plus`: the stored weight lies around zero and the multiplier is 1 + weight (the sum is formed
        once, in float32, when the weights are bound)."""
        super().__init__()
        self.size = size
        self.eps = eps
        self.one_plus = bool(one_plus)
        self._shifted = False
        self.add_param("weight", ParamSpec((size,), init=_around_zero if one_plus else "norm", dtype="float32"))
        self.out_dtype = torch.float32

    def set_param(self, local, tensor):
        super().set_param(local, tensor)
        self._shifted = False

    def finalize(self, device, dtype, max_positions):
        self.out_dtype = dtype
        if self.one_plus and not self._shifted:
            self.weight = self.weight + 1.0
            self._shifted = True

    def add_to(self, y, stream):
        """The norm on a sublayer's output: stream + weight * y / rms(y), all in float32. y: [T, n] or float32
        partial sums [P, T, n]. -> (the new stream in the compute dtype, the new stream in float32)."""
        return ops.add_rms_norm(y, self.weight, self.eps, stream, self.out_dtype)

    def add_terms(self, terms, stream):
        """`add_to` on a weighted sum that has not been formed yet: `terms.terms` lists (rows or float32 partial sums,
        scale, bias or None); sum, norm and residual sum are one kernel (`ops.weighted_sum`)."""
        return ops.weighted_sum(terms.terms, self.weight, self.eps, stream, self.out_dtype)

    def forward(self, x, residual, want_residual: bool = True):
        return ops.rms_norm(x, self.weight, self.eps, residual, self.out_dtype, want_residual)

    def linear_behind(self, x, residual, weight, out_dtype=None, gated: bool = False):
        if weight.dtype != self.out_dtype or not ops.norm_linear_fuses(x, weight):
            return None
        return ops.norm_linear(x, residual, self.weight, self.eps, weight, out_dtype, gated=gated)
