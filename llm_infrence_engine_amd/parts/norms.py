"""RMS norm: y = (offset + weight) * x * rsqrt(mean(x^2) + eps), computed in float on the float residual stream.
``offset`` is 0 for a scale stored as it is and 1 for one stored around zero; the sum is formed once, in float,
when the weights are loaded.

The reference computes the reduction in float, casts back and multiplies by the weight in the model's
type (src/miniserve/model.py:69-73); here the weight is applied in float too and the result is rounded once.
"""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Norm, register_part


class RMSNorm(Norm):
    def __init__(self, prefix: str, size: int, eps: float, offset: float = 0.0, name: str = "weight"):
        self.prefix, self.size, self.eps, self.offset, self.name = prefix, size, eps, float(offset), name

    def tensor_specs(self):
        # a scale stored around zero is drawn around zero by the random-weights mode too
        return [TensorSpec(self.prefix + self.name, (self.size,), "bias" if self.offset else "norm")]

    def load(self, get, rt):
        self.rt = rt
        self.weight = get(self.tensor_specs()[0])
        if self.offset:
            self.weight = (self.weight + self.offset).contiguous()

    def forward(self, x, delta=None, rows=None, write_back=True):
        n = x.shape[0] if rows is None else rows.numel()
        out = self.rt.empty(n, self.size)
        return ops.rms_norm(x, self.weight, self.eps, out, delta=delta, rows=rows, write_back=write_back)


    def forward_pair(self, other: "RMSNorm", x, delta=None):
        """(self's norm, ``other``'s norm) of the same rows of x (+ delta, kept in x): one pass when the two differ in
        their scales only, else two."""
        if not isinstance(other, RMSNorm) or other.size != self.size or other.eps != self.eps or \
                (delta is not None and delta.dim() != 2):
            first = self.forward(x, delta)
            return first, other.forward(x)
        n = x.shape[0]
        return ops.rms_norm_pair(x, self.weight, other.weight, self.eps, self.rt.empty(n, self.size),
                                 self.rt.empty(n, self.size), delta=delta)

    def lazy(self, x, delta=None, rows=None, write_back=True):
        """As ``forward``, for a consumer that can fold the norm into its first product: with few rows in
        bfloat16 the addend is summed into x now and the normalisation is left to that product."""
        n = x.shape[0] if rows is None else rows.numel()
        if self.rt.dtype != torch.bfloat16 or n > ops.SKINNY_MAX_ROWS or self.size % 8 or (delta is not None and not write_back):
            return self.forward(x, delta, rows, write_back)
        if delta is not None:
            ops.residual_add(x, delta)
        return linear.LazyNorm(x, self.weight, self.eps, self.rt.dtype, rows)


register_part("norm", "rms_norm", RMSNorm)
