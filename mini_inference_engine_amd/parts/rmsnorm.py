"""RMSNorm with the residual add folded in.

y = weight * x * rsqrt(mean(x^2) + eps), taken of the stream after the pending
branch output has been added to it (inference_engine/kernels/rmsnorm.py:56-65;
used at inference_engine/model.py:171,179,184).  The weight is a plain multiplier.
The stream and every intermediate are 32-bit; y is rounded once.
"""
from __future__ import annotations

from ..kernels.api import Normed
from .base import Norm, ParamSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, width: int, eps: float, weight_name: str):
        self.width = int(width)
        self.eps = float(eps)
        self.weight_name = weight_name
        self.weight = None

    def params(self):
        return [ParamSpec.single("weight", self.weight_name, (self.width,), init="scale")]

    def lazy(self, x, residual, rows=None):
        if isinstance(x, Normed):
            # the product before this norm already added its result to the stream (and may have prepared
            # this very norm's input)
            if x.weight is self.weight and x.residual is residual and x.eps == self.eps and x.pending is None:
                return x if rows is None else x.with_rows(rows)
            x = None
        return Normed(self.ops, x, residual, self.weight, self.eps, rows)

    def forward(self, x, residual, rows=None, out_dtype=None):
        if isinstance(x, Normed):
            return self.lazy(x, residual, rows).materialize(out_dtype)
        return self.ops.add_rmsnorm(x, residual, self.weight, self.eps, out_dtype=out_dtype, rows=rows)
