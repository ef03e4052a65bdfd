"""RMSNorm with the residual add folded in.

y = weight * x * rsqrt(mean(x^2) + eps), taken of the stream after the pending
branch output has been added to it (inference_engine/kernels/rmsnorm.py:56-65;
used at inference_engine/model.py:171,179,184).  The weight is a plain multiplier, or, with
``one_plus``, stored around zero and applied as 1 + weight (the sum is made once, in 32-bit, when
the weights are loaded).  The stream and every intermediate are 32-bit; y is rounded once.
"""
from __future__ import annotations

from ..kernels.api import Normed, NormedBranch, StreamCopy
from .base import Norm, ParamSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, width: int, eps: float, weight_name: str, one_plus: bool = False):
        self.width = int(width)
        self.eps = float(eps)
        self.weight_name = weight_name
        self.one_plus = bool(one_plus)
        self.weight = None
        self._summed = False

    def params(self):
        return [ParamSpec.single("weight", self.weight_name, (self.width,), init="weight" if self.one_plus else "scale")]

    def prepare(self, device, dtype):
        if self.one_plus and not self._summed:
            self._summed = True
            self.weight = (1.0 + self.weight.float()).contiguous()

    def lazy(self, x, residual, rows=None):
        if isinstance(x, NormedBranch):     # the block before left a normed branch output to be added: it is added now
            x = x.resolve()
        if isinstance(x, Normed):
            # the product before this norm already added its result to the stream (and may have prepared
            # this very norm's input)
            if x.weight is self.weight and x.residual is residual and x.eps == self.eps and x.pending is None:
                return x if rows is None else x.with_rows(rows)
            x = None
        if isinstance(x, StreamCopy):       # the block before left nothing pending
            x = None
        return Normed(self.ops, x, residual, self.weight, self.eps, rows)

    def forward(self, x, residual, rows=None, out_dtype=None):
        if isinstance(x, (Normed, NormedBranch, StreamCopy)):
            return self.lazy(x, residual, rows).materialize(out_dtype)
        return self.ops.add_rmsnorm(x, residual, self.weight, self.eps, out_dtype=out_dtype, rows=rows)

    def add_branch(self, y, stream, then=None):
        """stream += this norm of y (a sublayer's output).  ``then`` (a Norm): also returns that norm of the updated
        stream in the activation dtype."""
        self.ops.branch_norm_add(y, stream, self.weight, self.eps, copy=False)
        return None if then is None else then.forward(None, stream)
