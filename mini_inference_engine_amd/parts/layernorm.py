"""Layer norm with weight and bias, with the residual add folded in.

y = (x - mean) / sqrt(var + eps) * weight + bias, mean and var (the mean of the squared deviations) of the stream's
row after the pending branch output has been added to it.  The stream and every intermediate are 32-bit (weight and
bias are turned to 32-bit once, when the weights are loaded); y is rounded once.  ``add_branch`` is the other place a
block may put a norm: on a sublayer's output, before it is added to the stream.
"""
from __future__ import annotations

from ..kernels.api import Normed, NormedBranch, NormedLayer, StreamCopy
from .base import Norm, ParamSpec, register_norm


@register_norm("layernorm")
class LayerNorm(Norm):
    def __init__(self, width: int, eps: float, weight_name: str, bias_name: str | None = None):
        self.width = int(width)
        self.eps = float(eps)
        self.weight_name = weight_name
        self.bias_name = bias_name if bias_name is not None else weight_name + ".b"
        self.weight = self.bias = None

    def params(self):
        return [ParamSpec.single("weight", self.weight_name, (self.width,), init="scale"),
                ParamSpec.single("bias", self.bias_name, (self.width,))]

    def prepare(self, device, dtype):
        import torch
        for attr in ("weight", "bias"):
            t = getattr(self, attr)
            if t is not None and t.dtype != torch.float32:
                setattr(self, attr, t.float().contiguous())

    def _pending(self, x, residual):
        """What is still to be added to the stream before this norm reads it, as a tensor or None."""
        if isinstance(x, NormedBranch):
            x.resolve()
            return None
        if isinstance(x, Normed):       # a block of another kind before this one: its last add may be pending
            return x.pending
        if isinstance(x, StreamCopy):
            return None
        return x

    def lazy(self, x, residual, rows=None):
        return NormedLayer(self.ops, self._pending(x, residual), residual, self.weight, self.bias, self.eps, rows)

    def forward(self, x, residual, rows=None, out_dtype=None):
        return self.ops.add_layernorm(self._pending(x, residual), residual, self.weight, self.bias, self.eps,
                                      out_dtype=out_dtype, rows=rows)

    def add_branch(self, y, stream, then=None):
        """stream += this norm of y (a sublayer's output).  ``then`` (a Norm): also returns that norm of the updated
        stream in the activation dtype; where it is a layer norm too, both happen in one backend call."""
        if isinstance(then, LayerNorm):
            return self.ops.branch_layernorm_add(y, stream, self.weight, self.bias, self.eps,
                                                 next_norm=(then.weight, then.bias, then.eps))
        self.ops.branch_layernorm_add(y, stream, self.weight, self.bias, self.eps)
        return None if then is None else then.forward(None, stream)
