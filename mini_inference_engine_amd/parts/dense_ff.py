"""Dense feed-forward without a gate: down(act(up(x))), act the square of relu unless the constructor names another
of kernels.api.ACTIVATIONS.  ``tensor_names``: how the checkpoint calls the two matrices after the prefix.
``float32_output``: hand the caller the second product's 32-bit sums (where a norm reads them next)."""
from __future__ import annotations

from .base import FeedForward, ParamSpec, register_feed_forward


@register_feed_forward("dense")
class DenseFF(FeedForward):
    def __init__(self, width: int, inner: int, prefix: str, activation: str = "relu2", tensor_names=("up", "down"),
                 float32_output: bool = False):
        from ..kernels.api import ACTIVATIONS
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: one of {ACTIVATIONS}")
        self.width, self.inner, self.prefix, self.activation = int(width), int(inner), prefix, activation
        self.tensor_names = tuple(tensor_names)
        self.float32_output = bool(float32_output)
        self.w_up = self.w_down = None

    def params(self):
        up, down = self.tensor_names
        return [ParamSpec.single("w_up", f"{self.prefix}.{up}", (self.inner, self.width)),
                ParamSpec.single("w_down", f"{self.prefix}.{down}", (self.width, self.inner))]

    def forward(self, x, step, add_to=None):
        a = self.ops.linear_act(x, self.w_up, self.activation)
        if self.float32_output and add_to is None:
            import torch
            return self.ops.linear(a, self.w_down, out_dtype=torch.float32)
        return self.ops.linear(a, self.w_down, add_to=add_to)
