"""Several feed-forwards of the same input, added: a mixture of routed experts beside a shared expert that every
token runs, say.  The first part's output is wanted in 32-bit ([T, width] float32, as RoutedExperts gives it); every
further part adds its own into it, in its last product where the backend does that, and the sum goes on in 32-bit."""
from __future__ import annotations

from ..kernels.api import Normed, Sink
from .base import FeedForward, register_feed_forward


@register_feed_forward("summed")
class SummedFF(FeedForward):
    def __init__(self, parts):
        self.parts = list(parts)
        if not self.parts:
            raise ValueError("a sum of feed-forwards needs at least one")

    def children(self):
        return list(self.parts)

    def forward(self, x, step, add_to=None):
        import torch
        if isinstance(x, Normed):
            x = x.materialize()
        total = self.parts[0].forward(x, step)
        if total.dtype != torch.float32:
            total = total.float()
        for part in self.parts[1:]:
            y = part.forward(x, step, add_to=Sink(total))
            if isinstance(y, torch.Tensor):     # the part (or the backend) left the add to the caller
                total.add_(y.float())
        return total
