"""Feed-forward of routed experts: each token runs the ``top`` experts its router prefers.

Router logits z = W_r x (+ b_r) in 32-bit.  Two ways from logits to choice and shares:
  ``shares_over="chosen"``  the ``top`` largest logits are chosen; shares are the softmax over those alone;
  ``shares_over="all"``     scores s = softmax(z) over every router output; chosen are the ``top`` largest of
                            s + c (``choice_bias``: a checkpoint vector c that steers the choice only); shares are the
                            chosen outputs' s, not renormalised, or, with ``renormalise``, divided by their sum + 1e-20.
An expert is W_down act(W_up x) without biases (act: the square of relu unless another of kernels.api.ACTIVATIONS
is named), or, with ``gated=(limit, alpha)``, W_down (g * sigmoid(alpha g) * (u + 1)) with g = min(W_gate x, limit)
and u = clamp(W_up x, -limit, limit); ``gated=(limit, alpha, shift)`` adds ``shift`` to u instead of 1, and
``gated="silu"`` is the plain gated unit W_down (silu(W_gate x) * W_up x) (no clamp, alpha 1, shift 0).  The last ``identity`` router outputs have no tensors: they stand for experts
that return x itself.  The output is the share-weighted sum.  The experts' matrices are kept stacked, [experts, ff,
width] (gate rows before up rows, [experts, 2 ff, width], when gated) and [experts, width, ff], so that one grouped
product serves all of them.
"""
from __future__ import annotations

from .base import FeedForward, ParamSpec, register_feed_forward


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    def __init__(self, width: int, inner: int, num_experts: int, top: int, prefix: str, activation: str = "relu2",
                 router_bias: bool = True, tensor_names=None, shares_over: str = "chosen", choice_bias: bool = False,
                 gated=None, identity: int = 0, renormalise: bool = False):
        from ..kernels.api import ACTIVATIONS
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: one of {ACTIVATIONS}")
        if shares_over not in ("chosen", "all"):
            raise ValueError(f"shares_over {shares_over!r}: chosen or all")
        if identity < 0 or num_experts < 0 or not 1 <= top <= num_experts + identity:
            raise ValueError(f"top {top} of {num_experts} experts and {identity} identity outputs")
        if choice_bias and shares_over != "all":
            raise ValueError("a choice bias steers the choice among scores over all outputs (shares_over='all')")
        self.width, self.inner, self.num_experts, self.top = int(width), int(inner), int(num_experts), int(top)
        self.identity = int(identity)
        self.prefix, self.activation, self.router_bias = prefix, activation, bool(router_bias)
        self.shares_over, self.has_choice_bias = shares_over, bool(choice_bias)
        if renormalise and shares_over != "all":
            raise ValueError("shares over the chosen outputs alone already sum to one (renormalise goes with shares_over='all')")
        self.renormalise = bool(renormalise)
        if gated == "silu":
            gated = (float("inf"), 1.0, 0.0)
        self.gated = None if gated is None else tuple(float(g) for g in gated)
        if self.gated is not None and len(self.gated) not in (2, 3):
            raise ValueError("gated: (limit, alpha), (limit, alpha, shift) or 'silu'")
        self.names = dict(dict(router="router", router_bias="router.b", expert="e{e}", up="up", down="down", gate="gate",
                               choice_bias="correction"), **(tensor_names or {}))
        self.b_router = self.choice_bias = self.w_up = self.w_down = None

    def params(self):
        n, p, w, f, E = self.names, self.prefix, self.width, self.inner, self.num_experts
        R = E + self.identity
        expert = lambda e, m: f"{p}.{n['expert'].format(e=e)}.{n[m]}"        # noqa: E731
        specs = [ParamSpec.single("w_router", f"{p}.{n['router']}", (R, w))]
        if E:
            if self.gated is None:
                specs.append(ParamSpec.stacked("w_up", [(expert(e, "up"), (f, w)) for e in range(E)]))
            else:
                specs.append(ParamSpec.stacked("w_up", [(expert(e, m), (f, w)) for e in range(E) for m in ("gate", "up")]))
            specs.append(ParamSpec.stacked("w_down", [(expert(e, "down"), (w, f)) for e in range(E)]))
        if self.router_bias:
            specs.append(ParamSpec.single("b_router", f"{p}.{n['router_bias']}", (R,), init="zeros"))
        if self.has_choice_bias:
            specs.append(ParamSpec.single("choice_bias", f"{p}.{n['choice_bias']}", (R,)))
        return specs

    def prepare(self, device, dtype):
        first = not getattr(self, "_prepared", False)
        self._prepared = True
        for attr in ("b_router", "choice_bias"):        # router logits and scores are 32-bit
            t = getattr(self, attr, None)
            if t is not None:
                setattr(self, attr, t.float().contiguous())
        if first and self.gated is not None and self.num_experts:
            # the kernels may want a channel's gate row and up row near each other: blocks of n gate rows, n up rows
            self.glu_block = n = int(self.ops.glu_rows_block(self.inner))
            if n:
                E, f, w = self.num_experts, self.inner, self.width
                self.w_up = self.w_up.view(E, 2, f // n, n, w).transpose(1, 2).contiguous().view(E * 2 * f, w)

    def forward(self, x, step, add_to=None):
        import torch
        ops, E = self.ops, self.num_experts
        logits = ops.linear(x, self.w_router, out_dtype=torch.float32)
        if self.renormalise:
            experts, shares = ops.route_topk(logits, self.b_router if self.router_bias else None, self.top,
                                             over=self.shares_over, choice_bias=self.choice_bias, renormalise=True)
        else:
            experts, shares = ops.route_topk(logits, self.b_router if self.router_bias else None, self.top,
                                             over=self.shares_over, choice_bias=self.choice_bias)
        rows = self.inner if self.gated is None else 2 * self.inner
        w_up = None if not E else self.w_up.view(E, rows, self.width)
        w_down = None if not E else self.w_down.view(E, self.width, self.inner)
        if self.gated is None or not getattr(self, "glu_block", 0):
            return ops.routed_experts(x, experts, shares, w_up, w_down, self.activation, gated=self.gated,
                                      identity_from=E if self.identity else None)
        return ops.routed_experts(x, experts, shares, w_up, w_down, self.activation, gated=self.gated,
                                  identity_from=E if self.identity else None, glu_block=self.glu_block)
