"""Gated linear attention: a linear-attention state per head that decays per key channel.

Per head a state S [dim, vdim] (key channel i, value channel j), zero before a request's first token:
    S <- diag(alpha) S + k v^T,     o = S^T q
with q = W_q h * dim^(-1/2), k = W_k h, v = W_v h per head and a decay per head and key channel through a low-rank
pair of matrices, alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau).  Each head's o is divided by its root mean square and
multiplied by a weight of vdim numbers (one for all heads); the heads are concatenated, multiplied by silu(W_g h) and go
through the output projection.  Decay (through its logarithm), state and the whole recurrence are 32-bit; the state lives in
the request's state slot, which the cache zeroes when it hands the slot out, so a portion that starts anywhere goes on
from what the slot holds.

One product computes everything that reads h (q, k, v, g and the decay's inner activations); one backend call does the rest.
"""
from __future__ import annotations

from .base import FixedState, Mixer, ParamSpec, register_mixer

DEFAULT_NAMES = dict(q="q", k="k", v="v", g="g", a1="a1", a2="a2", a2_bias="a2.b", norm="norm", o="o")


@register_mixer("gla")
class GatedLinearAttention(Mixer):
    def __init__(self, width: int, num_heads: int, dim: int, vdim: int, rank: int, tau: float, eps: float, prefix: str,
                 q_scale: float | None = None, float32_output: bool = False, tensor_names=None):
        self.width, self.num_heads, self.dim, self.vdim, self.rank = int(width), int(num_heads), int(dim), int(vdim), int(rank)
        if self.dim > 256 or self.vdim > 256:
            raise ValueError(f"states of {dim} x {vdim} a head are beyond the 256 x 256 the recurrence kernel takes")
        if not tau > 0:
            raise ValueError(f"tau {tau} must be positive")
        self.tau, self.eps, self.prefix = float(tau), float(eps), prefix
        self.q_scale = float(q_scale) if q_scale is not None else self.dim ** -0.5
        self.float32_output = bool(float32_output)
        self.names = dict(DEFAULT_NAMES, **(tensor_names or {}))
        nk, nv = self.num_heads * self.dim, self.num_heads * self.vdim
        self.cols = dict(q=0, k=nk, v=2 * nk, g=2 * nk + nv, a=2 * nk + 2 * nv)

    def params(self):
        nm, w = self.names, self.width
        nk, nv = self.num_heads * self.dim, self.num_heads * self.vdim
        name = lambda k: f"{self.prefix}.{nm[k]}"        # noqa: E731
        return [ParamSpec.stacked("w_in", [(name("q"), (nk, w)), (name("k"), (nk, w)), (name("v"), (nv, w)), (name("g"), (nv, w)),
                                           (name("a1"), (self.rank, w))]),
                ParamSpec.single("w_decay", name("a2"), (nk, self.rank)),
                ParamSpec.single("decay_bias", name("a2_bias"), (nk,)),
                ParamSpec.single("norm", name("norm"), (self.vdim,), init="scale"),
                ParamSpec.single("w_o", name("o"), (w, nv))]

    def cache_requirement(self):
        return FixedState((self.num_heads, self.dim, self.vdim), "float32")

    def prepare(self, device, dtype):
        import torch
        if getattr(self, "_prepared", False):
            return
        self._prepared = True
        rows = self.w_in.shape[0]
        if rows % 16:       # the product kernels like whole tiles of weight rows: the sums get a few columns nobody reads
            padded = torch.zeros((-(-rows // 16) * 16, self.width), dtype=self.w_in.dtype, device=self.w_in.device)
            padded[:rows] = self.w_in
            self.w_in = padded
        # everything inside the recurrence is 32-bit whatever the checkpoint stores
        for attr in ("w_decay", "decay_bias", "norm"):
            setattr(self, attr, getattr(self, attr).float().contiguous())

    def forward(self, x, step, cache, add_to=None):
        import torch
        ops = self.ops
        sums = ops.linear(x, self.w_in, out_dtype=torch.float32)
        out = ops.gla(sums, self.cols, self.num_heads, self.dim, self.vdim, self.w_decay, self.decay_bias, self.tau, self.q_scale,
                      self.norm, self.eps, cache.state, step)
        if add_to is None and self.float32_output:
            return ops.linear(out, self.w_o, out_dtype=torch.float32)
        return ops.linear(out, self.w_o, add_to=add_to)
