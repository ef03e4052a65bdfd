"""Grouped-query attention whose weights are sigmoids: a visible key counts with sigmoid(score + b_h), b_h a number
per query head from the checkpoint, and the weights are not normalised over the keys.

score = cap * tanh((q . k) * scale / cap) with ``softcap`` = cap (None: the scaled product itself).  Visible are the
keys j <= i of the query's own chunk, floor(i / chunk) = floor(j / chunk), chunks counted from the request's first
position (``chunk`` None: all earlier keys).  Positions do not enter the scores.  With ``qk_norm`` queries and keys
are RMS-normed head by head over the head's ``dim`` numbers, with one weight of that size for all query heads and
one for all key heads.  Projections, cache layout, padded head size and the spread output matrix are
SoftmaxAttention's; pages that lie wholly before the chunk of a request's next token are given back (the cache
sees the chunk as a window of that many keys, which no chunk exceeds).
"""
from __future__ import annotations

from .base import ParamSpec, register_mixer
from .softmax_attention import SoftmaxAttention


@register_mixer("sigmoid_attention")
class SigmoidAttention(SoftmaxAttention):
    def __init__(self, width: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float, prefix: str,
                 chunk: int | None = None, softcap: float | None = None, head_bias: bool = True, qk_norm: bool = True,
                 eps: float = 1e-6, float32_output: bool = True, tensor_names=None):
        if chunk is not None and chunk < 1:
            raise ValueError("chunk must be >= 1 or None")
        if softcap is not None and not softcap > 0:
            raise ValueError("softcap must be positive or None")
        names = dict(dict(head_bias="pb"), **(tensor_names or {}))
        super().__init__(width, num_heads, num_kv_heads, dim, vdim, scale, None, prefix, window=chunk, qk_norm=qk_norm,
                         eps=eps, float32_output=float32_output, tensor_names=names)
        self.chunk = chunk
        self.softcap = None if softcap is None else float(softcap)
        self.has_head_bias = bool(head_bias)
        self.head_bias = None

    def params(self):
        n, w, H, G = self.names, self.width, self.num_heads, self.num_kv_heads
        name = lambda k: f"{self.prefix}.{n[k]}"        # noqa: E731
        specs = [ParamSpec.stacked("w_in", [(name("q"), (H * self.dim, w)), (name("k"), (G * self.dim, w)),
                                            (name("v"), (G * self.vdim, w))]),
                 ParamSpec.single("w_o", name("o"), (w, H * self.vdim))]
        if self.qk_norm:        # one weight of the head's size for all heads
            specs += [ParamSpec.single("q_norm", name("q_norm"), (self.dim,), init="scale"),
                      ParamSpec.single("k_norm", name("k_norm"), (self.dim,), init="scale")]
        if self.has_head_bias:
            specs.append(ParamSpec.single("head_bias", name("head_bias"), (H,)))
        return specs

    def prepare(self, device, dtype):
        first = not getattr(self, "_prepared", False)
        super().prepare(device, dtype)
        if first and self.head_bias is not None:
            self.head_bias = self.head_bias.float().contiguous()

    def forward(self, x, step, cache, add_to=None):
        import torch
        ops, H, G, P = self.ops, self.num_heads, self.num_kv_heads, self.padded_dim
        if cache.k.shape[-1] != P:
            raise ValueError(f"the cache holds heads of {cache.k.shape[-1]} numbers; this layer's are {P}")
        group = step.groups[cache.group]
        sums = ops.linear(x, self.w_in, out_dtype=torch.float32)
        q = ops.qkv_finish(sums, self.q_col, self.k_col, self.v_col, H, G, self.dim, self.vdim, P, step.positions, None,
                           "half", cache.k, cache.v, group.slot_mapping, q_norm=self.q_norm if self.qk_norm else None,
                           k_norm=self.k_norm if self.qk_norm else None, eps=self.eps, norm_per_head=True)
        o = ops.paged_attention(q, H, G, P, cache.k, cache.v, group, step, self.scale, None, weights="sigmoid",
                                softcap=self.softcap, chunk=self.chunk, head_bias=self.head_bias)
        if add_to is None and self.float32_output:
            return ops.linear(o, self.w_o, out_dtype=torch.float32)
        return ops.linear(o, self.w_o, add_to=add_to)
