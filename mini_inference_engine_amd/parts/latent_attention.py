"""Softmax attention whose keys and values are expanded from a cached low-rank latent.

Per token the layer keeps c = RMSNorm(W_dkv x)[:kv_rank] and one rotated key part k_r (the last rot_dim
outputs of W_dkv, position-encoded, shared by all heads).  Head h has key [W_uk,h c | k_r] and value
W_uv,h c; queries come through a latent of their own, q = W_uq RMSNorm(W_dq x), laid out per head as
[dim plain | rot_dim rotated].  Score (q_plain . k_plain + q_rot . k_r) * scale, causal (with ``window``: over the
last that many keys only, and pages the window has passed are given back), softmax.  The rotation pairs adjacent
numbers or the two halves of the turned part, as the position encoding says (``position.layout``).  The
concatenated heads are multiplied by sigmoid(W_g x) and projected by W_o.

Nothing but c and k_r is cached, and keys are never expanded: q_plain . (W_uk,h c) = (W_uk,h^T q_plain) . c,
so attention runs over the latents as one shared key/value head of kv_rank + rot_dim numbers, and W_uv is
applied to the attention's output.  W_uk is folded into the query up-projection once, when the weights are
loaded: head h of the folded matrix is [W_uk,h^T W_uq,h(plain rows) ; W_uq,h(rotated rows) ; 0], so that one
product gives every head's query against the cache's key rows [c | k_r | 0] and only the rotation is left to do.
The cache is what the attention kernels of the other mixers read: keys [c | k_r], values c, padded to a multiple of 16.

A layer built with ``has_kv`` False has no W_dkv: it reads another layer call's cache (same kv_rank,
rot_dim and position encoding) with its own W_uk, W_uv and queries.
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import CacheRequirement, Mixer, ParamSpec, register_mixer

DEFAULT_NAMES = dict(dq="dq", dq_norm="dq.norm", uq="uq", dkv="dkv", dkv_norm="dkv.norm", uk="uk", uv="uv", g="g", o="o")


@dataclass(frozen=True)
class PagedLatent(CacheRequirement):
    """A latent of ``kv_rank`` and a rotated key part of ``rot_dim`` per token, in pages, as one key/value head:
    keys [pages, 1, page, P] = [c | k_r | 0], values [pages, 1, P, page] = [c | 0] (transposed within a page), P the
    next multiple of 16."""
    kv_rank: int
    rot_dim: int
    window: int | None = None
    paged = True

    @property
    def padded_dim(self) -> int:
        return -(-(self.kv_rank + self.rot_dim) // 16) * 16

    def bytes_per_page(self, page_size, element_size):
        return 2 * page_size * self.padded_dim * element_size

    def allocate(self, num_pages, page_size, num_slots, device, act_dtype):
        import torch
        P = self.padded_dim
        return {"k": torch.zeros((num_pages, 1, page_size, P), dtype=act_dtype, device=device),
                "v": torch.zeros((num_pages, 1, P, page_size), dtype=act_dtype, device=device)}


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    MAX_PADDED_DIM = 1024       # what the attention kernels take as a head size (the matrix-core ones up to 256)

    def __init__(self, width: int, num_heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, q_rank: int,
                 scale: float, eps: float, position, prefix: str, has_kv: bool = True, gated: bool = True,
                 tensor_names=None, window: int | None = None):
        self.width, self.num_heads, self.dim, self.rot_dim = int(width), int(num_heads), int(dim), int(rot_dim)
        self.vdim, self.kv_rank, self.q_rank = int(vdim), int(kv_rank), int(q_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.position = position
        self.prefix = prefix
        self.has_kv, self.gated = bool(has_kv), bool(gated)
        if window is not None and window < 1:
            raise ValueError("window must be >= 1 or None")
        self.window = window
        self.layout = getattr(position, "layout", "interleaved")       # which numbers of the rotated part turn together
        self.names = dict(DEFAULT_NAMES, **(tensor_names or {}))
        if position.rotary_dim > self.rot_dim:
            raise ValueError(f"the position encoding turns {position.rotary_dim} dims; the rotated part has {self.rot_dim}")
        self.w_uq = self.w_uk = self.w_q = None
        self.padded_dim = PagedLatent(self.kv_rank, self.rot_dim).padded_dim
        if self.padded_dim > self.MAX_PADDED_DIM:
            raise ValueError(f"kv_rank {kv_rank} + rot_dim {rot_dim} is beyond the {self.MAX_PADDED_DIM} numbers a token "
                             "the attention kernels take")

    def children(self):
        return [self.position]

    def params(self):
        n, w, H = self.names, self.width, self.num_heads
        name = lambda k: f"{self.prefix}.{n[k]}"        # noqa: E731
        down = [(name("dq"), (self.q_rank, w))]
        if self.has_kv:
            down.append((name("dkv"), (self.kv_rank + self.rot_dim, w)))
        if self.gated:
            down.append((name("g"), (H * self.vdim, w)))
        specs = [ParamSpec.stacked("w_down", down),
                 ParamSpec.single("dq_norm", name("dq_norm"), (self.q_rank,), init="scale"),
                 ParamSpec.single("w_uq", name("uq"), (H * (self.dim + self.rot_dim), self.q_rank)),
                 ParamSpec.single("w_uk", name("uk"), (H * self.dim, self.kv_rank)),
                 ParamSpec.single("w_uv", name("uv"), (H * self.vdim, self.kv_rank)),
                 ParamSpec.single("w_o", name("o"), (w, H * self.vdim))]
        if self.has_kv:
            specs.append(ParamSpec.single("dkv_norm", name("dkv_norm"), (self.kv_rank,), init="scale"))
        return specs

    def cache_requirement(self):
        return PagedLatent(self.kv_rank, self.rot_dim, self.window)

    def prepare(self, device, dtype):
        """Fold W_uk into W_uq (in 32-bit, rounded once to the weights' dtype); the two are not needed afterwards."""
        import torch
        if self.w_uq is None:
            return
        H, d, dr, r, P = self.num_heads, self.dim, self.rot_dim, self.kv_rank, self.padded_dim
        uq = self.w_uq.float().view(H, d + dr, self.q_rank)
        uk = self.w_uk.float().view(H, d, r)
        folded = torch.zeros((H, P, self.q_rank), dtype=torch.float32, device=self.w_uq.device)
        folded[:, :r] = torch.einsum("hdr,hdq->hrq", uk, uq[:, :d])
        folded[:, r:r + dr] = uq[:, d:]
        self.w_q = folded.view(H * P, self.q_rank).to(self.w_uq.dtype).contiguous()
        self.w_uq = self.w_uk = None

    def forward(self, x, step, cache, add_to=None):
        import torch
        ops = self.ops
        if cache.read_only == self.has_kv:
            raise ValueError("a latent-attention part with a down-projection owns its cache; one without reads another's")
        if cache.k.shape[-1] != self.padded_dim:
            raise ValueError(f"the cache holds {cache.k.shape[-1]} numbers a token; this layer reads {self.padded_dim}")
        group = step.groups[cache.group]
        inv_freq = self.position.inv_freq
        # one product for everything that reads x: query latent, key/value latent + rotated key part, gate
        sums = ops.linear(x, self.w_down, out_dtype=torch.float32)
        col = self.q_rank
        half = {} if self.layout == "interleaved" else {"layout": self.layout}
        if self.has_kv:      # the token's cache entry and, in the same kernel, its normed query latent
            cq = ops.latent_kv_store(sums, col, self.kv_rank, self.rot_dim, self.dkv_norm, self.eps, step.positions, inv_freq,
                                     cache.k, cache.v, group.slot_mapping, also_norm=(0, self.q_rank, self.dq_norm), **half)
            col += self.kv_rank + self.rot_dim
        else:
            cq = ops.rmsnorm_columns(sums, 0, self.q_rank, self.dq_norm, self.eps)
        q = ops.latent_query_rotate_(ops.linear(cq, self.w_q), self.num_heads, self.kv_rank, self.padded_dim, step.positions,
                                     inv_freq, **half)
        o = ops.paged_attention(q, self.num_heads, 1, self.padded_dim, cache.k, cache.v, group, step, self.scale, self.window)
        heads = ops.latent_value_gate(o, self.w_uv, sums if self.gated else None, col, self.num_heads, self.vdim,
                                      self.kv_rank, self.padded_dim)
        return ops.linear(heads, self.w_o, out_dtype=torch.float32)
