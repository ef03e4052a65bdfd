"""Grouped-query softmax attention from one product's float32 sums, with the variations a design may ask for.

One product computes everything that reads the mixer's input: queries, keys, values (unless the values are the
keys as projected, ``values_from_keys``) and, with ``head_gate``, one gate number a query head.  From its float32
sums one kernel makes what attention reads (KernelBackend.qkv_finish): an optional RMS norm over the whole query
(key) projection with a weight of that size (``qk_norm``), the rotation of the first ``position.rotary_dim`` numbers
of every head by angles computed in 32-bit (``position``: RotaryInterleaved or RotaryHalfAngles), an optional
temperature a query head (``head_temperature``: a checkpoint vector that multiplies the head's scores), and the
key and value rows of the cache.  Attention: scores * scale over the last ``window`` keys (None: all earlier
keys), softmax in 32-bit, with ``sink`` (a number) one more term exp(sink) in every denominator that has no value.
Head h's output is multiplied by sigmoid(gate_h) (``head_gate``) and the heads go through the output projection.
With ``bias`` the query, key and value projections have biases.  ``position_temperature`` = (coef, every): the query at
position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).  ``distance_bias`` = (buckets, farthest): a
checkpoint table [buckets, heads] adds table[bucket(n), h] to head h's score of a key n positions back (after the
scale): one bucket a distance for n < buckets / 2, then buckets whose reach grows geometrically,
bucket(n) = min(buckets - 1, half + floor(ln(n / half) / ln(farthest / half) * (buckets - half))), half = buckets / 2.
The table is spread over distances once, when the weights are loaded ([heads, N], N the first distance of the last
bucket + 1: every key further back adds the last entry).

Keys and queries of ``dim`` and values of ``vdim`` numbers a head are kept in a cache of P = the next multiple of
16 of the larger one, zeros beyond their own size, so that every head size runs the same attention kernels; the
output projection's columns are spread to match when the weights are loaded.
"""
from __future__ import annotations

from .base import Mixer, PagedKV, ParamSpec, register_mixer

DEFAULT_NAMES = dict(q="q", k="k", v="v", g="g", o="o", temp="temp", q_norm="q.norm", k_norm="k.norm", q_bias="q.b",
                     k_bias="k.b", v_bias="v.b", distance_bias="rel")


def log_distance_buckets(buckets: int, farthest: float) -> list:
    """bucket(n) for n = 0 .. N - 1, N - 1 the first distance that falls into the last bucket (every larger one does too)."""
    import math
    half = buckets // 2
    if buckets < 2 or not farthest > half:
        raise ValueError(f"{buckets} distance buckets up to {farthest}: at least 2, and the farthest beyond the first half")
    out = []
    while True:
        n = len(out)
        b = n if n < half else min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(farthest / half) * (buckets - half))))
        out.append(b)
        if b == buckets - 1:
            return out


@register_mixer("softmax_attention")
class SoftmaxAttention(Mixer):
    def __init__(self, width: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float, position, prefix: str,
                 window: int | None = None, sink: float | None = None, values_from_keys: bool = False,
                 head_temperature: bool = False, head_gate: bool = False, qk_norm: bool = False, eps: float = 1e-6,
                 float32_output: bool = False, tensor_names=None, bias: bool = False, position_temperature=None,
                 distance_bias=None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if values_from_keys and vdim != dim:
            raise ValueError(f"values that are the keys have the keys' size {dim}, not {vdim}")
        if window is not None and window < 1:
            raise ValueError("window must be >= 1 or None")
        if position is not None and position.rotary_dim > dim:
            raise ValueError(f"the position encoding turns {position.rotary_dim} numbers; a head has {dim}")
        self.width, self.num_heads, self.num_kv_heads = int(width), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.scale = int(dim), int(vdim), float(scale)
        self.padded_dim = -(-max(self.dim, self.vdim) // 16) * 16
        if self.padded_dim > 1024:
            raise ValueError(f"heads of {max(dim, vdim)} numbers are beyond the 1024 the attention kernels take")
        self.position, self.prefix = position, prefix
        self.window = window
        self.sink = None if sink is None else float(sink)
        self.values_from_keys, self.head_temperature = bool(values_from_keys), bool(head_temperature)
        self.head_gate, self.qk_norm, self.eps = bool(head_gate), bool(qk_norm), float(eps)
        self.float32_output = bool(float32_output)
        self.names = dict(DEFAULT_NAMES, **(tensor_names or {}))
        self.has_bias = bool(bias)
        self.position_temperature = None
        if position_temperature is not None:
            coef, every = float(position_temperature[0]), int(position_temperature[1])
            if every < 1 or every != position_temperature[1]:
                raise ValueError(f"a query temperature every {position_temperature[1]} positions: a whole number >= 1")
            self.position_temperature = (coef, every)
        self.distance_buckets = None
        if distance_bias is not None:
            self.distance_buckets = log_distance_buckets(int(distance_bias[0]), float(distance_bias[1]))
            self.num_buckets = int(distance_bias[0])
        self.b_in = self.rel = self.distance_table = None
        H, G = self.num_heads, self.num_kv_heads
        self.q_col, self.k_col = 0, H * self.dim
        self.v_col = None if self.values_from_keys else self.k_col + G * self.dim
        self.gate_col = self.k_col + G * self.dim + (0 if self.values_from_keys else G * self.vdim)

    def children(self):
        return [self.position] if self.position is not None else []

    def params(self):
        n, w, H, G = self.names, self.width, self.num_heads, self.num_kv_heads
        name = lambda k: f"{self.prefix}.{n[k]}"        # noqa: E731
        pieces = [(name("q"), (H * self.dim, w)), (name("k"), (G * self.dim, w))]
        if not self.values_from_keys:
            pieces.append((name("v"), (G * self.vdim, w)))
        if self.head_gate:
            pieces.append((name("g"), (H, w)))
        specs = [ParamSpec.stacked("w_in", pieces), ParamSpec.single("w_o", name("o"), (w, H * self.vdim))]
        if self.head_temperature:
            specs.append(ParamSpec.single("temperature", name("temp"), (H,), init="scale"))
        if self.qk_norm:
            specs += [ParamSpec.single("q_norm", name("q_norm"), (H * self.dim,), init="scale"),
                      ParamSpec.single("k_norm", name("k_norm"), (G * self.dim,), init="scale")]
        if self.has_bias:
            if self.values_from_keys:
                raise ValueError("biased projections with values that are the keys are not built")
            specs.append(ParamSpec.stacked("b_in", [(name("q_bias"), (H * self.dim,)), (name("k_bias"), (G * self.dim,)),
                                                    (name("v_bias"), (G * self.vdim,))]))
        if self.distance_buckets is not None:
            specs.append(ParamSpec.single("rel", name("distance_bias"), (self.num_buckets, H)))
        return specs

    def cache_requirement(self):
        return PagedKV(self.num_kv_heads, self.padded_dim, self.window)

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
        P, H = self.padded_dim, self.num_heads
        if P != self.vdim:  # the attention's output has P numbers a head, the last P - vdim of them zero
            spread = torch.zeros((self.width, H, P), dtype=self.w_o.dtype, device=self.w_o.device)
            spread[:, :, :self.vdim] = self.w_o.view(self.width, H, self.vdim)
            self.w_o = spread.view(self.width, H * P)
        for attr in ("temperature", "q_norm", "k_norm"):     # 32-bit whatever the checkpoint stores
            if getattr(self, attr, None) is not None:
                setattr(self, attr, getattr(self, attr).float().contiguous())
        if self.b_in is not None:       # one number a column of the product's sums, zeros for the columns nobody reads
            b = torch.zeros(self.w_in.shape[0], dtype=torch.float32, device=self.w_in.device)
            b[:self.b_in.shape[0]] = self.b_in.float()
            self.b_in = b
        if self.rel is not None:        # [heads, distances]: the table's row for every distance up to the last bucket's first
            rows = torch.tensor(self.distance_buckets, dtype=torch.long, device=self.rel.device)
            self.distance_table = self.rel.float()[rows].t().contiguous()

    def _finish_options(self) -> dict:
        """What only some designs ask of qkv_finish (a backend that knows none of them is not handed any)."""
        opts = {}
        if self.b_in is not None:
            opts["col_bias"] = self.b_in
        if self.position_temperature is not None:
            opts["position_temperature"] = self.position_temperature
        return opts

    def forward(self, x, step, cache, add_to=None, sums=None, base=0):
        """``sums``: the float32 sums of a product that holds this part's ``w_in`` rows from column ``base`` on (a
        caller that stacked several parts' input matrices); ``x`` is then not read."""
        import torch
        ops, H, G, P = self.ops, self.num_heads, self.num_kv_heads, self.padded_dim
        if cache.k.shape[-1] != P:
            raise ValueError(f"the cache holds heads of {cache.k.shape[-1]} numbers; this layer's are {P}")
        group = step.groups[cache.group]
        if sums is None:
            sums, base = ops.linear(x, self.w_in, out_dtype=torch.float32), 0
        elif self.b_in is not None:
            raise ValueError("biased projections inside another part's product are not built")
        pos = self.position
        q = ops.qkv_finish(sums, base + self.q_col, base + self.k_col, None if self.v_col is None else base + self.v_col,
                           H, G, self.dim, self.vdim, P, step.positions,
                           pos.inv_freq if pos is not None else None, pos.layout if pos is not None else "half",
                           cache.k, cache.v, group.slot_mapping, q_norm=self.q_norm if self.qk_norm else None,
                           k_norm=self.k_norm if self.qk_norm else None, eps=self.eps,
                           q_head_scale=self.temperature if self.head_temperature else None,
                           **self._finish_options())
        if self.distance_table is not None:
            o = ops.paged_attention(q, H, G, P, cache.k, cache.v, group, step, self.scale, self.window, sink=self.sink,
                                    distance_bias=self.distance_table)
        else:
            o = ops.paged_attention(q, H, G, P, cache.k, cache.v, group, step, self.scale, self.window, sink=self.sink)
        if self.head_gate:
            o = ops.head_gate_(o, sums, base + self.gate_col, H, P)
        if add_to is None and self.float32_output:
            return ops.linear(o, self.w_o, out_dtype=torch.float32)
        return ops.linear(o, self.w_o, add_to=add_to)
