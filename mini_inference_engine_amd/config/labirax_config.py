"""Configuration of the Labirax decoder, read from its own ``config.json`` keys.

The file lists the layers one by one.  Each entry names its mixer kind, the mixer's sizes and constants and its
feed-forward.  Mixers: ``attention`` (grouped-query softmax attention with biased projections and no rotation; the
query grows with the logarithm of its position, ``q_temp``; a learned bias per head and bucketed distance joins the
scores, ``bias_max`` the distance at which the last bucket starts at the latest), ``latent_attention`` (keys and values
expanded from a cached low-rank latent, one rotated key part for all heads, a sliding window ``mask.size``, an output
gate), ``gla`` (gated linear attention: a state per head that decays per key channel, ``tau`` the root taken of the
decay's sigmoid).  The feed-forward is a mixture of gated experts (``router.experts``, of which a token runs
``router.top``) beside an optional shared expert, or none.  An entry with ``weights_of: j`` has no tensors: it runs with
layer j's, with a cache and state of its own.  Two sizes stand in no key of the file and are read from the checkpoint's
tensor shapes (``reads_tensor_shapes``): the number of distance buckets (rows of ``l<i>.mix.rel``) and the inner size
of the decay's pair of matrices (rows of ``l<i>.mix.a1``); ``to_dict`` writes them as ``buckets`` and ``rank``, which
the random-weights mode and the named sizes use.  Every size and constant that may differ between two models of the
design is a field here.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, ModelConfig, _take_float, _take_int
from .zifelorn_config import RotarySpec, _section


def _from_shape(d, key, shapes, tensor, where):
    """A size that config.json may leave to the checkpoint: key ``key`` of ``d``, else the first dim of ``tensor``."""
    v = d.get(key)
    if v is None and shapes is not None and tensor in shapes:
        v = int(shapes[tensor][0])
    if v is None:
        raise ConfigError(f"config.json: {where}{key} is not given and no checkpoint tensor {tensor} to read it from")
    if isinstance(v, bool) or not isinstance(v, int) or v < 1:
        raise ConfigError(f"config.json: {where}{key} must be a positive integer, found {v!r}")
    return v


@dataclass(frozen=True)
class BiasedAttentionSpec:
    """``temp_coef``, ``temp_every``: the query at position p times 1 + coef * ln(floor((p + 1) / every) + 1);
    ``buckets`` rows of the distance table (the first buckets // 2 one distance each), the last one reached at distance
    ``bias_max`` at the latest."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float
    temp_every: int
    buckets: int
    bias_max: float
    kind = "attention"

    @classmethod
    def from_dict(cls, d, where, shapes=None, owner=0):
        heads, kv_heads = _take_int(d, "heads"), _take_int(d, "kv_heads")
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}heads {heads} is not a multiple of kv_heads {kv_heads}")
        dim = _take_int(d, "dim")
        coef, every = 0.0, 1               # no q_temp: the query as projected
        if d.get("q_temp") is not None:
            temp = _section(d, "q_temp", where)
            every = temp.get("every")
            if isinstance(every, float) and every == int(every):
                every = int(every)
            if isinstance(every, bool) or not isinstance(every, int) or every < 1:
                raise ConfigError(f"config.json: {where}q_temp.every must be a whole number of positions >= 1, found {every!r}")
            coef = _take_float(temp, "coef")
        buckets = _from_shape(d, "buckets", shapes, f"l{owner}.mix.rel", where)
        spec = cls(heads, kv_heads, dim, _take_int(d, "vdim", default=dim), _take_float(d, "scale"),
                   coef, every, buckets, _take_float(d, "bias_max"))
        if buckets < 2:
            raise ConfigError(f"config.json: {where}a distance table of {buckets} rows: at least 2 are computed here")
        if not spec.bias_max > buckets // 2:
            raise ConfigError(f"config.json: {where}bias_max {spec.bias_max} must lie beyond the table's first half ({buckets // 2})")
        return spec

    def to_dict(self):
        return dict(heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim, scale=self.scale,
                    q_temp=dict(coef=self.temp_coef, every=self.temp_every), bias_max=self.bias_max, buckets=self.buckets)


@dataclass(frozen=True)
class WindowLatentAttentionSpec:
    """Attention through a low-rank latent: per head ``dim`` unrotated and ``rot_dim`` rotated query/key numbers, values of
    ``vdim``, keys and values expanded from a latent of ``kv_rank``, queries from one of ``q_rank``; ``window`` keys back
    at most (None: all)."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotarySpec
    window: int | None
    kind = "latent_attention"

    @classmethod
    def from_dict(cls, d, where, shapes=None, owner=0):
        rot = _section(d, "rot", where)
        mask = d.get("mask")
        spec = cls(heads=_take_int(d, "heads"), dim=_take_int(d, "dim"), rot_dim=_take_int(d, "rot_dim"),
                   vdim=_take_int(d, "vdim"), kv_rank=_take_int(d, "kv_rank"), q_rank=_take_int(d, "q_rank"),
                   scale=_take_float(d, "scale"), rot=RotarySpec(_take_float(rot, "base"), _take_int(rot, "dims")),
                   window=None if mask is None else _take_int(_section(d, "mask", where), "size"))
        if spec.rot.dims % 2 or spec.rot.dims > spec.rot_dim:
            raise ConfigError(f"config.json: {where}rot.dims {spec.rot.dims} must be even and at most rot_dim {spec.rot_dim}")
        if not spec.rot.base > 0:
            raise ConfigError(f"config.json: {where}rot.base must be positive")
        return spec

    def to_dict(self):
        d = dict(heads=self.heads, dim=self.dim, rot_dim=self.rot_dim, vdim=self.vdim, kv_rank=self.kv_rank,
                 q_rank=self.q_rank, scale=self.scale, rot=dict(base=self.rot.base, dims=self.rot.dims))
        if self.window is not None:
            d["mask"] = dict(size=self.window)
        return d


@dataclass(frozen=True)
class GlaSpec:
    """Gated linear attention: ``heads`` states of dim x vdim; ``rank`` the inner size of the decay's pair of matrices;
    the decay is the ``tau``-th root of a sigmoid."""
    heads: int
    dim: int
    vdim: int
    rank: int
    tau: float
    kind = "gla"

    @classmethod
    def from_dict(cls, d, where, shapes=None, owner=0):
        dim = _take_int(d, "dim")
        spec = cls(_take_int(d, "heads"), dim, _take_int(d, "vdim", default=dim),
                   _from_shape(d, "rank", shapes, f"l{owner}.mix.a1", where), _take_float(d, "tau"))
        if not spec.tau > 0:
            raise ConfigError(f"config.json: {where}tau must be positive, found {spec.tau}")
        return spec

    def to_dict(self):
        return dict(heads=self.heads, dim=self.dim, vdim=self.vdim, tau=self.tau, rank=self.rank)


@dataclass(frozen=True)
class SharedMoESpec:
    """``experts`` gated feed-forwards of inner size ``expert_ff``, of which a token runs ``top``, and a shared one of
    inner size ``shared_ff`` that every token runs (None: no shared expert)."""
    experts: int
    top: int
    expert_ff: int
    shared_ff: int | None
    kind = "moe"

    @classmethod
    def from_dict(cls, d, where):
        router, expert = _section(d, "router", where), _section(d, "expert", where)
        shared = d.get("shared")
        spec = cls(_take_int(router, "experts"), _take_int(router, "top"), _take_int(expert, "ff"),
                   None if shared is None else _take_int(_section(d, "shared", where), "ff"))
        if spec.top > spec.experts:
            raise ConfigError(f"config.json: {where}router.top {spec.top} exceeds router.experts {spec.experts}")
        return spec

    def to_dict(self):
        d = dict(kind="moe", expert=dict(ff=self.expert_ff), router=dict(experts=self.experts, top=self.top))
        if self.shared_ff is not None:
            d["shared"] = dict(ff=self.shared_ff)
        return d


def _feed_forward(d, where):
    if d is None:
        return None
    if not isinstance(d, Mapping):
        raise ConfigError(f"config.json: {where}mlp must be an object or null")
    kind = d.get("kind", "moe")
    if kind == "moe":
        return SharedMoESpec.from_dict(d, where + "mlp.")
    raise ConfigError(f"config.json: {where}mlp.kind {kind!r} is not computed here (moe)")


_MIXERS = {"attention": BiasedAttentionSpec, "latent_attention": WindowLatentAttentionSpec, "gla": GlaSpec}


@dataclass(frozen=True)
class LabiraxLayer:
    mixer: Any
    mlp: Any
    weights_of: int | None = None

    def to_dict(self):
        d = dict(type=self.mixer.kind, mixer=self.mixer.to_dict(), mlp=None if self.mlp is None else self.mlp.to_dict())
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class LabiraxConfig(ModelConfig):
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    logit_softcap: float | None

    architecture = "Labirax"
    reads_tensor_shapes = True          # from_dict takes the checkpoint's tensor shapes beside the dictionary

    def __post_init__(self):
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, found {self.norm_eps}")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError(f"config.json: logit_softcap must be positive, found {self.logit_softcap}")
        for i, layer in enumerate(self.layers):
            j = layer.weights_of
            if j is None:
                continue
            if not 0 <= j < len(self.layers) or j == i:
                raise ConfigError(f"config.json: layers[{i}].weights_of = {j} names no other layer")
            if self.layers[j].weights_of is not None:
                raise ConfigError(f"config.json: layers[{i}].weights_of = {j}, which has no tensors of its own")
            if (layer.mixer, layer.mlp) != (self.layers[j].mixer, self.layers[j].mlp):
                raise ConfigError(f"config.json: layers[{i}] runs with layer {j}'s tensors but describes another layer")

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs with."""
        j = self.layers[i].weights_of
        return i if j is None else j

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], tensor_shapes=None) -> "LabiraxConfig":
        raw = d.get("layers")
        if not isinstance(raw, (list, tuple)):
            raise ConfigError("config.json: 'layers' must be a list")
        layers = []
        for i, entry in enumerate(raw):
            where = f"layers[{i}]."
            if not isinstance(entry, Mapping):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            kind = entry.get("type")
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}type {kind!r} is not computed here ({sorted(_MIXERS)})")
            shared = None if entry.get("weights_of") is None else _take_int(entry, "weights_of", minimum=0)
            owner = i if shared is None else shared         # whose tensors' shapes give the sizes no key holds
            layers.append(LabiraxLayer(_MIXERS[kind].from_dict(_section(entry, "mixer", where), where + "mixer.", tensor_shapes, owner),
                                       _feed_forward(entry.get("mlp"), where), shared))
        cap = d.get("logit_softcap")
        return cls(vocab=_take_int(d, "vocab"), width=_take_int(d, "width"), layers=tuple(layers),
                   norm_eps=_take_float(_section(d, "norm", ""), "eps"),
                   embedding_scale=_take_float(d.get("embedding") or {}, "scale", default=1.0),
                   logit_scale=_take_float(d, "logit_scale", default=1.0),
                   logit_softcap=None if cap is None else _take_float(d, "logit_softcap"))

    def to_dict(self) -> dict:
        d = dict(architecture=self.architecture, vocab=self.vocab, width=self.width,
                 embedding=dict(scale=self.embedding_scale), norm=dict(eps=self.norm_eps), logit_scale=self.logit_scale,
                 layers=[layer.to_dict() for layer in self.layers])
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        return d
