"""Configuration of the Mutusun decoder, read from its own ``config.json`` keys.

The file lists the layers one by one.  Each entry names its mixer kind (``attention``: grouped-query attention
without positions, whose weights are sigmoids of capped scores and whose mask is causal within chunks of
``mask.size`` positions), the mixer's sizes and constants, and its feed-forward: ``dense`` (one matrix up, the
square of relu, one down), ``moe`` (gated experts with clamped inputs, of which a token runs ``top``; the last
``identity`` router outputs stand for experts that return their input) or none.  An entry with ``weights_of: j``
has no tensors: it runs with layer j's, with a cache and state of its own.  ``canon.taps`` is the length of the
short causal convolution on what every sublayer reads.  Every size and constant that may differ between two
models of the design is a field here.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, ModelConfig, _take_float, _take_int
from .zifelorn_config import DenseFFSpec, _section


@dataclass(frozen=True)
class SigmoidAttentionSpec:
    """``chunk``: a query sees the earlier keys of its own chunk of that many positions (None: all earlier keys);
    ``softcap``: scores pass through cap * tanh(score / cap) (None: as they are)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None
    chunk: int | None
    kind = "attention"

    @classmethod
    def from_dict(cls, d, where):
        heads, kv_heads = _take_int(d, "heads"), _take_int(d, "kv_heads")
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}heads {heads} is not a multiple of kv_heads {kv_heads}")
        dim = _take_int(d, "dim")
        mask = d.get("mask")
        chunk = None if mask is None else _take_int(_section(d, "mask", where), "size")
        cap = None if d.get("softcap") is None else _take_float(d, "softcap")
        if cap is not None and not cap > 0:
            raise ConfigError(f"config.json: {where}softcap must be positive, found {cap}")
        return cls(heads, kv_heads, dim, _take_int(d, "vdim", default=dim), _take_float(d, "scale"), cap, chunk)

    def to_dict(self):
        d = dict(heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim, scale=self.scale)
        if self.softcap is not None:
            d["softcap"] = self.softcap
        if self.chunk is not None:
            d["mask"] = dict(size=self.chunk)
        return d


@dataclass(frozen=True)
class GatedMoESpec:
    """``experts`` gated feed-forwards of inner size ``expert_ff`` whose gate and up inputs are clamped at ``limit``,
    and ``identity`` more router outputs that stand for experts returning their input; a token runs ``top``."""
    experts: int
    identity: int
    top: int
    expert_ff: int
    limit: float
    kind = "moe"

    @classmethod
    def from_dict(cls, d, where):
        router, expert = _section(d, "router", where), _section(d, "expert", where)
        spec = cls(_take_int(router, "experts", minimum=0), _take_int(router, "identity", default=0, minimum=0),
                   _take_int(router, "top"), _take_int(expert, "ff"), _take_float(expert, "limit"))
        if spec.top > spec.experts + spec.identity:
            raise ConfigError(f"config.json: {where}router.top {spec.top} exceeds the router's "
                              f"{spec.experts} + {spec.identity} outputs")
        if not spec.limit > 0:
            raise ConfigError(f"config.json: {where}expert.limit must be positive, found {spec.limit}")
        return spec

    def to_dict(self):
        return dict(kind="moe", expert=dict(ff=self.expert_ff, limit=self.limit),
                    router=dict(experts=self.experts, identity=self.identity, top=self.top))


def _feed_forward(d, where):
    if d is None:
        return None
    if not isinstance(d, Mapping):
        raise ConfigError(f"config.json: {where}mlp must be an object or null")
    kind = d.get("kind")
    if kind == "dense":
        return DenseFFSpec(_take_int(d, "ff"))
    if kind == "moe":
        return GatedMoESpec.from_dict(d, where + "mlp.")
    raise ConfigError(f"config.json: {where}mlp.kind {kind!r} is not computed here (dense, moe)")


_MIXERS = {"attention": SigmoidAttentionSpec}


@dataclass(frozen=True)
class MutusunLayer:
    mixer: Any
    mlp: Any
    weights_of: int | None = None

    def to_dict(self):
        d = dict(type=self.mixer.kind, mixer=self.mixer.to_dict(), mlp=None if self.mlp is None else self.mlp.to_dict())
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class MutusunConfig(ModelConfig):
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    canon_taps: int | None

    architecture = "Mutusun"

    def __post_init__(self):
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, found {self.norm_eps}")
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
    def from_dict(cls, d: Mapping[str, Any]) -> "MutusunConfig":
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
            layers.append(MutusunLayer(_MIXERS[kind].from_dict(_section(entry, "mixer", where), where + "mixer."),
                                       _feed_forward(entry.get("mlp"), where), shared))
        canon = d.get("canon")
        taps = None if canon is None else _take_int(_section(d, "canon", ""), "taps")
        return cls(vocab=_take_int(d, "vocab"), width=_take_int(d, "width"), layers=tuple(layers),
                   norm_eps=_take_float(_section(d, "norm", ""), "eps"), canon_taps=taps)

    def to_dict(self) -> dict:
        d = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.norm_eps),
                 layers=[layer.to_dict() for layer in self.layers])
        if self.canon_taps is not None:
            d["canon"] = dict(taps=self.canon_taps)
        return d
