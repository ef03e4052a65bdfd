"""Mutusun: a decoder whose layers are listed one by one in its configuration; a layer may run with the tensors
of another one, with a cache and state of its own.

A layer has a norm before and after each sublayer, stream += N1b(mixer(c1(N1 stream))) and then
stream += N2b(ff(c2(N2 stream))), every norm an RMS norm whose weight is stored around zero and applied as
1 + w, c1 and c2 a short causal convolution per channel that is added to what the sublayer reads.  The mixer is
grouped-query attention without positions: queries and keys normed head by head, scores capped by a tanh, a causal
mask within chunks of positions, sigmoid weights with a bias per head and no normalisation over the keys.  The
feed-forward is dense (the square of relu between two matrices), routed (gated experts with clamped inputs, scores
a softmax over all router outputs, a correction that steers the choice only, identity experts) or absent.  The
head has a matrix of its own.  Everything here is construction: sizes and constants come from MutusunConfig only.
Tensor names: ``embed``, ``head``, ``final.norm``, ``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.canon1|canon2``,
``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.mutusun_config import GatedMoESpec, MutusunConfig, SigmoidAttentionSpec
from ..config.registry import register_architecture
from ..config.zifelorn_config import DenseFFSpec
from ..parts import (DecoderSpec, DenseFF, Embedding, LayerCall, LMHead, ResidualConv, RMSNorm, RoutedExperts,
                     SandwichBlock, SigmoidAttention)

EXPERT_GATE_SLOPE = 1.702       # an expert's gate is g * sigmoid(1.702 g): fixed by the design


def build_mutusun(cfg: MutusunConfig) -> DecoderSpec:
    w, eps, taps = cfg.width, cfg.norm_eps, cfg.canon_taps
    norm = lambda name: RMSNorm(w, eps, name, one_plus=True)        # noqa: E731
    conv = lambda name: None if taps is None else ResidualConv(w, taps, name)        # noqa: E731
    layers, index = [], {}          # blocks that own tensors, and where layer i's block stands among them
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        m, f, p = layer.mixer, layer.mlp, f"l{i}"
        if not isinstance(m, SigmoidAttentionSpec):
            raise TypeError(f"layer {i}: no part for mixer {m!r}")
        mixer = SigmoidAttention(w, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, prefix=f"{p}.mix", chunk=m.chunk,
                                 softcap=m.softcap, head_bias=True, qk_norm=True, eps=eps, float32_output=True)
        if f is None:
            ff = None
        elif isinstance(f, DenseFFSpec):
            ff = DenseFF(w, f.ff, prefix=f"{p}.mlp", activation="relu2", float32_output=True)
        elif isinstance(f, GatedMoESpec):
            ff = RoutedExperts(w, f.expert_ff, f.experts, f.top, prefix=f"{p}.mlp", router_bias=False, shares_over="all",
                               choice_bias=True, gated=(f.limit, EXPERT_GATE_SLOPE), identity=f.identity)
        else:
            raise TypeError(f"layer {i}: no part for feed-forward {f!r}")
        index[i] = len(layers)
        if ff is None:
            layers.append(SandwichBlock(norm(f"{p}.norm1"), mixer, norm(f"{p}.norm1b"), conv_mixer=conv(f"{p}.canon1")))
        else:
            layers.append(SandwichBlock(norm(f"{p}.norm1"), mixer, norm(f"{p}.norm1b"), norm(f"{p}.norm2"), ff,
                                        norm(f"{p}.norm2b"), conv_mixer=conv(f"{p}.canon1"),
                                        conv_feed_forward=conv(f"{p}.canon2")))
    embedding = Embedding(cfg.vocab, w, "embed")
    return DecoderSpec(embedding=embedding, layers=layers, final_norm=norm("final.norm"),
                       head=LMHead(cfg.vocab, w, "head"),
                       schedule=[LayerCall(index[cfg.owner(i)]) for i in range(len(cfg.layers))], stop_token_ids=(),
                       max_position=None, vocab_size=cfg.vocab)


def _shape(vocab, width, heads, kv_heads, dim, chunk, ff, experts, identity, top, expert_ff, repeats, shared):
    """A named size: ``repeats`` times the run (dense layer, routed layer, ``shared`` more runs of the routed layer
    with its tensors)."""
    att = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, softcap=30.0, mask=dict(size=chunk))
    dense = dict(kind="dense", ff=ff)
    moe = dict(kind="moe", expert=dict(ff=expert_ff, limit=7.0), router=dict(experts=experts, identity=identity, top=top))
    layers = []
    for _ in range(repeats):
        layers.append(dict(type="attention", mixer=att, mlp=dense))
        owner = len(layers)
        layers.append(dict(type="attention", mixer=att, mlp=moe))
        layers += [dict(type="attention", mixer=att, mlp=moe, weights_of=owner) for _ in range(shared)]
    return dict(vocab=vocab, width=width, norm=dict(eps=1e-6), canon=dict(taps=4), layers=layers)


SHAPES = {
    "mutusun-tiny": _shape(vocab=320, width=64, heads=6, kv_heads=2, dim=16, chunk=24, ff=112, experts=5, identity=1, top=3,
                           expert_ff=48, repeats=1, shared=1),
    "mutusun-1b": _shape(vocab=32000, width=2048, heads=32, kv_heads=4, dim=64, chunk=1024, ff=5632, experts=16, identity=2,
                         top=4, expert_ff=1408, repeats=5, shared=1),
}

register_architecture("Mutusun", MutusunConfig, build_mutusun, shapes=SHAPES, replace=True)
