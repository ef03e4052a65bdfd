"""Labirax: a decoder whose layers are listed one by one in its configuration; a layer may run with the tensors of
another one, with a cache and state of its own.

A layer has a norm before and after each sublayer, stream += N1b(mixer(N1 stream)) and then
stream += N2b(ff(N2 stream)), every norm a layer norm with weight and bias.  Mixers: grouped-query softmax attention
with biased projections, no rotation, a query that grows with the logarithm of its position and a learned bias per
head and bucketed distance on the scores; attention through a cached low-rank latent with one rotated key part for
all heads (pairs i, i + dims / 2), a sliding window and an output gate; gated linear attention (a state per head that
decays per key channel).  The feed-forward is a mixture of gated experts (softmax over all experts, the ``top``
largest, their scores over their sum) beside a shared expert that every token runs, or absent.  The embedding is
scaled; the head has a matrix of its own, a logit scale and a tanh cap on the logits.  Everything here is
construction: sizes and constants come from LabiraxConfig only.
Tensor names: ``embed``, ``head``, ``final.norm``, ``l<i>.norm1|norm1b|norm2|norm2b`` (each with ``.b``), ``l<i>.mix.*``,
``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.labirax_config import BiasedAttentionSpec, GlaSpec, LabiraxConfig, SharedMoESpec, WindowLatentAttentionSpec
from ..config.registry import register_architecture
from ..parts import (DecoderSpec, Embedding, GatedLinearAttention, LatentAttention, LayerCall, LayerNorm, LMHead,
                     RotaryHalfAngles, RoutedExperts, SandwichBlock, SoftmaxAttention, SummedFF, SwiGLU)


def build_labirax(cfg: LabiraxConfig) -> DecoderSpec:
    w, eps = cfg.width, cfg.norm_eps
    norm = lambda name: LayerNorm(w, eps, name)        # noqa: E731
    rotations = {}          # one position-encoding part for each distinct (dims, base)
    layers, index = [], {}  # blocks that own tensors, and where layer i's block stands among them
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        m, f, p = layer.mixer, layer.mlp, f"l{i}"
        if isinstance(m, BiasedAttentionSpec):
            mixer = SoftmaxAttention(w, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, None, prefix=f"{p}.mix", bias=True,
                                     position_temperature=(m.temp_coef, m.temp_every),
                                     distance_bias=(m.buckets, m.bias_max), float32_output=True)
        elif isinstance(m, WindowLatentAttentionSpec):
            rot = rotations.setdefault((m.rot.dims, m.rot.base), RotaryHalfAngles(m.rot.dims, m.rot.base))
            mixer = LatentAttention(w, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.q_rank, m.scale, eps, rot,
                                    prefix=f"{p}.mix", window=m.window)
        elif isinstance(m, GlaSpec):
            mixer = GatedLinearAttention(w, m.heads, m.dim, m.vdim, m.rank, m.tau, eps, prefix=f"{p}.mix", float32_output=True)
        else:
            raise TypeError(f"layer {i}: no part for mixer {m!r}")
        if f is None:
            ff = None
        elif isinstance(f, SharedMoESpec):
            ff = RoutedExperts(w, f.expert_ff, f.experts, f.top, prefix=f"{p}.mlp", router_bias=False, shares_over="all",
                               renormalise=True, gated="silu")
            if f.shared_ff is not None:
                ff = SummedFF([ff, SwiGLU(w, f.shared_ff, prefix=f"{p}.mlp.shared", tensor_names=("gate", "up", "down"),
                                          float32_output=True)])
        else:
            raise TypeError(f"layer {i}: no part for feed-forward {f!r}")
        index[i] = len(layers)
        if ff is None:
            layers.append(SandwichBlock(norm(f"{p}.norm1"), mixer, norm(f"{p}.norm1b")))
        else:
            layers.append(SandwichBlock(norm(f"{p}.norm1"), mixer, norm(f"{p}.norm1b"), norm(f"{p}.norm2"), ff,
                                        norm(f"{p}.norm2b")))
    embedding = Embedding(cfg.vocab, w, "embed", scale=cfg.embedding_scale)
    return DecoderSpec(embedding=embedding, layers=layers, final_norm=norm("final.norm"),
                       head=LMHead(cfg.vocab, w, "head", scale=cfg.logit_scale, softcap=cfg.logit_softcap),
                       schedule=[LayerCall(index[cfg.owner(i)]) for i in range(len(cfg.layers))], stop_token_ids=(),
                       max_position=None, vocab_size=cfg.vocab)


def _shape(vocab, width, heads, kv_heads, dim, latent_heads, kv_rank, q_rank, rot_dim, window, gla_heads, gla_dim, gla_vdim,
           experts, top, expert_ff, shared_ff, repeats, shared):
    """A named size: ``repeats`` times the run (attention, gated linear attention, latent attention, each with the
    mixture of experts), then ``shared`` more runs of the first three layers with their tensors."""
    att = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, q_temp=dict(coef=0.2, every=256),
               bias_max=2048, buckets=32)
    lat = dict(heads=latent_heads, dim=dim, rot_dim=rot_dim, vdim=dim, kv_rank=kv_rank, q_rank=q_rank,
               scale=(dim + rot_dim) ** -0.5, rot=dict(base=10000.0, dims=rot_dim), mask=dict(size=window))
    gla = dict(heads=gla_heads, dim=gla_dim, vdim=gla_vdim, tau=16.0, rank=16)
    moe = dict(kind="moe", expert=dict(ff=expert_ff), router=dict(experts=experts, top=top), shared=dict(ff=shared_ff))
    layers = []
    for _ in range(repeats):
        layers += [dict(type="attention", mixer=att, mlp=moe), dict(type="gla", mixer=gla, mlp=moe),
                   dict(type="latent_attention", mixer=lat, mlp=moe)]
    kinds = (("attention", att), ("gla", gla), ("latent_attention", lat))
    layers += [dict(type=kinds[j % 3][0], mixer=kinds[j % 3][1], mlp=moe, weights_of=j % 3) for j in range(shared)]
    return dict(vocab=vocab, width=width, embedding=dict(scale=1.0), norm=dict(eps=1e-6), logit_scale=1.0, logit_softcap=30.0,
                layers=layers)


# Named sizes: one for tests and the command line's examples, one with the widths of a 1B-class model.
SHAPES = {
    "labirax-tiny": _shape(vocab=320, width=64, heads=6, kv_heads=2, dim=16, latent_heads=3, kv_rank=40, q_rank=24, rot_dim=8,
                           window=24, gla_heads=2, gla_dim=16, gla_vdim=32, experts=5, top=2, expert_ff=48, shared_ff=32,
                           repeats=1, shared=2),
    "labirax-1b": _shape(vocab=32000, width=2048, heads=32, kv_heads=4, dim=64, latent_heads=16, kv_rank=192, q_rank=768,
                         rot_dim=64, window=1024, gla_heads=16, gla_dim=64, gla_vdim=128, experts=16, top=4, expert_ff=1408,
                         shared_ff=1408, repeats=5, shared=1),
}

register_architecture("Labirax", LabiraxConfig, build_labirax, shapes=SHAPES, replace=True)
