"""Pre-norm block with the residual adds deferred into the norms.

stream += pending; y = norm1(stream); a = mixer(y); stream += a; y = norm2(stream);
pending' = feed_forward(y).  The block returns its feed-forward output still to
be added: the next block's first norm (or the final norm) adds it
(inference_engine/model.py:169-171,179,184).
"""
from __future__ import annotations

from ..kernels.api import Normed, NormedBranch, Sink, StreamCopy
from .base import Block, CombinedCache, register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    def __init__(self, norm_mixer, mixer, norm_feed_forward, feed_forward):
        self.norm_mixer = norm_mixer
        self.mixer = mixer
        self.norm_feed_forward = norm_feed_forward
        self.feed_forward = feed_forward

    def children(self):
        return [self.norm_mixer, self.mixer, self.norm_feed_forward, self.feed_forward]

    @property
    def first_norm(self):
        return self.norm_mixer

    def forward(self, h, residual, step, cache, next_norm=None):
        """``next_norm``: the norm that reads the stream after this block (the next block's first norm or
        the model's final norm), if the model knows it."""
        y = self.norm_mixer.lazy(h, residual)
        if not self.mixer.lazy_input:
            y = y.materialize()
        a = self.mixer.forward(y, step, cache, add_to=_sink(residual, self.norm_feed_forward))
        y = self.norm_feed_forward.lazy(a, residual)
        if not self.feed_forward.lazy_input:
            y = y.materialize()
        return self.feed_forward.forward(y, step, add_to=_sink(residual, next_norm)), residual


def _sink(residual, norm):
    weight, eps = getattr(norm, "weight", None), getattr(norm, "eps", None)
    if weight is None or eps is None or getattr(norm, "kind", "rmsnorm") != "rmsnorm":
        return Sink(residual)           # a sink names an RMS norm; any other kind is computed by the norm itself
    return Sink(residual, weight, eps)


@register_block("branch_norm")
class BranchNormBlock(Block):
    """The norm sits on each branch's output, and the branches read the stream itself:
    stream += norm_mixer(mixer(stream)); stream += norm_feed_forward(feed_forward(stream)).  ``feed_forward``
    (and its norm) may be None: the layer is its mixer alone.  Between the branches the stream travels in the
    activation dtype beside its float32 self (kernels.api.StreamCopy), made by the kernel that adds a branch."""

    def __init__(self, mixer, norm_mixer, feed_forward=None, norm_feed_forward=None):
        if (feed_forward is None) != (norm_feed_forward is None):
            raise ValueError("a feed-forward and its norm come together or not at all")
        self.mixer = mixer
        self.norm_mixer = norm_mixer
        self.feed_forward = feed_forward
        self.norm_feed_forward = norm_feed_forward

    def children(self):
        return [p for p in (self.mixer, self.norm_mixer, self.feed_forward, self.norm_feed_forward) if p is not None]

    def forward(self, h, residual, step, cache, next_norm=None):
        ops = self.ops
        if isinstance(h, NormedBranch):
            h = h.resolve()
        if isinstance(h, StreamCopy) and h.stream is residual:
            x = h.value
        else:
            if isinstance(h, Normed):         # a block of another kind before this one: its last add may be pending
                h, h_pending = None, h.pending
                if h_pending is not None:
                    residual.add_(h_pending.float())
            elif h is not None:
                residual.add_(h.float())
            x = ops.branch_norm_add(None, residual, None, 0.0)
        y = self.mixer.forward(x, step, cache)
        x = ops.branch_norm_add(y, residual, self.norm_mixer.weight, self.norm_mixer.eps)
        if self.feed_forward is not None:
            y = self.feed_forward.forward(x, step)
            x = ops.branch_norm_add(y, residual, self.norm_feed_forward.weight, self.norm_feed_forward.eps)
        return StreamCopy(residual, x), residual


@register_block("parallel")
class ParallelBlock(Block):
    """Mixer and feed-forward side by side, each behind a norm of its own of the same stream:
    stream += mixer(c(norm_mixer(stream))) + feed_forward(norm_feed_forward(stream)).  ``input_conv`` (c, a
    parts.ResidualConv, or None) is a short convolution on what the mixer reads; its last inputs are kept beside
    the mixer's cache (CombinedCache members ``mixer`` and ``conv``).  ``feed_forward`` (and its norm) may be None.
    Both norms are taken before either branch is added; the adds are 32-bit."""

    def __init__(self, norm_mixer, mixer, norm_feed_forward=None, feed_forward=None, input_conv=None):
        if (feed_forward is None) != (norm_feed_forward is None):
            raise ValueError("a feed-forward and its norm come together or not at all")
        self.norm_mixer, self.mixer = norm_mixer, mixer
        self.norm_feed_forward, self.feed_forward = norm_feed_forward, feed_forward
        self.input_conv = input_conv

    def children(self):
        return [p for p in (self.norm_mixer, self.input_conv, self.mixer, self.norm_feed_forward, self.feed_forward)
                if p is not None]

    def cache_requirement(self):
        if self.input_conv is None:
            return self.mixer.cache_requirement()
        return CombinedCache([("mixer", self.mixer.cache_requirement()), ("conv", self.input_conv.cache_requirement())])

    def prepare(self, device, dtype):
        # the norms' weights in 32-bit for the pass that makes both norms at once
        self._w_mixer = self.norm_mixer.weight.float().contiguous()
        self._w_ff = None if self.norm_feed_forward is None else self.norm_feed_forward.weight.float().contiguous()

    def forward(self, h, residual, step, cache, next_norm=None):
        import torch
        ops = self.ops
        if isinstance(h, NormedBranch):
            h = h.resolve()
        if isinstance(h, Normed):               # a block of another kind before this one: its last add may be pending
            h = h.pending
        elif isinstance(h, StreamCopy):
            h = None
        if h is not None:
            residual.add_(h.float())
        conv, nm, nf = self.input_conv, self.norm_mixer, self.norm_feed_forward
        if conv is not None and (nf is None or nf.eps == nm.eps):
            # both norms divide by the same root mean square: one pass over the stream makes both, and the convolution
            x, y = ops.norm_pair_conv(residual, self._w_mixer, None if nf is None else self._w_ff, nm.eps, conv.weight,
                                      cache.sub("conv").tensors["tail"], step)
        else:
            x = ops.add_rmsnorm(None, residual, nm.weight, nm.eps, out_dtype=torch.float32 if conv is not None else None)
            if conv is not None:
                x = conv.forward(x, step, cache.sub("conv"))
            y = None if nf is None else ops.add_rmsnorm(None, residual, nf.weight, nf.eps)
        sink = Sink(residual)
        a = self.mixer.forward(x, step, cache.sub("mixer") if conv is not None else cache, add_to=sink)
        if a is not None:
            residual.add_(a.float())
        if y is not None:
            f = self.feed_forward.forward(y, step, add_to=sink)
            if f is not None:
                residual.add_(f.float())
        return None, residual


@register_block("sandwich")
class SandwichBlock(Block):
    """A norm before and after each sublayer, and an optional short convolution on what each sublayer reads:
    stream += norm_mixer_out(mixer(c1(norm_mixer(stream)))); stream += norm_feed_forward_out(feed_forward(c2(
    norm_feed_forward(stream)))).  ``conv_mixer`` / ``conv_feed_forward`` (c1, c2: parts.ResidualConv or None) keep
    their last inputs beside the mixer's cache (CombinedCache members ``mixer``, ``conv1``, ``conv2``).  The
    feed-forward (with its two norms and its convolution) may be None.  The norms may be of any kind that has
    ``add_branch`` (RMS norms, layer norms with weight and bias).  Norms, convolutions and adds are 32-bit;
    the sublayers hand their 32-bit sums to the norm after them.  A sublayer's output is added by whoever reads the
    stream next (kernels.api.NormedBranch): where that is a sublayer with a convolution, one backend call adds the
    normed output and makes the next input."""

    def __init__(self, norm_mixer, mixer, norm_mixer_out, norm_feed_forward=None, feed_forward=None,
                 norm_feed_forward_out=None, conv_mixer=None, conv_feed_forward=None):
        if len({feed_forward is None, norm_feed_forward is None, norm_feed_forward_out is None}) != 1:
            raise ValueError("a feed-forward and its two norms come together or not at all")
        if feed_forward is None and conv_feed_forward is not None:
            raise ValueError("a convolution on the feed-forward's input needs a feed-forward")
        self.norm_mixer, self.mixer, self.norm_mixer_out = norm_mixer, mixer, norm_mixer_out
        self.norm_feed_forward, self.feed_forward = norm_feed_forward, feed_forward
        self.norm_feed_forward_out = norm_feed_forward_out
        self.conv_mixer, self.conv_feed_forward = conv_mixer, conv_feed_forward

    def children(self):
        return [p for p in (self.norm_mixer, self.conv_mixer, self.mixer, self.norm_mixer_out, self.norm_feed_forward,
                            self.conv_feed_forward, self.feed_forward, self.norm_feed_forward_out) if p is not None]

    def cache_requirement(self):
        if self.conv_mixer is None and self.conv_feed_forward is None:
            return self.mixer.cache_requirement()
        return CombinedCache([("mixer", self.mixer.cache_requirement()),
                              ("conv1", None if self.conv_mixer is None else self.conv_mixer.cache_requirement()),
                              ("conv2", None if self.conv_feed_forward is None else self.conv_feed_forward.cache_requirement())])

    def _read(self, pending, residual, norm, conv, cache, member, step):
        """What a sublayer reads: the normed stream (after the pending branch output, if any, has been added),
        through its convolution if it has one."""
        import torch
        ops = self.ops
        if conv is None:
            if pending is not None:
                return pending.resolve(then=norm)
            return norm.forward(None, residual)
        if getattr(norm, "kind", None) != "rmsnorm":     # another kind of norm: in 32-bit, then the convolution
            if pending is not None:
                pending.resolve()
            return conv.forward(norm.forward(None, residual, out_dtype=torch.float32), step, cache.sub(member))
        w = norm.weight if norm.weight.dtype == torch.float32 else norm.weight.float()
        tail = cache.sub(member).tensors["tail"]
        if (pending is not None and pending.y is not None and pending.stream is residual
                and getattr(pending.norm, "kind", "rmsnorm") == "rmsnorm"):
            y, pending.y = pending.y, None
            return ops.branch_norm_conv(y, residual, pending.weight, pending.eps, w, norm.eps, conv.weight, tail, step)
        if pending is not None:
            pending.resolve()
        return ops.norm_pair_conv(residual, w, None, norm.eps, conv.weight, tail, step)[0]

    def forward(self, h, residual, step, cache, next_norm=None):
        ops = self.ops
        pending = None
        if isinstance(h, NormedBranch):         # a block of this kind before this one: its last branch is still to be added
            pending, h = h, None
        elif isinstance(h, Normed):             # a block of another kind before this one: its last add may be pending
            h = h.pending
        elif isinstance(h, StreamCopy):
            h = None
        if h is not None:
            residual.add_(h.float())
        combined = self.conv_mixer is not None or self.conv_feed_forward is not None
        x = self._read(pending, residual, self.norm_mixer, self.conv_mixer, cache, "conv1", step)
        a = self.mixer.forward(x, step, cache.sub("mixer") if combined else cache)
        pending = NormedBranch(ops, a, residual, self.norm_mixer_out.weight, self.norm_mixer_out.eps, norm=self.norm_mixer_out)
        if self.feed_forward is not None:
            y = self._read(pending, residual, self.norm_feed_forward, self.conv_feed_forward, cache, "conv2", step)
            f = self.feed_forward.forward(y, step)
            pending = NormedBranch(ops, f, residual, self.norm_feed_forward_out.weight, self.norm_feed_forward_out.eps,
                                   norm=self.norm_feed_forward_out)
        return pending, residual
