"""The operations parts compute with.  The product has one implementation, the
HIP library (hip_backend.HipBackend); tests hand a model another one to check
the engine's host logic without a GPU.

Conventions: T tokens of a step, flattened; activations in ``act_dtype``
(bfloat16 or float32); the residual stream and logits in float32; int32 indices.
Every op runs on the current stream and allocates its outputs with torch.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any


ACTIVATIONS = ("silu", "gelu_tanh", "relu2")


@dataclass
class Sink:
    """Where a part's last product goes: added into the float32 ``stream``; and, if the block knows it,
    the norm that will read the stream next (its weight and eps), so that a backend can prepare that
    norm's input in the same kernel."""
    stream: Any
    norm_weight: Any = None
    norm_eps: float = 0.0


class Normed:
    """A normalised input that is not computed yet: rmsnorm(residual (+ pending)) * weight, of all
    rows or of ``rows``.  A backend's ``linear`` may take it whole (norm and product in one kernel);
    anything else calls ``materialize()``, which also performs the pending add exactly once."""

    def __init__(self, ops, pending, residual, weight, eps, rows=None, ready=None):
        self.ops, self.pending, self.residual, self.weight, self.eps, self.rows = ops, pending, residual, weight, eps, rows
        self.ready = ready        # backend-private: what an earlier kernel already prepared of this norm
        self._value = None

    def with_rows(self, rows):
        return Normed(self.ops, self.pending, self.residual, self.weight, self.eps, rows, self.ready)

    @property
    def shape(self):
        n = self.residual.shape[0] if self.rows is None else self.rows.shape[0]
        return (n, self.residual.shape[1])

    def materialize(self, out_dtype=None):
        if self._value is None:
            self._value = self.ops.add_rmsnorm(self.pending, self.residual, self.weight, self.eps,
                                               out_dtype=out_dtype, rows=self.rows)
            if self.rows is None:
                self.pending = None          # it is in the stream now
        return self._value


class NormedLayer(Normed):
    """The same for a layer norm with weight and bias: layernorm(residual (+ pending)) * weight + bias."""

    def __init__(self, ops, pending, residual, weight, bias, eps, rows=None):
        super().__init__(ops, pending, residual, weight, eps, rows)
        self.bias = bias

    def with_rows(self, rows):
        return NormedLayer(self.ops, self.pending, self.residual, self.weight, self.bias, self.eps, rows)

    def materialize(self, out_dtype=None):
        if self._value is None:
            self._value = self.ops.add_layernorm(self.pending, self.residual, self.weight, self.bias, self.eps,
                                                 out_dtype=out_dtype, rows=self.rows)
            if self.rows is None:
                self.pending = None
        return self._value


class NormedBranch:
    """A branch output that is still to be normed and added to the stream: stream += rmsnorm(y) * weight, or, with
    ``norm`` (a parts.Norm that has ``add_branch``), stream += norm(y) whatever kind of norm that is.  The block
    that made it hands it on so that the next reader of the stream may do the add in the kernel that makes its own
    input (``KernelBackend.branch_norm_conv``, or ``resolve(then=...)``); anyone else calls ``resolve()``, which
    performs the add exactly once."""

    def __init__(self, ops, y, stream, weight, eps, norm=None):
        self.ops, self.y, self.stream, self.weight, self.eps, self.norm = ops, y, stream, weight, eps, norm

    def resolve(self, then=None):
        """Adds the normed branch output to the stream.  ``then`` (a parts.Norm): also returns that norm of the updated
        stream, in the activation dtype; where both norms are of one kind that knows how, in the same kernel."""
        y, self.y = self.y, None
        if y is None:
            return None if then is None else then.forward(None, self.stream)
        if self.norm is not None:
            return self.norm.add_branch(y, self.stream, then)
        self.ops.branch_norm_add(y, self.stream, self.weight, self.eps, copy=False)
        return None if then is None else then.forward(None, self.stream)


class StreamCopy:
    """The residual stream as it stands, in the activation dtype (``value``; the stream itself where that is
    float32): what a block hands on when nothing is pending and its branches read the stream unnormed."""

    def __init__(self, stream, value):
        self.stream, self.value = stream, value


class KernelBackend:
    name = "?"
    act_dtype = None

    def prefer_rows(self, counts) -> None:
        """Row counts of steps that will recur (the batch sizes decode graphs are captured at, the token budget
        of a step): a backend may spend time once, outside any capture, to choose its kernels for them."""

    def embedding(self, ids, table, taken_from=None, earlier_tokens=None, scale=1.0):
        """stream[t, :] = float(table[ids[t], :]) * scale -> [T, width] float32.  With ``taken_from`` (int32 [T]):
        where it is >= 0 the token is ``earlier_tokens[taken_from[t]]`` instead of ``ids[t]`` (a token the
        step before chose, read on the device because the host has not seen it yet)."""
        raise NotImplementedError

    def add_rmsnorm(self, x, residual, weight, eps, out_dtype=None, rows=None):
        """If ``x`` is given: residual += float(x), in place.  y = residual *
        rsqrt(mean(residual^2) + eps) * weight, all in float32, rounded once to
        ``out_dtype`` (default act_dtype).  With ``rows`` only those rows are
        computed, y is [len(rows), width] and residual is not modified."""
        raise NotImplementedError

    def linear(self, x, w, bias=None, out_dtype=None, add_to=None):
        """y = x w^T (+ bias); w [out, in]; 32-bit accumulation.  ``x`` is a tensor or a Normed.
        With ``add_to`` (the float32 stream [T, out], or a Sink around it) the backend may add y into
        the stream in place and return None, or, for a Sink that names the next norm, a Normed of the
        updated stream for that norm; if it returns a plain tensor, the caller still has to add it."""
        raise NotImplementedError

    def linear_silu_mul(self, x, w_gate_up, intermediate):
        """gu = x w^T with w [2 * intermediate, in]; returns silu(gu[:, :I]) * gu[:, I:].
        ``x`` is a tensor or a Normed."""
        raise NotImplementedError

    def linear_act_mul(self, x, w_gate_up, intermediate, activation="silu"):
        """The same with another gate function: act(gu[:, :I]) * gu[:, I:], act one of ACTIVATIONS."""
        if activation == "silu":
            return self.linear_silu_mul(x, w_gate_up, intermediate)
        raise NotImplementedError

    def linear_act(self, x, w, activation="relu2"):
        """act(x w^T), act one of ACTIVATIONS, computed on the product's 32-bit sums and rounded once
        -> [T, out] in the activation dtype.  ``x`` is a tensor or a Normed."""
        raise NotImplementedError

    def scale_(self, t, factor):
        """t *= factor in place (float32), returns t."""
        raise NotImplementedError

    def scale_softcap_(self, t, scale, cap):
        """t = cap * tanh(t * scale / cap) in place (float32; ``cap`` None: t * scale), returns t."""
        raise NotImplementedError

    def add_layernorm(self, x, residual, weight, bias, eps, out_dtype=None, rows=None):
        """If ``x`` is given: residual += float(x), in place.  y = (residual - mean) / sqrt(var + eps) * weight + bias,
        mean and var (the mean of the squared deviations) of each row, all in float32 (weight, bias float32 [width]),
        rounded once to ``out_dtype`` (default act_dtype).  With ``rows`` only those rows are computed, y is
        [len(rows), width] and residual is not modified."""
        raise NotImplementedError

    def branch_layernorm_add(self, y, stream, weight, bias, eps, next_norm=None):
        """stream += layernorm(y) * weight + bias, row by row in float32 (y [T, width] of any float dtype).  With
        ``next_norm`` = (weight, bias, eps) also returns that layer norm of the updated stream in the activation dtype
        (a backend may do both in one kernel); else None."""
        raise NotImplementedError

    def branch_norm_add(self, y, stream, weight, eps, copy=True):
        """stream += y * rsqrt(mean(y^2) + eps) * weight, row by row in float32 (y [T, width] of any float
        dtype; None: nothing is added).  Returns the updated stream in the activation dtype, rounded once
        (the stream itself where that is float32); with ``copy`` False nothing is returned (and no copy made)."""
        raise NotImplementedError

    def rmsnorm_columns(self, x, col, n, weight, eps):
        """RMSNorm of columns [col, col + n) of x [T, *] float32, times weight [n] -> [T, n] in the activation dtype."""
        raise NotImplementedError

    # ---- attention through a cached latent (one shared latent "head" of kv_rank + rot_dim numbers a token)
    def latent_kv_store(self, sums, col, kv_rank, rot_dim, norm_weight, eps, positions, inv_freq, k_cache, v_cache,
                        slot_mapping, also_norm=None, layout="interleaved"):
        """Columns [col, col + kv_rank + rot_dim) of ``sums`` [T, *] float32 are a token's down-projection.  The
        first kv_rank, RMS-normed with ``norm_weight``, are its latent c; of the last rot_dim the first
        2 * len(inv_freq) turn in adjacent pairs (2i, 2i + 1) (``layout`` "half": pairs (i, i + len(inv_freq))) by the
        angle position * inv_freq[i] (32-bit).
        Token t's slot of k_cache [pages, 1, page, P] gets [c | turned part | zeros], of v_cache [pages, 1, P, page]
        [c | zeros] (P = the cache's padded size >= kv_rank + rot_dim).  ``also_norm`` = (col, n, weight): the same call
        also returns rmsnorm_columns(sums, col, n, weight, eps) (the query latent beside the key/value latent)."""
        raise NotImplementedError

    def latent_query_rotate_(self, q, num_heads, kv_rank, padded_dim, positions, inv_freq, layout="interleaved"):
        """q [T, H padded_dim], every head laid out as the cache's key rows are ([against the latent | rotated part | 0]):
        the first 2 * len(inv_freq) numbers of each head's rotated part (columns kv_rank ..) turn in place in adjacent
        pairs (``layout`` "half": element i with element i + len(inv_freq)) by the angle position * inv_freq[i].
        Returns q."""
        raise NotImplementedError

    def latent_value_gate(self, o, w_uv, gate, gate_col, num_heads, vdim, kv_rank, padded_dim):
        """o [T, H padded_dim] (attention over the latents; the first kv_rank of each head count); w_uv [H vdim,
        kv_rank]; gate [T, *] float32 whose columns [gate_col, gate_col + H vdim) are the gate before its sigmoid.
        -> (W_uv,h o_h) * sigmoid(gate) [T, H vdim] in the activation dtype."""
        raise NotImplementedError

    # ---- gated linear recurrence with a short convolution before it
    def causal_conv(self, x, col, channels, in_bias, taps, conv_bias, tail, step):
        """u[t, c] = conv_bias[c] + sum_k taps[c, k] * in(t - (K - 1 - k), c), in(t, c) = x[t, col + c] + in_bias[c]
        (x float32 [T, *]); inputs before a row's first token come from ``tail`` [slots, K - 1, channels] float32
        (the last K - 1 inputs of the row's request, zeros at its start), which this call only reads.
        -> [T, channels] float32."""
        raise NotImplementedError

    def grouped_linear(self, x, w, bias=None, x_groups=None):
        """x [T, Gx * in] float; w [G, out, in]; bias [G, out] or None.  Group g multiplies block g % Gx of x's
        columns (x_groups = Gx, default G): y[t, g, :] = w[g] x[t, g % Gx, :] + bias[g] -> [T, G * out] float32,
        32-bit arithmetic throughout."""
        raise NotImplementedError

    def rglru_scan(self, u, gates, lam, y, y_col, y_bias, x, x_col, x_bias, state, tail, step, taps, decay_scale=8.0):
        """Per row and channel, tokens in order: r, i = sigmoid of gates[t, c], gates[t, C + c];
        a = exp(-decay_scale * r * softplus(lam[c])); S = a S + sqrt(1 - a^2) * i * u[t, c] from the row's slot of
        ``state`` [slots, C] float32, left there afterwards; out[t, c] = S * gelu_tanh(y[t, y_col + c] + y_bias[c]).
        Also shifts the row's inputs x[t, x_col + c] + x_bias[c] into ``tail`` [slots, max(1, taps - 1), C].  All float32;
        -> [T, C] in the activation dtype."""
        raise NotImplementedError

    # ---- routed experts
    def route_topk(self, logits, bias, top, over="chosen", choice_bias=None, renormalise=False):
        """logits [T, E] float32 (+ bias [E]).  ``over`` "chosen": the ``top`` largest of a token (lowest index first
        among equals), in falling order, and the softmax over those alone.  ``over`` "all": scores = softmax over all
        E; chosen are the ``top`` largest of scores + choice_bias (float32 [E] or None; lowest index first among
        equals, falling order) and the shares are the chosen ones' scores as they are, or, with ``renormalise``,
        divided by their sum + 1e-20.
        -> (experts [T, top] int32, shares [T, top] float32)."""
        raise NotImplementedError

    def glu_rows_block(self, inner: int) -> int:
        """How ``routed_experts`` wants a gated expert's 2 * inner stacked rows: 0, the gate rows before the up rows; n
        (a divisor of inner), alternating blocks of n gate rows and n up rows (the kernels then meet a channel's gate
        and up sums in one place).  A part asks once, orders its rows so and passes the answer on as ``glu_block``."""
        return 0

    def routed_experts(self, x, experts, shares, w_up, w_down, activation="relu2", gated=None, identity_from=None,
                       glu_block=0):
        """y[t] = sum_j shares[t, j] * W_down[e] act(W_up[e] x[t]), e = experts[t, j]; w_up [E, ff, width],
        w_down [E, width, ff]; the hidden activation is rounded once to the activation dtype -> [T, width] float32.
        ``gated`` = (limit, alpha) or (limit, alpha, shift): w_up is [E, 2 ff, width], an expert's gate rows before its
        up rows (or in alternating blocks of ``glu_block`` gate rows and as many up rows: see glu_rows_block), and the
        hidden activation is g * sigmoid(alpha g) * (u + shift) with g = min(gate sum, limit), u = clamp(up sum, -limit,
        limit), shift 1 unless given (limit infinite, alpha 1, shift 0: silu(gate) * up), ``activation`` unused.  ``identity_from`` = E: a choice e >= E is an expert that returns x[t] itself (such
        choices may be all there are: w_up and w_down None)."""
        raise NotImplementedError

    # ---- a short convolution on a mixer's input, attention from one product's sums, the delta rule
    def residual_conv(self, h, taps, tail, step, out_dtype=None):
        """h [T, C] float32, taps [C, K] float32: y[t] = h[t] + sum_j taps[:, j] * h[t - (K - 1) + j], per row of the
        step; inputs before a row's first token come from ``tail`` [slots, max(1, K - 1), C] float32 (the last K - 1
        inputs of the row's request, oldest first; zeros at its start), which afterwards holds the last K - 1 inputs
        including this step's.  All float32 -> [T, C] in ``out_dtype`` (default: the activation dtype)."""
        raise NotImplementedError

    def norm_pair_conv(self, stream, w_first, w_second, eps, taps, tail, step):
        """Two RMS norms of the same float32 stream [T, width] and the short convolution of ``residual_conv`` on the
        first: x = residual_conv(rmsnorm(stream) * w_first), y = rmsnorm(stream) * w_second (None: no second norm),
        both in the activation dtype; ``tail`` moves on.  -> (x, y).  A backend may do it in one pass."""
        import torch
        h = self.add_rmsnorm(None, stream, w_first, eps, out_dtype=torch.float32)
        x = self.residual_conv(h, taps, tail, step)
        return x, (None if w_second is None else self.add_rmsnorm(None, stream, w_second, eps))

    def branch_norm_conv(self, y, stream, w_out, eps_out, w_next, eps_next, taps, tail, step):
        """``branch_norm_add`` of y (float32 [T, width]; weight w_out, eps_out) into the float32 stream, then the first
        result of ``norm_pair_conv`` of the updated stream (weight w_next, eps_next; no second norm) -> x in the
        activation dtype.  A backend may do both in one kernel."""
        self.branch_norm_add(y, stream, w_out, eps_out, copy=False)
        return self.norm_pair_conv(stream, w_next, None, eps_next, taps, tail, step)[0]

    def qkv_finish(self, sums, q_col, k_col, v_col, num_q_heads, num_kv_heads, dim, vdim, padded_dim, positions, inv_freq,
                   layout, k_cache, v_cache, slot_mapping, q_norm=None, k_norm=None, eps=0.0, q_head_scale=None,
                   norm_per_head=False, col_bias=None, position_temperature=None):
        """What lies between a q/k/v projection's float32 sums [T, *] and attention, in 32-bit: queries are columns
        [q_col, q_col + Hq dim), keys [k_col, k_col + Hkv dim), values [v_col, v_col + Hkv vdim), or, with ``v_col``
        None, the keys as projected (vdim = dim).  ``col_bias`` (float32, one number a column of the sums): the
        projection's biases, added first.  ``position_temperature`` = (coef, every): the query at position p is
        multiplied by 1 + coef * ln(floor((p + 1) / every) + 1), every a whole number of positions.  ``q_norm`` / ``k_norm`` (float32 [Hq dim] / [Hkv dim]): RMS norm over
        the whole of a token's queries (keys) at once, times that weight, before anything else; with ``norm_per_head`` the
        norm is taken head by head over the head's dim numbers and the weights are float32 [dim], one for all query
        heads and one for all key heads.  Then the first
        2 * len(inv_freq) numbers of every query and key head turn by the angles position * inv_freq[i]: ``layout``
        "interleaved" pairs (2i, 2i + 1), "half" pairs (i, i + len(inv_freq)).  ``q_head_scale`` (float32 [Hq]):
        head h's turned query times that number.  Keys and values go to the token's slot of k_cache [pages, Hkv, page, P]
        and v_cache [pages, Hkv, P, page], P = ``padded_dim`` >= dim, vdim, zeros beyond their own size.
        -> q [T, Hq * P] in the activation dtype, zeros beyond dim."""
        raise NotImplementedError

    def head_gate_(self, o, gate, gate_col, num_heads, head_dim):
        """o [T, H * head_dim] *= sigmoid(gate[t, gate_col + h]) for every number of head h, in place (gate float32
        [T, *]).  Returns o."""
        raise NotImplementedError

    def delta_rule(self, sums, cols, num_heads, dim, w_decay, decay_bias, decay_scale, removal_bias, norm_weight, eps,
                   state, step):
        """The delta-rule recurrence from one product's float32 sums [T, *].  ``cols``: first column of r, k, v (H dim
        each), of the output gate g and the removal gate a (H dim each) and of the decay's inner activations w
        (w_decay.shape[1] of them).  Per token, head and key channel i, all in 32-bit:
        decay = exp(-decay_scale * sigmoid(w_decay tanh(w) + decay_bias)), a = sigmoid(a + removal_bias),
        u = k / sqrt(sum(k^2) + 1e-6) per head.  Per row and head, tokens in order, from the row's slot of ``state``
        [slots, H, dim, dim] float32 (S[i, j]: key channel i, value channel j), left there afterwards:
        S <- diag(decay) S - (a * u) (u^T S) + k v^T with both terms of the old S; o = S^T r.
        -> rmsnorm(o over a head, eps) * norm_weight * sigmoid(g)  [T, H * dim] in the activation dtype."""
        raise NotImplementedError

    def normed_sum_add(self, stream, ys, weights, eps, scale):
        """stream += scale * sum_i rmsnorm(ys[i], eps) * weights[i], row by row in float32 (each y [T, width] float32,
        one or two of them).  Returns stream."""
        raise NotImplementedError

    def rotary_kv_store(self, qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                        k_cache, v_cache, slot_mapping):
        """Rotate the first ``rotary_dim`` dims of every q and k head of
        qkv [T, (Hq + 2 Hkv) D] in place (pairs j, j + rotary_dim / 2; angle tables
        cos, sin [positions, rotary_dim / 2] float32), then write k and v of token t to
        cache slot slot_mapping[t] of k_cache [pages, Hkv, page, D] and v_cache [pages, Hkv, D, page].
        rotary_dim 0: no rotation.  num_kv_heads 0 (k_cache None): q only, no write."""
        raise NotImplementedError

    def linear_rotary_kv_store(self, x, w_qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                               k_cache, v_cache, slot_mapping, for_attention: bool = False):
        """The fused q/k/v projection followed by rotary_kv_store.  Returns a tensor whose first
        Hq * D columns are the encoded q (the whole qkv, or q alone): a backend may do all of it in
        one kernel.  ``x`` is a tensor or a Normed.  ``for_attention``: the caller hands the result to this
        backend's ``paged_attention`` of the same step over the same caches, and to nothing else; a backend
        may then return an object of its own that only that call understands (work it has put off)."""
        qkv = self.linear(x, w_qkv)
        self.rotary_kv_store(qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim, k_cache,
                             v_cache, slot_mapping)
        return qkv

    def gla(self, sums, cols, num_heads, dim, vdim, w_decay, decay_bias, tau, q_scale, norm_weight, eps, state, step):
        """Gated linear attention from one product's float32 sums [T, *].  ``cols``: first column of q, k (H dim each),
        of v and the output gate g (H vdim each) and of the decay's inner activations a (w_decay.shape[1] of them).  Per
        token, head and key channel, in 32-bit: alpha = sigmoid(w_decay a + decay_bias)^(1 / tau).  Per row and head,
        tokens in order, from the row's slot of ``state`` [slots, H, dim, vdim] float32 (S[i, j]: key channel i, value
        channel j), left there afterwards: S <- diag(alpha) S + k v^T; o = S^T (q * q_scale).
        -> rmsnorm(o over a head, eps) * norm_weight [vdim] * silu(g)  [T, H * vdim] in the activation dtype."""
        raise NotImplementedError

    def paged_attention(self, qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group, step, scale,
                        window, sink=None, weights="softmax", softcap=None, chunk=None, head_bias=None,
                        distance_bias=None):
        """For token t of row r at position p: softmax over keys max(0, p - window + 1)..p
        of row r (read through group.block_tables[r]) of (q . k) * scale, times v.
        q head i uses kv head i // (Hq / Hkv).  q is the first Hq * D columns of
        qkv (row stride qkv.stride(0)).  ``sink`` (a number): one more term exp(sink) in every softmax's
        denominator, with no value.  ``chunk`` (a number of positions): keys before floor(p / chunk) * chunk are not
        seen either.  ``softcap`` (c > 0): the scaled scores pass through c * tanh(score / c).  ``weights`` "sigmoid":
        no softmax; a visible key counts with sigmoid(score + head_bias[i]) (head_bias float32 [Hq] or None), not
        normalised over the keys (no sink).  ``distance_bias`` (float32 [Hq, N]): a key n positions back of the query
        adds distance_bias[i, min(n, N - 1)] to query head i's score, after scale and cap.
        Returns [T, Hq * D] in act_dtype."""
        raise NotImplementedError

    def sample(self, logits, temperatures, seeds, counters, out=None):
        """Per row: argmax(logits) if temperature == 0, else argmax(logits / temperature + g)
        with Gumbel noise g from (seed, counter, vocabulary index).  -> [R] int32 (``out`` if given)."""
        raise NotImplementedError
