"""Plain references of every kernel, with the kernels' own signatures.

Two uses: the GPU tests compare each HIP kernel with the function of the same
name here, at sizes other than the engine's; and, handed to a model in place of
the HIP library, they let the host side of the engine (batching, block tables,
cache, scheduler, replay) run on the CPU.  Straightforward torch, float64
inside where it is cheap; nothing here is fast and nothing in the product
imports it.
"""
from __future__ import annotations

import numpy as np
import torch

from mini_inference_engine_amd.kernels.api import KernelBackend, Normed, Sink


def ref_embedding(ids, table, scale=1.0):
    out = table[ids.long()].float()
    return out if scale == 1.0 else out * scale


def ref_act(z, activation):
    if activation == "silu":
        return z * torch.sigmoid(z)
    if activation == "gelu_tanh":
        return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
    if activation == "relu2":
        return torch.relu(z) ** 2
    raise ValueError(activation)


def ref_branch_norm_add(y, stream, weight, eps, act_dtype):
    if y is not None:
        yd = y.double()
        stream.add_((yd * torch.rsqrt(yd.pow(2).mean(-1, keepdim=True) + eps) * weight.double()).float())
    return stream if act_dtype == torch.float32 else stream.to(act_dtype)


def ref_rmsnorm_columns(x, col, n, weight, eps, out_dtype):
    xd = x[:, col:col + n].double()
    return (xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + eps) * weight.double()).to(out_dtype)


def ref_turn_pairs(x, positions, inv_freq):
    """x [T, heads, d] float64: the first 2 * len(inv_freq) dims turn in adjacent pairs; the angle is a float32 product."""
    n = 2 * inv_freq.shape[0]
    angle = (positions.float()[:, None] * inv_freq.float()[None, :]).double()
    c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def ref_latent_kv_store(sums, col, kv_rank, rot_dim, norm_weight, eps, positions, inv_freq, k_cache, v_cache, slots,
                        layout="interleaved"):
    P = k_cache.shape[2]
    c = ref_rmsnorm_columns(sums, col, kv_rank, norm_weight, eps, torch.float64)
    kr = ref_turn(sums[:, None, col + kv_rank:col + kv_rank + rot_dim].double(), positions, inv_freq, layout)[:, 0]
    page, off = slots.long() // P, slots.long() % P
    k_cache[page, 0, off, :] = 0
    k_cache[page, 0, off, :kv_rank] = c.to(k_cache.dtype)
    k_cache[page, 0, off, kv_rank:kv_rank + rot_dim] = kr.to(k_cache.dtype)
    v_cache[page, 0, :, off] = 0
    v_cache[page, 0, :kv_rank, off] = c.to(v_cache.dtype)


def ref_latent_query_rotate(q, H, kv_rank, padded, positions, inv_freq, layout="interleaved"):
    T, n = q.shape[0], 2 * inv_freq.shape[0]
    heads = q.view(T, H, padded)
    heads[..., kv_rank:kv_rank + n] = ref_turn(heads[..., kv_rank:kv_rank + n].double(), positions, inv_freq, layout).to(q.dtype)
    return q


def ref_latent_value_gate(o, w_uv, gate, gate_col, H, vdim, kv_rank, padded, out_dtype):
    T = o.shape[0]
    v = torch.einsum("thr,hvr->thv", o.double().view(T, H, padded)[..., :kv_rank], w_uv.double().view(H, vdim, kv_rank))
    v = v.reshape(T, H * vdim)
    if gate is not None:
        v = v * torch.sigmoid(gate[:, gate_col:gate_col + H * vdim].double())
    return v.to(out_dtype)


def ref_causal_conv(x, col, C, in_bias, taps, conv_bias, tail, row_start, slots):
    K = taps.shape[1]
    out = torch.empty(x.shape[0], C, dtype=torch.float32, device=x.device)
    for r in range(len(slots)):
        a, b = int(row_start[r]), int(row_start[r + 1])
        inp = torch.cat([tail[int(slots[r])][:K - 1].double(), x[a:b, col:col + C].double() + in_bias.double()])
        acc = conv_bias.double().expand(b - a, C).clone()
        for k in range(K):
            acc += inp[k:k + b - a] * taps[:, k].double()
        out[a:b] = acc.float()
    return out


def ref_grouped_linear(x, w, bias, x_groups):
    G, n_out, n_in = w.shape
    gx = x_groups or G
    xb = x.double().view(x.shape[0], gx, n_in)
    y = torch.stack([xb[:, g % gx] @ w[g].double().T for g in range(G)], 1)
    if bias is not None:
        y = y + bias.double().view(1, G, n_out)
    return y.reshape(x.shape[0], G * n_out).float()


def ref_rglru_scan(u, gates, lam, y, y_col, y_bias, x, x_col, x_bias, state, tail, row_start, slots, taps, decay_scale, out_dtype):
    C = u.shape[1]
    K1 = taps - 1
    out = torch.empty(u.shape[0], C, dtype=torch.float64, device=u.device)
    sp = torch.nn.functional.softplus(lam.double())
    for r in range(len(slots)):
        a0, b0, slot = int(row_start[r]), int(row_start[r + 1]), int(slots[r])
        S = state[slot].double()
        for t in range(a0, b0):
            rg, ig = torch.sigmoid(gates[t, :C].double()), torch.sigmoid(gates[t, C:].double())
            a = torch.exp(-decay_scale * rg * sp)
            S = a * S + torch.sqrt(1.0 - a * a) * ig * u[t].double()
            out[t] = S * ref_act(y[t, y_col:y_col + C].double() + y_bias.double(), "gelu_tanh")
        state[slot] = S.float()
        if K1:
            inp = torch.cat([tail[slot][:K1].double(), x[a0:b0, x_col:x_col + C].double() + x_bias.double()])
            tail[slot][:K1] = inp[-K1:].float()
    return out.to(out_dtype)


def ref_route_topk(logits, bias, top, over="chosen", choice_bias=None, renormalise=False):
    z = logits.double() if bias is None else logits.double() + bias.double()
    if over == "all":
        scores = torch.softmax(z.float(), -1).double()
        by = scores if choice_bias is None else (scores.float() + choice_bias.float()).double()
        idx = torch.sort(by, dim=-1, descending=True, stable=True).indices[:, :top]
        shares = torch.gather(scores, 1, idx)
        if renormalise:
            shares = shares / (shares.sum(-1, keepdim=True) + 1e-20)
        return idx.to(torch.int32), shares.float()
    order = torch.sort(z, dim=-1, descending=True, stable=True)
    idx, val = order.indices[:, :top], order.values[:, :top]
    return idx.to(torch.int32), torch.softmax(val, -1).float()


def ref_clamped_glu(gu, inner, limit, alpha, shift=1.0):
    g, u = gu[..., :inner].clamp(max=limit), gu[..., inner:].clamp(min=-limit, max=limit)
    return g * torch.sigmoid(alpha * g) * (u + shift)


def ref_routed_experts(x, experts, shares, w_up, w_down, activation, act_dtype, gated=None, identity_from=None):
    y = torch.zeros(x.shape[0], x.shape[1], dtype=torch.float64, device=x.device)
    for t in range(x.shape[0]):
        for j in range(experts.shape[1]):
            e = int(experts[t, j])
            if identity_from is not None and e >= identity_from:
                y[t] += shares[t, j].double() * x[t].double()
                continue
            z = x[t].double() @ w_up[e].double().T
            h = ref_act(z, activation) if gated is None else ref_clamped_glu(z, z.shape[-1] // 2, *gated)
            y[t] += shares[t, j].double() * (h.to(act_dtype).double() @ w_down[e].double().T)
    return y.float()


def ref_add_rmsnorm(x, residual, weight, eps, out_dtype, rows=None):
    if rows is not None:
        r = residual[rows.long()]
        if x is not None:
            r = r + x[rows.long()].float()
    else:
        if x is not None:
            residual.add_(x.float())
        r = residual
    rd = r.double()
    y = rd * torch.rsqrt(rd.pow(2).mean(-1, keepdim=True) + eps) * weight.double()
    return y.to(out_dtype)


def ref_linear(x, w, bias=None, out_dtype=None):
    y = x.double() @ w.double().T
    if bias is not None:
        y = y + bias.double()
    return y.to(out_dtype or x.dtype)


def ref_silu_mul(gu, inter, out_dtype):
    g, u = gu[:, :inter].double(), gu[:, inter:].double()
    return (g * torch.sigmoid(g) * u).to(out_dtype)


def ref_rotary_kv_store(qkv, positions, cos, sin, rotary_dim, Hq, Hkv, D, k_cache, v_cache, slot_mapping):
    T = qkv.shape[0]
    heads = qkv.view(T, Hq + 2 * Hkv, D)
    if rotary_dim:
        half = rotary_dim // 2
        c = cos[positions.long()].double()[:, None, :]
        s = sin[positions.long()].double()[:, None, :]
        x = heads[:, :Hq + Hkv, :rotary_dim].double()
        x1, x2 = x[..., :half], x[..., half:]
        heads[:, :Hq + Hkv, :rotary_dim] = torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), -1).to(qkv.dtype)
    if Hkv and k_cache is not None:
        P = k_cache.shape[2]
        page, off = slot_mapping.long() // P, slot_mapping.long() % P
        k_cache[page, :, off, :] = heads[:, Hq:Hq + Hkv, :]
        v_cache[page, :, :, off] = heads[:, Hq + Hkv:, :]       # values: [pages, Hkv, D, page]


def ref_paged_attention(qkv, Hq, Hkv, D, k_cache, v_cache, block_tables, token_row, positions, scale, window,
                        out_dtype, sink=None, weights="softmax", softcap=None, chunk=None, head_bias=None, distance_bias=None):
    """Token by token, keys gathered through the block table."""
    T = qkv.shape[0]
    P = k_cache.shape[2]
    g = Hq // Hkv
    out = torch.empty(T, Hq * D, dtype=out_dtype, device=qkv.device)
    rows = token_row.tolist()
    pos = positions.tolist()
    bt = block_tables.long()
    for t in range(T):
        p = pos[t]
        lo = 0 if window is None else max(0, p - window + 1)
        if chunk is not None:
            lo = max(lo, p // chunk * chunk)
        keys = torch.arange(lo, p + 1, device=qkv.device)
        pages = bt[rows[t], keys // P]
        k = k_cache[pages, :, keys % P, :].double()          # [n, Hkv, D]
        v = v_cache[pages, :, :, keys % P].double()             # [n, Hkv, D]
        q = qkv[t, :Hq * D].double().view(Hkv, g, D)
        s = torch.einsum("hgd,nhd->hgn", q, k) * scale
        if softcap is not None:
            s = softcap * torch.tanh(s / softcap)
        if distance_bias is not None:
            n = (p - keys).clamp(max=distance_bias.shape[1] - 1)
            s = s + distance_bias.double()[:, n].view(Hkv, g, -1)
        if weights == "sigmoid":
            pr = torch.sigmoid(s if head_bias is None else s + head_bias.double().view(Hkv, g, 1))
        elif sink is None:
            pr = torch.softmax(s, dim=-1)
        else:               # one more term in the denominator, with no value
            top = s.max(-1, keepdim=True).values.clamp(min=sink)
            e = torch.exp(s - top)
            pr = e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))
        out[t] = torch.einsum("hgn,nhd->hgd", pr, v).reshape(Hq * D).to(out_dtype)
    return out


def ref_residual_conv(h, taps, tail, row_start, slots, out_dtype):
    K = taps.shape[1]
    out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
    for r in range(len(slots)):
        a, b, slot = int(row_start[r]), int(row_start[r + 1]), int(slots[r])
        inp = torch.cat([tail[slot][:K - 1].double(), h[a:b].double()])
        acc = h[a:b].double().clone()
        for j in range(K):
            acc += inp[j:j + b - a] * taps[:, j].double()
        out[a:b] = acc.to(out_dtype)
        if K > 1:
            tail[slot][:K - 1] = inp[-(K - 1):].float()
    return out


def ref_turn(x, positions, inv_freq, layout):
    """x [T, heads, d] float64: the first 2 * len(inv_freq) numbers of a head turn, adjacent pairs ("interleaved") or
    element i with i + len(inv_freq) ("half"); the angle is a float32 product."""
    if layout == "interleaved":
        return ref_turn_pairs(x, positions, inv_freq)
    n = inv_freq.shape[0]
    angle = (positions.float()[:, None] * inv_freq.float()[None, :]).double()
    c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    out = x.clone()
    out[..., :n] = u * c - v * s
    out[..., n:2 * n] = v * c + u * s
    return out


def ref_qkv_finish(sums, q_col, k_col, v_col, Hq, Hkv, dim, vdim, P, positions, inv_freq, layout, k_cache, v_cache, slots,
                   q_norm, k_norm, eps, q_head_scale, out_dtype, norm_per_head=False, col_bias=None, position_temperature=None):
    T = sums.shape[0]
    if col_bias is not None:
        sums = (sums.double() + col_bias.double()).float()
    q = sums[:, q_col:q_col + Hq * dim].double()
    k = sums[:, k_col:k_col + Hkv * dim].double()
    v = k if v_col is None else sums[:, v_col:v_col + Hkv * vdim].double()
    v = v.view(T, Hkv, -1)
    if norm_per_head:
        q, k = q.view(T, Hq, dim), k.view(T, Hkv, dim)
    if q_norm is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm.double()
    if k_norm is not None:
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm.double()
    q, k = q.reshape(T, Hq, dim), k.reshape(T, Hkv, dim)
    if inv_freq is not None:
        q, k = ref_turn(q, positions, inv_freq, layout), ref_turn(k, positions, inv_freq, layout)
    if q_head_scale is not None:
        q = q * q_head_scale.double()[None, :, None]
    if position_temperature is not None:
        coef, every = position_temperature
        q = q * (1.0 + coef * torch.log(torch.div(positions.long() + 1, every, rounding_mode="floor").double() + 1.0))[:, None, None]
    page_size = k_cache.shape[2]
    page, off = slots.long() // page_size, slots.long() % page_size
    k_cache[page, :, off, :] = 0
    k_cache[page, :, off, :dim] = k.to(k_cache.dtype)
    v_cache[page, :, :, off] = 0
    v_cache[page, :, :v.shape[-1], off] = v.to(v_cache.dtype)
    out = torch.zeros(T, Hq, P, dtype=out_dtype, device=sums.device)
    out[..., :dim] = q.to(out_dtype)
    return out.view(T, Hq * P)


def ref_head_gate(o, gate, gate_col, H, D):
    T = o.shape[0]
    g = torch.sigmoid(gate[:, gate_col:gate_col + H].double())
    return (o.double().view(T, H, D) * g[:, :, None]).view(T, H * D).to(o.dtype)


def ref_delta_rule(sums, cols, H, d, w_decay, decay_bias, decay_scale, removal_bias, norm_weight, eps, state, row_start, slots,
                   out_dtype):
    T, n = sums.shape[0], H * d
    x = sums.double()
    r, k, v, g, a = (x[:, cols[c]:cols[c] + n].view(T, H, d) for c in ("r", "k", "v", "g", "a"))
    inner = torch.tanh(x[:, cols["w"]:cols["w"] + w_decay.shape[1]])
    decay = torch.exp(-decay_scale * torch.sigmoid(inner @ w_decay.double().T + decay_bias.double())).view(T, H, d)
    a = torch.sigmoid(a + removal_bias.double().view(H, d))
    u = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    out = torch.empty(T, H, d, dtype=torch.float64, device=sums.device)
    for row in range(len(slots)):
        S = state[int(slots[row])].double()
        for t in range(int(row_start[row]), int(row_start[row + 1])):
            seen = torch.einsum("hi,hij->hj", u[t], S)
            S = decay[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * seen[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hij,hi->hj", S, r[t])
        state[int(slots[row])] = S.float()
    out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps)
    return (out.view(T, n) * norm_weight.double() * torch.sigmoid(g.reshape(T, n))).to(out_dtype)


def ref_normed_sum_add(stream, ys, weights, eps, scale):
    total = torch.zeros_like(stream, dtype=torch.float64)
    for y, w in zip(ys, weights):
        yd = y.double()
        total += yd * torch.rsqrt(yd.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    stream.add_((scale * total).float())
    return stream


def ref_layernorm(x, weight, bias, eps):
    xd = x.double()
    mean = xd.mean(-1, keepdim=True)
    var = (xd - mean).pow(2).mean(-1, keepdim=True)
    return (xd - mean) / torch.sqrt(var + eps) * weight.double() + bias.double()


def ref_add_layernorm(x, residual, weight, bias, eps, out_dtype, rows=None):
    if rows is not None:
        r = residual[rows.long()].double()
        if x is not None:
            r = r + x[rows.long()].double()
        return ref_layernorm(r, weight, bias, eps).to(out_dtype)
    if x is not None:
        residual.add_(x.float())
    return ref_layernorm(residual, weight, bias, eps).to(out_dtype)


def ref_branch_layernorm_add(y, stream, weight, bias, eps, next_norm, act_dtype):
    stream.add_(ref_layernorm(y, weight, bias, eps).float())
    if next_norm is None:
        return None
    return ref_layernorm(stream, next_norm[0], next_norm[1], next_norm[2]).to(act_dtype)


def ref_scale_softcap(t, scale, cap):
    v = t.double() * scale
    return (v if cap is None else cap * torch.tanh(v / cap)).float()


def ref_gla(sums, cols, H, d, dv, w_decay, decay_bias, tau, q_scale, norm_weight, eps, state, row_start, slots, out_dtype):
    T = sums.shape[0]
    x = sums.double()
    q = x[:, cols["q"]:cols["q"] + H * d].view(T, H, d) * q_scale
    k = x[:, cols["k"]:cols["k"] + H * d].view(T, H, d)
    v = x[:, cols["v"]:cols["v"] + H * dv].view(T, H, dv)
    g = x[:, cols["g"]:cols["g"] + H * dv]
    z = x[:, cols["a"]:cols["a"] + w_decay.shape[1]] @ w_decay.double().T
    if decay_bias is not None:
        z = z + decay_bias.double()
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(T, H, d)
    out = torch.empty(T, H, dv, dtype=torch.float64, device=sums.device)
    for row in range(len(slots)):
        S = state[int(slots[row])].double()
        for t in range(int(row_start[row]), int(row_start[row + 1])):
            S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hij,hi->hj", S, q[t])
        state[int(slots[row])] = S.float()
    out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_weight.double()
    return (out.view(T, H * dv) * g * torch.sigmoid(g)).to(out_dtype)


def _fmix32(x):
    m = np.uint64(0xFFFFFFFF)
    x = x ^ (x >> np.uint64(16))
    x = (x * np.uint64(0x85EBCA6B)) & m
    x = x ^ (x >> np.uint64(13))
    x = (x * np.uint64(0xC2B2AE35)) & m
    return x ^ (x >> np.uint64(16))


def ref_gumbel(seed, counter, vocab):
    m = np.uint64(0xFFFFFFFF)
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    key = _fmix32(_fmix32(_fmix32(np.uint64(seed & 0xFFFFFFFF)) ^ np.uint64(seed >> 32))
                  ^ np.uint64(int(counter) & 0xFFFFFFFF))
    v = np.arange(vocab, dtype=np.uint64)
    x = _fmix32(key ^ _fmix32((v + np.uint64(0x9E3779B9)) & m))
    u = ((x >> np.uint64(9)).astype(np.float32) + np.float32(0.5)) * np.float32(2.0 ** -23)
    return torch.from_numpy(-np.log(-np.log(u.astype(np.float64))))


def ref_perturbed(logits_row, temperature, seed, counter):
    z = logits_row.double().cpu()
    if temperature <= 0:
        return z
    return z / temperature + ref_gumbel(seed, counter, z.shape[0])


def ref_sample(logits, temperatures, seeds, counters):
    out = []
    for r in range(logits.shape[0]):
        out.append(int(torch.argmax(ref_perturbed(logits[r], float(temperatures[r]), int(seeds[r]), int(counters[r])))))
    return torch.tensor(out, dtype=torch.int32, device=logits.device)


class TorchBackend(KernelBackend):
    name = "torch-reference"

    def __init__(self, act_dtype=torch.float32, adds_in_place=True):
        self.act_dtype = act_dtype
        self.adds_in_place = adds_in_place      # linear(add_to=...) adds and returns None, or leaves it to the caller
        self.calls = {}

    def _count(self, name):
        self.calls[name] = self.calls.get(name, 0) + 1

    def embedding(self, ids, table, taken_from=None, earlier_tokens=None, scale=1.0):
        self._count("embedding")
        if taken_from is not None:
            ids = torch.where(taken_from >= 0, earlier_tokens[taken_from.clamp(min=0).long()], ids)
        return ref_embedding(ids, table, scale)

    def scale_(self, t, factor):
        return t.mul_(factor)

    def scale_softcap_(self, t, scale, cap):
        return t.copy_(ref_scale_softcap(t, scale, cap))

    def add_layernorm(self, x, residual, weight, bias, eps, out_dtype=None, rows=None):
        self._count("add_layernorm")
        return ref_add_layernorm(x, residual, weight, bias, eps, out_dtype or self.act_dtype, rows)

    def branch_layernorm_add(self, y, stream, weight, bias, eps, next_norm=None):
        self._count("branch_layernorm_add")
        return ref_branch_layernorm_add(y, stream, weight, bias, eps, next_norm, self.act_dtype)

    def gla(self, sums, cols, num_heads, dim, vdim, w_decay, decay_bias, tau, q_scale, norm_weight, eps, state, step):
        self._count("gla")
        return ref_gla(sums, cols, num_heads, dim, vdim, w_decay, decay_bias, tau, q_scale, norm_weight, eps, state,
                       step.host["row_start"], step.host["state_slots"], self.act_dtype)

    def linear_act(self, x, w, activation="relu2"):
        self._count("linear_act")
        if isinstance(x, Normed):
            x = x.materialize()
        return ref_act(ref_linear(x, w, None, torch.float32).double(), activation).to(self.act_dtype)

    def branch_norm_add(self, y, stream, weight, eps, copy=True):
        self._count("branch_norm_add")
        return ref_branch_norm_add(y, stream, weight, eps, self.act_dtype)

    def rmsnorm_columns(self, x, col, n, weight, eps):
        return ref_rmsnorm_columns(x, col, n, weight, eps, self.act_dtype)

    def linear_act_mul(self, x, w_gate_up, intermediate, activation="silu"):
        self._count("linear_act_mul")
        if isinstance(x, Normed):
            x = x.materialize()
        gu = ref_linear(x, w_gate_up, None, self.act_dtype).double()
        return (ref_act(gu[:, :intermediate], activation) * gu[:, intermediate:]).to(self.act_dtype)

    def latent_kv_store(self, sums, col, kv_rank, rot_dim, norm_weight, eps, positions, inv_freq, k_cache, v_cache,
                        slot_mapping, also_norm=None, layout="interleaved"):
        self._count("latent_kv_store")
        ref_latent_kv_store(sums, col, kv_rank, rot_dim, norm_weight, eps, positions, inv_freq, k_cache, v_cache, slot_mapping,
                            layout)
        if also_norm is not None:
            return ref_rmsnorm_columns(sums, also_norm[0], also_norm[1], also_norm[2], eps, self.act_dtype)
        return None

    def latent_query_rotate_(self, q, num_heads, kv_rank, padded_dim, positions, inv_freq, layout="interleaved"):
        return ref_latent_query_rotate(q, num_heads, kv_rank, padded_dim, positions, inv_freq, layout)

    def latent_value_gate(self, o, w_uv, gate, gate_col, num_heads, vdim, kv_rank, padded_dim):
        return ref_latent_value_gate(o, w_uv, gate, gate_col, num_heads, vdim, kv_rank, padded_dim, self.act_dtype)

    def causal_conv(self, x, col, channels, in_bias, taps, conv_bias, tail, step):
        return ref_causal_conv(x, col, channels, in_bias, taps, conv_bias, tail, step.host["row_start"],
                               step.host["state_slots"])

    def grouped_linear(self, x, w, bias=None, x_groups=None):
        return ref_grouped_linear(x, w, bias, x_groups)

    def rglru_scan(self, u, gates, lam, y, y_col, y_bias, x, x_col, x_bias, state, tail, step, taps, decay_scale=8.0):
        self._count("rglru_scan")
        return ref_rglru_scan(u, gates, lam, y, y_col, y_bias, x, x_col, x_bias, state, tail, step.host["row_start"],
                              step.host["state_slots"], taps, decay_scale, self.act_dtype)

    def route_topk(self, logits, bias, top, over="chosen", choice_bias=None, renormalise=False):
        return ref_route_topk(logits, bias, top, over, choice_bias, renormalise)

    def routed_experts(self, x, experts, shares, w_up, w_down, activation="relu2", gated=None, identity_from=None, glu_block=0):
        assert glu_block == 0, "the torch operations keep gate rows before up rows"
        self._count("routed_experts")
        return ref_routed_experts(x, experts, shares, w_up, w_down, activation, self.act_dtype, gated, identity_from)

    def add_rmsnorm(self, x, residual, weight, eps, out_dtype=None, rows=None):
        self._count("add_rmsnorm")
        return ref_add_rmsnorm(x, residual, weight, eps, out_dtype or self.act_dtype, rows)

    def linear(self, x, w, bias=None, out_dtype=None, add_to=None):
        self._count("linear")
        if isinstance(x, Normed):
            x = x.materialize()
        y = ref_linear(x, w, bias, out_dtype or self.act_dtype)
        sink = add_to if isinstance(add_to, Sink) else (Sink(add_to) if add_to is not None else None)
        if sink is not None and self.adds_in_place:
            sink.stream.add_(y.float())
            if sink.norm_weight is not None:      # as a fusing backend would: the next norm, prepared
                return Normed(self, None, sink.stream, sink.norm_weight, sink.norm_eps)
            return None
        return y

    def linear_silu_mul(self, x, w_gate_up, intermediate):
        self._count("linear_silu_mul")
        if isinstance(x, Normed):
            x = x.materialize()
        return ref_silu_mul(ref_linear(x, w_gate_up, None, self.act_dtype), intermediate, self.act_dtype)

    def rotary_kv_store(self, qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                        k_cache, v_cache, slot_mapping):
        self._count("rotary_kv_store")
        ref_rotary_kv_store(qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                            k_cache, v_cache, slot_mapping)

    def paged_attention(self, qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group, step, scale,
                        window, sink=None, weights="softmax", softcap=None, chunk=None, head_bias=None, distance_bias=None):
        self._count("paged_attention")
        return ref_paged_attention(qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group.block_tables,
                                   step.token_row, step.positions, scale, window, self.act_dtype, sink=sink,
                                   weights=weights, softcap=softcap, chunk=chunk, head_bias=head_bias,
                                   distance_bias=distance_bias)

    def residual_conv(self, h, taps, tail, step, out_dtype=None):
        self._count("residual_conv")
        return ref_residual_conv(h, taps, tail, step.host["row_start"], step.host["state_slots"], out_dtype or self.act_dtype)

    def qkv_finish(self, sums, q_col, k_col, v_col, num_q_heads, num_kv_heads, dim, vdim, padded_dim, positions, inv_freq,
                   layout, k_cache, v_cache, slot_mapping, q_norm=None, k_norm=None, eps=0.0, q_head_scale=None,
                   norm_per_head=False, col_bias=None, position_temperature=None):
        self._count("qkv_finish")
        return ref_qkv_finish(sums, q_col, k_col, v_col, num_q_heads, num_kv_heads, dim, vdim, padded_dim, positions, inv_freq,
                              layout, k_cache, v_cache, slot_mapping, q_norm, k_norm, eps, q_head_scale, self.act_dtype,
                              norm_per_head, col_bias, position_temperature)

    def head_gate_(self, o, gate, gate_col, num_heads, head_dim):
        o.copy_(ref_head_gate(o, gate, gate_col, num_heads, head_dim))
        return o

    def delta_rule(self, sums, cols, num_heads, dim, w_decay, decay_bias, decay_scale, removal_bias, norm_weight, eps,
                   state, step):
        self._count("delta_rule")
        return ref_delta_rule(sums, cols, num_heads, dim, w_decay, decay_bias, decay_scale, removal_bias, norm_weight, eps,
                              state, step.host["row_start"], step.host["state_slots"], self.act_dtype)

    def normed_sum_add(self, stream, ys, weights, eps, scale):
        self._count("normed_sum_add")
        return ref_normed_sum_add(stream, ys, weights, eps, scale)

    def sample(self, logits, temperatures, seeds, counters, out=None):
        self._count("sample")
        tokens = ref_sample(logits, temperatures, seeds, counters)
        if out is None:
            return tokens
        out.copy_(tokens)
        return out
