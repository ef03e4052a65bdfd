"""The Mutusun decoder written out plainly: whole sequence, no cache, float64, one function per mechanism.

It shares no code with the package.  ``forward(config, weights, ids)`` takes the config.json dictionary, a
name -> tensor dictionary and one request's token ids and returns the logits of every position; with
``streams`` (a list) it also appends the residual stream after every layer run (a layer that borrows another's
weights counts as a run of its own).

Notation: n tokens, stream s [n, width].  A layer is
    s += N1b(mixer(c1(N1 s)));  s += N2b(ff(c2(N2 s)))
with N(x) = x / rms(x) * (1 + w) and c(h) = h + conv(h), a short causal convolution per channel.
"""
from __future__ import annotations

import torch


def rms_norm(x, weight, eps, one_plus=False):
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    if weight is None:
        return y
    return y * (1.0 + weight) if one_plus else y * weight


def input_conv(h, taps):
    """h [n, channels] -> h + conv(h); taps [channels, K], the last column multiplies the current token, zeros
    stand before the sequence's start."""
    n, K = h.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, h.shape[1], dtype=h.dtype), h])
    return h + sum(padded[j:j + n] * taps[:, j] for j in range(K))


def chunk_mask(n, size):
    """[n, n] bool: query i sees key j <= i of its own chunk (chunks of ``size`` positions counted from 0; None: all)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if size is not None:
        seen = seen & (i // size == j // size)
    return seen


def soft_cap(scores, cap):
    return scores if cap is None else cap * torch.tanh(scores / cap)


def sigmoid_attention(q, k, v, scale, cap, head_bias, seen):
    """q [n, H, d], k [n, G, d], v [n, G, dv], head_bias [H], seen [n, n].  A visible key's weight is
    sigmoid(cap(q . k * scale) + bias of the head); the weights are not normalised.  -> [n, H, dv]"""
    H, G = q.shape[1], k.shape[1]
    rep = H // G
    scores = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, 1)) * scale
    weights = torch.sigmoid(soft_cap(scores, cap) + head_bias[:, None, None])
    weights = torch.where(seen[None], weights, torch.zeros_like(weights))
    return torch.einsum("hij,jhd->ihd", weights, v.repeat_interleave(rep, 1))


def attention_mixer(h, W, p, m, eps):
    """The mixer 'attention': projections, a norm per head on queries and keys (one weight of the head's size for all
    heads), no positions, capped scores, chunked causal mask, sigmoid weights, output projection."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ W[f"{p}.q"].T).view(n, H, d)
    k = (h @ W[f"{p}.k"].T).view(n, G, d)
    v = (h @ W[f"{p}.v"].T).view(n, G, dv)
    q = rms_norm(q, W[f"{p}.q.norm"], eps)
    k = rms_norm(k, W[f"{p}.k.norm"], eps)
    size = (m.get("mask") or {}).get("size")
    o = sigmoid_attention(q, k, v, m["scale"], m.get("softcap"), W[f"{p}.pb"], chunk_mask(n, size))
    return o.reshape(n, H * dv) @ W[f"{p}.o"].T


def dense_ff(h, W, p):
    return torch.relu(h @ W[f"{p}.up"].T).pow(2) @ W[f"{p}.down"].T


def expert(h, W, p, limit):
    g = (h @ W[f"{p}.gate"].T).clamp(max=limit)
    u = (h @ W[f"{p}.up"].T).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[f"{p}.down"].T


def route(h, W, p, top, margins=None):
    """-> (chosen [n, top], their weights [n, top]): softmax over all router outputs; the choice goes by the
    scores plus a correction, the weights are the scores themselves, not renormalised.  ``margins`` (a list)
    receives, per token, the gap between the last chosen and the first refused choice score."""
    s = torch.softmax(h @ W[f"{p}.router"].T, dim=-1)
    by = s + W[f"{p}.correction"]
    chosen = torch.topk(by, top, dim=-1).indices
    if margins is not None and top < by.shape[-1]:
        ranked = torch.sort(by, dim=-1, descending=True).values
        margins += (ranked[:, top - 1] - ranked[:, top]).tolist()
    return chosen, torch.gather(s, 1, chosen)


def moe_ff(h, W, p, f, margins=None):
    E, top = f["router"]["experts"], f["router"]["top"]
    chosen, weight = route(h, W, p, top, margins)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weight[t]):
            # router outputs beyond the experts are identity experts: the input itself
            y = h[t] if e >= E else expert(h[t:t + 1], W, f"{p}.e{e}", f["expert"]["limit"])[0]
            out[t] += w * y
    return out


def forward(config, weights, ids, streams=None, dtype=torch.float64, margins=None):
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    taps = (config.get("canon") or {}).get("taps")
    s = W["embed"][torch.as_tensor(ids, dtype=torch.long)]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i if layer.get('weights_of') is None else layer['weights_of']}"
        h = rms_norm(s, W[f"{p}.norm1"], eps, one_plus=True)
        if taps:
            h = input_conv(h, W[f"{p}.canon1"])
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        s = s + rms_norm(attention_mixer(h, W, f"{p}.mix", layer["mixer"], eps), W[f"{p}.norm1b"], eps, one_plus=True)
        f = layer.get("mlp")
        if f is not None:
            h = rms_norm(s, W[f"{p}.norm2"], eps, one_plus=True)
            if taps:
                h = input_conv(h, W[f"{p}.canon2"])
            y = dense_ff(h, W, f"{p}.mlp") if f["kind"] == "dense" else moe_ff(h, W, f"{p}.mlp", f, margins)
            s = s + rms_norm(y, W[f"{p}.norm2b"], eps, one_plus=True)
        if streams is not None:
            streams.append(s.clone())
    return rms_norm(s, W["final.norm"], eps, one_plus=True) @ W["head"].T

