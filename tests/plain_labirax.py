"""The Labirax decoder written out plainly: whole sequence, no cache, float64, one function per mechanism.

It shares no code with the package.  ``forward(config, weights, ids)`` takes the config.json dictionary, a
name -> tensor dictionary and one request's token ids and returns the logits of every position; with
``streams`` (a list) it also appends the residual stream after every layer run (a layer that borrows another's
weights counts as a run of its own).

Notation: n tokens, stream s [n, width].  A layer is
    s += L1b(mixer(L1 s));  s += L2b(ff(L2 s))
with L(x) = (x - mean) / sqrt(var + eps) * w + b.  Mixers: ``attention`` (grouped queries, biased projections, no
rotation, a temperature on the query that grows with the logarithm of the position, a learned bias per head and
bucketed distance on the scores), ``latent_attention`` (keys and values expanded from a low-rank latent, one rotated
key part for all heads, a sliding window, an output gate), ``gla`` (a linear-attention state per head that decays per
key channel).  The feed-forward is a mixture of gated experts beside a shared one.
"""
from __future__ import annotations

import math

import torch


def layer_norm(x, weight, bias, eps):
    mean = x.mean(-1, keepdim=True)
    var = (x - mean).pow(2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight + bias


def rms_norm(x, weight, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ attention with a distance bias
def distance_bucket(n: int, buckets: int, farthest: float) -> int:
    """The row of the bias table for a key ``n`` positions back: one row a distance for the first half of the
    table, then rows whose reach grows geometrically up to ``farthest``; the last row takes everything beyond."""
    half = buckets // 2
    if n < half:
        return n
    return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(farthest / half) * (buckets - half))))


def query_temperature(positions, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1) per position."""
    return 1.0 + coef * torch.log(torch.floor((positions + 1) / every) + 1.0)


def biased_attention(q, k, v, scale, table, farthest):
    """q [n, H, d], k [n, G, d], v [n, G, dv], table [buckets, H].  Causal softmax of q . k * scale + table[bucket(i - j), h].
    -> [n, H, dv]"""
    n, H = q.shape[0], q.shape[1]
    rep = H // k.shape[1]
    scores = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, 1)) * scale
    B = table.shape[0]
    rows = torch.tensor([[distance_bucket(i - j, B, farthest) if j <= i else 0 for j in range(n)] for i in range(n)])
    scores = scores + table[rows].permute(2, 0, 1)
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    scores = scores.masked_fill(j > i, float("-inf"))
    return torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), v.repeat_interleave(rep, 1))


def attention_mixer(h, W, p, m):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ W[f"{p}.q"].T + W[f"{p}.q.b"]).view(n, H, d)
    k = (h @ W[f"{p}.k"].T + W[f"{p}.k.b"]).view(n, G, d)
    v = (h @ W[f"{p}.v"].T + W[f"{p}.v.b"]).view(n, G, dv)
    pos = torch.arange(n, dtype=h.dtype)
    q = q * query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    o = biased_attention(q, k, v, m["scale"], W[f"{p}.rel"], m["bias_max"])
    return o.reshape(n, H * dv) @ W[f"{p}.o"].T


# ------------------------------------------------------------------ attention through a latent
def rotate_half(x, positions, base, dims):
    """x [n, ..., D]: of the first ``dims`` numbers, number i turns with number i + dims / 2 by positions * base^(-2i/dims)."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    a = positions.to(x.dtype)[:, None] * f
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (half,)
    cos, sin = torch.cos(a).view(shape), torch.sin(a).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def window_mask(n, size):
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if size is not None:
        seen = seen & (i - j < size)
    return seen


def latent_attention_mixer(h, W, p, m, eps):
    n = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n)
    cq = rms_norm(h @ W[f"{p}.dq"].T, W[f"{p}.dq.norm"], eps)
    q = (cq @ W[f"{p}.uq"].T).view(n, H, d + dr)
    down = h @ W[f"{p}.dkv"].T
    c = rms_norm(down[:, :r], W[f"{p}.dkv.norm"], eps)
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    k_rot = rotate_half(down[:, r:], pos, base, dims)                    # [n, dr], one for all heads
    q_rot = rotate_half(q[..., d:], pos, base, dims)                     # [n, H, dr]
    k_plain = (c @ W[f"{p}.uk"].T).view(n, H, d)
    v = (c @ W[f"{p}.uv"].T).view(n, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q[..., :d], k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    seen = window_mask(n, (m.get("mask") or {}).get("size"))
    scores = scores.masked_fill(~seen[None], float("-inf"))
    o = torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), v).reshape(n, H * dv)
    return (o * torch.sigmoid(h @ W[f"{p}.g"].T)) @ W[f"{p}.o"].T


# ------------------------------------------------------------------ gated linear attention
def gla_decay(h, W, p, tau):
    """sigmoid(z)^(1 / tau), z = W_a2 (W_a1 h) + b."""
    z = (h @ W[f"{p}.a1"].T) @ W[f"{p}.a2"].T + W[f"{p}.a2.b"]
    return torch.exp(torch.nn.functional.logsigmoid(z) / tau)


def gla_scan(q, k, v, alpha, state=None):
    """q, k, alpha [n, H, d], v [n, H, dv]; S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  -> (o [n, H, dv], S)"""
    n, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=q.dtype) if state is None else state.clone()
    out = []
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hij,hi->hj", S, q[t]))
    return torch.stack(out), S


def gla_mixer(h, W, p, m, eps):
    n = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ W[f"{p}.q"].T).view(n, H, d) * d ** -0.5
    k = (h @ W[f"{p}.k"].T).view(n, H, d)
    v = (h @ W[f"{p}.v"].T).view(n, H, dv)
    alpha = gla_decay(h, W, p, m["tau"]).view(n, H, d)
    o, _ = gla_scan(q, k, v, alpha)
    o = rms_norm(o, W[f"{p}.norm"], eps).reshape(n, H * dv)
    return (o * silu(h @ W[f"{p}.g"].T)) @ W[f"{p}.o"].T


# ------------------------------------------------------------------ feed-forward
def gated_ff(h, W, p):
    return (silu(h @ W[f"{p}.gate"].T) * (h @ W[f"{p}.up"].T)) @ W[f"{p}.down"].T


def route(h, W, p, top, margins=None):
    """-> (chosen [n, top], weights [n, top]): softmax over all experts, the ``top`` largest, their scores over
    their sum.  ``margins`` (a list) receives, per token, the gap between the last chosen and the first refused logit."""
    z = h @ W[f"{p}.router"].T
    s = torch.softmax(z, dim=-1)
    picked = torch.topk(s, top, dim=-1)
    if margins is not None and top < s.shape[-1]:
        ranked = torch.sort(z, dim=-1, descending=True).values
        margins += (ranked[:, top - 1] - ranked[:, top]).tolist()
    return picked.indices, picked.values / (picked.values.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, W, p, f, margins=None):
    chosen, weight = route(h, W, p, f["router"]["top"], margins)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weight[t]):
            out[t] += w * gated_ff(h[t:t + 1], W, f"{p}.e{e}")[0]
    if f.get("shared") is not None:
        out = out + gated_ff(h, W, f"{p}.shared")
    return out


# ------------------------------------------------------------------ the model
def forward(config, weights, ids, streams=None, dtype=torch.float64, margins=None):
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    norm = lambda x, name: layer_norm(x, W[name], W[name + ".b"], eps)        # noqa: E731
    s = W["embed"][torch.as_tensor(ids, dtype=torch.long)] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i if layer.get('weights_of') is None else layer['weights_of']}"
        h, m = norm(s, f"{p}.norm1"), layer["mixer"]
        if layer["type"] == "attention":
            y = attention_mixer(h, W, f"{p}.mix", m)
        elif layer["type"] == "latent_attention":
            y = latent_attention_mixer(h, W, f"{p}.mix", m, eps)
        elif layer["type"] == "gla":
            y = gla_mixer(h, W, f"{p}.mix", m, eps)
        else:
            raise ValueError(layer["type"])
        s = s + norm(y, f"{p}.norm1b")
        f = layer.get("mlp")
        if f is not None:
            s = s + norm(moe_ff(norm(s, f"{p}.norm2"), W, f"{p}.mlp", f, margins), f"{p}.norm2b")
        if streams is not None:
            streams.append(s.clone())
    logits = norm(s, "final.norm") @ W["head"].T * config.get("logit_scale", 1.0)
    cap = config.get("logit_softcap")
    return logits if cap is None else cap * torch.tanh(logits / cap)
