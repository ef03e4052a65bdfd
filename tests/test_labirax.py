"""Labirax through the engine against the plain implementation (tests/plain_labirax.py).

Configurations are made here, with sizes that differ from one another wherever the design lets them (query and key/value
head counts, head size and value size, windows that are no multiple of a page and a window of one key, distance tables of
few and many rows, a query temperature that moves every few positions, rotated parts turned whole and in part, states
that are not square, decay ranks, experts with and without a shared one, top = 1 and top = every expert, layers that run
with an earlier or a later layer's tensors, a layer without a feed-forward).  Host tests run the engine's own parts,
cache and step function on the CPU with the torch operations of tests/torch_backend.py; GPU tests run the HIP kernels,
each kernel against the torch operation of the same name and the whole model in the four trace families, in float32
(tight) and bfloat16.
"""
import json
import math

import pytest
import torch

import plain_labirax as plain
import trace_util
from torch_backend import TorchBackend
import torch_backend as ref

from mini_inference_engine_amd.config import EngineConfig, LabiraxConfig, load_model_config
from mini_inference_engine_amd.engine.batch import StepRow
from mini_inference_engine_amd.engine.runner import ModelRunner
from mini_inference_engine_amd.replay.trace import replay
from mini_inference_engine_amd.weights import random_tensors


def att(heads, kv_heads, dim, vdim=None, scale=None, coef=0.4, every=5, buckets=8, bias_max=30):
    d = dict(heads=heads, kv_heads=kv_heads, dim=dim, scale=scale if scale is not None else dim ** -0.5,
             q_temp=dict(coef=coef, every=every), bias_max=bias_max, buckets=buckets)
    if vdim is not None:
        d["vdim"] = vdim
    return d


def lat(heads, dim, rot_dim, vdim, kv_rank, q_rank, window=None, dims=None, base=100.0, scale=None):
    d = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank,
             scale=scale if scale is not None else (dim + rot_dim) ** -0.5, rot=dict(base=base, dims=dims if dims is not None else rot_dim))
    if window is not None:
        d["mask"] = dict(size=window)
    return d


def gla(heads, dim, vdim=None, tau=4.0, rank=4):
    d = dict(heads=heads, dim=dim, tau=tau, rank=rank)
    if vdim is not None:
        d["vdim"] = vdim
    return d


def moe(experts, top, ff, shared=None):
    d = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
    if shared is not None:
        d["shared"] = dict(ff=shared)
    return d


def layer(kind, mixer, mlp, weights_of=None):
    d = dict(type=kind, mixer=mixer, mlp=mlp)
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def model(vocab, width, eps, layers, emb=1.0, logit_scale=1.0, cap=None):
    d = dict(architecture="Labirax", vocab=vocab, width=width, norm=dict(eps=eps), embedding=dict(scale=emb),
             logit_scale=logit_scale, layers=layers)
    if cap is not None:
        d["logit_softcap"] = cap
    return d


A_ATT = att(6, 2, 16, vdim=24, scale=0.3, every=7, buckets=8, bias_max=40)
A_LAT = lat(3, 16, 8, 24, 40, 24, window=24)                              # a window of a page and a half
A_GLA = gla(2, 16, vdim=32, tau=4.0, rank=4)
A_MOE = moe(5, 2, 48, shared=32)
CFG_A = model(211, 64, 1e-5, [layer("attention", A_ATT, A_MOE),
                              layer("gla", A_GLA, A_MOE),
                              layer("latent_attention", A_LAT, A_MOE),
                              layer("gla", A_GLA, A_MOE, weights_of=1),
                              layer("attention", A_ATT, A_MOE, weights_of=0),
                              layer("latent_attention", A_LAT, A_MOE, weights_of=2)], emb=0.5, logit_scale=2.0, cap=20.0)
B_ATT = att(4, 4, 8, coef=0.25, every=1, buckets=4, bias_max=3)           # as many key heads; a table of four rows
B_LAT = lat(2, 24, 12, 8, 20, 10, window=16, dims=8, base=7.0)            # a window of a page; a part of the rotated part turns
B_GLA = gla(3, 24, vdim=8, tau=1.0, rank=2)
CFG_B = model(150, 48, 1e-3, [layer("latent_attention", B_LAT, moe(4, 4, 24), weights_of=3),   # runs with a later layer's tensors
                              layer("gla", B_GLA, moe(3, 1, 40, shared=16)),
                              layer("attention", B_ATT, None),
                              layer("latent_attention", B_LAT, moe(4, 4, 24)),            # every expert chosen, no shared expert
                              layer("gla", B_GLA, moe(3, 1, 40, shared=16), weights_of=1)], emb=3.0)   # no logit scale, no cap
# sizes the kernels' vector paths do not like: nothing a multiple of 8, an odd vocabulary
C_ATT = att(3, 1, 10, vdim=14, scale=0.4, every=3, buckets=6, bias_max=11.5)
CFG_C = model(101, 70, 1e-6, [layer("gla", gla(1, 10, vdim=14, tau=9.0, rank=3), moe(3, 2, 26, shared=18)),
                              layer("attention", C_ATT, moe(2, 1, 18)),
                              layer("latent_attention", lat(5, 6, 2, 10, 12, 6, window=5), moe(3, 3, 22, shared=50)),
                              layer("latent_attention", lat(1, 18, 6, 6, 9, 30), None)], logit_scale=0.7, cap=5.0)   # no window
# wider heads, a table of many rows, eight query heads on one key head, a window longer than most requests
D_ATT = att(8, 1, 40, vdim=56, scale=0.2, every=16, buckets=32, bias_max=64)
CFG_D = model(333, 96, 1e-4, [layer("attention", D_ATT, moe(9, 3, 32, shared=64)),
                              layer("latent_attention", lat(4, 32, 16, 48, 64, 40, window=100), moe(6, 2, 24)),
                              layer("gla", gla(2, 48, vdim=64, tau=16.0, rank=8), moe(9, 3, 32, shared=64), weights_of=None),
                              layer("attention", D_ATT, moe(9, 3, 32, shared=64), weights_of=0)], emb=0.7, cap=30.0)
CONFIGS = {"A": (CFG_A, 3), "B": (CFG_B, 4), "C": (CFG_C, 6), "D": (CFG_D, 8)}


def shape_weights(cfg, seed, sharp=True):
    """Random weights shaped so that faults show: products keep the scale of their input, norm weights and biases are far
    from their resting values, the distance tables spread scores over several units, decays range from fast to slow,
    routers are decisive.  ``sharp`` False leaves tables and routers at unit scale: the bfloat16 runs use it, because
    spread scores amplify the rounding of 8-bit values as much as they amplify faults."""
    w = random_tensors(cfg, seed, torch.float32, std=1.0)
    g = torch.Generator().manual_seed(seed + 100)
    for k, v in w.items():
        if k.endswith(".rel"):
            v.copy_(torch.randn(v.shape, generator=g) * (2.0 if sharp else 0.5))
        elif k.endswith(".a2.b"):
            v.copy_(torch.randn(v.shape, generator=g) * 2.0 + 2.0)
        elif k.endswith((".q.b", ".k.b", ".v.b")):
            v.copy_(torch.randn(v.shape, generator=g) * 0.5)
        elif k.endswith(".b"):                                             # a norm's bias
            v.copy_(torch.randn(v.shape, generator=g) * 0.3)
        elif "norm" in k:
            v.copy_(1.0 + 0.4 * torch.randn(v.shape, generator=g))
        elif v.dim() >= 2:
            v.mul_(v.shape[-1] ** -0.5)
        if k.endswith(".router") and sharp:
            v.mul_(4.0)
        if k.endswith((".mix.q", ".mix.uq")) and sharp:
            v.mul_(2.0)
    return w


def make(name, dtype=torch.float32, sharp=True):
    raw, seed = CONFIGS[name]
    cfg = LabiraxConfig.from_dict(raw)
    return raw, cfg, {k: v.to(dtype) for k, v in shape_weights(cfg, seed, sharp).items()}


def expected_logits(raw, weights, prompts):
    wf = {k: v.float() for k, v in weights.items()}
    return {rid: plain.forward(raw, wf, toks) for rid, toks in prompts.items()}


def host_runner(cfg, weights, pages=64, rows=8, tokens=256, slots=None):
    return ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                       num_pages=pages, max_rows=rows, max_step_tokens=tokens, max_model_len=pages * 16, num_state_slots=slots)


# float32 against the float64 plain implementation: rounding, amplified by scores that are spread on purpose; a fault
# (a lost key, a window that is one position off, a lost state, a wrong bucket or expert) moves logits by a hundred times this
F32_TOL = 3e-4
# bfloat16: every sublayer rounds a handful of values to 8 bits
BF16_TOL_PER_LAYER = 1.5e-2

FAMILIES = {"whole": trace_util.whole, "decode_tail": lambda p: trace_util.decode_tail(p, 40),
            "portions": trace_util.portions, "mixed": lambda p: trace_util.mixed(p, 4, seed=5)}
LENGTHS = [3, 70, 1, 37, 90, 18, 49]


def compare_most(got, expected, tol, what, over=0.1, cap=1.0):
    """The bfloat16 comparison.  A token whose router scores nearly tie may choose another expert once values are rounded
    to 8 bits, and then its logits (and, weakly, those after it) differ by design, not by fault: at most ``over`` of the
    rows may exceed ``tol``, none may exceed ``cap`` of the logit scale or be other than finite."""
    errs = []
    for (rid, p), row in got.items():
        err = float((row.double().cpu() - expected[rid][p]).abs().max()) / float(expected[rid].abs().max())
        assert math.isfinite(err) and err <= cap, f"{what}: request {rid} position {p}: error {err:.3e} of the logit scale"
        errs.append(err)
    bad = sum(e > tol for e in errs)
    assert errs and bad <= over * len(errs), f"{what}: {bad} of {len(errs)} rows beyond {tol:.1e} of the logit scale"
    return max(errs)


def run_family(name, family, tmp_path, device, dtype, tol):
    raw, cfg, weights = make(name, torch.float32 if dtype == "float32" else torch.bfloat16, sharp=dtype == "float32")
    prompts = trace_util.random_prompts(raw["vocab"], LENGTHS, seed=17)
    steps = FAMILIES[family](prompts)
    peak = trace_util.live_token_peak(steps)
    pages = peak // 16 + 1 + 4
    backend = TorchBackend(torch.float32) if device == "cpu" else None
    runner = ModelRunner(cfg, weights=weights, dtype=dtype, device=device, backend=backend, num_pages=pages, max_rows=4,
                         max_step_tokens=max(64, peak), max_model_len=(pages - 1) * 16, num_state_slots=5)
    if family == "mixed":
        assert peak < sum(-(-n // 64) * 64 for n in LENGTHS), "the pool must be smaller than all requests together"
    replay(runner, trace_util.to_lines(steps), str(tmp_path), lambda _: None, max_live=4)
    runner.cache.check()
    assert not runner.cache.live
    got = trace_util.read_outputs(str(tmp_path), steps, raw["vocab"])
    check = trace_util.compare if dtype == "float32" else compare_most
    return check(got, expected_logits(raw, weights, prompts), tol, f"labirax {name}/{family}/{dtype}")


# ------------------------------------------------------------------------------------------- configuration
def test_config_round_trip_registry_and_sizes_from_tensor_shapes(tmp_path):
    raw, cfg, _ = make("A")
    assert LabiraxConfig.from_dict(cfg.to_dict()) == cfg
    (tmp_path / "config.json").write_text(json.dumps(raw))
    loaded, arch = load_model_config(str(tmp_path))
    assert loaded == cfg and arch.name == "Labirax"
    assert cfg.layers[3].weights_of == 1 and cfg.owner(4) == 0 and cfg.owner(2) == 2
    assert cfg.layers[0].mixer.vdim == 24 and cfg.layers[2].mixer.window == 24 and cfg.layers[1].mixer.rank == 4
    b = LabiraxConfig.from_dict(CFG_B)
    assert b.logit_softcap is None and b.logit_scale == 1.0 and b.layers[2].mlp is None and b.layers[3].mlp.shared_ff is None
    assert LabiraxConfig.from_dict(CFG_C).layers[3].mixer.window is None
    # the table's rows and the decay's inner size stand in no key: they are the checkpoint's tensor shapes
    bare = json.loads(json.dumps(raw))
    for entry in bare["layers"]:
        entry["mixer"].pop("buckets", None)
        entry["mixer"].pop("rank", None)
    shapes = {"l0.mix.rel": (8, 6), "l1.mix.a1": (4, 64)}
    assert LabiraxConfig.from_dict(bare, tensor_shapes=shapes) == cfg
    from mini_inference_engine_amd.config import ConfigError
    with pytest.raises(ConfigError):
        LabiraxConfig.from_dict(bare)


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][3].update(weights_of=9),                         # no such layer
    lambda c: c["layers"][3].update(weights_of=3),                         # itself
    lambda c: c["layers"][4].update(weights_of=3),                         # a layer that has no tensors of its own
    lambda c: c["layers"][3].update(mixer=gla(2, 16, vdim=16)),            # another layer than the one whose tensors it runs with
    lambda c: c["layers"][0]["mlp"]["router"].update(top=6),               # more than there are experts
    lambda c: c["layers"][0]["mixer"].update(kv_heads=4),                  # 6 query heads over 4 key heads
    lambda c: c["layers"][0]["mixer"].update(bias_max=4),                  # not beyond the table's first half
    lambda c: c["layers"][0]["mixer"].update(buckets=1),
    lambda c: c["layers"][0]["mixer"]["q_temp"].update(every=0),
    lambda c: c["layers"][0]["mixer"]["q_temp"].update(every=2.5),
    lambda c: c["layers"][1]["mixer"].update(tau=0.0),
    lambda c: c["layers"][2]["mixer"]["rot"].update(dims=10),              # more than the rotated part
    lambda c: c["layers"][2]["mixer"]["rot"].update(dims=3),
    lambda c: c["layers"][0]["mlp"].update(kind="dense"),
    lambda c: c["layers"][0].update(type="conv"),
    lambda c: c.update(logit_softcap=0.0),
])
def test_config_refuses_what_cannot_be_computed(bad):
    from mini_inference_engine_amd.config import ConfigError
    raw = json.loads(json.dumps(CFG_A))
    bad(raw)
    with pytest.raises(ConfigError):
        LabiraxConfig.from_dict(raw)


def test_model_structure():
    _, cfg, weights = make("A")
    runner = host_runner(cfg, weights)
    m = runner.model
    # three layers own tensors; six runs, each with a cache or state of its own
    assert [c.layer for c in m.spec.schedule] == [0, 1, 2, 1, 0, 2]
    assert "l3.norm1" not in weights and "l4.mix.q" not in weights and "l2.norm2b.b" in weights and "final.norm.b" in weights
    assert tuple(weights["l0.mix.rel"].shape) == (8, 6) and tuple(weights["l0.mix.q.b"].shape) == (96,)
    assert tuple(weights["l1.mix.a1"].shape) == (4, 64) and tuple(weights["l1.mix.a2"].shape) == (32, 4)
    assert tuple(weights["l1.mix.norm"].shape) == (32,) and tuple(weights["l2.mix.dkv"].shape) == (48, 64)
    assert "l0.mlp.e4.gate" in weights and "l0.mlp.e5.gate" not in weights and "l0.mlp.shared.down" in weights
    assert len(runner.storage.entries) == 6
    # two page groups: every key for the biased attention, a window of 24 for the latent attention
    assert sorted(m.page_groups, key=lambda w: w or 0) == [None, 24]
    assert not m.padding_safe, "a model with a recurrent state takes no padding tokens"


# ------------------------------------------------------------------------------------- the plain implementation, by hand
def test_plain_buckets_temperature_and_norm_by_hand():
    # eight rows up to 40: distances 0..3 one row each, then 4 * 10^(k/4) starts row 4 + k
    got = [plain.distance_bucket(n, 8, 40) for n in range(45)]
    edges = [math.ceil(4 * 10 ** (k / 4) - 1e-9) for k in range(1, 4)]            # 8, 13, 23
    assert edges == [8, 13, 23]
    want = [n if n < 4 else 4 + sum(n >= e for e in edges) for n in range(45)]
    assert got == want and got[7] == 4 and got[8] == 5 and got[22] == 6 and got[23] == 7 and got[44] == 7
    assert plain.distance_bucket(3, 4, 3) == 3 and plain.distance_bucket(2, 4, 3) == 2 + int(math.log(1) // 1)
    t = plain.query_temperature(torch.arange(12, dtype=torch.float64), 0.5, 5)
    assert torch.allclose(t[:4], torch.ones(4, dtype=torch.float64)) and abs(float(t[4]) - (1 + 0.5 * math.log(2))) < 1e-12
    assert abs(float(t[8]) - (1 + 0.5 * math.log(2))) < 1e-12 and abs(float(t[9]) - (1 + 0.5 * math.log(3))) < 1e-12
    x = torch.tensor([[1.0, 3.0]], dtype=torch.float64)
    y = plain.layer_norm(x, torch.tensor([2.0, 0.5]).double(), torch.tensor([0.1, -0.1]).double(), 0.0)
    assert torch.allclose(y, torch.tensor([[-2.0 + 0.1, 0.5 - 0.1]]).double())
    y = plain.layer_norm(x, torch.ones(2).double(), torch.zeros(2).double(), 3.0)             # var 1, eps 3: a half
    assert torch.allclose(y, torch.tensor([[-0.5, 0.5]]).double())


def test_plain_rotation_window_and_recurrence_by_hand():
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0]]], dtype=torch.float64)              # [n = 1, heads = 1, 5]; four numbers turn
    out = plain.rotate_half(x, torch.tensor([2]), 4.0, 4)
    a0, a1 = 2.0, 2.0 * 4.0 ** -0.5
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0]
    assert torch.allclose(out[0, 0], torch.tensor(want, dtype=torch.float64))
    assert plain.window_mask(4, 2).tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [0, 1, 1, 0], [0, 0, 1, 1]]
    assert plain.window_mask(3, 1).tolist() == torch.eye(3).bool().tolist()
    assert plain.window_mask(3, None).tolist() == torch.ones(3, 3).tril().bool().tolist()
    # one head, two key channels, one value channel
    q = torch.tensor([[[1.0, 1.0]], [[1.0, 0.0]], [[0.0, 2.0]]], dtype=torch.float64)
    k = torch.tensor([[[1.0, 2.0]], [[3.0, 0.0]], [[0.0, 1.0]]], dtype=torch.float64)
    v = torch.tensor([[[10.0]], [[1.0]], [[100.0]]], dtype=torch.float64)
    alpha = torch.tensor([[[0.5, 0.5]], [[0.5, 0.1]], [[1.0, 0.5]]], dtype=torch.float64)
    o, S = plain.gla_scan(q, k, v, alpha)
    # S1 = [10, 20]; S2 = [5 + 3, 2]; S3 = [8, 1 + 100]
    assert o[:, 0, 0].tolist() == [30.0, 8.0, 202.0] and S[0, :, 0].tolist() == [8.0, 101.0]
    o2, _ = plain.gla_scan(q[2:], k[2:], v[2:], alpha[2:], state=plain.gla_scan(q[:2], k[:2], v[:2], alpha[:2])[1])
    assert o2[0, 0, 0].item() == 202.0
    W = {"m.a1": torch.tensor([[1.0, 0.0]]).double(), "m.a2": torch.tensor([[2.0], [0.0]]).double(), "m.a2.b": torch.tensor([0.0, 1.0]).double()}
    d = plain.gla_decay(torch.tensor([[3.0, 9.0]]).double(), W, "m", 2.0)
    assert torch.allclose(d, torch.tensor([[math.sqrt(1 / (1 + math.exp(-6.0))), math.sqrt(1 / (1 + math.exp(-1.0)))]]).double())


def test_plain_attention_and_router_by_hand():
    # one head, head size 1, three positions; a table of two rows: distance 0, and everything further back
    q = torch.tensor([[[1.0]], [[1.0]], [[2.0]]], dtype=torch.float64)
    k = torch.tensor([[[1.0]], [[2.0]], [[0.5]]], dtype=torch.float64)
    v = torch.tensor([[[1.0]], [[10.0]], [[100.0]]], dtype=torch.float64)
    table = torch.tensor([[0.5], [-1.0]], dtype=torch.float64)
    out = plain.biased_attention(q, k, v, 0.5, table, 1.5)
    e = math.exp
    w1 = [e(0.5 - 1.0), e(1.0 + 0.5)]
    w2 = [e(1.0 - 1.0), e(2.0 - 1.0), e(0.5 + 0.5)]
    assert abs(out[0, 0, 0].item() - 1.0) < 1e-12
    assert abs(out[1, 0, 0].item() - (w1[0] * 1 + w1[1] * 10) / sum(w1)) < 1e-12
    assert abs(out[2, 0, 0].item() - (w2[0] * 1 + w2[1] * 10 + w2[2] * 100) / sum(w2)) < 1e-12
    # router: softmax over all three, the two largest, their scores over their sum; the shared expert is added
    W = {"m.router": torch.eye(3).double()}
    for e_ in range(3):
        W[f"m.e{e_}.gate"] = torch.tensor([[1.0, 0.0, 0.0]]).double()
        W[f"m.e{e_}.up"] = torch.tensor([[0.0, float(e_ + 1), 0.0]]).double()
        W[f"m.e{e_}.down"] = torch.ones(3, 1).double()
    W["m.shared.gate"], W["m.shared.up"], W["m.shared.down"] = (torch.tensor([[0.0, 0.0, 1.0]]).double(),
                                                                torch.tensor([[1.0, 0.0, 0.0]]).double(), torch.full((3, 1), 2.0).double())
    h = torch.tensor([[1.0, 2.0, 0.5]], dtype=torch.float64)
    s = torch.softmax(h[0], 0)
    sil = lambda z: z / (1 + math.exp(-z))                                           # noqa: E731
    y = (s[1] * sil(1.0) * 2 * 2.0 + s[0] * sil(1.0) * 1 * 2.0) / (s[0] + s[1])
    out = plain.moe_ff(h, W, "m", dict(router=dict(experts=3, top=2), expert=dict(ff=1), shared=dict(ff=1)))
    assert torch.allclose(out, torch.full((1, 3), float(y) + 2.0 * sil(0.5) * 1.0, dtype=torch.float64))
    chosen, weight = plain.route(h, W, "m", 2)
    assert chosen.tolist() == [[1, 0]] and abs(float(weight.sum()) - 1.0) < 1e-12


def test_router_margins_of_the_test_models():
    """The comparisons are only fair if no token of the test prompts sits on a routing boundary."""
    for name in CONFIGS:
        raw, _, weights = make(name)
        margins = []
        for toks in trace_util.random_prompts(raw["vocab"], LENGTHS, seed=17).values():
            plain.forward(raw, weights, toks, margins=margins)
        assert margins and min(margins) > 1e-5, f"{name}: a token is routed with a margin of {min(margins):.1e}"


# ------------------------------------------------------------------------------------- mechanisms, one by one
def one_layer(kind, mixer, mlp, width=32, vocab=50, eps=1e-5, **kw):
    return model(vocab, width, eps, [layer(kind, mixer, mlp)], **kw)


MECHANISMS = {
    "attention": one_layer("attention", att(4, 2, 8, vdim=12, every=4, buckets=6, bias_max=9), None),
    "attention-one-head-no-temperature": one_layer("attention", att(1, 1, 24, vdim=40, coef=0.0, buckets=2, bias_max=1.5), None),
    "attention-table-longer-than-the-prompt": one_layer("attention", att(2, 1, 16, scale=0.2, buckets=64, bias_max=500), None),
    "latent": one_layer("latent_attention", lat(2, 8, 4, 12, 10, 6, window=6), None),
    "latent-window-of-one": one_layer("latent_attention", lat(2, 8, 8, 8, 16, 16, window=1), None),
    "latent-no-window-part-turned": one_layer("latent_attention", lat(3, 4, 12, 6, 7, 9, dims=4), None),
    "gla": one_layer("gla", gla(2, 8, vdim=12, tau=2.0, rank=3), None),
    "gla-one-head-rank-one": one_layer("gla", gla(1, 20, vdim=4, tau=30.0, rank=1), None),
    "experts-shared": one_layer("gla", gla(1, 8), moe(4, 2, 12, shared=20)),
    "experts-top1-no-shared": one_layer("gla", gla(1, 8), moe(3, 1, 12)),
    "experts-all-chosen": one_layer("gla", gla(1, 8), moe(2, 2, 20, shared=4)),
    "head-scaled-and-capped": one_layer("gla", gla(1, 8), None, emb=2.5, logit_scale=3.0, cap=4.0),
}


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_each_mechanism_alone_on_the_host(name):
    raw = MECHANISMS[name]
    cfg = LabiraxConfig.from_dict(raw)
    weights = shape_weights(cfg, 1)
    runner = host_runner(cfg, weights, pages=8, rows=2, tokens=64)
    toks = trace_util.random_prompts(raw["vocab"], [29], seed=2)["r0"]
    want = plain.forward(raw, weights, toks)
    rc = runner.cache.open("a")
    pos, rows = 0, []
    for n in (11, 1, 2, 15):                                  # a portion, a single token, two tokens, the rest
        assert runner.cache.reserve(rc, pos, n)
        row = StepRow(rc, toks[pos:pos + n], pos, list(range(n)))
        rows.append(runner.forward_step([row]))
        runner.after_step([row])
        pos += n
    got = torch.cat(rows).double()
    assert float((got - want).abs().max()) < 2e-5 * float(want.abs().max())


def test_prefill_equals_token_by_token_decoding():
    raw, cfg, weights = make("A")
    prompts = trace_util.random_prompts(raw["vocab"], [60], seed=21)
    whole = trace_util.run_on_runner(host_runner(cfg, weights), trace_util.whole(prompts))
    single = trace_util.run_on_runner(host_runner(cfg, weights), trace_util.decode_tail(prompts, 59))
    pairs = trace_util.run_on_runner(host_runner(cfg, weights), trace_util.portions(prompts, sizes=(2,)))
    scale = max(float(v.abs().max()) for v in whole.values())
    for key, row in whole.items():
        assert float((single[key] - row).abs().max()) < 1e-5 * scale, f"token by token differs at {key}"
        assert float((pairs[key] - row).abs().max()) < 1e-5 * scale, f"two by two differs at {key}"
    trace_util.compare(whole, expected_logits(raw, weights, prompts), F32_TOL, "whole")


# ------------------------------------------------------------------------------------------ whole models, host
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_on_the_host(name, family, tmp_path):
    run_family(name, family, tmp_path, "cpu", "float32", F32_TOL)


def window_model():
    """One latent-attention layer with a window of 20 keys (a page and a quarter) and no feed-forward: the logits of a
    position are a function of its own token and the 19 before it."""
    raw = one_layer("latent_attention", lat(3, 16, 8, 8, 24, 16, window=20, scale=0.5), None, width=48, vocab=90)
    cfg = LabiraxConfig.from_dict(raw)
    w = shape_weights(cfg, 5)
    w["embed"][89] = 4.0 * w["embed"][89].sign()              # the token that stands out
    return raw, cfg, w


def make_runner(device, cfg, w, pages, rows, tokens, dtype="float32"):
    if device == "cpu":
        return host_runner(cfg, w, pages=pages, rows=rows, tokens=tokens)
    return ModelRunner(cfg, weights=w, dtype=dtype, num_pages=pages, max_rows=rows, max_step_tokens=tokens,
                       max_model_len=(pages - 1) * 16)


def window_runs(device):
    """A token that stands out is put just inside and just outside the window of the positions asked for (and on a
    page's last and next first slot, and at the very first position), in a prompt's portion and for tokens decoded one by
    one.  Inside, it must move the logits; outside, the engine's logits must not move at all; both ways they follow the
    plain implementation."""
    raw, cfg, w = window_model()
    base = [t if t != 89 else 0 for t in trace_util.random_prompts(90, [75], seed=9)["r0"]]

    def run(tokens, cut):
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:cut], "want": list(range(cut))}], "end": []}]
        steps += [{"step": 1 + i, "entries": [{"id": "x", "tokens": tokens[cut + i:cut + i + 1], "want": [0]}], "end": []}
                  for i in range(len(tokens) - cut)]
        steps[-1]["end"] = ["x"]
        return {k: v.cpu() for k, v in trace_util.run_on_runner(make_runner(device, cfg, w, 8, 2, 80), steps).items()}

    for cut in (70, 42, 58):                 # asked-for positions in the portion; decoded; the window's edge among decoded tokens
        plain_run = run(base, cut)
        for needle in (40, 41, 47, 48, 0, 15, 16):
            tokens = list(base)
            tokens[needle] = 89
            want = plain.forward(raw, w, tokens)
            got = run(tokens, cut)
            trace_util.compare(got, {"x": want}, F32_TOL, f"needle at {needle}, portion of {cut}")
            for p in range(75):
                moved = float((got[("x", p)] - plain_run[("x", p)]).abs().max()) / float(want.abs().max())
                if needle <= p <= needle + 19:
                    assert moved > 2e-6, f"position {p} must see the token at {needle} (portion of {cut})"
                else:
                    assert moved < 2e-7, f"position {p} must not see the token at {needle} (portion of {cut}): moved {moved:.1e}"


def test_keys_just_inside_and_outside_a_window_on_the_host():
    window_runs("cpu")


def far_key_runs(device):
    """One key far back (hundreds of positions, through a dozen pages) is made to decide the biased attention's output.
    Its product with the last query is large because query and key matrices are made alike and the last token is the
    far key's own; the table's first row takes the last position's own key out of the way.  The key stands at a page's last slot, at the next page's
    first, and at the very first position."""
    raw = one_layer("attention", att(2, 1, 16, scale=0.25, coef=0.3, every=64, buckets=8, bias_max=24), None, width=32, vocab=64)
    cfg = LabiraxConfig.from_dict(raw)
    w = shape_weights(cfg, 7)
    w["l0.mix.q"].copy_(w["l0.mix.k"].repeat(2, 1) * 3.0)    # a token's queries are three times its key
    w["l0.mix.q.b"].zero_()
    w["l0.mix.k.b"].zero_()
    w["l0.mix.rel"].mul_(0.25)
    w["l0.mix.rel"][0] = -20.0                               # a position's own key (as large a product, the same value) counts for nothing
    toks = [t if t != 63 else 0 for t in trace_util.random_prompts(64, [230], seed=9)["r0"]]
    for needle in (31, 32, 0):
        tokens = list(toks)
        tokens[needle] = 63
        tokens[-1] = 63                                       # the last query is the far key's own token
        want = plain.forward(raw, w, tokens)
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:190], "want": [189]}], "end": []}]
        steps += [{"step": 1 + i, "entries": [{"id": "x", "tokens": tokens[190 + i:191 + i], "want": [0]}], "end": []}
                  for i in range(40)]
        steps[-1]["end"] = ["x"]
        got = {k: v.cpu() for k, v in trace_util.run_on_runner(make_runner(device, cfg, w, 16, 2, 192), steps).items()}
        trace_util.compare(got, {"x": want}, F32_TOL, f"far key at {needle}")
        other = list(tokens)
        other[needle] = toks[needle]
        moved = float((plain.forward(raw, w, other)[-1] - want[-1]).abs().max()) / float(want.abs().max())
        assert moved > 1e-2, "the far key must matter to the last position for this test to mean anything"


def test_a_far_key_and_the_first_token_are_seen():
    far_key_runs("cpu")


def bucket_edge_runs(device):
    """Keys and queries are made to count for nothing (their matrices are zero), so a position's output is decided by the
    distance table alone: one row of the table gets a large bonus, and the positions that fall into it, just inside and
    just outside its two edges, must be the ones that are attended to, in a prompt's portions and decoded one by one."""
    raw = one_layer("attention", att(2, 2, 8, buckets=8, bias_max=40, coef=0.0), None, width=32, vocab=64)
    cfg = LabiraxConfig.from_dict(raw)
    toks = trace_util.random_prompts(64, [60], seed=3)["r0"]
    for row in (2, 4, 5, 6, 7):                               # a single distance; 4..7; 8..12; 13..22; 23 and beyond
        w = shape_weights(cfg, 11)
        for k in ("l0.mix.q", "l0.mix.k", "l0.mix.q.b", "l0.mix.k.b"):
            w[k].zero_()
        w["l0.mix.rel"].zero_()
        w["l0.mix.rel"][row] = 9.0
        want = plain.forward(raw, w, toks)
        for steps in (trace_util.whole({"x": toks}), trace_util.decode_tail({"x": toks}, 45), trace_util.portions({"x": toks}, sizes=(5, 2, 16, 3))):
            got = {k: v.cpu() for k, v in trace_util.run_on_runner(make_runner(device, cfg, w, 8, 2, 64), steps).items()}
            trace_util.compare(got, {"x": want}, F32_TOL, f"bonus on table row {row}")


def test_distance_buckets_at_their_edges_on_the_host():
    bucket_edge_runs("cpu")


def test_state_slots_and_pages_are_used_again():
    """Five requests, one after another, through a runner with one usable state slot and pages for one request: each must
    start from an empty state and see no key of the one before."""
    raw, cfg, weights = make("B")
    prompts = trace_util.random_prompts(raw["vocab"], [40, 33, 40, 7, 25], seed=3)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                         num_pages=4, max_rows=1, max_step_tokens=64, max_model_len=48, num_state_slots=2)
    got = trace_util.run_on_runner(runner, trace_util.portions(prompts, sizes=(5, 2, 9)))
    trace_util.compare(got, expected_logits(raw, weights, prompts), F32_TOL, "reuse")
    states = [e.tensors["state"] for e in runner.storage.entries.values() if "state" in (e.tensors or {})]
    assert len(states) == 2
    for t in states:
        t.fill_(-2.0)
    rc = runner.cache.open("fresh")
    assert all(float(t[rc.state_slot].abs().max()) == 0.0 for t in states)
    runner.cache.close(rc)


def test_pages_before_the_window_are_given_back():
    """A request that decodes far beyond its window keeps the pages its window touches only."""
    raw = one_layer("latent_attention", lat(2, 8, 4, 8, 12, 8, window=32), None)
    cfg = LabiraxConfig.from_dict(raw)
    w = shape_weights(cfg, 2)
    prompts = trace_util.random_prompts(50, [150], seed=1)
    runner = ModelRunner(cfg, weights=w, dtype="float32", device="cpu", backend=TorchBackend(torch.float32), num_pages=6,
                         max_rows=1, max_step_tokens=64, max_model_len=160)          # five usable pages of 16 for 150 tokens
    got = trace_util.run_on_runner(runner, trace_util.portions(prompts, sizes=(20, 3, 1, 30)))
    trace_util.compare(got, expected_logits(raw, w, prompts), F32_TOL, "pages given back")


def test_long_decoding_carries_the_state():
    """Two hundred tokens one by one through a slow decay: what the first tokens wrote is still in the state at the end."""
    raw = one_layer("gla", gla(2, 8, vdim=12, tau=200.0, rank=2), None)
    cfg = LabiraxConfig.from_dict(raw)
    w = shape_weights(cfg, 4)
    prompts = trace_util.random_prompts(50, [200], seed=6)
    got = trace_util.run_on_runner(host_runner(cfg, w, pages=16, rows=1, tokens=64), trace_util.decode_tail(prompts, 199))
    want = expected_logits(raw, w, prompts)
    trace_util.compare(got, want, F32_TOL, "long decoding")
    other = dict(r0=[(prompts["r0"][0] + 1) % 50] + prompts["r0"][1:])
    moved = float((expected_logits(raw, w, other)["r0"][-1] - want["r0"][-1]).abs().max()) / float(want["r0"].abs().max())
    assert moved > 1e-4, "the first token must still matter at the end for this test to mean anything"


def test_batched_rows_equal_rows_alone():
    raw, cfg, weights = make("A")
    prompts = trace_util.random_prompts(raw["vocab"], [21, 5, 34, 1, 50], seed=12)
    alone = {}
    for rid, toks in prompts.items():
        alone.update(trace_util.run_on_runner(host_runner(cfg, weights), trace_util.decode_tail({rid: toks}, 1)))
    runner = host_runner(cfg, weights)
    ents = [{"id": rid, "tokens": toks[:-1], "want": list(range(len(toks) - 1))} for rid, toks in prompts.items() if len(toks) > 1]
    last = [{"id": rid, "tokens": toks[-1:], "want": [0]} for rid, toks in prompts.items()]
    got = trace_util.run_on_runner(runner, [{"step": 0, "entries": ents, "end": []}, {"step": 1, "entries": last, "end": list(prompts)}])
    assert set(got) == set(alone)
    for key, row in alone.items():
        assert float((got[key] - row).abs().max()) < 1e-5 * float(row.abs().max())


def generate(name, device, dtype, **engine):
    from mini_inference_engine_amd import LLMEngine, SamplingParams
    raw, cfg, weights = make(name, torch.float32 if dtype == "float32" else torch.bfloat16, sharp=dtype == "float32")
    prompts = list(trace_util.random_prompts(raw["vocab"], [9, 30, 2, 17, 23], seed=4).values())
    ecfg = EngineConfig(num_blocks=24, max_num_seqs=3, max_num_batched_tokens=32, max_model_len=128, **engine)
    kw = dict(device="cpu", backend=TorchBackend(torch.float32)) if device == "cpu" else {}
    eng = LLMEngine(cfg, ecfg, dtype=dtype, verbose=False, weights=weights, **kw)
    outs = eng.generate(prompts, SamplingParams(max_tokens=30, ignore_eos=True))          # through a window's edge
    wf = {k: v.float() for k, v in weights.items()}
    missed = 0
    for prompt, out in zip(prompts, outs):
        ids = list(prompt) + list(out.output_ids)
        assert len(out.output_ids) == 30
        logits = plain.forward(raw, wf, ids)
        for i, tok in enumerate(out.output_ids):
            row = logits[len(prompt) + i - 1]
            slack = (F32_TOL if dtype == "float32" else BF16_TOL_PER_LAYER * len(raw["layers"])) * float(row.abs().max())
            missed += float(row.max() - row[tok]) > slack
    # bfloat16: a token routed on a near-tie may differ (see compare_most); float32: every token is the plain choice
    assert missed <= (0 if dtype == "float32" else 6), f"{missed} of 150 tokens are not the plain implementation's choice"
    return eng


def test_greedy_generation_through_the_scheduler_on_the_host():
    eng = generate("A", "cpu", "float32", use_hip_graphs=False)
    assert eng.num_steps > 30, "five requests under three slots and a budget of 32 tokens come in several waves"


# ----------------------------------------------------------------------------------------------- GPU: kernels
def _rand(shape, dtype, g, scale=1.0):
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.fixture(scope="module")
def hip():
    from mini_inference_engine_amd.kernels.hip_backend import HipBackend
    return {torch.float32: HipBackend(torch.float32), torch.bfloat16: HipBackend(torch.bfloat16)}


def close(a, b, tol, what):
    err = float((a.double().cpu() - b.double().cpu()).abs().max()) / max(1e-9, float(b.double().abs().max()))
    assert err <= tol, f"{what}: {err:.3e} of the scale, tolerance {tol:.1e}"


TOL = {torch.float32: 2e-6, torch.bfloat16: 1e-2}


def step_of(rows, slots=None):
    """What the recurrence kernels read of a step: rows of (tokens) with a state slot each."""
    import numpy as np
    from types import SimpleNamespace
    rs = np.concatenate([[0], np.cumsum(rows)]).astype("int64")
    slots = np.asarray(slots if slots is not None else list(range(1, len(rows) + 1)), dtype="int64")
    token_row = torch.cat([torch.full((n,), r, dtype=torch.int32) for r, n in enumerate(rows)])
    return SimpleNamespace(num_rows=len(rows), num_tokens=int(rs[-1]), max_row_tokens=int(max(rows)),
                           row_start=torch.tensor(rs, dtype=torch.int32).cuda(), state_slots=torch.tensor(slots, dtype=torch.int32).cuda(),
                           token_row=token_row.cuda(), host={"row_start": rs, "state_slots": slots})


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_norm_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(21)
    for (T, W) in ((1, 64), (37, 70), (5, 320), (130, 2048), (3, 4096), (2, 5000)):
        stream = _rand((T, W), torch.float32, g, 3.0) + 1.5
        x = _rand((T, W), dtype, g)
        w, b = _rand((W,), torch.float32, g) + 1, _rand((W,), torch.float32, g)
        s1, s2 = stream.clone(), stream.clone()
        close(ops.add_layernorm(x, s1, w, b, 1e-5), ref.ref_add_layernorm(x, s2, w, b, 1e-5, dtype), TOL[dtype], f"add_layernorm {T}x{W}")
        close(s1, s2, 1e-6, "the stream after the add")
        rows = torch.tensor([T - 1, 0], dtype=torch.int32).cuda()
        close(ops.add_layernorm(x, s1, w, b, 1e-5, out_dtype=torch.float32, rows=rows),
              ref.ref_add_layernorm(x, s2, w, b, 1e-5, torch.float32, rows), 2e-6, "gathered rows")
        assert torch.equal(s1, s2.to(s1.dtype)) or float((s1 - s2).abs().max()) < 1e-5, "gathered rows leave the stream"
        y = _rand((T, W), torch.float32, g, 5.0) - 2.0
        w2, b2 = _rand((W,), torch.float32, g) + 1, _rand((W,), torch.float32, g)
        got = ops.branch_layernorm_add(y, s1, w, b, 1e-5, next_norm=(w2, b2, 1e-3))
        want = ref.ref_branch_layernorm_add(y, s2, w, b, 1e-5, (w2, b2, 1e-3), dtype)
        close(s1, s2, 2e-6, "the stream after the branch")
        close(got, want, TOL[dtype], f"branch_layernorm_add {T}x{W}")
        assert ops.branch_layernorm_add(y, s1, w, b, 1e-5) is None
        ref.ref_branch_layernorm_add(y, s2, w, b, 1e-5, None, dtype)
        close(s1, s2, 2e-6, "the stream after the branch alone")
    t = _rand((7, 333), torch.float32, g, 20.0)
    close(ops.scale_softcap_(t.clone(), 0.7, 5.0), ref.ref_scale_softcap(t, 0.7, 5.0), 2e-6, "scale and cap")
    close(ops.scale_softcap_(t.clone(), 0.7, None), ref.ref_scale_softcap(t, 0.7, None), 2e-6, "scale alone")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gla_kernel(hip, dtype):
    """Whole rows and (bfloat16 mode) rows in chunks, states that are not square, heads of sizes that are no multiple of
    16, slots that hold something, decays from fast to slow."""
    ops, g = hip[dtype], torch.Generator().manual_seed(22)
    for (rows, H, d, dv, rank, tau) in (([1, 1, 1], 2, 16, 32, 4, 4.0), ([37, 1, 5], 3, 24, 8, 2, 1.0), ([200], 1, 10, 14, 3, 9.0),
                                        ([130, 70, 1, 64, 65], 4, 48, 64, 16, 16.0), ([300, 2], 2, 64, 128, 8, 16.0),
                                        ([9], 1, 128, 64, 5, 2.0), ([3, 90], 1, 200, 40, 2, 50.0)):
        T = sum(rows)
        nk, nv = H * d, H * dv
        cols = dict(q=3, k=3 + nk, v=3 + 2 * nk, g=3 + 2 * nk + nv, a=3 + 2 * nk + 2 * nv)
        sums = _rand((T, cols["a"] + rank + 2), torch.float32, g)
        w2, b2 = _rand((nk, rank), torch.float32, g), _rand((nk,), torch.float32, g, 2.0) + 2.0
        nw = _rand((dv,), torch.float32, g) + 1
        state = _rand((len(rows) + 2, H, d, dv), torch.float32, g, 0.5)
        step = step_of(rows)
        s1, s2 = state.clone(), state.clone()
        got = ops.gla(sums, cols, H, d, dv, w2, b2, tau, d ** -0.5, nw, 1e-5, s1, step)
        want = ref.ref_gla(sums, cols, H, d, dv, w2, b2, tau, d ** -0.5, nw, 1e-5, s2, step.host["row_start"], step.host["state_slots"], dtype)
        close(got, want, 2e-5 if dtype == torch.float32 else 1e-2, f"gla rows {rows}, {H} heads of {d} x {dv}")
        close(s1, s2, 2e-5, f"gla state, rows {rows}")
        assert torch.equal(s1[0], state[0]) and torch.equal(s1[-1], state[-1]), "slots of no row are left alone"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_biased_attention_kernels(hip, dtype):
    """Decode rows and portions over random pages against the torch operation: tables shorter and longer than the
    contexts, grouped heads, padded and wide heads; the matrix-core kernels in bfloat16, the 32-bit kernel in float32."""
    from test_mutusun import AttentionCase
    ops, g = hip[dtype], torch.Generator().manual_seed(23)
    rows = [(0, 1), (23, 1), (24, 1), (47, 1), (200, 1), (0, 50), (17, 31), (63, 2), (100, 130), (0, 300)]
    for (Hq, Hkv, P, N, window) in ((6, 2, 16, 9, None), (3, 3, 32, 1, None), (4, 1, 16, 40, None), (2, 2, 48, 400, None),
                                    (8, 2, 64, 140, None), (4, 4, 128, 65, None), (16, 4, 64, 24, 50), (8, 4, 64, 200, None)):
        case = AttentionCase(rows, Hkv, P, dtype, g)
        q = _rand((case.num_tokens, Hq * P), dtype, g)
        table = _rand((Hq, N), torch.float32, g, 1.5)
        want = ref.ref_paged_attention(q, Hq, Hkv, P, case.k, case.v, case.block_tables, case.token_row, case.positions,
                                       P ** -0.5, window, torch.float32, distance_bias=table)
        got = ops.paged_attention(q, Hq, Hkv, P, case.k, case.v, case.group, case.step, P ** -0.5, window, distance_bias=table)
        close(got, want, 1e-5 if dtype == torch.float32 else 1.5e-2, f"heads {Hq}/{Hkv} of {P}, a table of {N}")
        if dtype == torch.bfloat16:
            slow = ops.paged_attention(q, Hq, Hkv, P, case.k, case.v, case.group, case.step, P ** -0.5, window, distance_bias=table,
                                       force_generic=True)
            close(slow, want, 1.5e-2, f"32-bit kernel on bfloat16, heads {Hq}/{Hkv} of {P}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_table_row_stands_out(hip, dtype):
    """Queries and keys are zero, so the weights are the table's alone: one distance gets a large bonus, and the output
    of a position is the value that many positions back (or, before there is such a key, a mean of what it sees)."""
    from test_mutusun import AttentionCase
    ops, g = hip[dtype], torch.Generator().manual_seed(24)
    Hq, Hkv, P, page = 4, 2, 32, 16
    for N, hot in ((70, 64), (70, 69), (20, 16), (20, 0), (130, 65)):
        rows = [(hot, 1), (hot + 1, 1), (150, 1), (0, 140), (hot, 2), (max(0, hot - 3), 70)]
        case = AttentionCase(rows, Hkv, P, dtype, g, page)
        q = torch.zeros(case.num_tokens, Hq * P, dtype=dtype).cuda()
        table = torch.zeros(Hq, N).cuda()
        table[:, hot] = 40.0
        got = ops.paged_attention(q, Hq, Hkv, P, case.k, case.v, case.group, case.step, 1.0, None, distance_bias=table).float().cpu()
        pos, row = case.positions.cpu().tolist(), case.token_row.cpu().tolist()
        for t in range(case.num_tokens):
            n = pos[t] - hot
            if n < 0 or (hot == N - 1 and n > 0):         # no key at that distance yet; or the last entry, which many keys share
                continue
            pg = int(case.block_tables[row[t], n // page])
            want = case.v[pg, :, :, n % page].float().cpu().repeat_interleave(Hq // Hkv, 0).reshape(-1)
            assert float((got[t] - want).abs().max()) < 2e-2, f"table of {N}, bonus at {hot}: position {pos[t]} of a row of {case.rows[row[t]]}"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_biased_projection_temperature_and_latent_layout_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(25)
    for (T, Hq, Hkv, dim, vdim, every) in ((1, 6, 2, 16, 24, 7), (37, 3, 3, 24, 8, 1), (130, 4, 1, 10, 14, 3), (64, 16, 4, 64, 64, 64)):
        P = -(-max(dim, vdim) // 16) * 16
        sums = _rand((T, 3 + Hq * dim + Hkv * dim + Hkv * vdim + 5), torch.float32, g, 2.0)
        bias = _rand((sums.shape[1],), torch.float32, g)
        positions = (torch.arange(T, dtype=torch.int32) * 3 + 5).cuda()
        pages, page = T // 16 + 3, 16
        slots = torch.randperm((pages - 1) * page, generator=g)[:T].to(torch.int32).cuda() + page
        kc, vc = torch.full((pages, Hkv, page, P), 7.0, dtype=dtype).cuda(), torch.full((pages, Hkv, P, page), 7.0, dtype=dtype).cuda()
        kw, vw = kc.clone(), vc.clone()
        cols = (3, 3 + Hq * dim, 3 + Hq * dim + Hkv * dim)
        want = ref.ref_qkv_finish(sums, *cols, Hq, Hkv, dim, vdim, P, positions, None, "half", kw, vw, slots, None, None, 0.0, None,
                                  dtype, col_bias=bias, position_temperature=(0.3, every))
        got = ops.qkv_finish(sums, *cols, Hq, Hkv, dim, vdim, P, positions, None, "half", kc, vc, slots, col_bias=bias,
                             position_temperature=(0.3, every))
        close(got, want, TOL[dtype], "queries")
        close(kc, kw, TOL[dtype], "keys")
        close(vc, vw, TOL[dtype], "values")
    for (T, H, r, dr, nf) in ((1, 3, 40, 8, 4), (70, 2, 20, 12, 4), (33, 5, 12, 2, 1), (9, 6, 128, 16, 8)):
        P = -(-(r + dr) // 16) * 16
        sums = _rand((T, 7 + r + dr), torch.float32, g, 2.0)
        nw = _rand((r,), torch.float32, g) + 1
        inv_freq = (50.0 ** -(torch.arange(nf, dtype=torch.float32) / nf)).cuda()
        positions = (torch.arange(T, dtype=torch.int32) * 2 + 1).cuda()
        pages, page = T // 16 + 3, 16
        slots = torch.randperm((pages - 1) * page, generator=g)[:T].to(torch.int32).cuda() + page
        kc, vc = torch.zeros((pages, 1, page, P), dtype=dtype).cuda(), torch.zeros((pages, 1, P, page), dtype=dtype).cuda()
        kw, vw = kc.clone(), vc.clone()
        ops.latent_kv_store(sums, 7, r, dr, nw, 1e-5, positions, inv_freq, kc, vc, slots, layout="half")
        ref.ref_latent_kv_store(sums, 7, r, dr, nw, 1e-5, positions, inv_freq, kw, vw, slots, layout="half")
        close(kc, kw, TOL[dtype], "latent keys, halves turned")
        close(vc, vw, TOL[dtype], "latent values")
        q = _rand((T, H * P), dtype, g)
        want = ref.ref_latent_query_rotate(q.clone(), H, r, P, positions, inv_freq, layout="half")
        close(ops.latent_query_rotate_(q, H, r, P, positions, inv_freq, layout="half"), want, TOL[dtype], "latent queries, halves turned")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_renormalised_routing_and_plain_gated_expert_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(26)
    silu = (float("inf"), 1.0, 0.0)
    for (T, W, E, top, ff) in ((1, 64, 5, 2, 48), (37, 48, 4, 4, 24), (300, 72, 3, 1, 40), (130, 128, 16, 4, 96), (700, 64, 200, 3, 32)):
        logits = _rand((T, E), torch.float32, g, 2.0)
        idx, shares = ops.route_topk(logits, None, top, over="all", renormalise=True)
        widx, wshares = ref.ref_route_topk(logits, None, top, over="all", renormalise=True)
        assert torch.equal(idx.cpu(), widx.cpu())
        close(shares, wshares, 2e-6, "shares")
        assert float((shares.sum(-1) - 1.0).abs().max()) < 1e-5, "a token's shares sum to one"
        x = _rand((T, W), dtype, g)
        w_up, w_down = _rand((E, 2 * ff, W), dtype, g, 2 * W ** -0.5), _rand((E, W, ff), dtype, g, ff ** -0.5)
        got = ops.routed_experts(x, idx, shares, w_up, w_down, "silu", gated=silu)
        want = ref.ref_routed_experts(x, idx, shares, w_up, w_down, "silu", dtype, gated=silu)
        close(got, want, 1e-5 if dtype == torch.float32 else 1e-2, f"experts {T} tokens, {E} experts")
        if ff % 16 == 0 and dtype == torch.bfloat16:
            mixed = w_up.view(E, 2, ff // 16, 16, W).transpose(1, 2).contiguous().view(E, 2 * ff, W)
            got = ops.routed_experts(x, idx, shares, mixed, w_down, "silu", gated=silu, glu_block=16)
            close(got, want, 1e-2, f"experts in blocks of 16, {T} tokens")


# ------------------------------------------------------------------------------------------- GPU: whole models
@pytest.mark.gpu
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_float32(name, family, tmp_path):
    run_family(name, family, tmp_path, "cuda", "float32", F32_TOL)


@pytest.mark.gpu
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_bfloat16(name, family, tmp_path):
    raw, _ = CONFIGS[name]
    run_family(name, family, tmp_path, "cuda", "bfloat16", BF16_TOL_PER_LAYER * len(raw["layers"]))


@pytest.mark.gpu
def test_keys_just_inside_and_outside_a_window():
    window_runs("cuda")


@pytest.mark.gpu
def test_a_far_key_and_the_first_token_are_seen_by_the_kernels():
    far_key_runs("cuda")


@pytest.mark.gpu
def test_distance_buckets_at_their_edges():
    bucket_edge_runs("cuda")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_in_chunks_of_the_recurrence(dtype):
    """Prompts of several hundred tokens, whole and in uneven portions: the recurrence runs in chunks side by side in
    bfloat16 and whole in float32; the distance table ends long before the prompt does."""
    raw, cfg, weights = make("D", torch.float32 if dtype == "float32" else torch.bfloat16, sharp=dtype == "float32")
    prompts = trace_util.random_prompts(raw["vocab"], [400, 129], seed=8)
    want = expected_logits(raw, weights, prompts)
    for steps in (trace_util.whole(prompts), trace_util.portions(prompts, sizes=(130, 2, 65, 64, 200))):
        runner = ModelRunner(cfg, weights=weights, dtype=dtype, num_pages=40, max_rows=2, max_step_tokens=512, max_model_len=39 * 16)
        got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, steps).items()}
        if dtype == "float32":
            trace_util.compare(got, want, F32_TOL, "long prompts")
        else:
            compare_most(got, want, BF16_TOL_PER_LAYER * len(raw["layers"]), "long prompts")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(dtype):
    eng = generate("A", "cuda", dtype)
    assert eng.num_graph_steps > 0, "decode steps run as captured graphs"


# --------------------------------------------------------------------------------------------- the command line
def run_cli(*args):
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-m", "mini_inference_engine_amd", *args], cwd=root, capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0, f"{args}: exit {proc.returncode}\n{proc.stderr[-2000:]}"
    return proc


def test_random_model_of_the_named_size_is_what_the_loader_reads(tmp_path):
    from safetensors.torch import load_file
    folder = str(tmp_path / "m")
    run_cli("random-model", "--shape", "labirax-tiny", "--seed", "3", "--dtype", "float32", "--out", folder)
    cfg, arch = load_model_config(folder)
    assert arch.name == "Labirax" and [layer.weights_of for layer in cfg.layers] == [None, None, None, 0, 1]
    stored = load_file(folder + "/model.safetensors")
    assert tuple(stored["l0.mix.rel"].shape) == (32, 6) and tuple(stored["l1.mix.a1"].shape) == (16, 64) and "l3.mix.q" not in stored
    raw = json.loads(open(folder + "/config.json").read())
    runner = host_runner(cfg, stored, pages=8, rows=2, tokens=64)
    toks = trace_util.random_prompts(raw["vocab"], [40], seed=1)
    got = trace_util.run_on_runner(runner, trace_util.portions(toks, sizes=(9, 2, 20)))
    trace_util.compare(got, expected_logits(raw, stored, toks), F32_TOL, "the named size")


@pytest.mark.gpu
def test_generate_from_the_command_line(tmp_path):
    from safetensors.torch import load_file
    folder = str(tmp_path / "m")
    run_cli("random-model", "--shape", "labirax-tiny", "--seed", "3", "--dtype", "float32", "--out", folder)
    prompts = [[5, 17, 3, 200, 41], list(range(20, 54)), [7]]
    args = ["generate", "--model", folder, "--dtype", "float32", "--max-tokens", "6", "--ignore-eos", "--num-blocks", "24", "--quiet"]
    for p in prompts:
        args += ["--prompt-ids", ",".join(map(str, p))]
    lines = [json.loads(line) for line in run_cli(*args).stdout.splitlines() if line.startswith("{")]
    raw, stored = json.loads(open(folder + "/config.json").read()), load_file(folder + "/model.safetensors")
    assert [r["prompt_len"] for r in lines] == [len(p) for p in prompts]
    for prompt, rec in zip(prompts, lines):
        ids = list(prompt)
        assert len(rec["output_ids"]) == 6
        for tok in rec["output_ids"]:
            row = plain.forward(raw, stored, ids)[-1]
            assert float(row.max() - row[tok]) <= 1e-5 * float(row.abs().max()), f"token {tok} after {len(ids)} tokens"
            ids.append(tok)
