"""Mutusun through the engine against the plain implementation (tests/plain_mutusun.py).

Configurations are made here, with sizes that differ from one another wherever the design lets them (query and
key/value head counts, head size and value size, chunks that are no multiple of a page, a chunk of one position and
no chunk at all, with and without a score cap, taps from one to four and no convolution, dense, routed and absent
feed-forwards, experts with none, some and only identity outputs, top = 1 and top = every output, layers that run
with an earlier or a later layer's tensors).  Host tests run the engine's own parts, cache and step function on
the CPU with the torch operations of tests/torch_backend.py; GPU tests run the HIP kernels, each kernel against the
torch operation of the same name and the whole model in the four trace families, in float32 (tight) and bfloat16.
"""
import json
import math

import pytest
import torch

import plain_mutusun as plain
import trace_util
from torch_backend import TorchBackend
import torch_backend as ref

from mini_inference_engine_amd.config import EngineConfig, MutusunConfig, load_model_config
from mini_inference_engine_amd.engine.batch import StepRow
from mini_inference_engine_amd.engine.runner import ModelRunner
from mini_inference_engine_amd.replay.trace import replay
from mini_inference_engine_amd.weights import random_tensors


def att(heads, kv_heads, dim, vdim=None, scale=None, softcap=None, chunk=None):
    d = dict(heads=heads, kv_heads=kv_heads, dim=dim, scale=scale if scale is not None else dim ** -0.5)
    if vdim is not None:
        d["vdim"] = vdim
    if softcap is not None:
        d["softcap"] = softcap
    if chunk is not None:
        d["mask"] = dict(size=chunk)
    return d


def layer(mixer, mlp, weights_of=None):
    d = dict(type="attention", mixer=mixer, mlp=mlp)
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def moe(experts, identity, top, ff, limit):
    return dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, identity=identity, top=top))


def model(vocab, width, eps, taps, layers):
    d = dict(architecture="Mutusun", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)
    if taps is not None:
        d["canon"] = dict(taps=taps)
    return d


A1 = att(6, 2, 16, vdim=24, scale=0.3, softcap=5.0, chunk=24)          # a chunk of a page and a half
A2 = att(3, 3, 24, vdim=8, chunk=7)                                    # no cap; heads padded 24 -> 32; as many key heads
M1 = moe(5, 2, 3, 48, 1.5)
CFG_A = model(211, 64, 1e-5, 4, [layer(A1, dict(kind="dense", ff=112)),
                                 layer(A1, M1),
                                 layer(A1, M1, weights_of=1),
                                 layer(A2, None),
                                 layer(A1, M1, weights_of=1),
                                 layer(A2, moe(3, 0, 1, 40, 0.8))])
B1 = att(4, 1, 8, softcap=2.0)                                         # one key head, every earlier key visible
B2 = att(2, 2, 32, vdim=16, scale=0.11, softcap=50.0, chunk=16)        # a chunk is a page
M2 = moe(4, 1, 5, 24, 3.0)                                             # every output chosen
CFG_B = model(150, 48, 1e-3, 2, [layer(B1, M2, weights_of=2),          # runs with a later layer's tensors
                                 layer(B2, dict(kind="dense", ff=64)),
                                 layer(B1, M2),
                                 layer(B2, dict(kind="dense", ff=64), weights_of=1),
                                 layer(B1, moe(0, 3, 2, 8, 1.0))])     # identity outputs only
# sizes the kernels' vector paths do not like: nothing a multiple of 8, an odd vocabulary, one tap
C1 = att(3, 1, 10, vdim=14, scale=0.4, softcap=9.0, chunk=5)
CFG_C = model(101, 70, 1e-6, 1, [layer(C1, moe(3, 1, 2, 26, 2.5)),
                                 layer(C1, dict(kind="dense", ff=50)),
                                 layer(att(5, 5, 6, chunk=33), moe(2, 2, 2, 18, 0.5))])
# a routed layer first, eight query heads on one key head, values wider than keys, a chunk longer than most requests,
# five taps, more router outputs than a token's choices by far
D1 = att(8, 1, 40, vdim=56, scale=0.2, softcap=12.0, chunk=100)          # heads padded to 64
D2 = att(2, 2, 72, softcap=3.0, chunk=50)                                # heads padded to 80
M4 = moe(9, 3, 6, 32, 4.0)
CFG_D = model(333, 96, 1e-4, 5, [layer(D1, M4),
                                 layer(D2, dict(kind="dense", ff=200)),
                                 layer(D1, M4, weights_of=0),
                                 layer(D2, dict(kind="dense", ff=200), weights_of=1),
                                 layer(D1, None)])
CONFIGS = {"A": (CFG_A, 3), "B": (CFG_B, 4), "C": (CFG_C, 6), "D": (CFG_D, 8)}


def shape_weights(cfg, seed, sharp=True):
    """Random weights shaped so that faults show: products keep the scale of their input, the norms' weights are far
    from their resting value, the query and key norms' weights are large (scores spread over several units, so that
    sigmoids saturate both ways and the cap bends them: which keys are seen matters), the head biases differ from head
    to head, routers are decisive and the correction moves the choice.  ``sharp`` False leaves queries, keys and
    routers at unit scale: the bfloat16 runs use it, because spread scores amplify the rounding of 8-bit values as much
    as they amplify faults."""
    w = random_tensors(cfg, seed, torch.float32, std=1.0)
    g = torch.Generator().manual_seed(seed + 100)
    for k, v in w.items():
        if k.endswith((".q.norm", ".k.norm")):
            v.copy_((1.0 + 0.3 * torch.randn(v.shape, generator=g)) * (1.6 if sharp else 1.0))
        elif "norm" in k:
            v.copy_(0.4 * torch.randn(v.shape, generator=g))               # stored around zero, applied as 1 + w
        elif k.endswith(".pb"):
            v.copy_(torch.randn(v.shape, generator=g) * 1.5 - 1.0)
        elif k.endswith(".correction"):
            v.copy_(torch.randn(v.shape, generator=g) * 0.25)
        elif "canon" in k:
            v.mul_(0.5)
        elif v.dim() >= 2:
            v.mul_(v.shape[-1] ** -0.5)
        if k.endswith(".router") and sharp:
            v.mul_(4.0)
    w["embed"].mul_(cfg.width ** 0.5 * 0.3)
    return w


def make(name, dtype=torch.float32, sharp=True):
    raw, seed = CONFIGS[name]
    cfg = MutusunConfig.from_dict(raw)
    return raw, cfg, {k: v.to(dtype) for k, v in shape_weights(cfg, seed, sharp).items()}


def expected_logits(raw, weights, prompts):
    wf = {k: v.float() for k, v in weights.items()}
    return {rid: plain.forward(raw, wf, toks) for rid, toks in prompts.items()}


def host_runner(cfg, weights, pages=64, rows=8, tokens=256, slots=None):
    return ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                       num_pages=pages, max_rows=rows, max_step_tokens=tokens, max_model_len=pages * 16, num_state_slots=slots)


# float32 against the float64 plain implementation: rounding, amplified by scores that are spread on purpose; a fault
# (a lost key, a chunk that is one position off, a stale tail, a wrong expert) moves logits by a hundred times this or more
F32_TOL = 3e-4
# bfloat16: every sublayer rounds a handful of values to 8 bits
BF16_TOL_PER_LAYER = 1.5e-2

FAMILIES = {"whole": trace_util.whole, "decode_tail": lambda p: trace_util.decode_tail(p, 40),
            "portions": trace_util.portions, "mixed": lambda p: trace_util.mixed(p, 4, seed=5)}
LENGTHS = [3, 70, 1, 37, 90, 18, 49]


def compare_most(got, expected, tol, what, over=0.1, cap=1.0):
    """The bfloat16 comparison.  A token whose choice scores nearly tie may choose another expert once values are
    rounded to 8 bits, and then its logits (and, weakly, those after it) differ by design, not by fault: at most
    ``over`` of the rows may exceed ``tol``, none may exceed ``cap`` of the logit scale or be other than finite.  The
    float32 runs are the sharp test; this one is for the bfloat16 kernels taking a wrong path."""
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
    return check(got, expected_logits(raw, weights, prompts), tol, f"mutusun {name}/{family}/{dtype}")


# ------------------------------------------------------------------------------------------- configuration
def test_config_round_trip_and_registry(tmp_path):
    raw, cfg, _ = make("A")
    assert MutusunConfig.from_dict(cfg.to_dict()) == cfg
    (tmp_path / "config.json").write_text(json.dumps(raw))
    loaded, arch = load_model_config(str(tmp_path))
    assert loaded == cfg and arch.name == "Mutusun"
    assert cfg.layers[2].weights_of == 1 and cfg.owner(4) == 1 and cfg.owner(3) == 3 and cfg.layers[3].mlp is None
    assert cfg.layers[3].mixer.softcap is None and cfg.layers[3].mixer.chunk == 7 and cfg.layers[0].mixer.vdim == 24
    assert MutusunConfig.from_dict(CFG_B).layers[0].mixer.chunk is None and MutusunConfig.from_dict(CFG_B).canon_taps == 2


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][2].update(weights_of=9),                         # no such layer
    lambda c: c["layers"][2].update(weights_of=2),                         # itself
    lambda c: c["layers"][4].update(weights_of=2),                         # a layer that has no tensors of its own
    lambda c: c["layers"][2].update(mixer=A2),                             # another layer than the one whose tensors it runs with
    lambda c: c["layers"][5]["mlp"]["router"].update(top=4),               # more than the router has outputs
    lambda c: c["layers"][0]["mixer"].update(kv_heads=4),                  # 6 query heads over 4 key heads
    lambda c: c["layers"][0]["mixer"].update(softcap=0.0),
    lambda c: c["layers"][0]["mlp"].update(kind="glu"),
    lambda c: c["layers"][0].update(type="conv"),
])
def test_config_refuses_what_cannot_be_computed(bad):
    from mini_inference_engine_amd.config import ConfigError
    raw = json.loads(json.dumps(CFG_A))
    bad(raw)
    with pytest.raises(ConfigError):
        MutusunConfig.from_dict(raw)


def test_model_structure():
    _, cfg, weights = make("A")
    runner = host_runner(cfg, weights)
    m = runner.model
    # four layers own tensors; six runs, each with a cache and state of its own
    assert [c.layer for c in m.spec.schedule] == [0, 1, 1, 2, 1, 3]
    assert "l2.norm1" not in weights and "l4.mix.q" not in weights and "l3.norm2" not in weights and "l3.norm1b" in weights
    assert "l1.mlp.e4.gate" in weights and "l1.mlp.e5.gate" not in weights and tuple(weights["l1.mlp.router"].shape) == (7, 64)
    assert tuple(weights["l1.mix.q.norm"].shape) == (16,) and tuple(weights["l1.mix.pb"].shape) == (6,)
    assert "l5.mlp.correction" in weights and tuple(weights["l0.canon2"].shape) == (64, 4)
    assert len(runner.storage.entries) == 6
    # a run without a feed-forward keeps one tail, the others two
    assert sorted(len([n for n in _names(e) if "tail" in n]) for e in runner.storage.entries.values()) == [1, 2, 2, 2, 2, 2]


def _names(entry, prefix=""):
    """The names of an entry's tensors, members of combined entries included."""
    out = []
    for k, v in (getattr(entry, "tensors", None) or {}).items():
        out.append(prefix + k)
    for name, sub in (getattr(entry, "members", None) or {}).items():
        out += _names(sub, prefix + name + ".")
    return out


# ------------------------------------------------------------------------------------- the plain implementation, by hand
def test_plain_mask_conv_and_norm_by_hand():
    seen = plain.chunk_mask(7, 3)
    assert seen.tolist() == [[1, 0, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0, 0], [0, 0, 0, 1, 0, 0, 0],
                             [0, 0, 0, 1, 1, 0, 0], [0, 0, 0, 1, 1, 1, 0], [0, 0, 0, 0, 0, 0, 1]]
    assert plain.chunk_mask(4, None).tolist() == torch.ones(4, 4).tril().bool().tolist()
    h = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0]], dtype=torch.float64)
    taps = torch.tensor([[0.5, 0.0, 2.0], [0.0, 1.0, 0.0]], dtype=torch.float64)        # the last column is the current token's
    out = plain.input_conv(h, taps)
    assert out.tolist() == [[1 + 2 * 1, 10.0], [2 + 2 * 2, 20 + 10], [3 + 2 * 3 + 0.5 * 1, 30 + 20]]
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    r = math.sqrt(12.5 + 0.5)
    assert torch.allclose(plain.rms_norm(x, torch.tensor([0.5, -1.0]).double(), 0.5, one_plus=True),
                          torch.tensor([[3 / r * 1.5, 0.0]], dtype=torch.float64))
    assert torch.allclose(plain.rms_norm(x, torch.tensor([0.5, -1.0]).double(), 0.5), torch.tensor([[1.5 / r, -4 / r]]).double())


def test_plain_attention_and_router_by_hand():
    # two query heads on one key head, two positions, head size 1: weights are sigmoids, not shares of one
    q = torch.tensor([[[1.0], [2.0]], [[-1.0], [0.5]]], dtype=torch.float64)         # [n, H, d]
    k = torch.tensor([[[2.0]], [[4.0]]], dtype=torch.float64)
    v = torch.tensor([[[1.0, 10.0]], [[2.0, 20.0]]], dtype=torch.float64)
    pb = torch.tensor([0.25, -0.5], dtype=torch.float64)
    cap = lambda s: 3.0 * math.tanh(s / 3.0)                                         # noqa: E731
    sg = lambda z: 1 / (1 + math.exp(-z))                                            # noqa: E731
    out = plain.sigmoid_attention(q, k, v, 0.5, 3.0, pb, plain.chunk_mask(2, None))
    w00, w01 = sg(cap(1 * 2 * 0.5) + 0.25), sg(cap(2 * 2 * 0.5) - 0.5)
    w10a, w10b = sg(cap(-1 * 2 * 0.5) + 0.25), sg(cap(-1 * 4 * 0.5) + 0.25)
    w11a, w11b = sg(cap(0.5 * 2 * 0.5) - 0.5), sg(cap(0.5 * 4 * 0.5) - 0.5)
    want = [[[w00, 10 * w00], [w01, 10 * w01]], [[w10a + 2 * w10b, 10 * w10a + 20 * w10b], [w11a + 2 * w11b, 10 * w11a + 20 * w11b]]]
    assert torch.allclose(out, torch.tensor(want, dtype=torch.float64))
    # with chunks of one position the second query sees its own key only
    alone = plain.sigmoid_attention(q, k, v, 0.5, 3.0, pb, plain.chunk_mask(2, 1))
    assert torch.allclose(alone[1, 0], torch.tensor([2 * w10b, 20 * w10b], dtype=torch.float64))
    # router: three outputs, the last an identity expert; the correction moves the choice, not the weights
    W = {"m.router": torch.eye(3).double(), "m.correction": torch.tensor([0.0, -1.0, 0.0]).double(),
         "m.e0.gate": torch.tensor([[1.0, 0.0, 0.0]]).double(), "m.e0.up": torch.tensor([[0.0, 0.0, 5.0]]).double(),
         "m.e0.down": torch.ones(3, 1).double(),
         "m.e1.gate": torch.zeros(1, 3).double(), "m.e1.up": torch.zeros(1, 3).double(), "m.e1.down": torch.ones(3, 1).double()}
    h = torch.tensor([[1.0, 2.0, 0.5]], dtype=torch.float64)                          # scores favour output 1, which the correction bars
    s = torch.softmax(h[0], 0)
    out = plain.moe_ff(h, W, "m", dict(router=dict(experts=2, identity=1, top=2), expert=dict(ff=1, limit=1.5)))
    g, u = 1.0, 1.5                                                                 # gate 1 stays; up 2.5 is clamped to the limit
    y0 = g * sg(1.702 * g) * (u + 1.0)
    assert torch.allclose(out, s[0] * torch.full((1, 3), y0, dtype=torch.float64) + s[2] * h)
    # the gate is clamped from above only
    e = plain.expert(torch.tensor([[-4.0, 0.0, -4.0]]).double(), W, "m.e0", 1.5)
    assert torch.allclose(e, torch.full((1, 3), -4.0 * sg(1.702 * -4.0) * (-1.5 + 1.0), dtype=torch.float64))


def test_router_margins_of_the_test_models():
    """The comparisons are only fair if no token of the test prompts sits on a routing boundary."""
    for name in CONFIGS:
        raw, _, weights = make(name)
        margins = []
        for toks in trace_util.random_prompts(raw["vocab"], LENGTHS, seed=17).values():
            plain.forward(raw, weights, toks, margins=margins)
        assert margins and min(margins) > 1e-5, f"{name}: a token is routed with a margin of {min(margins):.1e}"


# ------------------------------------------------------------------------------------- mechanisms, one by one
def one_layer(mixer, mlp, width=32, vocab=50, taps=None, eps=1e-5):
    return model(vocab, width, eps, taps, [layer(mixer, mlp)])


MECHANISMS = {
    "attention": one_layer(att(4, 2, 8, vdim=12, softcap=4.0, chunk=6), None),
    "attention-no-cap-no-chunk": one_layer(att(2, 1, 16, scale=0.2), None),
    "attention-chunk-of-one": one_layer(att(2, 2, 8, softcap=1.0, chunk=1), None),
    "attention-one-head": one_layer(att(1, 1, 24, vdim=40, chunk=10), None),
    "conv-4-taps": one_layer(att(2, 1, 8, chunk=9), None, taps=4),
    "conv-1-tap": one_layer(att(2, 1, 8, chunk=9), dict(kind="dense", ff=40), taps=1),
    "dense": one_layer(att(2, 1, 8, chunk=9), dict(kind="dense", ff=40), taps=3),
    "experts": one_layer(att(2, 1, 8, chunk=9), moe(4, 2, 3, 12, 1.0), taps=2),
    "experts-top1-no-identity": one_layer(att(2, 1, 8, chunk=9), moe(3, 0, 1, 12, 0.3)),
    "experts-all-chosen": one_layer(att(2, 1, 8, chunk=9), moe(2, 1, 3, 20, 5.0), taps=2),
    "identity-only": one_layer(att(2, 1, 8, chunk=9), moe(0, 2, 1, 4, 1.0), taps=2),
}


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_each_mechanism_alone_on_the_host(name):
    raw = MECHANISMS[name]
    cfg = MutusunConfig.from_dict(raw)
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


def edge_model():
    """One layer, no convolution, chunks of 20 positions (a page and a quarter): the logits of a position are a
    function of the tokens of its own chunk up to itself and of nothing else."""
    raw = one_layer(att(4, 2, 16, vdim=8, scale=0.25, softcap=6.0, chunk=20), dict(kind="dense", ff=48), width=48, vocab=90)
    cfg = MutusunConfig.from_dict(raw)
    w = shape_weights(cfg, 5)
    w["embed"][89] = 4.0 * w["embed"][89].sign()              # the token that stands out
    return raw, cfg, w


def edge_runs(device):
    """A token that stands out is put just inside and just outside the chunk of the positions asked for (and on a
    page's last and next first slot, and at the very first position), in a prompt's portion and for tokens decoded one
    by one.  Inside, it must move the logits; outside, the engine's logits must not move at all; both ways they follow
    the plain implementation."""
    raw, cfg, w = edge_model()
    base = [t if t != 89 else 0 for t in trace_util.random_prompts(90, [75], seed=9)["r0"]]

    def run(tokens, cut):
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:cut], "want": list(range(cut))}], "end": []}]
        steps += [{"step": 1 + i, "entries": [{"id": "x", "tokens": tokens[cut + i:cut + i + 1], "want": [0]}], "end": []}
                  for i in range(len(tokens) - cut)]
        steps[-1]["end"] = ["x"]
        if device == "cpu":
            runner = host_runner(cfg, w, pages=8, rows=2, tokens=80)
        else:
            runner = ModelRunner(cfg, weights=w, dtype="float32", num_pages=8, max_rows=2, max_step_tokens=80, max_model_len=112)
        return {k: v.cpu() for k, v in trace_util.run_on_runner(runner, steps).items()}

    for cut in (70, 42, 58):                 # asked-for positions in the portion; decoded; the chunk's edge among decoded tokens
        plain_run = run(base, cut)
        for needle in (59, 60, 39, 40, 47, 48, 0, 19, 20):
            tokens = list(base)
            tokens[needle] = 89
            want = plain.forward(raw, w, tokens)
            got = run(tokens, cut)
            trace_util.compare(got, {"x": want}, F32_TOL, f"needle at {needle}, portion of {cut}")
            first, last = needle // 20 * 20, needle // 20 * 20 + 19
            for p in range(75):
                moved = float((got[("x", p)] - plain_run[("x", p)]).abs().max()) / float(want.abs().max())
                if needle <= p <= last:
                    assert moved > 1e-3, f"position {p} must see the token at {needle} (portion of {cut})"
                else:
                    assert moved < 1e-6, f"position {p} must not see the token at {needle} (portion of {cut}): moved {moved:.1e}"
            assert first <= needle


def test_keys_just_inside_and_outside_a_chunk_on_the_host():
    edge_runs("cpu")


def far_key_runs(device):
    """No chunks: one key far back (hundreds of positions, through a dozen pages) is made to decide the output.  Every
    other key's weight is next to nothing (a head bias far below zero); the far key's product with the last query is
    large, because query and key matrices are made equal and the last token is the far key's own.  The
    key stands at a page's last slot, at the next page's first, and at the very first position."""
    raw = one_layer(att(2, 1, 16, scale=0.25), None, width=32, vocab=64)
    cfg = MutusunConfig.from_dict(raw)
    w = shape_weights(cfg, 7)
    w["l0.mix.q"].copy_(w["l0.mix.k"].repeat(2, 1))          # a token's queries equal its key: a product of 16 * 2 * 2 * scale
    w["l0.mix.pb"].fill_(-12.0)                              # other keys score 0 +- 4
    w["l0.mix.q.norm"].fill_(2.0)
    w["l0.mix.k.norm"].fill_(2.0)
    toks = [t if t != 63 else 0 for t in trace_util.random_prompts(64, [230], seed=9)["r0"]]
    for needle in (31, 32, 0):
        tokens = list(toks)
        tokens[needle] = 63
        tokens[-1] = 63                                       # the last query is the far key's own token: their product is the largest there is
        want = plain.forward(raw, w, tokens)
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:190], "want": [189]}], "end": []}]
        steps += [{"step": 1 + i, "entries": [{"id": "x", "tokens": tokens[190 + i:191 + i], "want": [0]}], "end": []}
                  for i in range(40)]
        steps[-1]["end"] = ["x"]
        if device == "cpu":
            runner = host_runner(cfg, w, pages=16, rows=2, tokens=192)
        else:
            runner = ModelRunner(cfg, weights=w, dtype="float32", num_pages=16, max_rows=2, max_step_tokens=192, max_model_len=240)
        got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, steps).items()}
        trace_util.compare(got, {"x": want}, F32_TOL, f"far key at {needle}")
        other = list(tokens)
        other[needle] = toks[needle]
        moved = float((plain.forward(raw, w, other)[-1] - want[-1]).abs().max()) / float(want.abs().max())
        assert moved > 1e-2, "the far key must matter to the last position for this test to mean anything"


def test_a_far_key_and_the_first_token_are_seen():
    far_key_runs("cpu")


def test_state_slots_and_pages_are_used_again():
    """Five requests, one after another, through a runner with one usable state slot and pages for one request:
    each must start from an empty convolution tail and see no key of the one before."""
    raw, cfg, weights = make("B")
    prompts = trace_util.random_prompts(raw["vocab"], [40, 33, 40, 7, 25], seed=3)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                         num_pages=4, max_rows=1, max_step_tokens=64, max_model_len=48, num_state_slots=2)
    got = trace_util.run_on_runner(runner, trace_util.portions(prompts, sizes=(5, 2, 9)))
    trace_util.compare(got, expected_logits(raw, weights, prompts), F32_TOL, "reuse")
    tails = [t for name, t in _all_tensors(runner.storage) if "tail" in name]
    assert len(tails) == 2 * 5
    for t in tails:
        t.fill_(-2.0)
    rc = runner.cache.open("fresh")
    assert all(float(t[rc.state_slot].abs().max()) == 0.0 for t in tails)
    runner.cache.close(rc)


def _all_tensors(storage):
    out = []

    def walk(entry, prefix):
        for k, v in (getattr(entry, "tensors", None) or {}).items():
            out.append((prefix + k, v))
        for name, sub in (getattr(entry, "members", None) or {}).items():
            walk(sub, prefix + name + ".")
    for i, e in storage.entries.items():
        walk(e, f"{i}.")
    return out


def test_pages_before_the_chunk_are_given_back():
    """A request that decodes far beyond its chunk keeps the pages of its own chunk only."""
    raw = one_layer(att(2, 1, 8, chunk=32), None, taps=2)
    cfg = MutusunConfig.from_dict(raw)
    w = shape_weights(cfg, 2)
    prompts = trace_util.random_prompts(50, [150], seed=1)
    runner = ModelRunner(cfg, weights=w, dtype="float32", device="cpu", backend=TorchBackend(torch.float32), num_pages=6,
                         max_rows=1, max_step_tokens=64, max_model_len=160)          # five usable pages of 16 for 150 tokens
    got = trace_util.run_on_runner(runner, trace_util.portions(prompts, sizes=(20, 3, 1, 30)))
    trace_util.compare(got, expected_logits(raw, w, prompts), F32_TOL, "pages given back")


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
    outs = eng.generate(prompts, SamplingParams(max_tokens=30, ignore_eos=True))          # through a chunk's edge
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


class AttentionCase:
    """Rows of a step over a paged cache filled at random: single-token rows first, as the engine orders them."""

    def __init__(self, rows, Hkv, P, dtype, g, page=16):
        import numpy as np
        from types import SimpleNamespace
        rows = sorted(rows, key=lambda r: r[1] != 1)                       # (tokens so far, new tokens)
        self.rows = rows
        per = [-(-(have + new) // page) for have, new in rows]
        pages = 1 + sum(per)
        perm = (torch.randperm(pages - 1, generator=g) + 1).tolist()       # page 0 is scratch
        width = max(per) + 1
        bt = torch.zeros(len(rows), width, dtype=torch.int32)
        at = 0
        for r, n in enumerate(per):
            bt[r, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
            at += n
        self.k = _rand((pages, Hkv, page, P), dtype, g)
        self.v = _rand((pages, Hkv, P, page), dtype, g)
        token_row = torch.cat([torch.full((new,), r, dtype=torch.int32) for r, (_, new) in enumerate(rows)])
        positions = torch.cat([torch.arange(have, have + new, dtype=torch.int32) for have, new in rows])
        self.block_tables = bt.cuda()
        self.group = SimpleNamespace(block_tables=self.block_tables, slot_mapping=None,
                                     context_lens=torch.tensor([h + n for h, n in rows], dtype=torch.int32).cuda())
        self.token_row, self.positions = token_row.cuda(), positions.cuda()
        self.num_tokens = int(token_row.numel())
        self.num_decode_rows = sum(1 for _, new in rows if new == 1)
        rs = np.concatenate([[0], np.cumsum([n for _, n in rows])]).astype("int64")
        self.step = SimpleNamespace(token_row=self.token_row, positions=self.positions, num_tokens=self.num_tokens,
                                    num_rows=len(rows), num_decode_rows=self.num_decode_rows,
                                    row_start=torch.tensor(rs, dtype=torch.int32).cuda(), host={"row_start": rs},
                                    row_position=torch.tensor([h for h, _ in rows], dtype=torch.int32).cuda(),
                                    max_row_tokens=max(n for _, n in rows),
                                    groups=[self.group], max_context=max(h + n for h, n in rows))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sigmoid_attention_kernels(hip, dtype):
    """Decode rows and portions over random pages against the torch operation: chunks that are no multiple of a page,
    of a page, of one position and none; with and without a cap and head biases; padded and wide heads."""
    ops, g = hip[dtype], torch.Generator().manual_seed(11)
    rows = [(0, 1), (23, 1), (24, 1), (47, 1), (200, 1), (0, 50), (17, 31), (63, 2), (100, 130)]
    for (Hq, Hkv, P, chunk, cap, bias) in ((6, 2, 16, 24, 5.0, True), (3, 3, 32, 7, None, True), (4, 1, 16, None, 2.0, False),
                                           (2, 2, 48, 16, 50.0, True), (8, 2, 64, 64, 30.0, True), (4, 4, 128, 1, None, True),
                                           (16, 4, 64, 100, 30.0, True)):
        case = AttentionCase(rows, Hkv, P, dtype, g)
        q = _rand((case.num_tokens, Hq * P), dtype, g)
        hb = (_rand((Hq,), torch.float32, g) - 2.0) if bias else None
        want = ref.ref_paged_attention(q, Hq, Hkv, P, case.k, case.v, case.block_tables, case.token_row, case.positions,
                                       P ** -0.5, chunk, torch.float32, weights="sigmoid", softcap=cap, chunk=chunk, head_bias=hb)
        got = ops.paged_attention(q, Hq, Hkv, P, case.k, case.v, case.group, case.step, P ** -0.5, chunk, weights="sigmoid",
                                  softcap=cap, chunk=chunk, head_bias=hb)
        close(got, want, 1e-5 if dtype == torch.float32 else 1.5e-2, f"heads {Hq}/{Hkv} of {P}, chunk {chunk}, cap {cap}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_key_stands_out_at_every_edge(hip, dtype):
    """Every key's weight is next to nothing (head bias -30) but one key's, whose product with every query is large:
    the output is that key's value if the query sees it and nothing otherwise.  The key stands just inside and just
    outside chunks and pages, far back and at the first position; queries are decode rows and rows of portions."""
    ops, g = hip[dtype], torch.Generator().manual_seed(12)
    Hq, Hkv, P, page = 4, 2, 32, 16
    for chunk in (24, 16, 40, None):
        for needle in (0, 15, 16, 23, 24, 39, 40, 47, 48, 95, 96, 119, 120):
            rows = [(needle, 1), (needle + 1, 1), (130, 1), (0, 131), (needle, 2), (max(0, needle - 3), 7)]
            if chunk is not None:
                edge = (needle // chunk + 1) * chunk                    # the first position that no longer sees the key
                rows += [(edge - 1, 1), (edge, 1), (edge - 1, 2), (max(0, edge - 5), 9)]
            case = AttentionCase(rows, Hkv, P, dtype, g, page)
            case.k.mul_(0.05)
            direction = torch.ones(P).to(dtype).cuda()
            for r in range(len(case.rows)):                             # the key at ``needle`` of every row that holds it
                if sum(case.rows[r]) > needle:
                    pg = int(case.block_tables[r, needle // page])
                    case.k[pg, :, needle % page, :] = direction
            q = (torch.ones(case.num_tokens, Hq * P) * 2.5).to(dtype).cuda()         # q . k * scale = 2.5 * 32 / sqrt(32) * ... large
            hb = torch.full((Hq,), -30.0).cuda()
            got = ops.paged_attention(q, Hq, Hkv, P, case.k, case.v, case.group, case.step, 1.0, chunk, weights="sigmoid",
                                      softcap=None, chunk=chunk, head_bias=hb).float().cpu()
            pos, row = case.positions.cpu().tolist(), case.token_row.cpu().tolist()
            for t in range(case.num_tokens):
                sees = needle <= pos[t] and (chunk is None or pos[t] // chunk == needle // chunk)
                if sees:
                    pg = int(case.block_tables[row[t], needle // page])
                    want = case.v[pg, :, :, needle % page].float().cpu().repeat_interleave(Hq // Hkv, 0).reshape(-1)
                else:
                    want = torch.zeros(Hq * P)
                assert float((got[t] - want).abs().max()) < 2e-2, \
                    f"chunk {chunk}, key at {needle}: position {pos[t]} of a row of {case.rows[row[t]]} " \
                    f"{'must' if sees else 'must not'} see it"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_per_head_and_store_kernel(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(13)
    for (T, Hq, Hkv, dim, vdim) in ((1, 6, 2, 16, 24), (37, 3, 3, 24, 8), (130, 4, 1, 10, 14), (5, 2, 2, 48, 48), (64, 16, 4, 64, 64)):
        P = -(-max(dim, vdim) // 16) * 16
        sums = _rand((T, 3 + Hq * dim + Hkv * dim + Hkv * vdim + 5), torch.float32, g, 2.0)
        qn, kn = _rand((dim,), torch.float32, g) + 1, _rand((dim,), torch.float32, g) + 1
        positions = torch.arange(T, dtype=torch.int32).cuda()
        pages, page = T // 16 + 3, 16
        slots = torch.randperm((pages - 1) * page, generator=g)[:T].to(torch.int32).cuda() + page
        kc, vc = torch.full((pages, Hkv, page, P), 7.0, dtype=dtype).cuda(), torch.full((pages, Hkv, P, page), 7.0, dtype=dtype).cuda()
        kw, vw = kc.clone(), vc.clone()
        cols = (3, 3 + Hq * dim, 3 + Hq * dim + Hkv * dim)
        want = ref.ref_qkv_finish(sums, *cols, Hq, Hkv, dim, vdim, P, positions, None, "half", kw, vw, slots, qn, kn, 1e-5, None,
                                  dtype, norm_per_head=True)
        got = ops.qkv_finish(sums, *cols, Hq, Hkv, dim, vdim, P, positions, None, "half", kc, vc, slots, q_norm=qn, k_norm=kn,
                             eps=1e-5, norm_per_head=True)
        close(got, want, TOL[dtype], "queries")
        close(kc, kw, TOL[dtype], "keys")
        close(vc, vw, TOL[dtype], "values")
        assert torch.equal(kc[0], kw[0]), "the scratch page was not written"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routing_over_all_outputs_and_gated_expert_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(14)
    for (T, W, E, I, top, ff, limit) in ((1, 64, 5, 2, 3, 48, 1.5), (37, 48, 4, 1, 5, 24, 3.0), (300, 72, 3, 0, 1, 40, 0.8),
                                         (9, 64, 0, 3, 2, 8, 1.0), (130, 128, 16, 2, 4, 96, 7.0), (65, 70, 2, 2, 2, 18, 0.5),
                                         (700, 64, 4, 1, 2, 64, 2.0), (2, 256, 8, 0, 2, 160, 1.0)):
        R = E + I
        logits, corr = _rand((T, R), torch.float32, g, 2.0), _rand((R,), torch.float32, g, 0.25)
        idx, shares = ops.route_topk(logits, None, top, over="all", choice_bias=corr)
        widx, wshares = ref.ref_route_topk(logits, None, top, over="all", choice_bias=corr)
        assert torch.equal(idx.cpu(), widx.cpu())
        close(shares, wshares, 2e-6, "shares")
        assert float(shares.sum(-1).max()) <= 1.0 + 1e-5 and (top == R or float(shares.sum(-1).min()) < 0.999), \
            "shares are the scores themselves, not renormalised"
        x = _rand((T, W), dtype, g)
        w_up = _rand((E, 2 * ff, W), dtype, g, 2 * W ** -0.5) if E else None
        w_down = _rand((E, W, ff), dtype, g, ff ** -0.5) if E else None
        got = ops.routed_experts(x, idx, shares, w_up, w_down, "relu2", gated=(limit, 1.702), identity_from=E if I else None)
        want = ref.ref_routed_experts(x, idx, shares, w_up, w_down, "relu2", dtype, gated=(limit, 1.702), identity_from=E if I else None)
        close(got, want, 1e-5 if dtype == torch.float32 else 1e-2, f"experts {T} tokens, {E}+{I} outputs")
        if E and ff % 16 == 0:
            # rows in alternating blocks of 16 gate and 16 up rows: in bfloat16 the product's own epilogue gates
            assert ops.glu_rows_block(ff) == (16 if dtype == torch.bfloat16 else 0)
            mixed = w_up.view(E, 2, ff // 16, 16, W).transpose(1, 2).contiguous().view(E, 2 * ff, W)
            got = ops.routed_experts(x, idx, shares, mixed, w_down, "relu2", gated=(limit, 1.702),
                                     identity_from=E if I else None, glu_block=16)
            close(got, want, 1e-5 if dtype == torch.float32 else 1e-2, f"experts in blocks of 16, {T} tokens")
    tie = torch.zeros(2, 4).cuda()
    assert ops.route_topk(tie, None, 2, over="all")[0].tolist() == [[0, 1], [0, 1]], "lowest index first among equals"
    moved = ops.route_topk(tie, None, 2, over="all", choice_bias=torch.tensor([0.0, 0.0, 0.5, 0.25]).cuda())
    assert moved[0].tolist() == [[2, 3], [2, 3]] and torch.allclose(moved[1].cpu(), torch.full((2, 2), 0.25))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activation_on_sums_and_sandwich_norm_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(15)
    for T, W, F in ((1, 64, 112), (37, 70, 50), (300, 192, 384)):
        x, w = _rand((T, W), dtype, g), _rand((F, W), dtype, g, W ** -0.5)
        want = ref.ref_act(x.double() @ w.double().T, "relu2")
        close(ops.linear_act(x, w, "relu2"), want, 1e-5 if dtype == torch.float32 else 1e-2, f"relu2 at {T} rows")
        stream = _rand((T, W), torch.float32, g)
        y, wt = _rand((T, W), torch.float32, g, 3.0), _rand((W,), dtype, g, 0.4) + 1
        want = stream.clone()
        ref.ref_branch_norm_add(y, want, wt, 1e-5, dtype)
        assert ops.branch_norm_add(y, stream, wt, 1e-5, copy=False) is None
        close(stream, want, 2e-6, "stream after a normed branch")


class FakeStep:
    def __init__(self, lens, slots):
        import numpy as np
        rs = np.concatenate([[0], np.cumsum(lens)]).astype("int64")
        self.num_rows, self.num_tokens = len(lens), int(rs[-1])
        self.host = {"row_start": rs, "state_slots": np.asarray(slots)}
        self.row_start = torch.tensor(rs, dtype=torch.int32).cuda()
        self.state_slots = torch.tensor(slots, dtype=torch.int32).cuda()
        self.token_row = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(torch.int32).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_branch_added_and_next_input_made_in_one_kernel(hip, dtype):
    """Steps of single-token rows add a normed branch output and make the next sublayer's convolved input in one
    kernel; steps with longer rows in two.  Both against the torch operations, stream, input and tails."""
    ops, g = hip[dtype], torch.Generator().manual_seed(16)
    for (W, K, lens, slots) in ((64, 4, [1, 1, 1], [3, 1, 2]), (72, 1, [1], [1]), (2048, 3, [1] * 8, [8, 7, 6, 5, 4, 3, 2, 1]),
                                (64, 2, [1, 5, 1], [1, 2, 3]), (70, 3, [1, 1], [2, 1])):
        step = FakeStep(lens, slots)
        T = step.num_tokens
        stream, y = _rand((T, W), torch.float32, g), _rand((T, W), torch.float32, g, 3.0)
        w_out, w_next = _rand((W,), torch.float32, g, 0.4) + 1, _rand((W,), torch.float32, g, 0.4) + 1
        taps, tail = _rand((W, K), torch.float32, g, 0.5), _rand((9, max(1, K - 1), W), torch.float32, g)
        want_stream, want_tail = stream.clone(), tail.cpu().clone()
        ref.ref_branch_norm_add(y, want_stream, w_out, 1e-5, torch.float32)
        h = ref.ref_add_rmsnorm(None, want_stream.clone(), w_next, 1e-6, torch.float32)
        want = ref.ref_residual_conv(h.cpu(), taps.cpu(), want_tail, step.host["row_start"], step.host["state_slots"], dtype)
        got = ops.branch_norm_conv(y, stream, w_out, 1e-5, w_next, 1e-6, taps, tail, step)
        close(stream, want_stream, 2e-6, f"stream, width {W}, rows {lens}")
        close(got, want, TOL[dtype] if dtype == torch.bfloat16 else 1e-5, f"input, width {W}, rows {lens}")
        if K > 1:
            close(tail, want_tail, 1e-5, f"tails, width {W}, rows {lens}")


# ------------------------------------------------------------------------------------------ GPU: whole models
@pytest.mark.gpu
def test_keys_just_inside_and_outside_a_chunk_gpu():
    edge_runs("cuda")


@pytest.mark.gpu
def test_a_far_key_and_the_first_token_are_seen_gpu():
    far_key_runs("cuda")


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(MECHANISMS))
def test_each_mechanism_alone_gpu(name):
    raw = MECHANISMS[name]
    cfg = MutusunConfig.from_dict(raw)
    weights = shape_weights(cfg, 1)
    prompts = trace_util.random_prompts(raw["vocab"], [29, 40], seed=2)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", num_pages=10, max_rows=2, max_step_tokens=64, max_model_len=128)
    got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, trace_util.mixed(prompts, 2, seed=3, tail=6)).items()}
    trace_util.compare(got, expected_logits(raw, weights, prompts), F32_TOL, name)


@pytest.mark.gpu
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_float32_gpu(name, family, tmp_path):
    run_family(name, family, tmp_path, "cuda", "float32", F32_TOL)


@pytest.mark.gpu
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_bfloat16_gpu(name, family, tmp_path):
    """bfloat16: a value is rounded to 8 bits a handful of times a layer; a fault (a lost key, a stale tail, the
    wrong cache) moves logits by a large part of their scale."""
    run_family(name, family, tmp_path, "cuda", "bfloat16", BF16_TOL_PER_LAYER * len(CONFIGS[name][0]["layers"]))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_gpu(dtype):
    eng = generate("A", "cuda", dtype)
    assert eng.num_graph_steps > 0, "decode steps of this model run as captured graphs too"


@pytest.mark.gpu
def test_long_decoding_gpu():
    """200 tokens one by one after a short prompt, float32: tails and cache carried through a dozen pages and eight
    chunks, with the pages before a chunk given back on the way."""
    raw, cfg, weights = make("A")
    toks = trace_util.random_prompts(raw["vocab"], [210], seed=6)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", num_pages=16, max_rows=2, max_step_tokens=64, max_model_len=240)
    got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, trace_util.decode_tail(toks, 200)).items()}
    trace_util.compare(got, expected_logits(raw, weights, toks), F32_TOL, "long decoding")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_sizes_of_a_real_model_gpu(dtype):
    """Heads of 64 and 128 numbers, chunks of 256 and 1,024 positions, a width of 512: the kernels' wide paths, on a
    prompt that crosses chunks in one portion and on decoded tokens."""
    big = att(8, 2, 64, softcap=30.0, chunk=256)
    wide = att(4, 4, 128, vdim=64, softcap=20.0, chunk=1024)
    raw = model(500, 512, 1e-6, 4, [layer(big, dict(kind="dense", ff=1024)), layer(wide, moe(8, 1, 2, 256, 7.0)),
                                    layer(wide, moe(8, 1, 2, 256, 7.0), weights_of=1)])
    cfg = MutusunConfig.from_dict(raw)
    sharp = dtype == "float32"
    weights = {k: v.to(torch.float32 if sharp else torch.bfloat16) for k, v in shape_weights(cfg, 9, sharp).items()}
    prompts = trace_util.random_prompts(500, [700, 300], seed=1)
    runner = ModelRunner(cfg, weights=weights, dtype=dtype, num_pages=72, max_rows=2, max_step_tokens=1024, max_model_len=1088)
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": prompts["r0"][:600], "want": [0, 255, 256, 257, 511, 512, 599]}], "end": []},
             {"step": 1, "entries": [{"id": "r0", "tokens": prompts["r0"][600:690], "want": [0, 89]},
                                     {"id": "r1", "tokens": prompts["r1"][:290], "want": [255, 256, 289]}], "end": []}]
    steps += [{"step": 2 + i, "entries": [{"id": "r0", "tokens": prompts["r0"][690 + i:691 + i], "want": [0]},
                                          {"id": "r1", "tokens": prompts["r1"][290 + i:291 + i], "want": [0]}], "end": []}
              for i in range(10)]
    steps[-1]["end"] = ["r0", "r1"]
    got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, steps).items()}
    check = trace_util.compare if sharp else compare_most
    check(got, expected_logits(raw, weights, prompts), F32_TOL if sharp else 3 * BF16_TOL_PER_LAYER, f"real sizes {dtype}")


@pytest.mark.gpu
def test_command_line_and_trace_runner(tmp_path):
    """The named size as a user reaches it: ``random-model`` writes the folder, ``generate`` and ``bin/trace_run``
    load it by the architecture its config.json names; greedy tokens and replayed logits against the plain model."""
    import os
    import subprocess
    import sys
    from safetensors.torch import load_file
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = str(tmp_path / "model")

    def run(cmd, **kw):
        proc = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=600, **kw)
        assert proc.returncode == 0, f"{cmd}: exit {proc.returncode}\n{proc.stderr[-2000:]}"
        return proc

    cli = [sys.executable, "-m", "mini_inference_engine_amd"]
    run(cli + ["random-model", "--shape", "mutusun-tiny", "--seed", "3", "--dtype", "float32", "--out", folder])
    raw = json.load(open(os.path.join(folder, "config.json")))
    weights = load_file(os.path.join(folder, "model.safetensors"))
    assert raw["architecture"] == "Mutusun" and len(raw["layers"]) == 3 and raw["layers"][2]["weights_of"] == 1
    prompt = [5, 17, 3, 200, 41, 7, 7, 300]
    out = run(cli + ["generate", "--model", folder, "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)),
                     "--max-tokens", "6", "--ignore-eos", "--quiet"])
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    ids = list(prompt)
    for tok in rec["output_ids"]:
        logits = plain.forward(raw, weights, ids)[-1]
        assert float(logits.max() - logits[tok]) <= F32_TOL * float(logits.abs().max())
        ids.append(tok)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:9], "want": [0, 8]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": ids[9:11], "want": []}, {"id": "b", "tokens": ids[:3], "want": [2]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": ids[11:12], "want": [0]}], "end": ["a"]}]
    out_dir = str(tmp_path / "out")
    proc = run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out_dir,
                "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n")
    assert [ln for ln in proc.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    got = trace_util.read_outputs(out_dir, steps, raw["vocab"])
    want = {"a": plain.forward(raw, weights, ids[:12]), "b": plain.forward(raw, weights, ids[:3])}
    trace_util.compare(got, want, F32_TOL, "trace_run")
