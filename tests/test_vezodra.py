"""Vezodra through the engine against the plain implementation (tests/plain_vezodra.py).

Configurations are made here, with sizes that differ from one another wherever the design lets them (query and
kv heads, key and value sizes that are no multiple of 16 and differ from each other, turned parts smaller than a
head, windows shorter than a page, of exactly one key and longer than two pages, one state head, an inner decay
size of 3, convolutions of 1, 2 and 4 taps and none, a looped stretch of one and of two layers, a layer without
feed-forward).  Host tests run the engine's own parts, cache and step function on the CPU with the torch
operations of tests/torch_backend.py; GPU tests run the HIP kernels, each kernel against the torch operation of
the same name and the whole model in the four trace families, in float32 (tight) and bfloat16.
"""
import json
import math

import pytest
import torch

import plain_vezodra as plain
import trace_util
from torch_backend import TorchBackend
import torch_backend as ref

from mini_inference_engine_amd.config import ConfigError, EngineConfig, VezodraConfig, load_model_config
from mini_inference_engine_amd.engine.batch import StepRow
from mini_inference_engine_amd.engine.runner import ModelRunner
from mini_inference_engine_amd.replay.trace import replay
from mini_inference_engine_amd.weights import random_tensors


def sink_att(heads, kv_heads, dim, dims=None, base=1000.0, scale=None):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale if scale is not None else dim ** -0.5,
                rot=dict(base=base, dims=dims or dim))


def par(heads, kv_heads, dim, vdim, window, rec_heads, rec_dim, rank, dims=None, base=1000.0, factor=None, scale=None):
    rot = dict(base=base, dims=dims or dim)
    if factor is not None:
        rot["scaling"] = dict(factor=factor)
    return dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else dim ** -0.5,
                          mask=dict(size=window), rot=rot),
                right=dict(heads=rec_heads, dim=rec_dim, rank=rank))


def layer(kind, mixer, ff):
    return dict(type=kind, mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff))


CFG_A = dict(architecture="Vezodra", vocab=211, width=64, norm=dict(eps=1e-5), canon=dict(taps=4), loop=dict(start=1, stop=3, times=2),
             layers=[layer("parallel", par(4, 2, 16, 24, 20, 2, 16, 8, dims=8, factor=4.0), 112),
                     layer("attention", sink_att(6, 3, 32, dims=16, base=77.0, scale=0.21), 80),
                     layer("parallel", par(2, 1, 32, 16, 33, 3, 8, 5, base=50.0), None),
                     layer("attention", sink_att(2, 2, 16), 72)])
CFG_B = dict(architecture="Vezodra", vocab=150, width=48, norm=dict(eps=1e-3), canon=dict(taps=2),
             layers=[layer("attention", sink_att(3, 3, 48, dims=24, base=300.0), None),
                     layer("parallel", par(3, 1, 16, 16, 1, 1, 32, 3, factor=1.5), 64),
                     layer("parallel", par(4, 4, 16, 32, 16, 2, 24, 16, dims=4), 40)])
# sizes the kernels' vector paths do not like: nothing a multiple of 8, an odd vocabulary, one tap, a single looped layer
CFG_C = dict(architecture="Vezodra", vocab=101, width=70, norm=dict(eps=1e-6), canon=dict(taps=1), loop=dict(start=0, stop=1, times=3),
             layers=[layer("parallel", par(3, 3, 10, 14, 7, 5, 12, 5, dims=6, base=30.0, factor=2.0), 50),
                     layer("attention", sink_att(5, 1, 22, dims=10), 34)])
CONFIGS = {"A": (CFG_A, 3), "B": (CFG_B, 4), "C": (CFG_C, 6)}


def shaped(cfg, seed, dtype=torch.float32, sharp=True):
    """Random weights shaped so that faults show: products keep the scale of their input, query and key projections
    are doubled (scores spread over several units: which keys are seen, and whether the sink is there, matters),
    temperatures, norm weights and biases are not 1 or 0, decays cover slow and fast channels.  ``sharp`` False
    leaves queries and keys at unit scale: the bfloat16 runs use it, because spread scores amplify the rounding of
    8-bit values as much as they amplify faults."""
    w = random_tensors(cfg, seed, torch.float32, std=1.0)
    g = torch.Generator().manual_seed(seed + 100)
    for k, v in w.items():
        if v.dim() >= 2 and "canon" not in k:
            v.mul_(v.shape[-1] ** -0.5)
        if k.endswith((".q", ".k")) and sharp:
            v.mul_(2.0)
        if k.endswith((".a.b", ".w0")):
            v.copy_(torch.randn(v.shape, generator=g) * 1.5)
        if k.endswith(".temp"):
            v.copy_(torch.rand(v.shape, generator=g) + 0.5)
        if "norm" in k or k.endswith(".out"):
            v.copy_(torch.randn(v.shape, generator=g) * 0.3 + 1.0)
        if "canon" in k:
            v.mul_(0.5)
        if k.endswith(".w2"):
            v.mul_(3.0)
    w["embed"].mul_(0.5)
    return {k: v.to(dtype) for k, v in w.items()}


def make(name, dtype=torch.float32, sharp=True):
    raw, seed = CONFIGS[name]
    cfg = VezodraConfig.from_dict(raw)
    return raw, cfg, shaped(cfg, seed, dtype, sharp)


def expected_logits(raw, weights, prompts):
    wf = {k: v.float() for k, v in weights.items()}
    return {rid: plain.forward(raw, wf, toks) for rid, toks in prompts.items()}


def host_runner(cfg, weights, pages=64, rows=8, tokens=256):
    return ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                       num_pages=pages, max_rows=rows, max_step_tokens=tokens, max_model_len=pages * 16)


def any_runner(device, cfg, weights, dtype="float32", **kw):
    if device == "cpu":
        kw.update(device="cpu", backend=TorchBackend(torch.float32))
    return ModelRunner(cfg, weights=weights, dtype=dtype, **kw)


# float32 against the float64 plain implementation: rounding, amplified by scores that are spread on purpose; a fault
# (a lost key, a window one token off, a stale state, a sink left out) moves logits by a hundred times this or more
F32_TOL = 3e-4
# bfloat16: every layer run rounds a handful of values to 8 bits
BF16_TOL_PER_LAYER = 1.5e-2

FAMILIES = {"whole": trace_util.whole, "decode_tail": lambda p: trace_util.decode_tail(p, 40),
            "portions": trace_util.portions, "mixed": lambda p: trace_util.mixed(p, 4, seed=5)}
LENGTHS = [3, 70, 1, 37, 90, 18, 49]


def compare_most(got, expected, tol, what, over=0.1, cap=1.0):
    """The bfloat16 comparison: at most ``over`` of the rows may exceed ``tol``, none may exceed ``cap`` of the logit
    scale or be other than finite.  The float32 runs are the sharp test; this one is for the bfloat16 kernels
    taking a wrong path."""
    errs = []
    for (rid, p), row in got.items():
        err = float((row.double().cpu() - expected[rid][p]).abs().max()) / float(expected[rid].abs().max())
        assert math.isfinite(err) and err <= cap, f"{what}: request {rid} position {p}: error {err:.3e} of the logit scale"
        errs.append(err)
    bad = sum(e > tol for e in errs)
    assert errs and bad <= over * len(errs), f"{what}: {bad} of {len(errs)} rows beyond {tol:.1e} of the logit scale"
    return max(errs)


def layer_runs(raw):
    return len(plain.run_order(raw))


def run_family(name, family, tmp_path, device, dtype, tol):
    raw, cfg, weights = make(name, torch.float32 if dtype == "float32" else torch.bfloat16, sharp=dtype == "float32")
    prompts = trace_util.random_prompts(raw["vocab"], LENGTHS, seed=17)
    steps = FAMILIES[family](prompts)
    peak = trace_util.live_token_peak(steps)
    pages = peak // 16 + 1 + 4
    runner = any_runner(device, cfg, weights, dtype, num_pages=pages, max_rows=4, max_step_tokens=max(64, peak),
                        max_model_len=(pages - 1) * 16, num_state_slots=5)
    if family == "mixed":
        assert peak < sum(-(-n // 64) * 64 for n in LENGTHS), "the pool must be smaller than all requests together"
    replay(runner, trace_util.to_lines(steps), str(tmp_path), lambda _: None, max_live=4)
    runner.cache.check()
    assert not runner.cache.live
    got = trace_util.read_outputs(str(tmp_path), steps, raw["vocab"])
    check = trace_util.compare if dtype == "float32" else compare_most
    return check(got, expected_logits(raw, weights, prompts), tol, f"vezodra {name}/{family}/{dtype}")


# ------------------------------------------------------------------------------------------- configuration
def test_config_round_trip_registry_and_the_size_read_from_a_tensor(tmp_path):
    from safetensors.torch import save_file
    raw, cfg, weights = make("A")
    assert VezodraConfig.from_dict(cfg.to_dict()) == cfg
    assert cfg.run_order() == [0, 1, 2, 1, 2, 3] == plain.run_order(raw)
    # a config.json that does not say the decay's inner size: it is the checkpoint tensor's first dim
    bare = json.loads(json.dumps(raw))
    for entry in bare["layers"]:
        if entry["type"] == "parallel":
            del entry["mixer"]["right"]["rank"]
    (tmp_path / "config.json").write_text(json.dumps(bare))
    with pytest.raises(ConfigError):
        VezodraConfig.from_dict(bare)
    save_file({k: v.contiguous() for k, v in weights.items()}, str(tmp_path / "model.safetensors"))
    loaded, arch = load_model_config(str(tmp_path))
    assert loaded == cfg and arch.name == "Vezodra"
    assert cfg.layers[0].mixer.right.rank == 8 and cfg.layers[2].mixer.right.rank == 5 and cfg.layers[2].mlp is None
    assert cfg.layers[0].mixer.left.rot.factor == 4.0 and cfg.layers[2].mixer.left.rot.factor == 1.0


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][1]["mixer"].update(vdim=24),                      # values are the keys: one size
    lambda c: c["layers"][1]["mixer"].update(kv_heads=4),                   # 6 query heads on 4
    lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18),        # more than a head has
    lambda c: c["loop"].update(stop=5),
    lambda c: c["layers"][0].update(type="conv"),
    lambda c: c["layers"][0]["mlp"].update(kind="moe"),
])
def test_config_refuses_what_cannot_be_computed(bad):
    raw = json.loads(json.dumps(CFG_A))
    bad(raw)
    with pytest.raises(ConfigError):
        VezodraConfig.from_dict(raw)


def test_model_structure():
    _, cfg, weights = make("A")
    runner = host_runner(cfg, weights)
    model = runner.model
    # six layer runs, each with a cache entry of its own (the looped layers twice); one page group per distinct window
    assert [c.layer for c in model.spec.schedule] == [0, 1, 2, 1, 2, 3] and sorted(model.cache_entries) == list(range(6))
    assert model.page_groups == [20, None, 33]
    assert not model.padding_safe
    assert "l2.mlp.up" not in weights and "l2.norm2" not in weights and "l1.mix.v" not in weights
    t = runner.storage.entries[0].tensors
    assert t["mixer.left.k"].shape[-1] == 32 and t["mixer.right.state"].shape[1:] == (2, 16, 16) and t["conv.tail"].shape[1:] == (3, 64)
    assert runner.storage.entries[1].tensors["mixer.k"].data_ptr() != runner.storage.entries[3].tensors["mixer.k"].data_ptr()


# ------------------------------------------------------------------------------------- mechanisms, one by one
def one_layer(kind, mixer, ff, width=32, vocab=50, taps=3):
    raw = dict(architecture="Vezodra", vocab=vocab, width=width, norm=dict(eps=1e-5), layers=[layer(kind, mixer, ff)])
    if taps is not None:
        raw["canon"] = dict(taps=taps)
    return raw


@pytest.mark.parametrize("raw", [
    one_layer("attention", sink_att(4, 2, 16), None, taps=None),
    one_layer("attention", sink_att(1, 1, 24, dims=8, base=3.0), None, taps=None),
    one_layer("parallel", par(4, 2, 8, 8, 5, 2, 8, 4), None, taps=None),
    one_layer("parallel", par(2, 2, 16, 8, 100, 1, 16, 2, dims=4, factor=8.0), None, taps=None),
    one_layer("attention", sink_att(2, 1, 16), None, taps=5),
    one_layer("attention", sink_att(2, 1, 16), None, taps=1),
    one_layer("attention", sink_att(2, 1, 16), 40, taps=2),
], ids=["sink-attention", "sink-attention-one-head", "parallel", "parallel-wide-window", "conv-5", "conv-1", "dense"])
def test_each_mechanism_alone_on_the_host(raw):
    cfg = VezodraConfig.from_dict(raw)
    weights = shaped(cfg, 1)
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


def test_rotation_layouts():
    x = torch.randn(6, 2, 12, dtype=torch.float64)
    pos = torch.arange(6)
    for layout, first, second in (("interleaved", slice(0, 8, 2), slice(1, 8, 2)), ("half", slice(0, 4), slice(4, 8))):
        rot = dict(base=100.0, dims=8)
        y = plain.rotate(x, pos, rot, layout)
        assert torch.equal(y[..., 8:], x[..., 8:]) and torch.allclose(y[0], x[0])
        assert torch.allclose(y[..., first] ** 2 + y[..., second] ** 2, x[..., first] ** 2 + x[..., second] ** 2)
        a, b = (0, 1) if layout == "interleaved" else (0, 4)      # pair 0 turns one radian a position
        assert torch.allclose(y[3, 0, a], x[3, 0, a] * math.cos(3.0) - x[3, 0, b] * math.sin(3.0))
        assert torch.allclose(y[3, 0, b], x[3, 0, b] * math.cos(3.0) + x[3, 0, a] * math.sin(3.0))
        # linear scaling: position 6 with factor 2 is position 3 without
        z = plain.rotate(x[:1].expand(6, 2, 12), torch.full((6,), 6), dict(rot, scaling=dict(factor=2.0)), layout)
        assert torch.allclose(z[0], plain.rotate(x[:1], torch.tensor([3]), rot, layout)[0])
        q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
        dots = [float((plain.rotate(q, torch.tensor([p + 4]), rot, layout) * plain.rotate(k, torch.tensor([p]), rot, layout)).sum())
                for p in (0, 9, 300)]
        assert max(dots) - min(dots) < 1e-9


def test_plain_mechanisms_by_hand():
    # softmax with a sink of score 0: one key of score s gets exp(s) / (1 + exp(s))
    q, k = torch.tensor([[[2.0]]], dtype=torch.float64), torch.tensor([[[1.5]]], dtype=torch.float64)
    o = plain.softmax_attention(q, k, torch.tensor([[[7.0]]], dtype=torch.float64), 0.5, sink=0.0)
    assert torch.allclose(o, torch.tensor(7.0 * math.exp(1.5) / (1 + math.exp(1.5)), dtype=torch.float64))
    # window of 2: query 2 sees keys 1 and 2 only
    q3 = torch.zeros(3, 1, 1, dtype=torch.float64)
    v3 = torch.tensor([[[1.0]], [[10.0]], [[100.0]]], dtype=torch.float64)
    assert torch.allclose(plain.softmax_attention(q3, q3, v3, 1.0, window=2)[:, 0, 0], torch.tensor([1.0, 5.5, 55.0], dtype=torch.float64))
    # convolution: taps [a, b] give h[t] + a h[t - 1] + b h[t]
    h = torch.tensor([[1.0], [2.0], [4.0]], dtype=torch.float64)
    assert torch.allclose(plain.input_conv(h, torch.tensor([[0.5, 0.25]], dtype=torch.float64))[:, 0],
                          torch.tensor([1.25, 2.0 + 0.5 + 0.5, 4.0 + 1.0 + 1.0], dtype=torch.float64))
    # delta rule, one head of two channels, two tokens: the second token removes along its unit key from the old state
    z = torch.zeros(2, 2)
    w = {"p.r": torch.eye(2), "p.k": torch.eye(2), "p.v": torch.tensor([[0.0, 1.0], [1.0, 0.0]]), "p.g": z, "p.a": z, "p.a.b": torch.zeros(2),
         "p.w1": torch.zeros(1, 2), "p.w2": torch.zeros(2, 1), "p.w0": torch.zeros(2), "p.norm": torch.ones(2), "p.o": torch.eye(2)}
    w = {n: t.double() for n, t in w.items()}
    hh = torch.tensor([[3.0, 0.0], [3.0, 4.0]], dtype=torch.float64)
    out = plain.delta_rule(w, "p.", dict(heads=1, dim=2), hh, 0.0)
    decay = math.exp(-math.exp(-0.5) * 0.5)
    S0 = torch.tensor([[0.0, 9.0], [0.0, 0.0]], dtype=torch.float64)                        # k v^T of token 0
    u = torch.tensor([0.6, 0.8], dtype=torch.float64)
    S1 = decay * S0 - (0.5 * u)[:, None] * (u @ S0)[None, :] + torch.outer(hh[1], torch.tensor([4.0, 3.0], dtype=torch.float64))
    o0, o1 = S0.T @ hh[0], S1.T @ hh[1]
    want = torch.stack([o0 / o0.pow(2).mean().sqrt(), o1 / o1.pow(2).mean().sqrt()]) * 0.5
    assert torch.allclose(out, want, atol=1e-6)


# ------------------------------------------------------------------------------------------ whole models, host
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_on_the_host(name, family, tmp_path):
    run_family(name, family, tmp_path, "cpu", "float32", F32_TOL)


def edge_runs(device):
    """Windows and the sink, where it shows.  One layer of each mixer kind, scores spread wide.  The engine must follow
    the plain implementation at every position of a prompt portion and of tokens decoded one by one, across the
    window's edge; and the test means something: a window one key longer or shorter, or no sink, moves the plain
    implementation's own logits at those positions by far more than the tolerance."""
    for window in (1, 7, 16, 17, 40):
        raw = one_layer("parallel", par(2, 1, 16, 16, window, 1, 8, 2), None, width=32, vocab=60, taps=2)
        cfg = VezodraConfig.from_dict(raw)
        w = shaped(cfg, 5)
        for n in ("l0.mix.left.q", "l0.mix.left.k"):
            w[n].mul_(3.0)
        toks = trace_util.random_prompts(60, [100], seed=window)["r0"]
        want = plain.forward(raw, w, toks)
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:50], "want": list(range(50))}], "end": []}]
        steps += [{"step": 1 + i, "entries": [{"id": "x", "tokens": toks[50 + i:51 + i], "want": [0]}], "end": []} for i in range(50)]
        steps[-1]["end"] = ["x"]
        runner = any_runner(device, cfg, w, num_pages=9, max_rows=2, max_step_tokens=64, max_model_len=128, num_state_slots=3)
        got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, steps).items()}
        trace_util.compare(got, {"x": want}, F32_TOL, f"window {window}")
        runner.cache.check()
        for other in (window - 1, window + 1):
            if other < 1:
                continue
            varied = json.loads(json.dumps(raw))
            varied["layers"][0]["mixer"]["left"]["mask"]["size"] = other
            moved = (plain.forward(varied, w, toks) - want).abs().amax(-1) / float(want.abs().max())
            edge = max(window, other)                      # the first position whose visible keys differ
            if edge < 100:
                assert float(moved[edge:].min()) > 0 and float(moved[edge:60].max() if edge < 60 else moved[edge:].max()) > 30 * F32_TOL, \
                    f"a window of {other} instead of {window} must show"
            assert float(moved[:min(window, other)].max()) == 0.0
    raw = one_layer("attention", sink_att(2, 1, 16), None, width=32, vocab=60, taps=2)
    cfg = VezodraConfig.from_dict(raw)
    w = shaped(cfg, 6)
    toks = trace_util.random_prompts(60, [60], seed=3)["r0"]
    want = plain.forward(raw, w, toks)
    runner = any_runner(device, cfg, w, num_pages=6, max_rows=2, max_step_tokens=64, max_model_len=80, num_state_slots=3)
    got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, trace_util.decode_tail({"x": toks}, 30)).items()}
    trace_util.compare(got, {"x": want}, F32_TOL, "sink")
    moved = (plain.forward(raw, w, toks, sink=None) - want).abs().amax(-1) / float(want.abs().max())
    assert float(moved[0]) > 30 * F32_TOL and float(moved[:8].min()) > 3 * F32_TOL and float(moved[30:].max()) > 3 * F32_TOL, \
        "leaving the sink out must show, at the first position above all (one key, and the sink beside it)"


def test_window_edges_and_the_sink():
    edge_runs("cpu")


@pytest.mark.gpu
def test_window_edges_and_the_sink_gpu():
    edge_runs("cuda")


def far_key_runs(device):
    """One token is made to stand out (an embedding no other position has): far back, at the last slot of a page and the
    first of the next, and at the very first position.  The engine must follow the plain implementation through 13
    pages, a portion of 150 tokens and 50 single tokens; and the token must matter to the last position."""
    raw, cfg, weights = make("A")
    toks = [t if t != 210 else 0 for t in trace_util.random_prompts(raw["vocab"], [200], seed=9)["r0"]]
    for needle in (37, 15, 16, 0):
        tokens = list(toks)
        tokens[needle] = 210                                   # a token no other position holds
        assert tokens.count(210) == 1
        w = {k: v.clone() for k, v in weights.items()}
        w["embed"][210] = 3.0 * w["embed"][210].sign()
        want = plain.forward(raw, w, tokens)
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:150], "want": [149]}], "end": []}]
        steps += [{"step": 1 + i, "entries": [{"id": "x", "tokens": tokens[150 + i:151 + i], "want": [0]}], "end": []}
                  for i in range(50)]
        steps[-1]["end"] = ["x"]
        runner = any_runner(device, cfg, w, num_pages=16, max_rows=2, max_step_tokens=160, max_model_len=240, num_state_slots=3)
        got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, steps).items()}
        trace_util.compare(got, {"x": want}, F32_TOL, f"needle at {needle}")
        other = list(tokens)
        other[needle] = toks[needle]
        moved = float((plain.forward(raw, w, other)[-1] - want[-1]).abs().max()) / float(want.abs().max())
        assert moved > 1e-3, "the far token must matter to the last position for this test to mean anything"


def test_a_far_key_and_the_first_token_are_seen():
    far_key_runs("cpu")


@pytest.mark.gpu
def test_a_far_key_and_the_first_token_are_seen_gpu():
    far_key_runs("cuda")


def test_state_slots_and_pages_are_used_again():
    """Five requests, one after another, through a runner with one usable state slot and pages for one request:
    each must start from zero state and an empty convolution, and see no key of the one before."""
    raw, cfg, weights = make("B")
    prompts = trace_util.random_prompts(raw["vocab"], [40, 33, 40, 7, 25], seed=3)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                         num_pages=4, max_rows=1, max_step_tokens=64, max_model_len=48, num_state_slots=2)
    got = trace_util.run_on_runner(runner, trace_util.portions(prompts, sizes=(5, 2, 9)))
    trace_util.compare(got, expected_logits(raw, weights, prompts), F32_TOL, "reuse")
    for entry in runner.storage.entries.values():
        for name, t in entry.tensors.items():
            if name.endswith(("state", "tail")):
                t.fill_(3.0)
    rc = runner.cache.open("fresh")
    for entry in runner.storage.entries.values():
        for name, t in entry.tensors.items():
            if name.endswith(("state", "tail")):
                assert float(t[rc.state_slot].abs().max()) == 0.0 and float(t[0].abs().max()) == 3.0
    runner.cache.close(rc)


def test_batched_rows_equal_rows_alone():
    raw, cfg, weights = make("A")
    prompts = trace_util.random_prompts(raw["vocab"], [21, 5, 34], seed=12)
    alone = {}
    for rid, toks in prompts.items():
        runner = host_runner(cfg, weights)
        alone.update(trace_util.run_on_runner(runner, trace_util.whole({rid: toks})))
    runner = host_runner(cfg, weights)
    ents = [{"id": rid, "tokens": toks[:-1], "want": list(range(len(toks) - 1))} for rid, toks in prompts.items()]
    last = [{"id": rid, "tokens": toks[-1:], "want": [0]} for rid, toks in prompts.items()]
    got = trace_util.run_on_runner(runner, [{"step": 0, "entries": ents, "end": []}, {"step": 1, "entries": last, "end": list(prompts)}])
    for key, row in alone.items():
        assert float((got[key] - row).abs().max()) < 1e-5 * float(row.abs().max())


def generate(name, device, dtype, **engine):
    from mini_inference_engine_amd import LLMEngine, SamplingParams
    raw, cfg, weights = make(name, torch.float32 if dtype == "float32" else torch.bfloat16, sharp=dtype == "float32")
    prompts = list(trace_util.random_prompts(raw["vocab"], [9, 30, 2, 17, 23], seed=4).values())
    ecfg = EngineConfig(num_blocks=24, max_num_seqs=3, max_num_batched_tokens=32, max_model_len=128, **engine)
    kw = dict(device="cpu", backend=TorchBackend(torch.float32)) if device == "cpu" else {}
    eng = LLMEngine(cfg, ecfg, dtype=dtype, verbose=False, weights=weights, **kw)
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    wf = {k: v.float() for k, v in weights.items()}
    missed = 0
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        assert len(out.output_ids) == 12
        for tok in out.output_ids:
            logits = plain.forward(raw, wf, ids)[-1]
            slack = (F32_TOL if dtype == "float32" else BF16_TOL_PER_LAYER * layer_runs(raw)) * float(logits.abs().max())
            missed += float(logits.max() - logits[tok]) > slack
            ids.append(tok)
    assert missed == 0, f"{missed} of 60 tokens are not the plain implementation's choice"
    return eng


def test_greedy_generation_through_the_scheduler_on_the_host():
    eng = generate("A", "cpu", "float32", use_hip_graphs=False)
    assert eng.num_steps > 12, "five requests under three slots and a budget of 32 tokens come in several waves"


# ----------------------------------------------------------------------------------------------- GPU: kernels
def _rand(shape, dtype, g, scale=1.0):
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


class FakeStep:
    def __init__(self, lens, slots):
        import numpy as np
        rs = np.concatenate([[0], np.cumsum(lens)]).astype("int64")
        self.num_rows, self.num_tokens = len(lens), int(rs[-1])
        self.host = {"row_start": rs, "state_slots": np.asarray(slots)}
        self.row_start = torch.tensor(rs, dtype=torch.int32).cuda()
        self.state_slots = torch.tensor(slots, dtype=torch.int32).cuda()
        self.token_row = torch.repeat_interleave(torch.arange(len(lens)), torch.tensor(lens)).to(torch.int32).cuda()


@pytest.fixture(scope="module")
def hip():
    from mini_inference_engine_amd.kernels.hip_backend import HipBackend
    return {torch.float32: HipBackend(torch.float32), torch.bfloat16: HipBackend(torch.bfloat16)}


def close(a, b, tol, what):
    err = float((a.double().cpu() - b.double().cpu()).abs().max()) / max(1e-9, float(b.double().abs().max()))
    assert err <= tol, f"{what}: {err:.3e} of the scale, tolerance {tol:.1e}"


TOL = {torch.float32: 3e-6, torch.bfloat16: 1e-2}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_and_joined_norm_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(0)
    for (C, K, lens, slots) in ((64, 4, [1, 1, 9, 2, 300], [4, 1, 3, 5, 2]), (70, 1, [5, 1], [1, 2]), (520, 6, [3, 2, 40], [2, 3, 1]),
                                (48, 2, [1], [3])):
        step = FakeStep(lens, slots)
        h = _rand((step.num_tokens, C), torch.float32, g)
        taps = _rand((C, K), torch.float32, g, 0.5)
        tail = _rand((6, max(1, K - 1), C), torch.float32, g)
        want_tail = tail.cpu().clone()
        want = ref.ref_residual_conv(h.cpu(), taps.cpu(), want_tail, step.host["row_start"], step.host["state_slots"], dtype)
        got = ops.residual_conv(h, taps, tail, step)
        assert got.dtype == dtype
        close(got, want, TOL[dtype], "conv")
        if K > 1:
            assert torch.equal(tail.cpu(), want_tail), "the tail holds the last inputs as they were given"
        # the same behind two norms of one stream, in one pass
        stream, w1, w2 = _rand((step.num_tokens, C), torch.float32, g, 2.0), _rand((C,), torch.float32, g) + 1, _rand((C,), torch.float32, g) + 1
        tail2 = _rand((6, max(1, K - 1), C), torch.float32, g)
        want_tail = tail2.cpu().clone()
        hn = ref.ref_add_rmsnorm(None, stream.cpu(), w1.cpu(), 1e-5, torch.float32)
        want_x = ref.ref_residual_conv(hn, taps.cpu(), want_tail, step.host["row_start"], step.host["state_slots"], dtype)
        for second in (w2, None):
            tl = tail2.clone()
            x, y = ops.norm_pair_conv(stream, w1, second, 1e-5, taps, tl, step)
            close(x, want_x, TOL[dtype], "norms and conv in one pass")
            close(tl, want_tail, 3e-6, "tail behind the norm")
            assert (y is None) == (second is None)
            if y is not None:
                close(y, ref.ref_add_rmsnorm(None, stream.cpu(), w2.cpu(), 1e-5, dtype), TOL[dtype], "second norm")
    for T, W in ((1, 64), (5, 70), (3, 4100)):
        stream = _rand((T, W), torch.float32, g)
        ys = [_rand((T, W), torch.float32, g, 3.0), _rand((T, W), torch.float32, g, 0.2)]
        ws = [_rand((W,), torch.float32, g) + 1, _rand((W,), torch.float32, g) + 1]
        for n in (2, 1):
            want = ref.ref_normed_sum_add(stream.clone(), ys[:n], ws[:n], 1e-5, 0.5)
            got = ops.normed_sum_add(stream.clone(), ys[:n], ws[:n], 1e-5, 0.5)
            close(got, want, 2e-6, "joined norms")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_preparation_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(2)
    cases = ((4, 2, 16, 24, 32, 4, "half", True, False, True, 37), (6, 3, 32, 32, 32, 8, "interleaved", False, True, False, 3),
             (3, 3, 10, 14, 16, 3, "half", True, True, True, 130), (5, 1, 22, 22, 32, 5, "interleaved", False, True, False, 300),
             (2, 1, 96, 96, 96, 48, "interleaved", False, False, False, 20), (2, 2, 16, 16, 16, 0, "half", True, False, True, 9))
    for (Hq, Hkv, dim, vdim, P, nf, layout, normed, temp, own_v, T) in cases:
        inv_freq = (50.0 ** -(torch.arange(nf).double() * 2 / max(1, 2 * nf))).float().cuda() if nf else None
        positions = torch.randint(0, 5000, (T,), generator=g).to(torch.int32).cuda()
        q_col, k_col = 3, 3 + Hq * dim + 2
        v_col = k_col + Hkv * dim + 1 if own_v else None
        sums = _rand((T, k_col + Hkv * dim + 1 + Hkv * vdim + 5), torch.float32, g, 2.0)
        qn = (_rand((Hq * dim,), torch.float32, g) + 1) if normed else None
        kn = (_rand((Hkv * dim,), torch.float32, g) + 1) if normed else None
        hs = (torch.rand(Hq, generator=g) + 0.5).cuda() if temp else None
        pages, page = T // 16 + 3, 16
        slots = torch.randperm((pages - 1) * page, generator=g)[:T].to(torch.int32).cuda() + page
        kc = torch.full((pages, Hkv, page, P), 7.0, dtype=dtype).cuda()
        vc = torch.full((pages, Hkv, P, page), 7.0, dtype=dtype).cuda()
        kw, vw = kc.clone(), vc.clone()
        if not own_v and vdim != dim:
            continue
        want = ref.ref_qkv_finish(sums, q_col, k_col, v_col, Hq, Hkv, dim, vdim, P, positions, inv_freq, layout, kw, vw, slots,
                                  qn, kn, 1e-5, hs, dtype)
        got = ops.qkv_finish(sums, q_col, k_col, v_col, Hq, Hkv, dim, vdim, P, positions, inv_freq, layout, kc, vc, slots,
                             q_norm=qn, k_norm=kn, eps=1e-5, q_head_scale=hs)
        close(got, want, TOL[dtype], f"queries {layout}")
        close(kc, kw, TOL[dtype], f"keys {layout}")
        close(vc, vw, TOL[dtype], "values")
        assert torch.equal(kc[0], kw[0]), "the scratch page was not written"
        assert float(got.view(T, Hq, P)[..., dim:].abs().max() if P > dim else 0.0) == 0.0
        o = _rand((T, Hq * P), dtype, g)
        gate = _rand((T, 7 + Hq), torch.float32, g, 2.0)
        want_o = ref.ref_head_gate(o, gate, 7, Hq, P)
        assert ops.head_gate_(o, gate, 7, Hq, P) is o
        close(o, want_o, TOL[dtype], "head gate")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_delta_rule_kernel(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(3)
    for (H, d, rank, lens, slots) in ((2, 16, 8, [1, 1, 9, 2, 70], [4, 1, 3, 5, 2]), (1, 32, 3, [5, 1], [1, 2]), (5, 12, 5, [3, 2, 40], [2, 3, 1]),
                                      (3, 8, 5, [33], [5]), (2, 64, 16, [1, 20], [1, 2]), (1, 128, 4, [6], [3]), (1, 144, 4, [3, 1], [3, 1]),
                                      # rows beyond 64 tokens: the bfloat16 mode runs them in chunks of 64 side by side
                                      (2, 64, 8, [1, 64, 65, 300, 128], [5, 4, 3, 2, 1]), (3, 24, 4, [129, 2], [1, 2]), (1, 80, 4, [70], [2]),
                                      # inner sizes beyond what the prepare kernel keeps in registers, and no multiple of 4; the widest heads
                                      (2, 16, 70, [3, 1, 20], [1, 2, 3]), (1, 32, 128, [2, 90], [4, 5]), (1, 200, 6, [5, 1, 66], [1, 2, 3]), (1, 128, 6, [130, 3], [1, 2])):
        step = FakeStep(lens, slots)
        T, n = step.num_tokens, H * d
        cols = dict(r=2, k=2 + n, v=3 + 2 * n, g=3 + 3 * n, a=4 + 4 * n, w=4 + 5 * n)
        sums = _rand((T, 4 + 5 * n + rank + 3), torch.float32, g)
        w_decay, db, rb = _rand((n, rank), torch.float32, g, 1.5), _rand((n,), torch.float32, g), _rand((n,), torch.float32, g)
        nw = _rand((n,), torch.float32, g) + 1
        state = _rand((6, H, d, d), torch.float32, g, 0.5)
        st_w = state.cpu().clone()
        want = ref.ref_delta_rule(sums.cpu(), cols, H, d, w_decay.cpu(), db.cpu(), 0.6, rb.cpu(), nw.cpu(), 1e-5, st_w,
                                  step.host["row_start"], step.host["state_slots"], dtype)
        got = ops.delta_rule(sums, cols, H, d, w_decay, db, 0.6, rb, nw, 1e-5, state, step)
        close(got, want, 3e-5 if dtype == torch.float32 else 1e-2, f"delta rule {H} x {d}")
        close(state, st_w, 3e-5, "state")
        assert torch.equal(state[0].cpu(), st_w[0]), "slots of no row are left alone"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_kernels_with_a_sink(hip, dtype):
    """The three attention kernels (32-bit, matrix-core decode with and without splits, matrix-core prompt portions)
    with one more term in the denominator; scores spread so that the term matters (and so that it is sometimes the
    largest)."""
    from test_kernels_gpu import paged_setup
    ops = hip[dtype]
    for (Hq, Hkv, D, ctx, lens, window, sink) in ((4, 2, 32, [3, 18, 1], [1, 1, 1], None, -0.5), (6, 3, 96, [6, 140, 7], [1, 40, 7], None, 0.0),
                                                  (2, 1, 64, [2001, 901], [1, 1], None, 8.0), (4, 4, 16, [33, 66], [33, 2], 20, 3.0)):
        q, kc, vc, group, step = paged_setup(ctx, lens, Hq, Hkv, D, 16, dtype)
        scale = 2.0 / math.sqrt(D)
        expect = ref.ref_paged_attention(q, Hq, Hkv, D, kc, vc, group.block_tables, step.token_row, step.positions, scale, window,
                                         torch.float64, sink=sink)
        plain_softmax = ref.ref_paged_attention(q, Hq, Hkv, D, kc, vc, group.block_tables, step.token_row, step.positions, scale,
                                                window, torch.float64)
        assert float((expect - plain_softmax).abs().max()) > 0.05 * float(expect.abs().max()), "the sink must matter here"
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        close(ops.paged_attention(q, Hq, Hkv, D, kc, vc, group, step, scale, window, sink=sink), expect, tol, "sink")
        close(ops.paged_attention(q, Hq, Hkv, D, kc, vc, group, step, scale, window, sink=sink, force_generic=True), expect, tol, "sink, 32-bit kernel")
        if all(n == 1 for n in lens):
            for splits in (1, 3):
                close(ops.paged_attention(q, Hq, Hkv, D, kc, vc, group, step, scale, window, sink=sink, num_splits=splits), expect, tol,
                      f"sink, {splits} splits")


# ------------------------------------------------------------------------------------------ GPU: whole models
@pytest.mark.gpu
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_float32_gpu(name, family, tmp_path):
    run_family(name, family, tmp_path, "cuda", "float32", F32_TOL)


@pytest.mark.gpu
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_bfloat16_gpu(name, family, tmp_path):
    run_family(name, family, tmp_path, "cuda", "bfloat16", BF16_TOL_PER_LAYER * layer_runs(CONFIGS[name][0]))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_gpu(dtype):
    eng = generate("A", "cuda", dtype)
    assert eng.num_graph_steps > 0, "decode steps of this model run as captured graphs too"


@pytest.mark.gpu
def test_long_decoding_gpu():
    """160 tokens one by one after a short prompt, float32: state, convolution tails, windows and cache carried through
    ten pages, the windows' passed pages given back on the way."""
    raw, cfg, weights = make("A")
    toks = trace_util.random_prompts(raw["vocab"], [170], seed=6)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", num_pages=14, max_rows=2, max_step_tokens=64,
                         max_model_len=208, num_state_slots=3)
    runner.cache.keep_log = True
    got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, trace_util.decode_tail(toks, 160)).items()}
    trace_util.compare(got, expected_logits(raw, weights, toks), F32_TOL, "long decoding")
    assert any(g != 1 for g, _ in runner.cache.released_log[:5]), "a windowed group gave pages back while the request ran"


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
    run(cli + ["random-model", "--shape", "vezodra-tiny", "--seed", "3", "--dtype", "float32", "--out", folder])
    raw = json.load(open(os.path.join(folder, "config.json")))
    weights = load_file(os.path.join(folder, "model.safetensors"))
    assert raw["architecture"] == "Vezodra" and len(raw["layers"]) == 3 and raw["loop"]["times"] == 2
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
