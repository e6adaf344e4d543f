"""Zifelorn through the engine against the plain implementation (tests/plain_zifelorn.py).

Configurations are made here, with sizes that differ from one another wherever the design lets them (plain
and rotated head dims, value size, both latent ranks, channels, blocks, taps, experts, top; a layer without
a feed-forward; rot.dims below rot_dim; kv_rank + rot_dim no multiple of 16; top = 1 and top = experts).
Host tests run the engine's own parts, cache and step function on the CPU with the torch operations of
tests/torch_backend.py; GPU tests run the HIP kernels, each kernel against the torch operation of the same
name and the whole model in the four trace families, in float32 (tight) and bfloat16.
"""
import json
import math

import pytest
import torch

import plain_zifelorn as plain
import trace_util
from torch_backend import TorchBackend
import torch_backend as ref

from mini_inference_engine_amd.config import EngineConfig, ZifelornConfig, load_model_config
from mini_inference_engine_amd.engine.batch import StepRow
from mini_inference_engine_amd.engine.runner import ModelRunner
from mini_inference_engine_amd.replay.trace import replay
from mini_inference_engine_amd.weights import random_tensors


def att(heads, dim, rot_dim, vdim, kv_rank, q_rank, dims=None, base=1000.0, scale=None, kv_from=None):
    d = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank,
             scale=scale if scale is not None else (dim + rot_dim) ** -0.5, rot=dict(base=base, dims=dims or rot_dim))
    if kv_from is not None:
        d["kv_from"] = kv_from
    return d


def layer(kind, mixer, mlp):
    return dict(type=kind, mixer=mixer, mlp=mlp)


def moe(experts, top, ff):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


A1 = att(3, 16, 8, 24, 40, 48)
A2 = att(2, 8, 16, 16, 24, 16, dims=8, base=77.0, scale=0.31)          # turns half of the rotated part; padded 40 -> 48
CFG_A = dict(architecture="Zifelorn", vocab=211, width=64, embedding=dict(scale=5.5), norm=dict(eps=1e-5), logit_scale=0.7,
             layers=[layer("latent_attention", A1, dict(kind="dense", ff=112)),
                     layer("latent_attention", A1, moe(5, 2, 48)),
                     layer("rglru", dict(width=96, blocks=3, conv=4), dict(kind="dense", ff=80)),
                     layer("latent_attention", dict(A1, kv_from=1), moe(5, 2, 48)),
                     layer("rglru", dict(width=64, blocks=1, conv=2), None),
                     layer("latent_attention", A2, dict(kind="dense", ff=72)),
                     layer("latent_attention", dict(A1, heads=5, vdim=8, q_rank=24, kv_from=1), moe(3, 3, 40))])
B1 = att(4, 24, 4, 12, 28, 20, base=50.0)
CFG_B = dict(architecture="Zifelorn", vocab=150, width=48, embedding=dict(scale=1.0), norm=dict(eps=1e-3), logit_scale=1.0,
             layers=[layer("rglru", dict(width=40, blocks=5, conv=1), moe(4, 1, 24)),
                     layer("latent_attention", B1, None),
                     layer("latent_attention", dict(B1, kv_from=1), moe(6, 4, 16)),
                     layer("rglru", dict(width=48, blocks=2, conv=6), dict(kind="dense", ff=64))])
# sizes the kernels' vector paths do not like: nothing a multiple of 8, an odd vocabulary
C1 = att(3, 10, 6, 14, 22, 18, base=300.0)
CFG_C = dict(architecture="Zifelorn", vocab=101, width=70, embedding=dict(scale=3.0), norm=dict(eps=1e-6), logit_scale=1.3,
             layers=[layer("latent_attention", C1, moe(3, 2, 26)),
                     layer("rglru", dict(width=30, blocks=3, conv=3), dict(kind="dense", ff=50)),
                     layer("latent_attention", dict(C1, kv_from=0), dict(kind="dense", ff=34))])
CONFIGS = {"A": (CFG_A, 3), "B": (CFG_B, 4), "C": (CFG_C, 6)}


def make(name, dtype=torch.float32, sharp=True):
    """(config dict, typed config, weights): random weights shaped so that faults show: products keep the scale of
    their input, query and key projections are doubled (scores spread over several units: which keys are seen
    matters), routers are decisive, decays cover slow and fast channels, biases are not zero.  ``sharp`` False
    leaves queries, keys and routers at unit scale: the bfloat16 runs use it, because spread scores amplify the
    rounding of 8-bit values as much as they amplify faults."""
    raw, seed = CONFIGS[name]
    cfg = ZifelornConfig.from_dict(raw)
    w = random_tensors(cfg, seed, torch.float32, std=1.0)
    g = torch.Generator().manual_seed(seed + 100)
    for k, v in w.items():
        if v.dim() >= 2 and not k.endswith("conv"):
            v.mul_(v.shape[-1] ** -0.5)
        if k.endswith((".uq", ".dkv")) and sharp:
            v.mul_(2.0)
        if k.endswith(".router") and sharp:
            v.mul_(4.0)
        if k.endswith((".b", ".lam")) or "norm" in k:
            v.copy_(torch.randn(v.shape, generator=g) * (0.5 if k.endswith(".b") else 1.0) + (1.0 if "norm" in k else 0.0))
        if k.endswith(".conv"):
            v.mul_(0.5)
    w["embed"].mul_(0.3)
    w = {k: v.to(dtype) for k, v in w.items()}
    return raw, cfg, w


def expected_logits(raw, weights, prompts):
    wf = {k: v.float() for k, v in weights.items()}
    return {rid: plain.forward(raw, wf, toks) for rid, toks in prompts.items()}


def host_runner(cfg, weights, pages=64, rows=8, tokens=256):
    return ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                       num_pages=pages, max_rows=rows, max_step_tokens=tokens, max_model_len=pages * 16)


# float32 against the float64 plain implementation: rounding, amplified by scores that are spread on purpose; a fault
# (a lost key, a stale state, a wrong expert) moves logits by a hundred times this or more
F32_TOL = 3e-4
# bfloat16: every layer rounds a handful of values to 8 bits, and the spread scores amplify that; measured 1.2e-2 of the
# logit scale a layer at the worst of some 50,000 logits
BF16_TOL_PER_LAYER = 1.5e-2

FAMILIES = {"whole": trace_util.whole, "decode_tail": lambda p: trace_util.decode_tail(p, 40),
            "portions": trace_util.portions, "mixed": lambda p: trace_util.mixed(p, 4, seed=5)}
LENGTHS = [3, 70, 1, 37, 90, 18, 49]


def compare_most(got, expected, tol, what, over=0.1, cap=1.0):
    """The bfloat16 comparison.  A token whose router logits nearly tie may choose another expert once values are
    rounded to 8 bits, and then its logits (and, weakly, those after it) differ by design, not by fault: at most
    ``over`` of the rows may exceed ``tol``, none may exceed ``cap`` of the logit scale or be other than finite.
    (The same model run on the CPU with the torch operations rounding to bfloat16 at the same places differs from
    the plain implementation by as much: 2e-2 of the logit scale at the median, 0.2 at the 97th percentile of rows
    for the seven-layer configuration.  The float32 runs are the sharp test; this one is for the bfloat16 kernels
    taking a wrong path.)"""
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
    return check(got, expected_logits(raw, weights, prompts), tol, f"zifelorn {name}/{family}/{dtype}")


# ------------------------------------------------------------------------------------------- configuration
def test_config_round_trip_and_registry(tmp_path):
    raw, cfg, _ = make("A")
    assert ZifelornConfig.from_dict(cfg.to_dict()) == cfg
    (tmp_path / "config.json").write_text(json.dumps(raw))
    loaded, arch = load_model_config(str(tmp_path))
    assert loaded == cfg and arch.name == "Zifelorn"
    assert cfg.layers[3].mixer.kv_from == 1 and cfg.layers[4].mlp is None and cfg.layers[5].mixer.rot.dims == 8


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][3]["mixer"].update(kv_from=5),                  # a later layer
    lambda c: c["layers"][3]["mixer"].update(kv_from=2),                  # not an attention layer
    lambda c: c["layers"][3]["mixer"].update(kv_rank=32),                 # another latent size than its source's
    lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
    lambda c: c["layers"][2]["mixer"].update(blocks=5),
    lambda c: c["layers"][0].update(type="conv"),
])
def test_config_refuses_what_cannot_be_computed(bad):
    from mini_inference_engine_amd.config import ConfigError
    raw = json.loads(json.dumps(CFG_A))
    bad(raw)
    with pytest.raises(ConfigError):
        ZifelornConfig.from_dict(raw)


def test_model_structure():
    _, cfg, weights = make("A")
    runner = host_runner(cfg, weights)
    model = runner.model
    # the two layers that borrow layer 1's latent own no cache; one page group; a layer without feed-forward has no second norm
    assert sorted(model.cache_entries) == [0, 1, 2, 4, 5] and model.page_groups == [None]
    assert [c.cache_of for c in model.spec.schedule] == [None, None, None, 1, None, None, 1]
    assert not model.padding_safe
    assert "l4.norm2" not in weights and "l3.mix.dkv" not in weights and "l5.mix.dkv" in weights
    k = runner.storage.entries[5].tensors["k"]
    assert k.shape[-1] == 48 and runner.storage.entries[1].tensors["k"].shape[-1] == 48


# ------------------------------------------------------------------------------------- mechanisms, one by one
def one_layer(mixer_kind, mixer, mlp, width=32, vocab=50):
    return dict(architecture="Zifelorn", vocab=vocab, width=width, embedding=dict(scale=2.0), norm=dict(eps=1e-5),
                logit_scale=1.0, layers=[layer(mixer_kind, mixer, mlp)])


@pytest.mark.parametrize("raw", [
    one_layer("latent_attention", att(2, 8, 4, 12, 20, 16), None),
    one_layer("latent_attention", att(1, 16, 2, 8, 10, 12, base=3.0), None),
    one_layer("rglru", dict(width=24, blocks=2, conv=3), None),
    one_layer("rglru", dict(width=16, blocks=4, conv=1), None),
    one_layer("rglru", dict(width=8, blocks=1, conv=2), dict(kind="dense", ff=40)),
    one_layer("rglru", dict(width=8, blocks=1, conv=2), moe(4, 2, 12)),
    one_layer("rglru", dict(width=8, blocks=1, conv=2), moe(3, 1, 12)),
], ids=["latent", "latent-one-head", "rglru", "rglru-no-conv", "dense", "experts-top2", "experts-top1"])
def test_each_mechanism_alone_on_the_host(raw):
    cfg = ZifelornConfig.from_dict(raw)
    weights = random_tensors(cfg, 1, torch.float32, std=0.3)
    for k in weights:
        if k.endswith(".b"):
            weights[k] = torch.linspace(-0.4, 0.6, weights[k].numel()).view(weights[k].shape)
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


def test_rotation_pairs_neighbours_and_scores_depend_on_distance_only():
    x = torch.randn(6, 2, 12, dtype=torch.float64)
    pos = torch.arange(6)
    y = plain.rotate_interleaved(x, pos, 100.0, 8)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.allclose(y[0], x[0])
    assert torch.allclose(y[..., 0:8:2] ** 2 + y[..., 1:8:2] ** 2, x[..., 0:8:2] ** 2 + x[..., 1:8:2] ** 2)
    # pair 0 turns one radian a position
    assert torch.allclose(y[3, 0, 0], x[3, 0, 0] * math.cos(3.0) - x[3, 0, 1] * math.sin(3.0))
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    dots = [float((plain.rotate_interleaved(q, torch.tensor([p + 4]), 100.0, 8) *
                   plain.rotate_interleaved(k, torch.tensor([p]), 100.0, 8)).sum()) for p in (0, 9, 300)]
    assert max(dots) - min(dots) < 1e-9


def test_plain_recurrence_and_router_by_hand():
    w = {"p.y": torch.zeros(2, 3), "p.y.b": torch.tensor([1.0, -2.0]), "p.x": torch.eye(2, 3), "p.x.b": torch.zeros(2),
         "p.conv": torch.tensor([[0.0, 1.0], [0.5, 0.5]]), "p.conv.b": torch.tensor([0.0, 1.0]),
         "p.ra": torch.zeros(1, 2, 2), "p.ra.b": torch.zeros(1, 2), "p.ri": torch.zeros(1, 2, 2), "p.ri.b": torch.zeros(1, 2),
         "p.lam": torch.tensor([0.0, 1.0]), "p.o": torch.eye(2)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.tensor([[2.0, 4.0, 0.0], [6.0, 8.0, 0.0]], dtype=torch.float64)
    out = plain.rglru(w, "p.", dict(width=2, blocks=1, conv=2), h)
    a = [math.exp(-8 * 0.5 * math.log(2.0)), math.exp(-8 * 0.5 * math.log(1 + math.e))]
    u = [[2.0, 0.5 * 4 + 1], [6.0, 0.5 * 4 + 0.5 * 8 + 1]]
    s0 = [math.sqrt(1 - a[c] ** 2) * 0.5 * u[0][c] for c in range(2)]
    s1 = [a[c] * s0[c] + math.sqrt(1 - a[c] ** 2) * 0.5 * u[1][c] for c in range(2)]
    y = [float(plain.gelu_tanh(torch.tensor(b, dtype=torch.float64))) for b in (1.0, -2.0)]
    assert torch.allclose(out, torch.tensor([[s0[0] * y[0], s0[1] * y[1]], [s1[0] * y[0], s1[1] * y[1]]], dtype=torch.float64))
    wr = {"m.router": torch.eye(3).double(), "m.router.b": torch.tensor([0.0, 0.0, 2.5]).double()}
    for e in range(3):
        wr[f"m.e{e}.up"] = torch.full((1, 3), float(e + 1)).double()
        wr[f"m.e{e}.down"] = torch.ones(3, 1).double()
    hh = torch.tensor([[1.0, 2.0, -1.0]], dtype=torch.float64)            # logits 1, 2, 1.5: experts 1 and 2
    p1, p2 = math.exp(2.0) / (math.exp(2.0) + math.exp(1.5)), math.exp(1.5) / (math.exp(2.0) + math.exp(1.5))
    out = plain.moe_ff(wr, "m.", dict(router=dict(experts=3, top=2)), hh)
    assert torch.allclose(out, torch.full((1, 3), p1 * (2 * 2.0) ** 2 + p2 * (3 * 2.0) ** 2, dtype=torch.float64))


def test_router_margins_of_the_test_models():
    """The comparisons are only fair if no token of the test prompts sits on a routing boundary."""
    for name in CONFIGS:
        raw, _, weights = make(name)
        margins = []
        for toks in trace_util.random_prompts(raw["vocab"], LENGTHS, seed=17).values():
            plain.forward(raw, weights, toks, margins=margins)
        assert min(margins) > 1e-4, f"{name}: a token is routed with a margin of {min(margins):.1e}"


# ------------------------------------------------------------------------------------------ whole models, host
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_families_on_the_host(name, family, tmp_path):
    run_family(name, family, tmp_path, "cpu", "float32", F32_TOL)


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
        if device == "cpu":
            runner = host_runner(cfg, w, pages=16, rows=2, tokens=160)
        else:
            runner = ModelRunner(cfg, weights=w, dtype="float32", num_pages=16, max_rows=2, max_step_tokens=160, max_model_len=240)
        got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, steps).items()}
        trace_util.compare(got, {"x": want}, F32_TOL, f"needle at {needle}")
        # and the needle matters: without it the last logits are different
        other = list(tokens)
        other[needle] = toks[needle]
        moved = float((plain.forward(raw, w, other)[-1] - want[-1]).abs().max()) / float(want.abs().max())
        assert moved > 1e-3, "the far token must matter to the last position for this test to mean anything"


def test_a_far_key_and_the_first_token_are_seen():
    far_key_runs("cpu")


@pytest.mark.gpu
def test_a_far_key_and_the_first_token_are_seen_gpu():
    far_key_runs("cuda")


def test_state_slots_and_pages_are_used_again(tmp_path):
    """Five requests, one after another, through a runner with one usable state slot and pages for one request:
    each must start from zero state and see no key of the one before."""
    raw, cfg, weights = make("B")
    prompts = trace_util.random_prompts(raw["vocab"], [40, 33, 40, 7, 25], seed=3)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                         num_pages=4, max_rows=1, max_step_tokens=64, max_model_len=48, num_state_slots=2)
    got = trace_util.run_on_runner(runner, trace_util.portions(prompts, sizes=(5, 2, 9)))
    trace_util.compare(got, expected_logits(raw, weights, prompts), F32_TOL, "reuse")
    entry = next(t for t in runner.storage.entries.values() if "tail" in (t.tensors or {}))
    entry.tensors["state"].fill_(3.0)
    entry.tensors["tail"].fill_(-2.0)
    rc = runner.cache.open("fresh")
    assert float(entry.tensors["state"][rc.state_slot].abs().max()) == 0.0
    assert float(entry.tensors["tail"][rc.state_slot].abs().max()) == 0.0
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
            slack = (F32_TOL if dtype == "float32" else BF16_TOL_PER_LAYER * len(raw["layers"])) * float(logits.abs().max())
            missed += float(logits.max() - logits[tok]) > slack
            ids.append(tok)
    # bfloat16: a token routed on a near-tie may differ (see compare_most); float32: every token is the plain choice
    assert missed <= (0 if dtype == "float32" else 3), f"{missed} of 60 tokens are not the plain implementation's choice"
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


TOL = {torch.float32: 2e-6, torch.bfloat16: 1e-2}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_branch_norm_and_column_norm_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(0)
    for T, W in ((1, 64), (5, 70), (3, 4100)):
        stream = _rand((T, W), torch.float32, g)
        y = _rand((T, W), dtype, g, 3.0)
        wt = _rand((W,), dtype, g) + 1
        want = stream.clone()
        want_copy = ref.ref_branch_norm_add(y, want, wt, 1e-5, dtype)
        got_copy = ops.branch_norm_add(y, stream, wt, 1e-5)
        close(stream, want, 2e-6, "stream")
        close(got_copy, want_copy, TOL[dtype], "copy")
        assert got_copy.dtype == dtype and (dtype != torch.float32 or got_copy is stream)
        close(ops.branch_norm_add(None, stream, None, 0.0), stream, TOL[dtype], "copy alone")
        x = _rand((T, W + 9), torch.float32, g)
        close(ops.rmsnorm_columns(x, 4, W, wt, 1e-3), ref.ref_rmsnorm_columns(x, 4, W, wt, 1e-3, dtype), TOL[dtype], "columns")
    t = _rand((7, 33), torch.float32, g)
    want = t * 0.37
    close(ops.scale_(t, 0.37), want, 1e-7, "scale")
    ids = torch.tensor([3, 0, 6], dtype=torch.int32).cuda()
    table = _rand((8, 20), dtype, g)
    close(ops.embedding(ids, table, scale=2.5), table[ids.long()].float() * 2.5, 1e-7, "scaled embedding")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act", ["gelu_tanh", "relu2", "silu"])
def test_gated_activation_kernel(hip, dtype, act):
    ops, g = hip[dtype], torch.Generator().manual_seed(1)
    for T in (3, 40, 200):
        x, w = _rand((T, 72), dtype, g), _rand((2 * 56, 72), dtype, g, 0.2)
        gu = (x.double() @ w.double().T)
        want = ref.ref_act(gu[:, :56], act) * gu[:, 56:]
        close(ops.linear_act_mul(x, w, 56, act), want, 3 * TOL[dtype] if dtype == torch.bfloat16 else 1e-5, f"{act} at {T} rows")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(2)
    for (H, dim, rot, vdim, r, n_freq, T) in ((3, 16, 8, 24, 40, 4, 37), (5, 8, 16, 8, 24, 4, 3), (2, 24, 4, 12, 28, 2, 130), (4, 32, 16, 40, 48, 8, 300)):
        P = -(-(r + rot) // 16) * 16
        inv_freq = (50.0 ** -(torch.arange(n_freq).double() * 2 / (2 * n_freq))).float().cuda()
        positions = torch.randint(0, 5000, (T,), generator=g).to(torch.int32).cuda()
        sums = _rand((T, 11 + r + rot + 5), torch.float32, g, 2.0)
        nw = _rand((r,), dtype, g) + 1
        pages, page = T // 16 + 3, 16
        slots = torch.randperm((pages - 1) * page, generator=g)[:T].to(torch.int32).cuda() + page
        kc = torch.full((pages, 1, page, P), 7.0, dtype=dtype).cuda()
        vc = torch.full((pages, 1, P, page), 7.0, dtype=dtype).cuda()
        kw, vw = kc.clone(), vc.clone()
        ref.ref_latent_kv_store(sums, 11, r, rot, nw, 1e-5, positions, inv_freq, kw, vw, slots)
        qw = _rand((9,), dtype, g) + 1
        cq = ops.latent_kv_store(sums, 11, r, rot, nw, 1e-5, positions, inv_freq, kc, vc, slots, also_norm=(1, 9, qw))
        close(cq, ref.ref_rmsnorm_columns(sums, 1, 9, qw, 1e-5, dtype), TOL[dtype], "query latent normed beside")
        close(kc, kw, TOL[dtype], "keys")
        close(vc, vw, TOL[dtype], "values")
        assert torch.equal(kc[0], kw[0]), "the scratch page was not written"
        q = _rand((T, H * P), dtype, g)
        want = ref.ref_latent_query_rotate(q.clone(), H, r, P, positions, inv_freq)
        assert ops.latent_query_rotate_(q, H, r, P, positions, inv_freq) is q
        close(q, want, TOL[dtype], "query rotation")
        untouched = torch.ones(P, dtype=torch.bool)
        untouched[r:r + 2 * n_freq] = False
        assert torch.equal(q.view(T, H, P)[..., untouched], want.view(T, H, P)[..., untouched]), "only the turned pairs change"
        o = _rand((T, H * P), dtype, g)
        w_uv = _rand((H * vdim, r), dtype, g, 0.3)
        gate = _rand((T, 7 + H * vdim), torch.float32, g, 2.0)
        close(ops.latent_value_gate(o, w_uv, gate, 7, H, vdim, r, P),
              ref.ref_latent_value_gate(o, w_uv, gate, 7, H, vdim, r, P, dtype), TOL[dtype], "gated values")
        close(ops.latent_value_gate(o, w_uv, None, 0, H, vdim, r, P),
              ref.ref_latent_value_gate(o, w_uv, None, 0, H, vdim, r, P, dtype), TOL[dtype], "values")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_recurrence_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(3)
    # rows of 32, 33, 64 and 65 tokens: the scan's chunks are 32 long, and a row of up to 32 runs in one pass
    for (C, B, K, lens, slots) in ((96, 3, 4, [1, 1, 9, 2, 300], [4, 1, 3, 5, 2]), (40, 5, 1, [5, 1], [1, 2]), (520, 1, 6, [3, 2, 40], [2, 3, 1]),
                                   (64, 2, 3, [32, 33, 64, 65, 1], [5, 4, 3, 2, 1]), (64, 2, 3, [32, 2], [1, 2])):
        step = FakeStep(lens, slots)
        T = step.num_tokens
        x = _rand((T, 2 * C + 3), torch.float32, g)
        b_in, taps, cb = _rand((2 * C,), torch.float32, g, 0.3), _rand((C, K), torch.float32, g, 0.5), _rand((C,), torch.float32, g, 0.3)
        tail = _rand((6, max(1, K - 1), C), torch.float32, g)
        state = _rand((6, C), torch.float32, g)
        u = ops.causal_conv(x, C + 3, C, b_in[C:], taps, cb, tail, step)
        close(u, ref.ref_causal_conv(x.cpu(), C + 3, C, b_in[C:].cpu(), taps.cpu(), cb.cpu(), tail.cpu(), step.host["row_start"],
                                     step.host["state_slots"]), 2e-6, "conv")
        wg = _rand((2 * B, C // B, C // B), dtype, g, 0.2)
        bg = _rand((2 * B, C // B), torch.float32, g)
        gates = ops.grouped_linear(u, wg, bg, x_groups=B)
        close(gates, ref.ref_grouped_linear(u, wg, bg, B), 2e-6, "block-diagonal gates")
        lam = _rand((C,), torch.float32, g, 2.0)
        st_w, tl_w = state.cpu().clone(), tail.cpu().clone()
        want = ref.ref_rglru_scan(u.cpu(), gates.cpu(), lam.cpu(), x.cpu(), 0, b_in[:C].cpu(), x.cpu(), C + 3, b_in[C:].cpu(), st_w,
                                  tl_w, step.host["row_start"], step.host["state_slots"], K, 8.0, dtype)
        got = ops.rglru_scan(u, gates, lam, x, 0, b_in[:C], x, C + 3, b_in[C:], state, tail, step, K, 8.0)
        close(got, want, 2e-5 if dtype == torch.float32 else 1e-2, "scan")
        close(state, st_w, 2e-5, "state")
        if K > 1:
            close(tail, tl_w, 1e-6, "tail")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routing_and_expert_kernels(hip, dtype):
    ops, g = hip[dtype], torch.Generator().manual_seed(4)
    for (T, W, E, top, ff) in ((1, 64, 5, 2, 48), (37, 48, 6, 4, 16), (300, 72, 3, 3, 40), (9, 64, 4, 1, 24), (130, 128, 16, 2, 96)):
        logits, bias = _rand((T, E), torch.float32, g, 2.0), _rand((E,), torch.float32, g)
        idx, shares = ops.route_topk(logits, bias, top)
        widx, wshares = ref.ref_route_topk(logits, bias, top)
        assert torch.equal(idx.cpu(), widx.cpu())
        close(shares, wshares, 2e-6, "shares")
        x = _rand((T, W), dtype, g)
        w_up, w_down = _rand((E, ff, W), dtype, g, W ** -0.5), _rand((E, W, ff), dtype, g, ff ** -0.5)
        got = ops.routed_experts(x, idx, shares, w_up, w_down, "relu2")
        close(got, ref.ref_routed_experts(x, idx, shares, w_up, w_down, "relu2", dtype), 1e-5 if dtype == torch.float32 else 1e-2,
              f"experts {T} tokens")
    tie = torch.zeros(2, 4).cuda()
    assert ops.route_topk(tie, None, 2)[0].tolist() == [[0, 1], [0, 1]], "lowest index first among equals"


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
    """bfloat16: a value is rounded to 8 bits a handful of times a layer; a fault (a lost key, a stale state, the
    wrong cache) moves logits by a large part of their scale, since scores are spread over several units."""
    run_family(name, family, tmp_path, "cuda", "bfloat16", BF16_TOL_PER_LAYER * len(CONFIGS[name][0]["layers"]))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_gpu(dtype):
    eng = generate("A", "cuda", dtype)
    assert eng.num_graph_steps > 0, "decode steps of this model run as captured graphs too"


@pytest.mark.gpu
def test_long_decoding_gpu():
    """160 tokens one by one after a short prompt, float32: recurrent state and cache carried through ten pages."""
    raw, cfg, weights = make("A")
    toks = trace_util.random_prompts(raw["vocab"], [170], seed=6)
    runner = ModelRunner(cfg, weights=weights, dtype="float32", num_pages=14, max_rows=2, max_step_tokens=64,
                         max_model_len=208)
    got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, trace_util.decode_tail(toks, 160)).items()}
    trace_util.compare(got, expected_logits(raw, weights, toks), F32_TOL, "long decoding")


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
    run(cli + ["random-model", "--shape", "zifelorn-tiny", "--seed", "3", "--dtype", "float32", "--out", folder])
    raw = json.load(open(os.path.join(folder, "config.json")))
    weights = load_file(os.path.join(folder, "model.safetensors"))
    assert raw["architecture"] == "Zifelorn" and len(raw["layers"]) == 4
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


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_latent_wider_than_the_matrix_core_kernels_gpu(dtype):
    """kv_rank + rot_dim = 288 numbers a token: beyond the head sizes of the matrix-core attention kernels, so both
    dtypes run the 32-bit attention kernel; a portion, single tokens and a second request beside it."""
    raw = one_layer("latent_attention", att(2, 16, 16, 16, 272, 32), dict(kind="dense", ff=48), width=64, vocab=90)
    cfg = ZifelornConfig.from_dict(raw)
    weights = random_tensors(cfg, 8, torch.float32, std=0.2)
    weights = {k: v.to(torch.float32 if dtype == "float32" else torch.bfloat16) for k, v in weights.items()}
    prompts = trace_util.random_prompts(90, [50, 21], seed=1)
    runner = ModelRunner(cfg, weights=weights, dtype=dtype, num_pages=12, max_rows=2, max_step_tokens=64, max_model_len=128)
    got = {k: v.cpu() for k, v in trace_util.run_on_runner(runner, trace_util.mixed(prompts, 2, seed=2, tail=5)).items()}
    check = trace_util.compare if dtype == "float32" else compare_most
    check(got, expected_logits(raw, weights, prompts), F32_TOL if dtype == "float32" else BF16_TOL_PER_LAYER, f"wide latent {dtype}")
