"""Defosun through the engine's own logic on the CPU (the kernel library replaced by the
plain-torch stand-in of tests/cpu_ops.py): configuration and weights, layers that are passed
several times with a cache layer and state of their own a pass, all ways of cutting the work,
slots and pages that change hands, and greedy generation through the scheduler, against the plain
implementation; and the plain implementation's own facts by hand."""
import json
import math

import numpy as np
import pytest
import torch

import plain_defosun
from cpu_ops import CpuOps
from defosun_helpers import SMALL, make_weights, plain_greedy, plain_logits, write_folder
from helpers import collect, max_error, random_prompt, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
from tiny_llm_infer_amd.config import ConfigError, DefosunConfig
from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
from tiny_llm_infer_amd.engine.loading import load_model
from tiny_llm_infer_amd.engine.replay import Replayer
from tiny_llm_infer_amd.engine.runner import ModelRunner, StepEntry
from tiny_llm_infer_amd.registry import architecture_of
from tiny_llm_infer_amd.sampling.params import SamplingParams
from tiny_llm_infer_amd.weights.loader import WeightError

F64 = torch.float64


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("defosun")
    return {name: write_folder(str(root / name), cfg, make_weights(cfg, seed)) for name, (cfg, _, seed) in SMALL.items()}


def _runner(folder, page, max_tokens, max_requests=4):
    model, _ = load_model(folder, "float32", "cpu", max_model_len=1024, ops=CpuOps())
    return ModelRunner(model, model.env, page_size=page, num_pages=max_tokens // page,
                       max_requests=max_requests, max_batch_tokens=512)


def _replay(runner, steps):
    rp = Replayer(runner)
    return {st["step"]: rp.run_step(st) for st in steps}


def _requests(name, lengths, seed):
    vocab = SMALL[name][0]["vocab"]
    return {f"r{i}": random_prompt(vocab, n, seed + i) for i, n in enumerate(lengths)}


# ------------------------------------------------------------ configuration ---
def test_config_round_trip_registry_and_run_order():
    from tiny_llm_infer_amd.models.defosun import defosun_spec
    for name, (cfg, _, _) in SMALL.items():
        typed = DefosunConfig.from_dict(cfg)
        assert typed.to_dict() == cfg
        assert architecture_of(cfg).name == "Defosun"
        spec = defosun_spec(typed)
        order = plain_defosun.run_order(cfg)
        assert [c.block for c in spec.schedule] == order and len(spec.blocks) == len(cfg["layers"])
        kept = [c.cache for c, i in zip(spec.schedule, order) if cfg["layers"][i]["type"] != "lightning"]
        assert kept == list(range(len(kept)))                       # a cache layer of its own a pass
        assert all(c.cache == -1 for c, i in zip(spec.schedule, order) if cfg["layers"][i]["type"] == "lightning")
        assert spec.blocks[0].arrangement == ("hyper_prenorm" if "streams" in cfg else "prenorm")
    assert plain_defosun.run_order(SMALL["A"][0]) == [0, 1, 2, 1, 2]
    assert plain_defosun.run_order(SMALL["C"][0]) == [0, 1, 2] * 2


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="conv"), "layer type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "values of this attention are its keys"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=4), "whole turned part"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5]), "one a head"),
    (lambda c: c["layers"][0]["mlp"].update(kind="conv"), "feed-forward kind"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "cannot give"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["layers"][1]["mlp"]["shared"].update(limit=0.0), "limit"),
    (lambda c: c["loop"].update(stop=4), "loop"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_config_errors(change, message):
    cfg = json.loads(json.dumps(SMALL["A"][0]))
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        DefosunConfig.from_dict(cfg)


def test_a_checkpoint_that_does_not_fit_is_refused(tmp_path):
    cfg, _, seed = SMALL["A"]
    w = make_weights(cfg, seed)
    del w["l0.mix.sink"]
    w["l1.mlp.e2.up"] = w["l1.mlp.e2.up"][:-1]
    w["l0.mix.v"] = w["l0.mix.k"].clone()                           # the values are the keys: there is no such matrix
    w["l0.hc1.mix"] = w["l0.hc1.mix"][:2]
    folder = write_folder(str(tmp_path / "bad"), cfg, w)
    with pytest.raises(WeightError) as err:
        load_model(folder, "float32", "cpu", ops=CpuOps())
    assert err.value.missing == ["l0.mix.sink"] and err.value.unexpected == ["l0.mix.v"]
    assert sorted(n for n, _, _ in err.value.wrong_shape) == ["l0.hc1.mix", "l1.mlp.e2.up"]


def test_every_pass_of_a_layer_has_a_cache_layer_and_state_of_its_own(folders):
    runner = _runner(folders["A"], 16, 256)
    # run order 0 1 2 1 2: attention, latent, lightning, latent, lightning
    groups = {tuple(g.cache_layers): [r.dims for r in g.need.records] for g in runner.cache.groups}
    assert set(groups) == {(0,), (1, 2)} and groups[(1, 2)] == [(-1, 32 + 8)]
    states = [s for s in runner.states if s is not None]
    assert len(states) == 2 and states[0]["mixer"].data_ptr() != states[1]["mixer"].data_ptr()
    assert tuple(states[0]["mixer"].shape) == (4 + 1, 2, 24, 16) and states[0]["mixer"].dtype == torch.float32
    assert [s is not None for s in runner.states] == [False, False, True, False, True]


# ------------------------------------------------------------------ all the cuts ---
@pytest.mark.parametrize("name", list(SMALL))
def test_all_cuts_match_plain(folders, name):
    folder = folders[name]
    reqs = _requests(name, [70, 45, 97, 33, 1, 58, 2], seed=5)
    want = plain_logits(folder, reqs)
    max_tokens = 256
    cuts = {
        "whole": trace_whole(reqs),
        "decode": trace_prefill_then_decode(reqs),
        "portions": trace_portions(reqs, seed=3),
        "mixed": trace_mixed(reqs, max_tokens=max_tokens, seed=9),
    }
    for cut, steps in cuts.items():
        runner = _runner(folder, SMALL[name][1], max_tokens)
        got = collect(steps, _replay(runner, steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], want[rid])
            assert err <= 2e-5 * max(1.0, scale), f"{name}/{cut}/{rid}: error {err} at token {row}"
        runner.cache.check()
        assert not runner.cache.live()
        assert runner.cache.free_pages() == runner.cache.pages_per_group()


def test_token_by_token_equals_whole(folders):
    """Every token decoded alone from position 0 against the whole prompt: the first tokens of a sequence and the
    state as it builds up."""
    for name in ("A", "B"):
        folder = folders[name]
        reqs = _requests(name, [60], seed=21)
        want = plain_logits(folder, reqs)
        steps = trace_prefill_then_decode(reqs, tail=59)
        runner = _runner(folder, SMALL[name][1], 64)
        got = collect(steps, _replay(runner, steps))
        err, row, scale = max_error(got["r0"], want["r0"])
        assert err <= 2e-5 * scale, (name, err, row)


def test_pages_and_slots_that_change_hands_carry_nothing_over(folders):
    """Few pages and one state slot, used by request after request; portions down to two tokens."""
    folder = folders["C"]
    reqs = _requests("C", [37, 29, 41], seed=40)
    want = plain_logits(folder, reqs)
    runner = _runner(folder, 16, 48, max_requests=1)
    steps = trace_portions(reqs, seed=1)
    got = collect(steps, _replay(runner, steps))
    for rid in reqs:
        err, row, scale = max_error(got[rid], want[rid])
        assert err <= 2e-5 * scale, (rid, err, row)
    assert runner.cache.pages_taken_total > runner.cache.num_pages


def test_unequal_requests_together_equal_each_alone(folders):
    folder = folders["R"]
    reqs = _requests("R", [3, 130, 34, 65], seed=60)
    alone = {}
    for rid, toks in reqs.items():
        runner = _runner(folder, 32, 256)
        alone[rid] = _replay(runner, trace_whole({rid: toks}))[0]
    runner = _runner(folder, 32, 512)
    step = {"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in reqs.items()],
            "end": list(reqs)}
    together = collect([step], _replay(runner, [step]))
    for rid in reqs:
        assert np.abs(together[rid] - alone[rid]).max() <= 4e-6 * np.abs(alone[rid]).max()      # (the stand-in's products round by their shape)


# ------------------------------------------------- generation through the scheduler ---
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_matches_plain(folders, name):
    folder = folders[name]
    vocab = SMALL[name][0]["vocab"]
    prompts = [random_prompt(vocab, n, 40 + n) for n in (5, 17, 33)]
    want = [plain_greedy(folder, p, 12) for p in prompts]
    args = dict(dtype="float32", device="cpu", max_model_len=128, page_size=SMALL[name][1], num_kv_blocks=64,
                max_num_seqs=4, max_num_batched_tokens=24, ops=CpuOps())
    eng = LLMEngine.from_folder(folder, **args)
    got = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    assert [r.token_ids for r in got] == want
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()


# ------------------------------------------------------ the plain implementation itself ---
def test_plain_mechanisms_by_hand():
    """The plain implementation's own small facts, so that an oracle that is wrong in the same way as
    the engine does not go unnoticed."""
    x = torch.tensor([[3.0, 4.0, 0.0, 0.0]], dtype=F64)
    y = plain_defosun.zero_centred_norm(x, torch.tensor([0.0, 1.0, 0.0, 0.0], dtype=F64), 0.0)      # rms 2.5; weights 1 2 1 1
    assert torch.allclose(y, torch.tensor([[1.2, 3.2, 0.0, 0.0]], dtype=F64))
    assert torch.allclose(plain_defosun.unit_rms(x, 2.75), x / 3.0)            # eps inside the root: sqrt(6.25 + 2.75)
    # a quarter of the way round for pair 0 at position 1; base 1: every frequency is 1; element 4 passes
    z = torch.zeros(2, 5, dtype=F64)
    z[1] = torch.tensor([1.0, 0.0, 0.0, 2.0, 9.0])
    c, s = math.cos(1.0), math.sin(1.0)
    r = plain_defosun.turn(z, torch.arange(2), 4, 1.0, False)                  # pairs (0, 2) and (1, 3)
    assert torch.allclose(r[1], torch.tensor([c, -2 * s, s, 2 * c, 9.0], dtype=F64))
    r = plain_defosun.turn(z, torch.arange(2), 4, 1.0, True)                   # pairs (0, 1) and (2, 3)
    assert torch.allclose(r[1], torch.tensor([c, s, -2 * s, 2 * c, 9.0], dtype=F64))
    assert torch.allclose(r[0], z[0])
    # frequencies: pair i of 4 turned elements turns by base^(-2 i / 4)
    r = plain_defosun.turn(torch.tensor([[0.0, 1.0, 0.0, 0.0]], dtype=F64), torch.tensor([3]), 4, 100.0, False)
    assert torch.allclose(r[0], torch.tensor([0.0, math.cos(0.3), 0.0, math.sin(0.3)], dtype=F64))
    # the sink counts once, unscaled, and has no value: two equal scores of 0 and a sink of ln 2 weigh 1/4 each
    p = plain_defosun.softmax_with_sink(torch.zeros(2, 2, dtype=F64), math.log(2.0))
    assert torch.allclose(p, torch.tensor([[1 / 3, 0.0], [0.25, 0.25]], dtype=F64))
    assert torch.allclose(plain_defosun.softmax_with_sink(torch.zeros(2, 2, dtype=F64), None)[1], torch.tensor([0.5, 0.5], dtype=F64))
    # the limited activation: g = min(3, 1) = 1, u = clamp(-5, -1, 1) = -1: the unit is 0; u + 1 = 2 at the upper limit
    w = {"gate": torch.tensor([[3.0]], dtype=F64), "up": torch.tensor([[-5.0]], dtype=F64), "down": torch.tensor([[1.0]], dtype=F64)}
    h = torch.tensor([[1.0]], dtype=F64)
    assert float(plain_defosun.limited_ff(h, w, "", 1.0)) == 0.0
    w["up"] = torch.tensor([[5.0]], dtype=F64)
    assert math.isclose(float(plain_defosun.limited_ff(h, w, "", 1.0)), 2.0 / (1.0 + math.exp(-1.702)))
    w["gate"] = torch.tensor([[-3.0]], dtype=F64)                                # the gate has no lower limit
    assert math.isclose(float(plain_defosun.limited_ff(h, w, "", 1.0)), -3.0 / (1.0 + math.exp(3 * 1.702)) * 2.0)
    # the router: the largest scores, weighing as they are
    s = torch.tensor([0.30, 0.05, 0.25, 0.02, 0.20, 0.18], dtype=F64)
    ids, wts = plain_defosun.route(torch.log(s).view(1, 6), {"router": {"experts": 6, "top": 3}}, {"router": torch.eye(6, dtype=F64)}, "")
    assert ids == [[0, 2, 4]] and np.allclose(wts, [[0.30, 0.25, 0.20]])
    # lightning: one head of one key and one value element, decay 1/2: S = 1, 1.5, 1.75; o = S q
    m = {"heads": 1, "dim": 1, "vdim": 1, "decay": [0.5]}
    big = 40.0                                                                   # silu(40) = 40, sigmoid(40) = 1 to float64
    w = {"q": torch.tensor([[big]], dtype=F64), "k": torch.tensor([[big]], dtype=F64), "v": torch.tensor([[big]], dtype=F64),
         "g": torch.tensor([[big]], dtype=F64), "o": torch.tensor([[1.0]], dtype=F64), "norm": torch.tensor([2.0], dtype=F64)}
    out = plain_defosun.lightning(torch.ones(3, 1, dtype=F64), m, w, "", 0.0)
    assert torch.allclose(out, torch.full((3, 1), 2.0, dtype=F64))              # one element: the unit norm leaves its sign, times the weight
    state = torch.zeros(1, 1, 1, dtype=F64)
    plain_defosun.lightning(torch.ones(3, 1, dtype=F64), m, w, "", 0.0, state=state)
    assert math.isclose(float(state), big * big * 1.75, rel_tol=1e-12)
    # hyper-connections: two streams, the sublayer's output written to stream 1 only, stream 0 handed to both
    cfg = {"architecture": "Defosun", "vocab": 3, "width": 2, "norm": {"eps": 1e-9}, "streams": 2,
           "layers": [{"type": "lightning", "mixer": {"heads": 1, "dim": 1, "vdim": 1, "decay": [0.0]}, "mlp": None}]}
    w = {"embed": torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]], dtype=F64), "final.norm": torch.zeros(2, dtype=F64),
         "head": torch.eye(2, dtype=F64)[[0, 1, 0]], "l0.norm1": torch.zeros(2, dtype=F64),
         "l0.hc1.in": torch.tensor([1.0, 0.0], dtype=F64), "l0.hc1.out": torch.tensor([0.0, 1.0], dtype=F64),
         "l0.hc1.mix": torch.tensor([[1.0, 1.0], [0.0, 0.0]], dtype=F64),
         "l0.mix.q": torch.zeros(1, 2, dtype=F64), "l0.mix.k": torch.zeros(1, 2, dtype=F64), "l0.mix.v": torch.zeros(1, 2, dtype=F64),
         "l0.mix.g": torch.zeros(1, 2, dtype=F64), "l0.mix.o": torch.zeros(2, 1, dtype=F64), "l0.mix.norm": torch.ones(1, dtype=F64)}
    res = []
    plain_defosun.forward(cfg, w, [0, 1], residuals=res)
    # the mixer gives 0: both streams become stream 0 (mix [from, to] = [[1, 1], [0, 0]]): their sum is twice the embedding
    assert torch.allclose(res[0], 2.0 * w["embed"][[0, 1]])
