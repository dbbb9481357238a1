"""Gimipel through the engine's own logic on the CPU (the kernel library replaced by the
plain-torch stand-in of tests/cpu_ops.py): configuration and weights, layers that run with
another layer's weights, window pages that are given back while the first ones stay, all ways of
cutting the work, and greedy generation through the scheduler, against the plain implementation."""
import json
import math

import numpy as np
import pytest
import torch

import plain_gimipel
from cpu_ops import CpuOps
from gimipel_helpers import SMALL, _attention, _config, _layer, make_weights, plain_greedy, plain_logits, write_folder
from helpers import collect, max_error, random_prompt, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
from tiny_llm_infer_amd.config import ConfigError, GimipelConfig
from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
from tiny_llm_infer_amd.engine.loading import load_model
from tiny_llm_infer_amd.engine.replay import Replayer
from tiny_llm_infer_amd.engine.runner import ModelRunner, StepEntry
from tiny_llm_infer_amd.registry import architecture_of
from tiny_llm_infer_amd.sampling.params import SamplingParams
from tiny_llm_infer_amd.weights.loader import WeightError

F64 = torch.float64


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
    from tiny_llm_infer_amd.models.gimipel import gimipel_spec
    for name, (cfg, _, _) in SMALL.items():
        typed = GimipelConfig.from_dict(cfg)
        assert typed.to_dict() == cfg
        assert architecture_of(cfg).name == "Gimipel"
        spec = gimipel_spec(typed)
        own = [i for i, layer in enumerate(cfg["layers"]) if "weights_of" not in layer]
        assert len(spec.blocks) == len(own) and len(spec.schedule) == len(cfg["layers"])
        for i, (layer, call) in enumerate(zip(cfg["layers"], spec.schedule)):
            assert call.block == own.index(layer.get("weights_of", i))
            assert call.cache == i                                  # every layer keeps a cache of its own


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="conv"), "layer type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"].pop("diff"), "diff"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "feed-forward kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(experts=5), "equal groups"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=1), "cannot give"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=1), "other sizes"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_config_errors(change, message):
    cfg = json.loads(json.dumps(SMALL["A"][0]))
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        GimipelConfig.from_dict(cfg)


def test_a_layer_may_name_a_layer_that_names_another():
    cfg = json.loads(json.dumps(SMALL["A"][0]))
    cfg["layers"].append(dict(cfg["layers"][2], weights_of=2))
    typed = GimipelConfig.from_dict(cfg)
    assert typed.layers[4].weights_of == 0


def test_a_checkpoint_that_does_not_fit_is_refused(tmp_path):
    cfg, _, seed = SMALL["A"]
    w = make_weights(cfg, seed)
    del w["l0.mix.lq2"]
    w["l1.mlp.e2.up"] = w["l1.mlp.e2.up"][:-1]
    w["l2.norm1"] = torch.zeros(64, dtype=torch.bfloat16)           # layer 2 runs with the weights of layer 0
    w["l0.mlp.e6.gate"] = w["l0.mlp.e5.gate"].clone()               # router outputs 6 and 7 have no matrices
    folder = write_folder(str(tmp_path / "bad"), cfg, w)
    with pytest.raises(WeightError) as err:
        load_model(folder, "float32", "cpu", ops=CpuOps())
    assert err.value.missing == ["l0.mix.lq2"] and sorted(err.value.unexpected) == ["l0.mlp.e6.gate", "l2.norm1"]
    assert [n for n, _, _ in err.value.wrong_shape] == ["l1.mlp.e2.up"]


def test_cache_layers_of_layers_that_share_weights_and_pages_that_stay(gimipel_folders):
    """Two attention layers with the same weights keep their keys apart (one group of cache layers, two layers in
    it), and so do the two latent layers (a group that keeps everything); the window gives pages back but for
    those of the first positions."""
    runner = _runner(gimipel_folders["A"], 16, 256)
    groups = {tuple(g.cache_layers): g.need for g in runner.cache.groups}
    assert set(groups) == {(0, 2), (1, 3)}
    assert groups[(0, 2)].window == 20 and groups[(0, 2)].keep_first == 3 and groups[(1, 3)].keeps_all
    assert [r.dims for r in groups[(1, 3)].records] == [(-1, 32 + 8)]                 # the latent vector and the turned part
    windowed = [tuple(g.cache_layers) for g in runner.cache.groups].index((0, 2))
    runner.admit("a")
    toks = random_prompt(160, 100, 1)
    runner.step([StepEntry("a", toks[:90], [])])
    tables = runner.cache.get("a").tables
    held = [b for b, p in enumerate(tables[windowed]) if p >= 0]
    assert held == [0, 4, 5]                                       # block 0 (kept); a query at 90 reads 71..89
    assert sum(p >= 0 for p in tables[1 - windowed]) == 6
    runner.release("a")
    runner.cache.check()

    runner = _runner(gimipel_folders["K"], 8, 256)                  # 20 kept first keys: three blocks of eight stay
    runner.admit("a")
    runner.step([StepEntry("a", random_prompt(300, 90, 2), [])])
    g7 = [i for i, g in enumerate(runner.cache.groups) if g.need.window == 7][0]
    assert [b for b, p in enumerate(runner.cache.get("a").tables[g7]) if p >= 0] == [0, 1, 2, 10, 11]
    runner.release("a")


# ------------------------------------------------------------------ all the cuts ---
@pytest.mark.parametrize("name", list(SMALL))
def test_all_cuts_match_plain(gimipel_folders, name):
    folder = gimipel_folders[name]
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


def test_token_by_token_equals_whole(gimipel_folders):
    """Every token decoded alone from position 0 against the whole prompt: the first tokens of a sequence, the
    kept first keys as they are written, the window as it starts to pass."""
    for name in ("A", "K"):
        folder = gimipel_folders[name]
        reqs = _requests(name, [60], seed=21)
        want = plain_logits(folder, reqs)
        steps = trace_prefill_then_decode(reqs, tail=59)
        runner = _runner(folder, SMALL[name][1], 64)
        got = collect(steps, _replay(runner, steps))
        err, row, scale = max_error(got["r0"], want["r0"])
        assert err <= 2e-5 * scale, (name, err, row)


def test_pages_that_change_hands_carry_nothing_over(gimipel_folders):
    """Few pages, used by request after request; portions down to two tokens."""
    folder = gimipel_folders["C"]
    reqs = _requests("C", [37, 29, 41], seed=40)
    want = plain_logits(folder, reqs)
    runner = _runner(folder, 16, 48, max_requests=1)
    steps = trace_portions(reqs, seed=1)
    got = collect(steps, _replay(runner, steps))
    for rid in reqs:
        err, row, scale = max_error(got[rid], want[rid])
        assert err <= 2e-5 * scale, (rid, err, row)
    assert runner.cache.pages_taken_total > runner.cache.num_pages


def test_unequal_requests_together_equal_each_alone(gimipel_folders):
    folder = gimipel_folders["R"]
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
        assert np.abs(together[rid] - alone[rid]).max() <= 1e-5


# ------------------------------------------------- generation through the scheduler ---
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_matches_plain(gimipel_folders, name):
    folder = gimipel_folders[name]
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
def test_plain_mechanisms_by_hand(tmp_path):
    """The plain implementation's own small facts, so that an oracle that is wrong in the same way as
    the engine does not go unnoticed."""
    x = torch.tensor([[3.0, 4.0, 0.0, 0.0]], dtype=F64)
    y = plain_gimipel.rms_norm(x, torch.tensor([1.0, 2.0, 1.0, 1.0], dtype=F64), 0.0)
    assert torch.allclose(y, torch.tensor([[1.2, 3.2, 0.0, 0.0]], dtype=F64))
    y = plain_gimipel.rms_norm(x, None, 2.75)                       # eps inside the root: sqrt(6.25 + 2.75) = 3
    assert torch.allclose(y, x / 3.0)
    # a window of 3 with the first 2 kept: row 6 sees 0, 1 (kept) and 4, 5, 6
    ok = plain_gimipel.visible(7, 3, 2)
    assert ok[6].tolist() == [True, True, False, False, True, True, True]
    assert ok[2].tolist() == [True, True, True, False, False, False, False]
    assert plain_gimipel.visible(4, None, 0).tolist() == torch.tril(torch.ones(4, 4)).bool().tolist()
    # a quarter turn of the pair (0, 2) at position 1; base 1: every frequency is 1; element 4 passes
    z = torch.zeros(2, 5, dtype=F64)
    z[1] = torch.tensor([1.0, 0.0, 0.0, 2.0, 9.0])
    r = plain_gimipel.rotate_half(z, torch.arange(2), 4, 1.0)
    c, s = math.cos(1.0), math.sin(1.0)
    assert torch.allclose(r[1], torch.tensor([c, -2 * s, s, 2 * c, 9.0], dtype=F64))
    # frequencies: pair i of a part of 4 turns by base^(-2 i / 4)
    r = plain_gimipel.rotate_half(torch.tensor([[0.0, 1.0, 0.0, 0.0]], dtype=F64), torch.tensor([3]), 4, 100.0)
    assert torch.allclose(r[0], torch.tensor([0.0, math.cos(0.3), 0.0, math.sin(0.3)], dtype=F64))
    # the router: six outputs in three groups of two, of which two stay; the correction enters the choice only
    s = torch.tensor([0.30, 0.05, 0.25, 0.02, 0.20, 0.18], dtype=F64)
    w = {"router": torch.eye(6, dtype=F64), "correction": torch.tensor([0.0, 0.0, -0.3, 0.0, 0.0, 0.1], dtype=F64)}
    f = {"router": {"experts": 5, "identity": 1, "top": 3, "groups": {"count": 3, "keep": 2}}}
    ids, wts = plain_gimipel.route(torch.log(s).view(1, 6), f, w, "")
    # choice scores .30 .05 -.05 .02 .20 .28: groups 0 and 2 stay; inside them 0, 5, 4; a negative choice
    # score (2) would still beat an expert of a group that does not stay
    assert ids == [[0, 5, 4]] and np.allclose(wts, [[0.30, 0.18, 0.20]])
    f["router"]["groups"] = {"count": 3, "keep": 3}
    f["router"]["top"] = 5
    ids, wts = plain_gimipel.route(torch.log(s).view(1, 6), f, w, "")
    assert ids == [[0, 5, 4, 1, 3]]
    # an expert without matrices hands its input on, times its weight; nothing is renormalized
    f = {"router": {"experts": 0, "identity": 2, "top": 1, "groups": {"count": 1, "keep": 1}}}
    h = torch.tensor([[1.0, 2.0]], dtype=F64)
    out = plain_gimipel.routed_experts(h, f, {"router": torch.tensor([[1.0, 0.0], [0.0, 0.0]], dtype=F64)}, "")
    assert torch.allclose(out, h * (math.e / (math.e + 1.0)))
    # two maps: with equal queries for both maps a1 = a2, so o = (1 - lambda) a and the unit norm takes the factor out
    cfg = _config(20, 16, [_layer("attention", _attention(2, 1, 4, 4, None, 0, diff=0.25), None)])
    wts = {k: v.to(F64) for k, v in make_weights(cfg, 1).items()}
    q = wts["l0.mix.q"].view(2, 2, 4, 16)
    q[:, 1] = q[:, 0]
    k = wts["l0.mix.k"].view(1, 2, 4, 16)
    k[:, 1] = k[:, 0]
    h = torch.randn(5, 16, dtype=F64, generator=torch.Generator().manual_seed(0))
    a = plain_gimipel.differential_attention(h, cfg["layers"][0]["mixer"], wts, "l0.mix.", 1e-9)
    wts2 = dict(wts)
    wts2["l0.mix.lq1"] = wts["l0.mix.lq1"] * 3.0                    # another lambda (of the same sign of 1 - lambda)
    lam = lambda w: math.exp(float((w["l0.mix.lq1"] * w["l0.mix.lk1"]).sum())) - math.exp(float((w["l0.mix.lq2"] * w["l0.mix.lk2"]).sum())) + 0.25
    b = plain_gimipel.differential_attention(h, cfg["layers"][0]["mixer"], wts2, "l0.mix.", 1e-9)
    sign = 1.0 if (1 - lam(wts)) * (1 - lam(wts2)) > 0 else -1.0
    assert torch.allclose(a, sign * b, atol=1e-6)
    heads = (a @ torch.linalg.pinv(wts["l0.mix.o"].T)).view(5, 2, 4)
    gate = torch.sigmoid(h @ wts["l0.mix.g"].T)
    assert torch.allclose((heads / gate[..., None]).pow(2).mean(-1).sqrt(), torch.full((5, 2), 0.75, dtype=F64), atol=1e-5)
