"""Defosun on the GPU: each mechanism's kernels alone against the plain implementation's function
for it, then the model through the step function in every cut, in float32 and in bfloat16, keys far
back and at the edges of pages, a sink that takes most of the weight, a state that remembers
hundreds of tokens, long decoding through recorded launches, and greedy generation through the
engine and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_defosun
from defosun_helpers import (SMALL, _attention, _config, _dense, _latent, _layer, _lightning, _moe, make_weights,
                             plain_greedy, plain_logits, write_folder)
from helpers import collect, max_error, random_prompt, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole

pytestmark = pytest.mark.gpu
F64 = torch.float64
# of the largest logit; bfloat16: rounding of the small widths, whose largest errors the plain-torch stand-in
# of the kernels (the same places of rounding, other code) shows alike
TOL = {"float32": 2e-5, "bfloat16": 4e-2}
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from tiny_llm_infer_amd.kernels.ops import HipOps
    return HipOps("cuda:0")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("defosun")
    return {name: write_folder(str(root / name), cfg, make_weights(cfg, seed)) for name, (cfg, _, seed) in SMALL.items()}


@pytest.fixture(scope="module")
def clear_folders(tmp_path_factory):
    """Weights whose routers read nothing that rounding touches and whose queries are smaller (for bfloat16)."""
    root = tmp_path_factory.mktemp("defosun_clear")
    return {name: write_folder(str(root / name), cfg, make_weights(cfg, seed, clear_routing=True, mild=True))
            for name, (cfg, _, seed) in SMALL.items()}


def _runner(folder, dtype, max_tokens, page, max_requests=4):
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    model, _ = load_model(folder, dtype, "cuda:0", max_model_len=2048)
    return ModelRunner(model, model.env, page_size=page, num_pages=max_tokens // page,
                       max_requests=max_requests, max_batch_tokens=1024)


def _replay(runner, steps):
    from tiny_llm_infer_amd.engine.replay import Replayer
    rp = Replayer(runner)
    return {st["step"]: rp.run_step(st) for st in steps}


def _requests(vocab, lengths, seed):
    return {f"r{i}": random_prompt(vocab, n, seed + i) for i, n in enumerate(lengths)}


def _close(got, want, tol, what):
    got, want = got.detach().double().cpu(), want.double()
    err, scale = float((got - want).abs().max()), float(want.abs().max())
    assert err <= tol * max(scale, 1e-6), f"{what}: error {err:.3e}, scale {scale:.3e}"


def _all_cuts(folder, dtype, reqs, want, page, max_tokens, tol, what):
    cuts = {
        "whole": trace_whole(reqs),
        "decode": trace_prefill_then_decode(reqs),
        "portions": trace_portions(reqs, seed=3),
        "mixed": trace_mixed(reqs, max_tokens=max_tokens, seed=9),
    }
    for cut, steps in cuts.items():
        runner = _runner(folder, dtype, max_tokens, page)
        got = collect(steps, _replay(runner, steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], want[rid])
            assert err <= tol * scale, f"{what}/{dtype}/{cut}/{rid}: error {err:.3e} at token {row} (scale {scale:.3e})"
        runner.cache.check()
        assert not runner.cache.live() and runner.cache.free_pages() == runner.cache.pages_per_group()
        if cut == "mixed" and runner.cache.groups:
            assert runner.cache.pages_taken_total > runner.cache.num_pages


def _view(starts, counts, slots):
    """A step of sequences that stand at ``starts`` and bring ``counts`` rows, as the step function packs it."""
    from tiny_llm_infer_amd.parts.base import StepView
    i32 = lambda v: torch.tensor([int(x) for x in v], dtype=torch.int32, device="cuda")
    row_start = [0] + list(np.cumsum(counts))
    pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
    sor = [i for i, c in enumerate(counts) for _ in range(c)]
    totals = [s + c for s, c in zip(starts, counts)]
    return StepView(num_rows=sum(counts), num_seqs=len(counts), token_ids=i32(pos), positions=i32(pos), seq_of_row=i32(sor),
                    row_start=i32(row_start), seq_start=i32(starts), seq_len=i32(totals), slots=i32(slots),
                    sample_rows=i32([0]), h_row_start=[int(r) for r in row_start], h_seq_start=list(starts),
                    h_seq_len=totals, h_slots=list(slots), max_rows_per_seq=max(counts), max_seq_len=max(totals),
                    reach=max(128, 1 << (max(totals) - 1).bit_length()))


# -------------------------------------------------- the small kernels, each alone ---
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows, n, limit", [(1, 40, 1.0), (33, 64, 0.5), (7, 136, 7.0), (5, 25, 2.0)])
def test_limited_gated_units(ops, dtype, rows, n, limit):
    """g <- min(g, limit), u <- clamp(u, -limit, limit), g sigmoid(1.702 g) (u + 1): values on both sides of every limit."""
    g = torch.Generator().manual_seed(n)
    gu = (torch.randn(rows, 2 * n, generator=g) * 2 * limit).to(DTYPES[dtype])
    got = ops.swiglu(gu.cuda(), limit=limit, slope=1.702)
    pick = torch.eye(2 * n, dtype=F64)                               # a feed-forward whose gate and up sums are the row's halves
    want = plain_defosun.limited_ff(gu.double(), {"gate": pick[:n], "up": pick[n:], "down": torch.eye(n, dtype=F64)}, "", limit)
    _close(got, want, 2e-6 if dtype == "float32" else 5e-3, "limited units")
    a, b = gu[:, :n].double(), gu[:, n:].double()
    _close(ops.swiglu(gu.cuda()), a * torch.sigmoid(a) * b, 2e-6 if dtype == "float32" else 5e-3, "without a limit: silu(g) u")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16-plain"])
@pytest.mark.parametrize("T, E, top, n, ff, limit", [(1, 4, 2, 48, 40, 1.0), (40, 8, 3, 104, 24, 0.5), (300, 10, 4, 128, 64, 2.0),
                                                     (130, 3, 3, 136, 200, 7.0)])
def test_experts_with_the_limited_activation(ops, dtype, T, E, top, n, ff, limit):
    g = torch.Generator().manual_seed(T)
    dtype, _, variant = dtype.partition("-")
    dt = DTYPES[dtype]
    x = torch.randn(T, n, generator=g).to(dt)
    w_gu = (torch.randn(E, 2 * ff, n, generator=g) * n ** -0.5 * 2).to(dt)
    w_down = (torch.randn(E, n, ff, generator=g) * ff ** -0.5).to(dt)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wts = torch.rand(T, top, generator=g) + 0.2
    shared = torch.randn(T, n, generator=g).to(dt)
    gate = torch.rand(T, generator=g)
    want = gate.double()[:, None] * shared.double()
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            w = {"gate": w_gu[e, :ff].double(), "up": w_gu[e, ff:].double(), "down": w_down[e].double()}
            want[t] += wts[t, j].double() * plain_defosun.limited_ff(x[t:t + 1].double(), w, "", limit)[0]
    packed = None if variant == "plain" else ops.pack_experts(w_gu.cuda(), w_down.cuda())
    rowmajor = (None, None) if packed is not None else (w_gu.cuda(), w_down.cuda())
    got = ops.apply_experts(x.cuda(), ids.cuda(), wts.cuda(), *rowmajor, packed, shared.cuda(), gate.cuda(), limit=limit, slope=1.702)
    _close(got, want, 2e-5 if dtype == "float32" else 2e-2, "limited experts beside a gated shared one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("lanes", [16, 64])
@pytest.mark.parametrize("heads, dk, dv", [(2, 16, 24), (3, 20, 12), (1, 40, 20), (4, 64, 32), (2, 128, 128), (1, 200, 50), (5, 8, 7),
                                           (1, 256, 16)])
def test_lightning_recurrence_in_portions_and_slots_that_are_used_again(ops, dtype, heads, dk, dv, lanes, monkeypatch):
    """Three sequences cut into portions of 1 to 43 rows side by side, in slots that are never cleared and are
    used again by the next sequences; decays from 0.5 to 1; a column of the state in 16 lanes and in 64."""
    monkeypatch.setattr(ops, "lightning_lanes", lanes)
    g = torch.Generator().manual_seed(dk * dv)
    dt = DTYPES[dtype]
    decay = torch.linspace(0.5, 1.0, heads)
    m = {"heads": heads, "dim": dk, "vdim": dv, "decay": decay.tolist()}
    width = 2 * heads * dk + 2 * heads * dv
    eye = torch.eye(width, dtype=F64)
    names = {"q": eye[:heads * dk], "k": eye[heads * dk:2 * heads * dk], "v": eye[2 * heads * dk:2 * heads * dk + heads * dv],
             "g": eye[2 * heads * dk + heads * dv:], "o": torch.eye(heads * dv, dtype=F64), "norm": torch.ones(heads * dv, dtype=F64)}
    state = torch.full((3, *ops.lightning_state_shape(heads, dk, dv)), 7.0, device="cuda")       # what another request left
    for round_ in range(2):
        lengths = [61 + round_, 97, 5 + 40 * round_]
        proj = [(torch.randn(n, width, generator=g) * 0.7).to(dt) for n in lengths]
        slots = [2, 0, 1] if round_ else [0, 1, 2]
        got = [[] for _ in lengths]
        at = [0, 0, 0]
        cuts = [1, 43, 2, 16, 33, 7]
        k = 0
        while any(a < n for a, n in zip(at, lengths)):
            live = [i for i in range(3) if at[i] < lengths[i]]
            counts = [min(cuts[(k + i) % len(cuts)], lengths[i] - at[i]) for i in live]
            k += 1
            rows = torch.cat([proj[i][at[i]:at[i] + c] for i, c in zip(live, counts)]).cuda()
            view = _view([at[i] for i in live], counts, [slots[i] for i in live])
            o = ops.lightning_attention(rows, decay.cuda(), state, view, heads, dk, dv)
            y = ops.lightning_norm(o, rows, 2 * heads * dk + heads * dv, torch.ones(heads * dv, device="cuda"), 1e-5, dt)
            r = 0
            for i, c in zip(live, counts):
                got[i].append(y[r:r + c].cpu())
                r += c
                at[i] += c
        for i, n in enumerate(lengths):
            final = torch.zeros(heads, dk, dv, dtype=F64)
            want = plain_defosun.lightning(proj[i].double(), m, names, "", 1e-5, state=final)
            _close(torch.cat(got[i]), want, 2e-5 if dtype == "float32" else 1.5e-2, f"sequence {i} of round {round_}")
            _close(state[slots[i]].transpose(1, 2), final, 2e-5, f"state of sequence {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads, dk, dv", [(2, 64, 32), (1, 128, 128), (3, 20, 12), (2, 30, 70), (1, 256, 40)])
def test_lightning_long_portions_walked_in_segments(ops, dtype, heads, dk, dv):
    """Portions of hundreds of rows are cut into segments that are walked side by side and joined afterwards: two
    steps of three sequences (900 + 650, 300 + 1, 5 + 700 rows), the second from the states that the first left, beside
    a short sequence that is not cut."""
    g = torch.Generator().manual_seed(dk + dv)
    dt = DTYPES[dtype]
    decay = torch.tensor([1.0, 0.99, 0.9][:heads])
    m = {"heads": heads, "dim": dk, "vdim": dv, "decay": decay.tolist()}
    width = 2 * heads * dk + 2 * heads * dv
    eye = torch.eye(width, dtype=F64)
    names = {"q": eye[:heads * dk], "k": eye[heads * dk:2 * heads * dk], "v": eye[2 * heads * dk:2 * heads * dk + heads * dv],
             "g": eye[2 * heads * dk + heads * dv:], "o": torch.eye(heads * dv, dtype=F64), "norm": torch.ones(heads * dv, dtype=F64)}
    state = torch.full((3, *ops.lightning_state_shape(heads, dk, dv)), -3.0, device="cuda")
    steps = [[900, 300, 5], [650, 1, 700]]
    proj = [(torch.randn(sum(c), width, generator=g) * 0.5).to(dt) for c in zip(*steps)]
    got, at = [[], [], []], [0, 0, 0]
    for counts in steps:
        rows = torch.cat([proj[i][at[i]:at[i] + c] for i, c in enumerate(counts)]).cuda()
        view = _view(at, counts, [1, 2, 0])
        o = ops.lightning_attention(rows, decay.cuda(), state, view, heads, dk, dv)
        y = ops.lightning_norm(o, rows, 2 * heads * dk + heads * dv, torch.ones(heads * dv, device="cuda"), 1e-5, dt)
        r = 0
        for i, c in enumerate(counts):
            got[i].append(y[r:r + c].cpu())
            r += c
            at[i] += c
    for i in range(3):
        final = torch.zeros(heads, dk, dv, dtype=F64)
        want = plain_defosun.lightning(proj[i].double(), m, names, "", 1e-5, state=final)
        _close(torch.cat(got[i]), want, 2e-5 if dtype == "float32" else 1.5e-2, f"sequence {i}")
        _close(state[[1, 2, 0][i]].transpose(1, 2), final, 2e-5, f"state of sequence {i}")


# ------------------------------------------------------- one mixer alone, every cut ---
MIXERS = {
    # grouped heads whose values are their keys: sizes in and out of sixteens, all and part of a head turned
    "keys as values 4/2 16 (8 turned)": ("attention", _attention(4, 2, 16, 8)),
    "keys as values 6/1 24 (6 turned)": ("attention", _attention(6, 1, 24, 6, scale=0.3)),
    "keys as values 2/2 32 (all turned)": ("attention", _attention(2, 2, 32, 32, base=500.0)),
    "keys as values 8/2 64 (16 turned)": ("attention", _attention(8, 2, 64, 16)),
    "keys as values 2/1 128 (64 turned)": ("attention", _attention(2, 1, 128, 64, base=1e6)),
    "keys as values 34/2 16 (2 turned)": ("attention", _attention(34, 2, 16, 2)),
    "keys as values 3/3 20 (10 turned)": ("attention", _attention(3, 3, 20, 10)),
    "keys as values 4/2 48 (24 turned)": ("attention", _attention(4, 2, 48, 24)),
    "keys as values 5/1 96 (32 turned)": ("attention", _attention(5, 1, 96, 32, base=1e5)),
    # one latent vector a position, the key part turned in pairs of neighbours
    "latent 3 64+16 -> 96 of 80": ("latent_attention", _latent(3, 64, 16, 96, 80, base=1e6)),
    "latent 5 24+6 -> 20 of 40": ("latent_attention", _latent(5, 24, 6, 20, 40)),
    "latent 20 32+16 -> 32 of 112": ("latent_attention", _latent(20, 32, 16, 32, 112)),
    "latent 1 16+2 -> 16 of 8": ("latent_attention", _latent(1, 16, 2, 16, 8)),
    "latent 2 32+16 -> 48 of 144": ("latent_attention", _latent(2, 32, 16, 48, 144)),
    # a matrix of state a head
    "lightning 2 x 16 x 24": ("lightning", _lightning(2, 16, 24, [0.9, 0.99])),
    "lightning 3 x 20 x 12": ("lightning", _lightning(3, 20, 12, [0.5, 1.0, 0.97])),
    "lightning 1 x 200 x 50": ("lightning", _lightning(1, 200, 50, [0.98])),
    "lightning 4 x 128 x 64": ("lightning", _lightning(4, 128, 64, [0.7, 0.9, 0.99, 0.999])),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(MIXERS))
def test_one_mixer_alone_in_every_cut(tmp_path, name, dtype):
    """A model of one layer without feed-forward and without streams: the mixer's kernels (what they make of the
    projections, what they write into the cache or the state and read back) between an embedding and the head."""
    kind, mixer = MIXERS[name]
    cfg = _config(120, 64 if mixer["heads"] < 20 else 96, [_layer(kind, mixer, None)])
    folder = write_folder(str(tmp_path / "one"), cfg, make_weights(cfg, len(name), mild=dtype == "bfloat16"))
    reqs = _requests(120, [70, 45, 137, 33, 1, 58, 2, 3], seed=5)
    _all_cuts(folder, dtype, reqs, plain_logits(folder, reqs), 16, 384, TOL[dtype], name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("streams", [1, 2, 5])
def test_streams_around_a_dense_feed_forward(tmp_path, dtype, streams):
    """Hyper-connections of one, two and five streams around a small attention and the gated dense feed-forward."""
    cfg = _config(90, 48, [_layer("attention", _attention(2, 1, 16, 16), _dense(72))] * 2, streams=streams)
    folder = write_folder(str(tmp_path / "streams"), cfg, make_weights(cfg, 10 + streams, mild=True))
    reqs = _requests(90, [50, 3, 77], seed=8)
    _all_cuts(folder, dtype, reqs, plain_logits(folder, reqs), 8, 128, TOL[dtype], f"{streams} streams")


# ---------------------------------------------- a key far back, at the borders of pages; the sink ---
def _last_token_three_ways(folder, dtype, page, toks, want, what):
    """The last token in a whole prompt, decoded alone, and at the end of a portion of two."""
    from tiny_llm_infer_amd.engine.runner import StepEntry
    n = len(toks)
    for tail in (0, 1, 2):
        runner = _runner(folder, dtype, 512, page)
        runner.admit("x")
        if tail:
            runner.step([StepEntry("x", toks[:n - tail], [])])
            got = runner.step([StepEntry("x", toks[n - tail:], [tail - 1])])
        else:
            got = runner.step([StepEntry("x", toks, [n - 1])])
        err = np.abs(got[0].double().cpu().numpy() - want).max()
        assert err <= TOL[dtype] * np.abs(want).max(), (what, tail, err)


def _needle_attention(tmp_path, sink, scale=1.5):
    """One layer of attention in which a token's query finds the key of a like token among hundreds.  Of a head's 16
    elements the turned pair (0, 1) says nothing, elements 2..7 are the same for queries and keys (the same rows of
    the two matrices, reading the first half of the width), and elements 8..15 are the keys' own and read the second
    half of the width, where queries have zeros.  Tokens 88 and 89 have the same first half and opposite second
    halves: the query of 89 scores the key of 88 as it scores its own, and the value there (the key itself) differs."""
    cfg = _config(90, 32, [_layer("attention", _attention(2, 2, 16, 2, scale=scale), None)])
    w = {k: v.float() for k, v in make_weights(cfg, 4).items()}
    q, k = w["l0.mix.q"].view(2, 16, 32), w["l0.mix.k"].view(2, 16, 32)
    q[:, :, 16:] = 0.0
    q[:, :2] = 0.0
    q[:, 8:] = 0.0
    k[:, :8] = q[:, :8]
    k[:, 8:, :16] = 0.0
    w["l0.mix.q.b"], w["l0.mix.k.b"] = torch.zeros(32), torch.zeros(32)
    w["l0.mix.sink"] = torch.full((2,), float(sink))
    w["embed"][88, :16] = w["embed"][89, :16]
    w["embed"][88, 16:] = -w["embed"][89, 16:]
    return cfg, write_folder(str(tmp_path / f"needle{sink}"), cfg, {k: v.to(torch.bfloat16) for k, v in w.items()})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page, at", [(16, 2), (16, 15), (16, 16), (8, 263), (32, 31), (32, 32)])
def test_one_key_far_back_and_at_the_borders_of_pages(tmp_path, dtype, page, at):
    """The token that the last query looks for stands hundreds of positions back, in the last slot of a page or the
    first of the next."""
    cfg, folder = _needle_attention(tmp_path, sink=0.0)
    w = plain_defosun.read_model(folder)[1]
    n = 430
    toks = [t % 88 for t in random_prompt(88, n, 6)]
    toks[n - 1] = 89
    without = plain_defosun.forward(cfg, w, toks)[-1].numpy()
    toks[at] = 88
    want = plain_defosun.forward(cfg, w, toks)[-1].numpy()
    assert np.abs(want - without).max() > 0.04 * np.abs(without).max()       # the needle matters
    _last_token_three_ways(folder, dtype, page, toks, want, f"needle at {at}")


@pytest.mark.parametrize("page", [4, 16])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sink_that_takes_most_of_the_weight(tmp_path, dtype, page):
    """With a sink far above every score the heads give next to nothing; with one far below, the softmax is the plain one;
    a kernel that left the sink out, scaled it, or counted it a key at a time would show in either."""
    logits = {}
    for sink in (-30.0, 6.0, 12.0):
        cfg, folder = _needle_attention(tmp_path, sink=sink, scale=0.1)
        w = plain_defosun.read_model(folder)[1]
        toks = [t % 88 for t in random_prompt(88, 150, 3)]
        logits[sink] = plain_defosun.forward(cfg, w, toks)[-1].numpy()
        _last_token_three_ways(folder, dtype, page, toks, logits[sink], f"sink {sink}")
    assert np.abs(logits[6.0] - logits[-30.0]).max() > 0.04 * np.abs(logits[-30.0]).max()
    assert np.abs(logits[12.0] - logits[6.0]).max() > 0.04 * np.abs(logits[6.0]).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads, dim, rot, vdim, rank, page", [(2, 16, 8, 16, 24, 8), (4, 32, 16, 48, 64, 16)])
def test_one_latent_key_hundreds_of_positions_back(tmp_path, dtype, heads, dim, rot, vdim, rank, page):
    """Latent attention sees everything: the query of the last token is made (by a change of rank one to the query
    matrix) to point at what the latent vector of token 88 becomes as a key, and that token stands at position 2 of
    430.  In a whole prompt, in portions, and with the last 40 tokens decoded one by one."""
    cfg = _config(90, 32, [_layer("latent_attention", _latent(heads, dim, rot, vdim, rank, scale=1.0, base=100.0), None)])
    w = {k: v.float() for k, v in make_weights(cfg, 9).items()}
    eps = cfg["norm"]["eps"]
    wq = w["l0.mix.q"].view(heads, dim + rot, 32)
    wq[:, dim:] *= 0.05                                              # the turned parts say little
    n1 = 1.0 + w["l0.norm1"].to(torch.bfloat16).double()

    def normed(token):
        return (plain_defosun.unit_rms(w["embed"][token].to(torch.bfloat16).double(), eps) * n1).float()
    x_a, x_b = normed(88), normed(89)
    c = (plain_defosun.unit_rms((w["l0.mix.dkv"][:rank].to(torch.bfloat16).float() @ x_a).double(), eps)
         * w["l0.mix.dkv.norm"].to(torch.bfloat16).double()).float()
    key = (w["l0.mix.uk"].to(torch.bfloat16).float() @ c).view(heads, dim)
    target = key * (30.0 / (key * key).sum(-1, keepdim=True))         # a score of 30 in every head
    wq[:, :dim] += ((target - wq[:, :dim] @ x_b)[..., None] * x_b) / (x_b * x_b).sum()
    folder = write_folder(str(tmp_path / "far"), cfg, {k: v.to(torch.bfloat16) for k, v in w.items()})
    wd = plain_defosun.read_model(folder)[1]
    n = 430
    toks = [t % 88 for t in random_prompt(88, n, 11)]
    toks[n - 1] = 89
    without = plain_defosun.forward(cfg, wd, toks)[-1].numpy()
    toks[2] = 88
    want = plain_defosun.forward(cfg, wd, toks)
    assert np.abs(want[-1].numpy() - without).max() > 0.04 * np.abs(without).max()
    _last_token_three_ways(folder, dtype, page, toks, want[-1].numpy(), "far")
    reqs = {"r0": toks}
    for steps in (trace_prefill_then_decode(reqs, tail=40), trace_portions(reqs, seed=5)):
        got = collect(steps, _replay(_runner(folder, dtype, 448, page), steps))
        first = 0 if dtype == "float32" else n - 1
        err, row, scale = max_error(got["r0"][first:], want.numpy()[first:])
        assert err <= TOL[dtype] * scale, (err, row)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_state_that_remembers_a_token_hundreds_of_positions_back(tmp_path, dtype):
    """Decays of 1 and near 1: a token changed 400 positions back moves the last logits; decoded, in portions and in
    a mixed batch the state carries it."""
    cfg = _config(90, 32, [_layer("lightning", _lightning(2, 16, 16, [1.0, 0.998]), None)])
    folder = write_folder(str(tmp_path / "long"), cfg, make_weights(cfg, 12))
    w = plain_defosun.read_model(folder)[1]
    n = 430
    toks = random_prompt(90, n, 2)
    other = list(toks)
    other[30] = (toks[30] + 1) % 90
    want, moved = plain_defosun.forward(cfg, w, toks), plain_defosun.forward(cfg, w, other)
    assert np.abs(want[-1].numpy() - moved[-1].numpy()).max() > 50 * TOL["float32"] * np.abs(want[-1].numpy()).max()
    reqs = {"r0": toks, "r1": other, "r2": toks[:77]}
    full = {"r0": want.numpy(), "r1": moved.numpy(), "r2": want.numpy()[:77]}
    for steps in (trace_prefill_then_decode(reqs, tail=40), trace_portions(reqs, seed=5), trace_mixed(reqs, max_tokens=1024, seed=2)):
        got = collect(steps, _replay(_runner(folder, dtype, 1024, 16), steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], full[rid])
            assert err <= TOL[dtype] * scale, (rid, err, row)


# ------------------------------------------------------------- the model, every cut ---
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SMALL))
def test_all_cuts_match_plain(folders, clear_folders, name, dtype):
    """float32: weights that are random throughout.  bfloat16: weights whose routers read nothing that rounding
    touches, so that no close call is turned, and whose scores are smaller."""
    folder = (clear_folders if dtype == "bfloat16" else folders)[name]
    reqs = _requests(SMALL[name][0]["vocab"], [70, 45, 197, 33, 1, 58, 2, 3], seed=5)
    _all_cuts(folder, dtype, reqs, plain_logits(folder, reqs), SMALL[name][1], 384, TOL[dtype], name)


def test_token_by_token_from_the_first(folders):
    """Every token decoded alone from position 0: the first keys as they are written, the state from nothing."""
    for name in ("A", "B"):
        folder = folders[name]
        reqs = _requests(SMALL[name][0]["vocab"], [60], seed=21)
        want = plain_logits(folder, reqs)
        steps = trace_prefill_then_decode(reqs, tail=59)
        got = collect(steps, _replay(_runner(folder, "float32", 64, SMALL[name][1]), steps))
        err, row, scale = max_error(got["r0"], want["r0"])
        assert err <= TOL["float32"] * scale, (name, err, row)


def test_unequal_requests_together_equal_each_alone(folders):
    """float32: a request's logits in a batch of unequal requests are those it has alone, to rounding."""
    folder = folders["R"]
    reqs = _requests(320, [3, 130, 34, 65], seed=60)
    alone = {rid: _replay(_runner(folder, "float32", 256, 32), trace_whole({rid: toks}))[0] for rid, toks in reqs.items()}
    step = {"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in reqs.items()], "end": list(reqs)}
    together = collect([step], _replay(_runner(folder, "float32", 512, 32), [step]))
    for rid in reqs:
        assert np.abs(together[rid] - alone[rid]).max() <= 2e-5 * np.abs(alone[rid]).max()


def test_bfloat16_through_the_plain_kernels_does_not_depend_on_the_cut(clear_folders):
    """Through the plain kernels a row's arithmetic is the same whatever stands beside it: bfloat16 logits are the same
    bits in every cut, which would show a stale slot or a page used again however small the difference."""
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    from tiny_llm_infer_amd.kernels.ops import HipOps
    folder = clear_folders["A"]
    reqs = _requests(160, [70, 45, 97, 33, 1, 58], seed=15)
    results = []
    for steps in (trace_whole(reqs), trace_portions(reqs, seed=3), trace_mixed(reqs, max_tokens=256, seed=9)):
        ops = HipOps("cuda:0")
        ops.use_plain_kernels()
        model, _ = load_model(folder, "bfloat16", "cuda:0", max_model_len=512, ops=ops)
        runner = ModelRunner(model, model.env, page_size=16, num_pages=16, max_requests=4, max_batch_tokens=512)
        results.append(collect(steps, _replay(runner, steps)))
    for rid in reqs:
        assert np.array_equal(results[0][rid], results[1][rid]) and np.array_equal(results[0][rid], results[2][rid]), rid


def test_long_decoding_through_recorded_launches(clear_folders):
    """150 tokens decoded one by one for three requests at once (bfloat16: the steps are replayed from
    recordings), caches and states of every pass of the looped layers moving on with them."""
    folder = clear_folders["R"]
    reqs = _requests(320, [160, 171, 183], seed=77)
    want = plain_logits(folder, reqs)
    runner = _runner(folder, "bfloat16", 768, 32)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:len(t) - 150], "want": []} for r, t in reqs.items()], "end": []}]
    for j in range(150):
        steps.append({"step": j + 1, "entries": [{"id": r, "tokens": [t[len(t) - 150 + j]], "want": [0]} for r, t in reqs.items()],
                      "end": list(reqs) if j == 149 else []})
    got = collect(steps, _replay(runner, steps))
    assert runner.graph_replays > 100
    for rid, toks in reqs.items():
        err, row, scale = max_error(got[rid], want[rid][len(toks) - 150:])
        assert err <= TOL["bfloat16"] * scale, (rid, err, row)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(folders, clear_folders, dtype):
    from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = (clear_folders if dtype == "bfloat16" else folders)["A"]
    prompts = [random_prompt(160, n, 90 + n) for n in (4, 19, 30, 41)]
    eng = LLMEngine.from_folder(folder, dtype=dtype, max_model_len=128, page_size=16, num_kv_blocks=32, max_num_seqs=3,
                                max_num_batched_tokens=32)
    got = eng.generate(prompts, SamplingParams(max_tokens=10, ignore_eos=True))
    if dtype == "float32":
        assert [r.token_ids for r in got] == [plain_greedy(folder, p, 10) for p in prompts]
    else:
        # rounding may turn a close call: every token must be the plain implementation's choice or within
        # the rounding error of it, given the tokens before
        cfg, w = plain_defosun.read_model(folder)
        for p, r in zip(prompts, got):
            logits = plain_defosun.forward(cfg, w, p + r.token_ids)[len(p) - 1:-1]
            for z, t in zip(logits, r.token_ids):
                assert float(z.max() - z[t]) <= 2 * TOL["bfloat16"] * float(z.abs().max())
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()


# ------------------------------------------------------------------ the command line ---
def test_the_programs_take_a_defosun_folder(folders, tmp_path):
    """bin/trace_run replays a mixed trace, model_main --infer generates greedily, and a model of random
    weights made from a config.json alone loads and generates."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, vocab = folders["C"], SMALL["C"][0]["vocab"]
    reqs = _requests(vocab, [40, 9, 77, 23, 52], seed=12)
    want = plain_logits(folder, reqs)
    steps = trace_mixed(reqs, max_tokens=192, seed=4)
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(tmp_path / "out"), "--max-tokens", "192"],
                          input="".join(json.dumps(s) + "\n" for s in steps), text=True, stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    outputs = {s["step"]: np.fromfile(tmp_path / "out" / f"{s['step']}.f32", dtype="<f4").reshape(-1, vocab)
               for s in steps if sum(len(e["want"]) for e in s["entries"])}
    got = collect(steps, outputs)
    for rid in reqs:
        err, row, scale = max_error(got[rid], want[rid])
        assert err <= TOL["float32"] * scale, (rid, err, row)
    prompt = random_prompt(vocab, 21, 3)
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "model_main"), "--infer", "--model", folder, "--dtype",
                           "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "8", "--ignore-eos",
                           "--max-seq-len", "64", "--num-kv-blocks", "16"],
                          text=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == plain_greedy(folder, prompt, 8)
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(SMALL["R"][0]))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "model_main"), "--infer", "--config", str(cfg_file),
                           "--random-weights", "--seed", "5", "--prompt-ids", "1,2,3,4,5", "--max-new-tokens", "6",
                           "--ignore-eos", "--max-seq-len", "64", "--num-kv-blocks", "16"],
                          text=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert len(proc.stdout.split()) == 6
