"""Shared by the Gimipel tests: small configurations that differ in every size and option,
weights drawn so that every mechanism matters, and model folders of them."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import numpy as np
import torch


def _attention(heads, kv_heads, dim, vdim, window, keep_first, diff=0.5, scale=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
           "scale": float(dim ** -0.5 if scale is None else scale)}
    if window is not None:
        out["mask"] = {"size": window, "keep_first": keep_first}
    return out


def _latent(heads, dim, rot_dim, vdim, rank, base=10000.0, scale=None, dims=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
            "scale": float((dim + rot_dim) ** -0.5 if scale is None else scale),
            "rot": {"dims": rot_dim if dims is None else dims, "base": base}}


def _moe(experts, identity, top, groups, keep, ff, shared):
    out = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "top": top, "identity": identity, "groups": {"count": groups, "keep": keep}}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def _layer(kind, mixer, mlp, weights_of=None):
    out = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def _config(vocab, width, layers, emb_scale=4.0, eps=1e-5):
    return {"architecture": "Gimipel", "vocab": vocab, "width": width, "embedding": {"scale": emb_scale},
            "norm": {"eps": eps}, "layers": layers}


_A_ATT, _A_LAT, _A_MOE = _attention(4, 2, 16, 32, 20, 3), _latent(2, 16, 8, 24, 32), _moe(6, 2, 3, 4, 2, 32, 48)
_C_ATT, _C_MOE = _attention(6, 1, 24, 40, 100, 9, diff=0.3, scale=0.3), _moe(7, 1, 3, 8, 3, 24, 16)
# name -> (config.json, page size of the engine in its tests, seed)
SMALL = {
    # a window that is no multiple of the page with three kept first keys; value heads larger than key heads; eight
    # router outputs (two of them without matrices) in four groups; layers 2 and 3 run with the weights of 0 and 1
    "A": (_config(160, 64, [_layer("attention", _A_ATT, _A_MOE), _layer("latent_attention", _A_LAT, _A_MOE),
                            _layer("attention", _A_ATT, _A_MOE, 0), _layer("latent_attention", _A_LAT, _A_MOE, 1)]), 16, 3),
    # as many key heads as query heads, no window at all, one head of latent attention whose values are as long as its
    # keys, one group of experts with one chosen, none without matrices and no shared expert, a layer without
    # feed-forward, embedding scale 1, fewer turned elements than the turned part holds
    "B": (_config(211, 96, [_layer("latent_attention", _latent(1, 16, 16, 32, 16, dims=8), _moe(4, 0, 1, 1, 1, 40, None)),
                            _layer("attention", _attention(2, 2, 16, 16, None, 0, diff=0.8), None)], emb_scale=1.0, eps=3e-6), 8, 5),
    # a width that is no multiple of 8, six query heads on one key head, sizes that are no multiples of 16, a window
    # longer than every test sequence, groups of one router output
    "C": (_config(257, 100, [_layer("attention", _C_ATT, _C_MOE), _layer("latent_attention", _latent(3, 40, 6, 20, 40, base=500.0), _C_MOE),
                             _layer("attention", _C_ATT, _C_MOE, 0)], emb_scale=2.0, eps=1e-6), 16, 11),
    # a window shorter than a page and more kept first keys than two pages hold; a window without kept keys
    "K": (_config(300, 128, [_layer("attention", _attention(2, 1, 32, 32, 7, 20), _moe(4, 4, 2, 2, 1, 48, 64)),
                             _layer("attention", _attention(4, 4, 16, 48, 13, 0, diff=0.1), _moe(4, 4, 2, 2, 1, 48, 64)),
                             _layer("latent_attention", _latent(4, 32, 16, 16, 48), None)], emb_scale=3.0), 8, 13),
    # sizes in sixteens (the matrix-core kernels), pages of 32, sixteen experts in four groups of which two stay
    "R": (_config(320, 128, [_layer("attention", _attention(4, 2, 64, 64, 48, 5), _moe(15, 1, 4, 4, 2, 64, 128)),
                             _layer("latent_attention", _latent(4, 64, 32, 48, 96, base=50000.0), _moe(15, 1, 4, 4, 2, 64, 128))]), 32, 7),
}


def make_weights(cfg: dict, seed: int, clear_routing: bool = False, mild: bool = False) -> Dict[str, torch.Tensor]:
    """bfloat16 weights of a size that makes every mechanism show in the logits.  ``mild``: scores a quarter as
    large, so that a softmax does not multiply the rounding of bfloat16 queries and keys (scores of 20 and more move
    by a tenth when their inputs are rounded, and so do the weights made of them).  ``clear_routing``: no router's
    logits depend on anything that rounding touches, so that a run in bfloat16 chooses as the plain implementation
    does (a row that goes to another expert is another computation, and so are the rows behind it).  The last n
    elements of the width are set aside (n router outputs): a token's embedding has one of them set (which one: its
    id modulo n), no sublayer writes to them, and the routers read nothing else, output e taking element j with the
    weight 3 / n (((p(e) + j) mod n) - (n - 1) / 2) for a permutation p a layer; all of it exact in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]
    sharp = 0.5 if mild else 1.0

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    w = {"embed": normal(cfg["vocab"], D, std=0.5), "final.norm": normal(D, std=0.1, mean=1.0),
         "head": normal(cfg["vocab"], D, std=D ** -0.5 * 4)}
    for i, layer in enumerate(cfg["layers"]):
        if "weights_of" in layer:
            continue
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = normal(D, std=0.1, mean=1.0)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[p + "mix.q"] = normal(H * 2 * d, D, std=D ** -0.5 * 2)
            w[p + "mix.k"] = normal(G * 2 * d, D, std=D ** -0.5 * 2)
            w[p + "mix.v"] = normal(G * e, D, std=D ** -0.5 * 1.5)
            w[p + "mix.g"] = normal(H, D, std=D ** -0.5 * 2)
            w[p + "mix.o"] = normal(D, H * e, std=(H * e) ** -0.5 * 1.5)
            w[p + "mix.q.norm"] = normal(d, std=0.2 * sharp, mean=2.0 * sharp)
            w[p + "mix.k.norm"] = normal(d, std=0.2 * sharp, mean=2.0 * sharp)
            for r in ("lq1", "lk1", "lq2", "lk2"):
                w[p + "mix." + r] = normal(d, std=0.15)
        else:
            H, d, r, e, n = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w[p + "mix.q"] = normal(H * (d + r), D, std=D ** -0.5 * 3 * sharp * sharp)
            w[p + "mix.dkv"] = normal(n + r, D, std=D ** -0.5 * 2)
            w[p + "mix.dkv.norm"] = normal(n, std=0.1, mean=1.0)
            w[p + "mix.uk"] = normal(H * d, n, std=n ** -0.5 * 2)
            w[p + "mix.uv"] = normal(H * e, n, std=n ** -0.5 * 1.5)
            w[p + "mix.o"] = normal(D, H * e, std=(H * e) ** -0.5 * 1.5)
        f = layer["mlp"]
        if f is not None:
            ff, outs = f["expert"]["ff"], f["router"]["experts"] + f["router"].get("identity", 0)
            w[p + "norm2"] = normal(D, std=0.1, mean=1.0)
            w[p + "mlp.router"] = normal(outs, D, std=D ** -0.5 * 0.6)
            w[p + "mlp.correction"] = normal(outs, std=0.05)
            for j in range(f["router"]["experts"]):
                w[f"{p}mlp.e{j}.gate"] = normal(ff, D, std=D ** -0.5 * 1.5)
                w[f"{p}mlp.e{j}.up"] = normal(ff, D, std=D ** -0.5 * 1.5)
                w[f"{p}mlp.e{j}.down"] = normal(D, ff, std=ff ** -0.5 * 1.5)
            if f.get("shared") is not None:
                sf = f["shared"]["ff"]
                w[p + "mlp.shared.gate"] = normal(sf, D, std=D ** -0.5 * 1.5)
                w[p + "mlp.shared.up"] = normal(sf, D, std=D ** -0.5 * 1.5)
                w[p + "mlp.shared.down"] = normal(D, sf, std=sf ** -0.5 * 1.5)
    if clear_routing:
        sizes = {layer["mlp"]["router"]["experts"] + layer["mlp"]["router"].get("identity", 0)
                 for layer in cfg["layers"] if layer["mlp"] is not None}
        assert len(sizes) == 1, "one number of router outputs in all layers"
        n = sizes.pop()
        w["embed"][:, D - n:] = 0.0
        w["embed"][torch.arange(cfg["vocab"]), D - n + torch.arange(cfg["vocab"]) % n] = 4.0 / cfg["embedding"]["scale"]
        for name in list(w):
            if name.endswith(("mix.o", ".down")):
                w[name][D - n:] = 0.0                            # nothing is written where the routers read
            if name.endswith("mlp.router"):
                order = torch.randperm(n, generator=g)
                w[name] = torch.zeros(n, D)
                w[name][:, D - n:] = (((order[:, None] + torch.arange(n)[None, :]) % n) - (n - 1) / 2) * 0.5
                w[name.replace("router", "correction")] = (torch.randperm(n, generator=g).float() - (n - 1) / 2) * 0.125
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


def write_folder(folder: str, cfg: dict, weights: Dict[str, torch.Tensor]) -> str:
    from tiny_llm_infer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(folder, "model.safetensors"), list(weights.items()))
    return folder


def make_folder(folder: str, name: str, clear_routing: bool = False, mild: bool = False) -> str:
    cfg, _, seed = SMALL[name]
    return write_folder(folder, cfg, make_weights(cfg, seed, clear_routing=clear_routing, mild=mild))


def plain_logits(folder: str, reqs: Dict[str, List[int]]) -> Dict[str, np.ndarray]:
    import plain_gimipel
    cfg, w = plain_gimipel.read_model(folder)
    return {rid: plain_gimipel.forward(cfg, w, toks).numpy() for rid, toks in reqs.items()}


def rows_with_a_clear_choice(folder: str, reqs: Dict[str, List[int]], margin: float) -> Dict[str, int]:
    """For every request, the number of leading rows whose routers all choose by more than ``margin``.  Rounding
    in bfloat16 can turn a closer call, after which that row and the rows behind it are another computation."""
    import plain_gimipel
    cfg, w = plain_gimipel.read_model(folder)
    out = {}
    for rid, toks in reqs.items():
        margins = []
        plain_gimipel.forward(cfg, w, toks, margins=margins)
        close = [any(layer[t] < margin for layer in margins) for t in range(len(toks))]
        out[rid] = close.index(True) if True in close else len(toks)
    return out


def plain_greedy(folder: str, prompt: List[int], new_tokens: int) -> List[int]:
    import plain_gimipel
    cfg, w = plain_gimipel.read_model(folder)
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(plain_gimipel.forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]
