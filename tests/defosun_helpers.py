"""Shared by the Defosun tests: small configurations that differ in every size and option,
weights drawn so that every mechanism matters, and model folders of them."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import numpy as np
import torch


def _attention(heads, kv_heads, dim, dims, base=10000.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": float(dim ** -0.5 if scale is None else scale),
            "rot": {"dims": dims, "base": base}}


def _latent(heads, dim, rot_dim, vdim, rank, base=10000.0, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
            "scale": float((dim + rot_dim) ** -0.5 if scale is None else scale), "rot": {"dims": rot_dim, "base": base}}


def _lightning(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, limit, shared=None, shared_limit=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared, "limit": limit if shared_limit is None else shared_limit}
    return out


def _layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def _config(vocab, width, layers, streams=None, loop=None, eps=1e-5):
    out = {"architecture": "Defosun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        out["streams"] = streams
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


_A_MOE = _moe(6, 2, 32, 1.5, 48, 0.75)
_R_MOE = _moe(16, 4, 64, 1.25, 128, 2.0)
# name -> (config.json, page size of the engine in its tests, seed)
SMALL = {
    # three streams; the last two layers are passed twice; a quarter of every attention head is turned; value heads
    # of the latent attention longer than its key heads; experts and a shared expert with limits of their own
    "A": (_config(160, 64, [_layer("attention", _attention(4, 2, 16, 8), _dense(96)),
                            _layer("latent_attention", _latent(2, 16, 8, 24, 32), _A_MOE),
                            _layer("lightning", _lightning(2, 16, 24, [0.9, 0.99]), _A_MOE)], streams=3, loop=(1, 3, 2)), 16, 3),
    # one plain residual and no loop; as many key heads as query heads, every element of a head turned; a layer
    # without feed-forward; three lightning heads of sizes that are no multiples of 16, one of them without decay;
    # one latent head; one expert chosen of four, no shared expert, a limit that is rarely met
    "B": (_config(211, 96, [_layer("attention", _attention(2, 2, 32, 32, base=500.0), None),
                            _layer("lightning", _lightning(3, 20, 12, [0.5, 1.0, 0.97]), _dense(80)),
                            _layer("latent_attention", _latent(1, 16, 16, 32, 16), _moe(4, 1, 40, 7.0))], eps=3e-6), 8, 5),
    # one stream (hyper-connections all the same), a width that is no multiple of 8, six query heads on one key head,
    # one lightning head, every expert chosen, all layers passed twice
    "C": (_config(257, 100, [_layer("attention", _attention(6, 1, 24, 6, scale=0.3), _moe(3, 3, 24, 0.5, 16, 0.5)),
                             _layer("lightning", _lightning(1, 40, 20, [0.93]), None),
                             _layer("latent_attention", _latent(3, 40, 6, 20, 40, base=500.0), _dense(56))],
                  streams=1, loop=(0, 3, 2), eps=1e-6), 16, 11),
    # sizes in sixteens (the matrix-core kernels), pages of 32, two streams, the first two layers passed twice
    "R": (_config(320, 128, [_layer("attention", _attention(8, 2, 64, 16, base=100000.0), _R_MOE),
                             _layer("lightning", _lightning(4, 64, 32, [0.8, 0.95, 0.99, 0.999]), _dense(256)),
                             _layer("latent_attention", _latent(4, 64, 32, 48, 80, base=30000.0), _R_MOE)],
                  streams=2, loop=(0, 2, 2)), 32, 7),
}


def make_weights(cfg: dict, seed: int, clear_routing: bool = False, mild: bool = False) -> Dict[str, torch.Tensor]:
    """bfloat16 weights of a size that makes every mechanism show in the logits.  ``mild``: queries and keys half as large,
    so that a softmax does not multiply the rounding of bfloat16 queries and keys.  ``clear_routing``: no router's
    choice depends on anything that rounding touches, so that a run in bfloat16 chooses as the plain
    implementation does (a row that goes to another expert is another computation).  The last n elements of the
    width are set aside (n: the most experts of a layer): a token's embedding has one of them set (which one: its
    id modulo n), no sublayer writes to them, and the routers read nothing else, expert e taking element j with
    one of n levels; a row's logits are then those levels times one positive factor, whose order no rounding changes."""
    g = torch.Generator().manual_seed(seed)
    D, S = cfg["width"], cfg.get("streams")
    sharp = 0.5 if mild else 1.0

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    w = {"embed": normal(cfg["vocab"], D, std=0.5), "final.norm": normal(D, std=0.1),
         "head": normal(cfg["vocab"], D, std=D ** -0.5 * 4)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = normal(D, std=0.1)
        if layer["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            w[p + "mix.q"] = normal(H * d, D, std=D ** -0.5 * 3 * sharp)
            w[p + "mix.q.b"] = normal(H * d, std=0.3)
            w[p + "mix.k"] = normal(G * d, D, std=D ** -0.5 * 2 * sharp)
            w[p + "mix.k.b"] = normal(G * d, std=0.3)
            w[p + "mix.sink"] = normal(H, std=1.0, mean=1.0)
            w[p + "mix.o"] = normal(D, H * d, std=(H * d) ** -0.5 * 1.5)
            w[p + "mix.o.b"] = normal(D, std=0.2)
        elif layer["type"] == "latent_attention":
            H, d, r, e, n = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w[p + "mix.q"] = normal(H * (d + r), D, std=D ** -0.5 * 3 * sharp)
            w[p + "mix.dkv"] = normal(n + r, D, std=D ** -0.5 * 2)
            w[p + "mix.dkv.norm"] = normal(n, std=0.1, mean=1.0)
            w[p + "mix.uk"] = normal(H * d, n, std=n ** -0.5 * 2 * sharp)
            w[p + "mix.uv"] = normal(H * e, n, std=n ** -0.5 * 1.5)
            w[p + "mix.sink"] = normal(H, std=1.0, mean=1.0)
            w[p + "mix.o"] = normal(D, H * e, std=(H * e) ** -0.5 * 1.5)
        else:
            H, d, e = m["heads"], m["dim"], m["vdim"]
            for r, n in (("q", H * d), ("k", H * d), ("v", H * e), ("g", H * e)):
                w[p + "mix." + r] = normal(n, D, std=D ** -0.5 * 1.5)
            w[p + "mix.norm"] = normal(H * e, std=0.1, mean=1.0)
            w[p + "mix.o"] = normal(D, H * e, std=(H * e) ** -0.5 * 1.5)
        f = layer["mlp"]
        if f is not None:
            w[p + "norm2"] = normal(D, std=0.1)
            if f["kind"] == "dense":
                ff = f["ff"]
                w[p + "mlp.gate"] = normal(ff, D, std=D ** -0.5 * 1.5)
                w[p + "mlp.up"] = normal(ff, D, std=D ** -0.5 * 1.5)
                w[p + "mlp.down"] = normal(D, ff, std=ff ** -0.5 * 1.5)
            else:
                ff, E = f["expert"]["ff"], f["router"]["experts"]
                w[p + "mlp.router"] = normal(E, D, std=D ** -0.5 * 1.5)
                for j in range(E):
                    w[f"{p}mlp.e{j}.gate"] = normal(ff, D, std=D ** -0.5 * 1.5)
                    w[f"{p}mlp.e{j}.up"] = normal(ff, D, std=D ** -0.5 * 1.5)
                    w[f"{p}mlp.e{j}.down"] = normal(D, ff, std=ff ** -0.5 * 1.5)
                if f.get("shared") is not None:
                    sf = f["shared"]["ff"]
                    w[p + "mlp.shared.gate"] = normal(sf, D, std=D ** -0.5 * 1.5)
                    w[p + "mlp.shared.up"] = normal(sf, D, std=D ** -0.5 * 1.5)
                    w[p + "mlp.shared.down"] = normal(D, sf, std=sf ** -0.5 * 1.5)
                    w[p + "mlp.shared.sg"] = normal(1, D, std=D ** -0.5 * 2)
        if S:
            for q in (1, 2) if f is not None else (1,):
                w[f"{p}hc{q}.in"] = normal(S, std=0.1, mean=1.0 / S)
                w[f"{p}hc{q}.out"] = normal(S, std=0.15, mean=0.6)
                w[f"{p}hc{q}.mix"] = torch.eye(S) * (1.0 if S == 1 else 0.8) + normal(S, S, std=0.1).abs()      # (one stream: nothing else keeps the embedding)
    if clear_routing:
        n = max([layer["mlp"]["router"]["experts"] for layer in cfg["layers"]
                 if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe"], default=0)
        if n:
            w["embed"][:, D - n:] = 0.0
            w["embed"][torch.arange(cfg["vocab"]), D - n + torch.arange(cfg["vocab"]) % n] = 4.0
            for name in list(w):
                if name.endswith(("mix.o", ".down", "mix.o.b")):
                    w[name][D - n:] = 0.0                            # nothing is written where the routers read
                if name.endswith("mlp.router"):
                    E = w[name].shape[0]
                    order = torch.randperm(n, generator=g)[:E]
                    w[name] = torch.zeros(E, D)
                    w[name][:, D - n:] = (((order[:, None] + torch.arange(n)[None, :]) % n) - (n - 1) / 2) * 0.5
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
    import plain_defosun
    cfg, w = plain_defosun.read_model(folder)
    return {rid: plain_defosun.forward(cfg, w, toks).numpy() for rid, toks in reqs.items()}


def plain_greedy(folder: str, prompt: List[int], new_tokens: int) -> List[int]:
    import plain_defosun
    cfg, w = plain_defosun.read_model(folder)
    toks = list(prompt)
    for _ in range(new_tokens):
        toks.append(int(plain_defosun.forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]
