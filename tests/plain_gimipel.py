"""The Gimipel decoder written out plainly: one function a mechanism, float64, whole sequences,
no cache, no batching, loops where a loop says it best.  What the engine is compared with; it
shares no code with the engine.

Notation: T positions, width D.  A block is  x <- x + n1(mixer(x)),  x <- x + n2(ff(x))  with
n1, n2 RMS norms of the sublayer's output; the sublayers read x itself.

``cfg`` is the parsed config.json (a dict), ``w`` maps tensor names to float64 tensors.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import torch

F = torch.float64


def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    kinds = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "I32": torch.int32}
    with open(path, "rb") as fh:
        raw = fh.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        t = torch.frombuffer(bytearray(raw[8 + hlen + b:8 + hlen + e]), dtype=kinds[info["dtype"]]).reshape(info["shape"])
        out[name] = t.to(F) if t.dtype.is_floating_point else t.clone()
    return out


def read_model(folder: str):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def visible(T: int, window: Optional[int], keep_first: int) -> torch.Tensor:
    """[T, T] booleans: row i sees column j."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    ok = j <= i
    if window is not None:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def softmax_rows(scores: torch.Tensor, ok: torch.Tensor) -> torch.Tensor:
    scores = scores.masked_fill(~ok, float("-inf"))
    return torch.softmax(scores, dim=-1)


def differential_attention(h: torch.Tensor, m: Dict, w: Dict[str, torch.Tensor], p: str, eps: float) -> torch.Tensor:
    """Two softmax maps a head over the same values, o = a1 - lambda a2, a unit-RMS head times
    (1 - diff), a gate a head, the output projection."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    diff = float(m["diff"])
    mask = m.get("mask") or {}
    q = (h @ w[p + "q"].T).view(T, H, 2, d)
    k = (h @ w[p + "k"].T).view(T, G, 2, d)
    v = (h @ w[p + "v"].T).view(T, G, e)
    q = rms_norm(q, w[p + "q.norm"], eps)
    k = rms_norm(k, w[p + "k.norm"], eps)
    lam = math.exp(float((w[p + "lq1"] * w[p + "lk1"]).sum())) - math.exp(float((w[p + "lq2"] * w[p + "lk2"]).sum())) + diff
    ok = visible(T, mask.get("size"), int(mask.get("keep_first", 0)))
    gate = torch.sigmoid(h @ w[p + "g"].T)                      # [T, H]
    heads = []
    for a in range(H):
        g = a // (H // G)
        maps = []
        for n in range(2):
            s = (q[:, a, n] @ k[:, g, n].T) * float(m["scale"])
            maps.append(softmax_rows(s, ok) @ v[:, g])
        o = maps[0] - lam * maps[1]
        o = rms_norm(o, None, eps) * (1.0 - diff)
        heads.append(o * gate[:, a:a + 1])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


def rotate_half(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """The first ``dims`` elements of the last axis turned: pair (i, i + dims/2) by the angle
    position * base^(-2i/dims); x is [T, ..., n] with positions [T]."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    a = positions.to(F).view(-1, *([1] * (x.dim() - 1))) * f
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), x[..., dims:]], dim=-1)


def latent_attention(h: torch.Tensor, m: Dict, w: Dict[str, torch.Tensor], p: str, eps: float) -> torch.Tensor:
    """Keys and values made from one normed latent vector a position, beside one turned key part
    that all heads share."""
    T = h.shape[0]
    H, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ w[p + "q"].T).view(T, H, d + r)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    k_turned = rotate_half(down[:, rank:], pos, m["rot"]["dims"], float(m["rot"]["base"]))          # [T, r]
    q_plain = q[..., :d]
    q_turned = rotate_half(q[..., d:], pos, m["rot"]["dims"], float(m["rot"]["base"]))             # [T, H, r]
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, e)
    ok = visible(T, None, 0)
    heads = []
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_turned[:, a] @ k_turned.T) * float(m["scale"])
        heads.append(softmax_rows(s, ok) @ v[:, a])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


def gated_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    z = h @ w[p + "gate"].T
    return ((z * torch.sigmoid(z)) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h: torch.Tensor, f: Dict, w: Dict[str, torch.Tensor], p: str, margins: Optional[list] = None):
    """Per position the chosen router outputs and their weights (lists of lists).  ``margins``: a list
    that takes, per position, by how much the choice was made (the smallest difference of choice scores
    between a group or an output that was taken and one that was not)."""
    r = f["router"]
    E, ident, top = r["experts"], int(r.get("identity", 0)), r["top"]
    groups = r.get("groups") or {}
    count = int(groups.get("count", 1))
    keep = int(groups.get("keep", count))
    n = E + ident
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)            # [T, n]
    choice = s + w[p + "correction"] if (p + "correction") in w else s.clone()
    per = n // count
    ids, weights = [], []
    for t in range(h.shape[0]):
        c = choice[t].clone()
        margin = float("inf")
        if keep < count:
            best = c.view(count, per).max(dim=1).values
            order = sorted(range(count), key=lambda g: (-float(best[g]), g))
            margin = float(best[order[keep - 1]] - best[order[keep]])
            for g in order[keep:]:
                c[g * per:(g + 1) * per] = float("-inf")
        ranked = sorted(range(n), key=lambda j: (-float(c[j]), j))
        chosen = ranked[:top]
        if top < n and c[ranked[top]] > float("-inf"):
            margin = min(margin, float(c[ranked[top - 1]] - c[ranked[top]]))
        if margins is not None:
            margins.append(margin)
        ids.append(chosen)
        weights.append([float(s[t, j]) for j in chosen])
    return ids, weights


def routed_experts(h: torch.Tensor, f: Dict, w: Dict[str, torch.Tensor], p: str, margins: Optional[list] = None) -> torch.Tensor:
    E = f["router"]["experts"]
    ids, weights = route(h, f, w, p, margins)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        row = h[t:t + 1]
        for j, a in zip(ids[t], weights[t]):
            out[t] += a * (row[0] if j >= E else gated_ff(row, w, f"{p}e{j}.")[0])
    if f.get("shared") is not None:
        out = out + gated_ff(h, w, p + "shared.")
    return out


def owner(cfg: Dict, i: int) -> int:
    while cfg["layers"][i].get("weights_of") is not None:
        i = cfg["layers"][i]["weights_of"]
    return i


def forward(cfg: Dict, w: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None,
            margins: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``residuals``: a list that takes the residual
    stream after every layer; ``margins``: one that takes, layer by layer, a list of every position's
    margin of the router's choice."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{owner(cfg, i)}."
        if layer["type"] == "attention":
            a = differential_attention(x, layer["mixer"], w, p + "mix.", eps)
        elif layer["type"] == "latent_attention":
            a = latent_attention(x, layer["mixer"], w, p + "mix.", eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(a, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            by_row = None if margins is None else []
            x = x + rms_norm(routed_experts(x, layer["mlp"], w, p + "mlp.", by_row), w[p + "norm2"], eps)
            if margins is not None:
                margins.append(by_row)
        if residuals is not None:
            residuals.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
