"""The Defosun decoder written out plainly: one function a mechanism, float64, whole sequences,
no cache, no batching, loops where a loop says it best.  What the engine is compared with; it
shares no code with the engine.

Notation: T positions, width D, S residual streams.  A sublayer reads u = sum_s in[s] x_s,
gives y = sublayer(norm(u)) and is written back as x_t = sum_s mix[s, t] x_s + out[t] y; without
streams it is x = x + sublayer(norm(x)).  A norm's weight is stored around zero: the multiplier
is 1 + w.

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


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def zero_centred_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * (1.0 + weight)


def turn(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, neighbours: bool) -> torch.Tensor:
    """The first ``dims`` elements of the last axis turned by the position; pair i is (i, i + dims/2),
    or (2i, 2i + 1) with ``neighbours``; angle = position * base^(-2i/dims).  x is [T, ..., n]."""
    out = x.clone()
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if neighbours else (i, i + dims // 2)
        angle = positions.to(F) * base ** (-2.0 * i / dims)
        angle = angle.view(-1, *([1] * (x.dim() - 2)))
        c, s = torch.cos(angle), torch.sin(angle)
        out[..., a] = x[..., a] * c - x[..., b] * s
        out[..., b] = x[..., b] * c + x[..., a] * s
    return out


def softmax_with_sink(scores: torch.Tensor, sink: Optional[float]) -> torch.Tensor:
    """Causal softmax over the rows of [T, T] scores whose denominator also holds exp(sink)."""
    T = scores.shape[0]
    out = torch.zeros_like(scores)
    for i in range(T):
        row = scores[i, :i + 1]
        top = max(float(row.max()), float("-inf") if sink is None else sink)
        e = torch.exp(row - top)
        out[i, :i + 1] = e / (e.sum() + (0.0 if sink is None else math.exp(sink - top)))
    return out


def key_valued_attention(h: torch.Tensor, m: Dict, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    """Grouped heads; the values are the keys as projected, before they are turned."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    G = m.get("kv_heads") or H
    pos = torch.arange(T)
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
    v = k
    rot = m["rot"]
    q = turn(q, pos, rot["dims"], float(rot["base"]), False)
    k = turn(k, pos, rot["dims"], float(rot["base"]), False)
    heads = []
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * float(m["scale"])
        heads.append(softmax_with_sink(s, float(w[p + "sink"][a])) @ v[:, g])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T + w[p + "o.b"]


def latent_attention(h: torch.Tensor, m: Dict, w: Dict[str, torch.Tensor], p: str, eps: float) -> torch.Tensor:
    """Keys and values made from one normed latent vector a position, beside one turned key part
    that all heads share."""
    T = h.shape[0]
    H, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    base = float(m["rot"]["base"])
    q = (h @ w[p + "q"].T).view(T, H, d + r)
    down = h @ w[p + "dkv"].T
    c = unit_rms(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_turned = turn(down[:, rank:], pos, r, base, True)                 # [T, r]
    q_turned = turn(q[..., d:], pos, r, base, True)                    # [T, H, r]
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, e)
    heads = []
    for a in range(H):
        s = (q[:, a, :d] @ k_plain[:, a].T + q_turned[:, a] @ k_turned.T) * float(m["scale"])
        heads.append(softmax_with_sink(s, float(w[p + "sink"][a])) @ v[:, a])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def lightning(h: torch.Tensor, m: Dict, w: Dict[str, torch.Tensor], p: str, eps: float,
              state: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A matrix of state a head that decays by a constant a token and takes k v^T."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).view(T, H, d)
    k = silu(h @ w[p + "k"].T).view(T, H, d)
    v = silu(h @ w[p + "v"].T).view(T, H, e)
    S = torch.zeros(H, d, e, dtype=F) if state is None else state
    o = torch.zeros(T, H, e, dtype=F)
    for t in range(T):
        for a in range(H):
            S[a] = float(m["decay"][a]) * S[a] + torch.outer(k[t, a], v[t, a])
            o[t, a] = S[a].T @ q[t, a]
    y = unit_rms(o.reshape(T, H * e), eps) * w[p + "norm"]
    return (y * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def gated_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def limited_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route(h: torch.Tensor, f: Dict, w: Dict[str, torch.Tensor], p: str, margins: Optional[list] = None):
    """Per position the chosen experts and their weights (lists of lists).  ``margins`` takes, per
    position, the difference of the scores of the last expert taken and the first one left."""
    E, top = f["router"]["experts"], f["router"]["top"]
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)
    ids, weights = [], []
    for t in range(h.shape[0]):
        ranked = sorted(range(E), key=lambda j: (-float(s[t, j]), j))
        if margins is not None:
            margins.append(float(s[t, ranked[top - 1]] - s[t, ranked[top]]) if top < E else float("inf"))
        ids.append(ranked[:top])
        weights.append([float(s[t, j]) for j in ranked[:top]])
    return ids, weights


def routed_experts(h: torch.Tensor, f: Dict, w: Dict[str, torch.Tensor], p: str, margins: Optional[list] = None) -> torch.Tensor:
    ids, weights = route(h, f, w, p, margins)
    limit = float(f["expert"]["limit"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j, a in zip(ids[t], weights[t]):
            out[t] += a * limited_ff(h[t:t + 1], w, f"{p}e{j}.", limit)[0]
    if f.get("shared") is not None:
        gate = torch.sigmoid(h @ w[p + "shared.sg"].T)                  # [T, 1]
        out = out + gate * limited_ff(h, w, p + "shared.", float(f["shared"]["limit"]))
    return out


def run_order(cfg: Dict) -> List[int]:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg: Dict, w: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None,
            margins: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``residuals`` takes the residual stream (the sum of
    the streams) after every layer run; ``margins``, run by run, every position's router margin."""
    eps = float(cfg["norm"]["eps"])
    S = cfg.get("streams")
    x = w["embed"][torch.tensor(tokens)]
    xs = [x.clone() for _ in range(S)] if S else None

    def sublayer(q: int, p: str, fn):
        nonlocal x, xs
        if xs is None:
            x = x + fn(zero_centred_norm(x, w[f"{p}norm{q}"], eps))
            return
        hc = f"{p}hc{q}."
        u = sum(w[hc + "in"][s] * xs[s] for s in range(S))
        y = fn(zero_centred_norm(u, w[f"{p}norm{q}"], eps))
        xs = [sum(w[hc + "mix"][s, t] * xs[s] for s in range(S)) + w[hc + "out"][t] * y for t in range(S)]

    for i in run_order(cfg):
        layer, p = cfg["layers"][i], f"l{i}."
        m = layer["mixer"]
        if layer["type"] == "attention":
            sublayer(1, p, lambda h: key_valued_attention(h, m, w, p + "mix."))
        elif layer["type"] == "latent_attention":
            sublayer(1, p, lambda h: latent_attention(h, m, w, p + "mix.", eps))
        elif layer["type"] == "lightning":
            sublayer(1, p, lambda h: lightning(h, m, w, p + "mix.", eps))
        else:
            raise ValueError(layer["type"])
        f = layer.get("mlp")
        if f is not None:
            if f["kind"] == "dense":
                sublayer(2, p, lambda h: gated_ff(h, w, p + "mlp."))
            elif f["kind"] == "moe":
                by_row = None if margins is None else []
                sublayer(2, p, lambda h: routed_experts(h, f, w, p + "mlp.", by_row))
                if margins is not None:
                    margins.append(by_row)
            else:
                raise ValueError(f["kind"])
        if residuals is not None:
            residuals.append((sum(xs) if xs is not None else x).clone())
    final = sum(xs) if xs is not None else x
    return zero_centred_norm(final, w["final.norm"], eps) @ w["head"].T
