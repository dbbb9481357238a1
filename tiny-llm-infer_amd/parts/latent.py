"""Attention whose keys and values are made from one latent vector a position ("latent attention").

With H heads, ``head_dim`` d elements of a query/key head that are not turned and ``rotary_dim``
r that are, value heads of e and a latent vector of ``kv_rank`` n:

    q = W_q x                       [H, d + r] a position, head by head as [plain, turned part]
    W_down x                        [n + r]: the first n, RMS-normed with a weight, are the latent
                                    vector c; the last r, not normed, are one key part for all heads
    k_h = [W_uk,h c | key part],  v_h = W_uv,h c
    s_ij = (q_plain . k_plain + q_turned . k_turned) * scale,   j <= i,   softmax, sum of values

The position encoding (``position``) turns the r-part of every query head and the shared key
part (pairs (i, i + dims/2), or neighbours for an encoding that says so).  With a ``sink`` (one
learned logit a head) the softmax's denominator also holds exp(sink).  The cache keeps, for a position, c and the turned key part and nothing else (record
"latent", ``[slot, n + r]``): q_plain . (W_uk,h c) = (W_uk,h^T q_plain) . c, so every head's
query is taken into the latent space by a small product of its own and all heads then read the
same cached vectors, and the weighted sum of the c of the seen positions goes through W_uv,h
afterwards (sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import PAGE, CacheNeed, CacheRecord
from ..weights.loader import TensorDecl
from .base import ROTARY_PAIRINGS, BuildEnv, Mixer, RotaryTables, StepView, build_part, register_part
from .linear import as_matrix, fuse_rows


class LatentAttention(Mixer):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.dim = int(p["head_dim"])
        self.rot = int(p["rotary_dim"])
        self.vdim = int(p.get("value_dim") or self.dim)
        self.rank = int(p["kv_rank"])
        self.scale = float(p["scale"])
        self.position = build_part("position", spec.parts["position"])
        self.latent_norm = build_part("norm", spec.parts["latent_norm"])

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        return [TensorDecl(n["q"], (self.heads * (self.dim + self.rot), self.hidden)),
                TensorDecl(n["down"], (self.rank + self.rot, self.hidden)),
                TensorDecl(n["up_k"], (self.heads * self.dim, self.rank)),
                TensorDecl(n["up_v"], (self.heads * self.vdim, self.rank)),
                TensorDecl(n["o"], (self.hidden, self.heads * self.vdim))] + \
            ([TensorDecl(n["sink"], (self.heads,), "normal(0.0,1.0)")] if "sink" in n else []) + \
            self.latent_norm.tensors() + self.position.tensors()

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_sized_attention(self.heads, 1, self.rank + self.rot, self.rank)
        self.position.load(weights, env)
        self.latent_norm.load(weights, env)
        tables = self.position.rotary()
        if tables is None:
            raise ValueError("the position encoding of this attention must be a rotation")
        tables = RotaryTables(*tables)
        if tables.pairing not in ROTARY_PAIRINGS:
            raise ValueError(f"rotary pairing '{tables.pairing}' is not known; known: {', '.join(ROTARY_PAIRINGS)}")
        if tables.rotary_dim > self.rot:
            raise ValueError(f"{tables.rotary_dim} turned elements do not fit a part of {self.rot}")
        self.rotary = (tables.cos, tables.sin, int(tables.rotary_dim))
        # The kernels turn the pairs (i, i + dims / 2).  An encoding that pairs neighbours (2i, 2i + 1) is served
        # by them all the same: a score does not change when the turned parts of q and of the key are permuted
        # alike, so the rows that make those parts are put in the order 0, 2, 4, .., 1, 3, 5, .. once, here.
        w_q, w_down = weights[n["q"]], weights[n["down"]]
        if tables.pairing == "interleaved":
            rd = int(tables.rotary_dim)
            order = torch.cat([torch.arange(0, rd, 2), torch.arange(1, rd, 2), torch.arange(rd, self.rot)]).to(w_q.device)
            per = self.dim + self.rot
            q_rows = torch.cat([torch.arange(self.dim, device=w_q.device), self.dim + order])
            w_q = w_q.view(self.heads, per, self.hidden)[:, q_rows].reshape(self.heads * per, self.hidden)
            w_down = torch.cat([w_down[:self.rank], w_down[self.rank:][order]], dim=0)
        rms = self.latent_norm.as_rms()
        if rms is None or tuple(rms[0].shape) != (self.rank,):
            raise ValueError("the norm of the latent vector must be an RMS norm over its elements")
        self.norm_weight, self.norm_eps = rms[0], float(rms[1])
        self.w_in = fuse_rows([w_q, w_down], env)
        # a sink: one learned logit a head in the softmax's denominator, with no key and no value
        self.sinks = weights[n["sink"]].to(torch.float32).contiguous() if "sink" in n else None
        # a matrix a head, row-major: into the latent space [H, n, d] (W_uk of the head, transposed) and out of it [H, e, n]
        self.w_qk = weights[n["up_k"]].to(env.dtype).view(self.heads, self.dim, self.rank).transpose(1, 2).contiguous()
        self.w_v = weights[n["up_v"]].to(env.dtype).view(self.heads, self.vdim, self.rank).contiguous()
        self.w_o = as_matrix(weights[n["o"]], env)

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed((CacheRecord("latent", (PAGE, self.rank + self.rot)),))

    def workspace_elems(self, rows: int) -> int:
        key = self.rank + self.rot
        return rows * (2 * (self.heads * (self.dim + self.rot) + key) + self.heads * (key + self.rank + self.vdim))

    def forward(self, x: torch.Tensor, step: StepView) -> torch.Tensor:
        ops = self.env.ops
        proj = ops.linear(x, self.w_in)
        o = ops.latent_attention(proj, step, step.cache, self.heads, self.dim, self.rot, self.rank, self.vdim,
                                 self.norm_weight, self.norm_eps, self.rotary, self.scale, self.w_qk, self.w_v,
                                 **({} if self.sinks is None else {"sinks": self.sinks}))
        return ops.linear(o, self.w_o)


register_part("mixer", "latent_attention", LatentAttention)
