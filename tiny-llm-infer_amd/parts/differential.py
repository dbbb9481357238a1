"""Attention with two softmax maps a head ("differential attention") over the paged cache.

q has heads * 2 * dim rows and k has kv_heads * 2 * dim, head by head as [map 1, map 2]; v has
kv_heads * vdim.  Every head and map of q and of k is RMS-normed over its dim elements with one
weight vector (``q_norm``, ``k_norm``).  There is no rotation: positions enter through the mask
alone.  Map m of head h scores against map m of key head h // (heads / kv_heads),

    s_ij = (q_i . k_j) * scale,      i sees j  <=>  j <= i and (i - j < window or j < keep_first)

(no ``window``: every j <= i), softmax over the seen keys, and both maps weigh the same values.
With a1, a2 the two outputs of a head:

    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff          (one number a layer, float32, at load)
    o = a1 - lambda a2;   o <- o / sqrt(mean(o^2) + eps) * (1 - diff);   o <- o * sigmoid(w_g[h] . x)

and the output projection reads the heads side by side.  The gate's logits are rows of the same
product that gives q, k and v.

The cache keeps the normed keys ``[kv head * 2 + map, slot, dim]`` and the values transposed
``[kv head, vdim, slot]``; with a window its pages are given back as the window passes, those of
the first ``keep_first`` positions excepted.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..cache.manager import PAGE, CacheNeed, CacheRecord
from ..weights.loader import TensorDecl
from .base import BuildEnv, Mixer, StepView, build_part, register_part
from .linear import as_matrix, fuse_rows


class DifferentialAttention(Mixer):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.dim = int(p["head_dim"])
        self.vdim = int(p.get("value_dim") or self.dim)
        self.scale = float(p["scale"])
        self.diff = float(p["diff"])
        self.eps = float(p["norm_eps"])
        self.window = None if p.get("window") is None else int(p["window"])
        self.keep_first = int(p.get("keep_first") or 0) if self.window is not None else 0
        if self.heads % self.kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if self.window is not None and self.window <= 0:
            raise ValueError("window must be positive")
        self.q_norm = build_part("norm", spec.parts["q_norm"])
        self.k_norm = build_part("norm", spec.parts["k_norm"])

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        out = [TensorDecl(n["q"], (self.heads * 2 * self.dim, self.hidden)),
               TensorDecl(n["k"], (self.kv_heads * 2 * self.dim, self.hidden)),
               TensorDecl(n["v"], (self.kv_heads * self.vdim, self.hidden)),
               TensorDecl(n["gate"], (self.heads, self.hidden)),
               TensorDecl(n["o"], (self.hidden, self.heads * self.vdim))]
        out += [TensorDecl(n[role], (self.dim,)) for role in ("lq1", "lk1", "lq2", "lk2")]
        return out + self.q_norm.tensors() + self.k_norm.tensors()

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_sized_attention(self.heads, self.kv_heads, self.dim, self.vdim)
        self.head_norms = []
        for role, norm in (("q", self.q_norm), ("k", self.k_norm)):
            norm.load(weights, env)
            rms = norm.as_rms()
            if rms is None or abs(float(rms[1]) - self.eps) > 0.0:
                raise ValueError(f"the {role} norm of this attention must be an RMS norm with the layer's eps")
            if tuple(rms[0].shape) != (self.dim,):
                raise ValueError(f"the {role} norm has {tuple(rms[0].shape)} weights, a head's map has {self.dim} elements")
            self.head_norms.append(rms[0])
        l = {role: weights[n[role]].to(torch.float32) for role in ("lq1", "lk1", "lq2", "lk2")}
        first = float((l["lq1"] * l["lk1"]).sum(dtype=torch.float32))
        second = float((l["lq2"] * l["lk2"]).sum(dtype=torch.float32))
        self.lam = math.exp(first) - math.exp(second) + self.diff
        self.w_in = fuse_rows([weights[n["q"]], weights[n["k"]], weights[n["v"]], weights[n["gate"]]], env)
        self.w_o = as_matrix(weights[n["o"]], env)

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed((CacheRecord("k", (self.kv_heads * 2, PAGE, self.dim)),
                          CacheRecord("v", (self.kv_heads, self.vdim, PAGE))), self.window, keep_first=self.keep_first)

    def workspace_elems(self, rows: int) -> int:
        q, k, v = self.heads * 2 * self.dim, self.kv_heads * 2 * self.dim, self.kv_heads * self.vdim
        return rows * (2 * (q + k + v + self.heads) + q + 3 * 2 * self.heads * self.vdim)

    def forward(self, x: torch.Tensor, step: StepView) -> torch.Tensor:
        ops = self.env.ops
        proj = ops.linear(x, self.w_in)
        o = ops.differential_attention(proj, step, step.cache, self.heads, self.kv_heads, self.dim, self.vdim,
                                       self.head_norms[0], self.head_norms[1], self.eps, self.scale, self.lam,
                                       1.0 - self.diff, self.window, self.keep_first)
        return ops.linear(o, self.w_o)


register_part("mixer", "differential_attention", DifferentialAttention)
