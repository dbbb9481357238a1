"""Attention with grouped heads over the paged cache whose softmax may have a sink, whose
projections may have biases, and whose values may be its keys.

For the rows h_p of one sequence (H query heads, G key/value heads of size d, query head a reads
key head a // (H / G)):

    q_p = Wq h_p (+ bq),  k_p = Wk h_p (+ bk)
    v_p = k_p as projected, before it is turned    (``values`` = "keys": there is no Wv)
          or Wv h_p (+ bv)                          (``values`` = "projected")
    q, k: the first ``rotary_dim`` elements of every head turned by the position (``position``)
    s_ij = (q_i . k_j) * scale,   j <= i (and i - j < ``window``, if one is given)
    w_ij = exp(s_ij) / (sum_j' exp(s_ij') + exp(sink_a))        (``sink``: one learned logit a head
                                                                   that has no key and no value)
    out_i = Wo [sum_j w_ij v_j]_a (+ bo)

Names of weights that the spec leaves out do not exist: ``q_bias``, ``k_bias``, ``v_bias``,
``o_bias``, ``sink``, ``v``.  Turned keys and the values go into the cache (records "k" and "v" of
the stock attention part); scores, softmax and the sink are float32.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import CacheNeed
from ..weights.loader import TensorDecl
from .base import BuildEnv, Mixer, RotaryTables, StepView, build_part, register_part
from .linear import as_matrix, fuse_rows

VALUES = ("keys", "projected")


class SinkAttention(Mixer):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.scale = float(p["scale"])
        self.values = str(p.get("values", "projected"))
        self.window = None if p.get("window") is None else int(p["window"])
        if self.values not in VALUES:
            raise ValueError(f"values '{self.values}' are not known; known: {', '.join(VALUES)}")
        if self.heads % self.kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if self.window is not None and self.window <= 0:
            raise ValueError("window must be positive")
        self.q_dim = self.heads * self.head_dim
        self.kv_dim = self.kv_heads * self.head_dim
        self.position = build_part("position", spec.parts["position"]) if "position" in spec.parts else None

    def _roles(self):
        return ["q", "k"] + (["v"] if self.values == "projected" else [])

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        sizes = {"q": self.q_dim, "k": self.kv_dim, "v": self.kv_dim}
        out = []
        for r in self._roles():
            out.append(TensorDecl(n[r], (sizes[r], self.hidden)))
            if r + "_bias" in n:
                out.append(TensorDecl(n[r + "_bias"], (sizes[r],)))
        out.append(TensorDecl(n["o"], (self.hidden, self.q_dim)))
        if "o_bias" in n:
            out.append(TensorDecl(n["o_bias"], (self.hidden,)))
        if "sink" in n:
            out.append(TensorDecl(n["sink"], (self.heads,), "normal(0.0,1.0)"))
        return out + (self.position.tensors() if self.position is not None else [])

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_sized_attention(self.heads, self.kv_heads, self.head_dim, self.head_dim)
        self.rotary = None
        if self.position is not None:
            self.position.load(weights, env)
            tables = self.position.rotary()
            if tables is not None:
                tables = RotaryTables(*tables)
                if tables.pairing != "half":
                    raise ValueError(f"the kernel of this attention turns the pairs (i, i + dims / 2), not '{tables.pairing}'")
                if tables.rotary_dim > self.head_dim:
                    raise ValueError(f"{tables.rotary_dim} turned elements do not fit a head of {self.head_dim}")
                self.rotary = (tables.cos, tables.sin, int(tables.rotary_dim))
        roles = self._roles()
        self.w_in = fuse_rows([weights[n[r]] for r in roles], env)
        self.bias = None
        if any(r + "_bias" in n for r in roles):
            sizes = {"q": self.q_dim, "k": self.kv_dim, "v": self.kv_dim}
            self.bias = torch.cat([weights[n[r + "_bias"]].to(torch.float32) if r + "_bias" in n
                                   else torch.zeros(sizes[r], dtype=torch.float32, device=env.device) for r in roles]).contiguous()
        self.sinks = weights[n["sink"]].to(torch.float32).contiguous() if "sink" in n else None
        self.w_o = as_matrix(weights[n["o"]], env)
        self.o_bias = weights[n["o_bias"]].to(torch.float32).contiguous() if "o_bias" in n else None

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed.keys_and_values(self.kv_heads, self.head_dim, self.window)

    def workspace_elems(self, rows: int) -> int:
        return rows * (2 * (self.q_dim + 2 * self.kv_dim) + 2 * self.q_dim)

    def forward(self, x: torch.Tensor, step: StepView):
        ops = self.env.ops
        proj = ops.linear(x, self.w_in)
        o = ops.sink_attention(proj, step, step.cache, self.heads, self.kv_heads, self.head_dim, self.bias, self.rotary,
                               self.scale, self.sinks, self.window, self.values == "keys")
        if self.o_bias is None:
            return ops.linear(o, self.w_o, deferred=True)
        return ops.add_bias(ops.linear(o, self.w_o), self.o_bias)


register_part("mixer", "sink_attention", SinkAttention)
