"""Routed experts: a feed-forward of E small gated feed-forwards of which every row uses ``top``,
beside an optional shared one that every row uses.

    s = sigmoid(W_router h)   or   softmax(W_router h)        [E + I], float32     (``score``)
    c = s + correction   (a vector of the checkpoint, where the spec names one): what the choice looks at
    the router's outputs form ``groups`` equal groups of neighbours; a group's score is the sum of its two
        largest c, or its largest c (``group_score``: "top2", "max"); outputs outside the ``keep`` best
        groups cannot be chosen
    chosen = the ``top`` largest c among the rest;  weight_j = s_j / (sum of the chosen s + 1e-20) * scale,
        or s_j * scale (``normalize`` false)
    out = sum_j weight_j expert_j(h)  +  sigmoid(w_sg . h) * shared(h)   (or + shared(h), where the spec
        names no gate for the shared expert)
    expert(h) = W_down (silu(W_gate h) * (W_up h));  the last I (``identity``) router outputs stand for
        experts without matrices whose output is h itself
    ``activation`` "limited": an expert's hidden units are g * sigmoid(slope * g) * (u + 1) with
        g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit)  (``limit``, ``gate_slope``; the shared
        expert with ``shared_limit``)

The router's product gives float32 (the row of the shared expert's gate rides along as one more
row of that matrix); scores, choice and weights are float32.  A row's chosen experts are added
in the order of the choice, whatever else is in the step.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorDecl
from .base import BuildEnv, FeedForward, StepView, register_part
from .linear import GatedMatrix, as_matrix, fuse_rows


class RoutedExperts(FeedForward):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.experts = int(p["experts"])                  # experts with matrices
        self.identity = int(p.get("identity") or 0)       # router outputs behind them whose expert hands h on
        self.outputs = self.experts + self.identity
        self.score = str(p.get("score", "sigmoid"))
        self.group_score = str(p.get("group_score", "top2"))
        self.normalize = bool(p.get("normalize", True))
        self.top = int(p["top"])
        self.groups = int(p.get("groups") or 1)
        self.keep = int(p.get("keep") or self.groups)
        self.scale = float(p.get("scale", 1.0))
        self.inter = int(p["intermediate_size"])
        shared = p.get("shared_intermediate_size")
        self.shared_inter = None if shared is None else int(shared)
        if self.experts < 1 or self.outputs % self.groups or not 1 <= self.keep <= self.groups \
                or not 1 <= self.top <= self.keep * (self.outputs // self.groups):
            raise ValueError(f"{self.outputs} router outputs in {self.groups} groups, {self.keep} kept, cannot give {self.top}")
        self.activation = str(p.get("activation", "silu"))
        if self.activation not in ("silu", "limited"):
            raise ValueError(f"activation '{self.activation}' is not known; known: silu, limited")
        self.limit = float(p.get("limit", 0.0)) if self.activation == "limited" else 0.0
        self.shared_limit = float(p.get("shared_limit", self.limit)) if self.activation == "limited" else 0.0
        self.slope = float(p.get("gate_slope", 1.0))
        if self.activation == "limited" and (self.limit <= 0.0 or self.shared_limit <= 0.0):
            raise ValueError("the limited activation needs a positive limit")
        self.correction_name = spec.names.get("correction")
        self.shared_gated = "shared_scale" in spec.names

    def _expert(self, j: int, role: str) -> str:
        return self.spec.names["experts"].format(j) + role

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        out = [TensorDecl(n["router"], (self.outputs, self.hidden))]
        if self.correction_name is not None:
            out.append(TensorDecl(self.correction_name, (self.outputs,)))
        for j in range(self.experts):
            out += [TensorDecl(self._expert(j, "gate"), (self.inter, self.hidden)),
                    TensorDecl(self._expert(j, "up"), (self.inter, self.hidden)),
                    TensorDecl(self._expert(j, "down"), (self.hidden, self.inter))]
        if self.shared_inter is not None:
            out += [TensorDecl(n["shared_gate"], (self.shared_inter, self.hidden)),
                    TensorDecl(n["shared_up"], (self.shared_inter, self.hidden)),
                    TensorDecl(n["shared_down"], (self.hidden, self.shared_inter))]
            if self.shared_gated:
                out.append(TensorDecl(n["shared_scale"], (1, self.hidden)))
        return out

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_expert_sizes(self.outputs, self.top, self.groups, self.keep, self.hidden, self.inter)
        if (self.score, self.group_score) != ("sigmoid", "top2"):
            env.ops.check_router(self.score, self.group_score)
        self.has_gate = self.shared_inter is not None and self.shared_gated
        rows = [weights[n["router"]]] + ([weights[n["shared_scale"]]] if self.has_gate else [])
        self.correction = None
        if self.correction_name is not None:
            self.correction = weights[self.correction_name].to(torch.float32).contiguous()
        self.w_router = torch.cat([r.to(env.dtype) for r in rows], dim=0).contiguous()       # few rows: kept row-major
        # the experts' matrices side by side: [E, 2 ff, hidden] (an expert's gate rows, then its up rows), [E, hidden, ff]
        self.w_gate_up = torch.stack([torch.cat([weights[self._expert(j, "gate")], weights[self._expert(j, "up")]], dim=0)
                                      for j in range(self.experts)]).to(env.dtype).contiguous()
        self.w_down = torch.stack([weights[self._expert(j, "down")] for j in range(self.experts)]).to(env.dtype).contiguous()
        # (where the kernels for the matrix cores apply they read a layout of their own, and the row-major
        # matrices are not kept beside it)
        self.packed = env.ops.pack_experts(self.w_gate_up, self.w_down)
        if self.packed is not None:
            self.w_gate_up = self.w_down = None
        self.shared_gate_up = self.shared_down = None
        if self.shared_inter is not None:
            if self.activation == "silu":
                self.shared_gate_up = GatedMatrix(weights[n["shared_gate"]], weights[n["shared_up"]], env)
            else:       # (the products' own epilogue is silu(gate) * up: gate and up rows stacked, the activation in a pass of its own)
                self.shared_gate_up = fuse_rows([weights[n["shared_gate"]], weights[n["shared_up"]]], env)
            self.shared_down = as_matrix(weights[n["shared_down"]], env)

    def workspace_elems(self, rows: int) -> int:
        return rows * (self.top * (3 * self.inter + self.hidden) + 3 * (self.shared_inter or 0) + 2 * self.outputs)

    def forward(self, x: torch.Tensor, step: StepView):
        ops = self.env.ops
        z, transposed = ops.small_product(x, self.w_router)
        how = {}
        if (self.score, self.group_score, self.normalize, self.correction) != ("sigmoid", "top2", True, None):
            how = dict(score=self.score, group_score=self.group_score, normalize=self.normalize, correction=self.correction)
        ids, weights, shared_gate = ops.route_experts(z, self.outputs, self.top, self.groups, self.keep, self.scale,
                                                      self.has_gate, transposed, **how)
        shared = None
        if self.shared_inter is not None:
            if self.activation == "silu":
                hidden = ops.linear_swiglu(x, self.shared_gate_up)
            else:
                hidden = ops.swiglu(ops.linear(x, self.shared_gate_up), limit=self.shared_limit, slope=self.slope)
            shared = ops.linear(hidden, self.shared_down)
        how = {} if self.activation == "silu" else {"limit": self.limit, "slope": self.slope}
        return ops.apply_experts(x, ids, weights, self.w_gate_up, self.w_down, self.packed, shared, shared_gate, **how)


register_part("ffn", "routed_experts", RoutedExperts)
