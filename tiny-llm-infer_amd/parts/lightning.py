"""Lightning attention: a recurrent mixer that keeps a matrix of state a head, decaying by a
constant a token, instead of keys and values a token.

For the rows h_t of one sequence (H heads, key size dk, value size dv, one decay c_a a head from
the configuration):

    q = silu(Wq h),  k = silu(Wk h)   [H dk],    v = silu(Wv h)   [H dv]       (no biases)
    per head:  S_t = c_a S_(t-1) + k_t v_t^T,    o_t = S_t^T q_t                 (no other scale)
    y = o / sqrt(mean(o^2) + eps) * w * sigmoid(Wg h)      the heads side by side, normed together
    out = Wo y

S [dk, dv] starts at zero and is per-request state in float32; the recurrence, the norm and the
gate are float32.  Nothing is kept in the paged cache.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..cache.manager import StateNeed
from ..weights.loader import TensorDecl
from .base import BuildEnv, Mixer, StepView, register_part
from .linear import as_matrix, fuse_rows


class LightningAttention(Mixer):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.dk = int(p["key_dim"])
        self.dv = int(p["value_dim"])
        self.eps = float(p["norm_eps"])
        self.decay_values = [float(c) for c in p["decay"]]
        if len(self.decay_values) != self.heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.heads} heads")
        self.qk_dim = self.heads * self.dk
        self.v_dim = self.heads * self.dv

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        return [TensorDecl(n["q"], (self.qk_dim, self.hidden)), TensorDecl(n["k"], (self.qk_dim, self.hidden)),
                TensorDecl(n["v"], (self.v_dim, self.hidden)), TensorDecl(n["gate"], (self.v_dim, self.hidden)),
                TensorDecl(n["o"], (self.hidden, self.v_dim)), TensorDecl(n["norm"], (self.v_dim,), "ones_normal")]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        env.ops.check_lightning_sizes(self.heads, self.dk, self.dv)
        # one product for q, k, v and, behind them, the gate's logits
        self.w_in = fuse_rows([weights[n[r]] for r in ("q", "k", "v", "gate")], env)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=env.device)
        self.norm = weights[n["norm"]].to(torch.float32).contiguous()
        self.w_o = as_matrix(weights[n["o"]], env)

    def state_need(self) -> StateNeed:
        # (the kernel library says in which order it keeps a head's matrix)
        return StateNeed(tuple(self.env.ops.lightning_state_shape(self.heads, self.dk, self.dv)), torch.float32)

    def workspace_elems(self, rows: int) -> int:
        # the projections, then q, k, v (padded at worst to twice their size) and o in float32 (two elements of the run's type each at worst)
        return rows * (2 * self.qk_dim + 2 * self.v_dim + 2 * (4 * self.qk_dim + 2 * self.v_dim) + 2 * self.v_dim + self.v_dim)

    def forward(self, x: torch.Tensor, step: StepView):
        ops = self.env.ops
        proj = ops.linear(x, self.w_in)
        o = ops.lightning_attention(proj, self.decay, step.state, step, self.heads, self.dk, self.dv)
        y = ops.lightning_norm(o, proj, 2 * self.qk_dim + self.v_dim, self.norm, self.eps, self.env.dtype)
        return ops.linear(y, self.w_o, deferred=True)


register_part("mixer", "lightning_attention", LightningAttention)
