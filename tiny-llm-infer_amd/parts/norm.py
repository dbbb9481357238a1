"""RMSNorm: y_j = w_j * x_j / sqrt(mean(x^2) + eps), all in float32
(kernels/src/rmsnorm_kernel_cpu.cpp:27-43).  The weight is a plain multiplier; a
norm whose spec names no weight has none (all ones).  ``weight_offset`` c: the checkpoint stores
the multiplier less c (a weight kept around zero is ``weight_offset`` 1), added in float32 when
the weight is loaded.
The residual stream is float32; the norm adds what the previous part owes the
residual before it normalises, so the residual sum is never rounded.

LayerNorm: y_j = w_j * (x_j - m) / sqrt(mean((x - m)^2) + eps) with m = mean(x), a
weight and no bias, float32 likewise."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorDecl
from .base import BuildEnv, Norm, register_part


class RMSNorm(Norm):
    replayable = True
    supports_lazy = True
    takes_unfinished_products = True

    def __init__(self, spec):
        super().__init__(spec)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight_name = spec.names.get("weight")             # None: a norm without weights
        self.offset = float(spec.params.get("weight_offset", 0.0))
        self.weight: Optional[torch.Tensor] = None

    def tensors(self) -> List[TensorDecl]:
        init = "ones_normal" if self.offset == 0.0 else f"normal({1.0 - self.offset},0.02)"
        return [TensorDecl(self.weight_name, (self.size,), init)] if self.weight_name is not None else []

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        # vectors are held in float32: exact for 16-bit storage, unchanged for 32-bit
        if self.weight_name is None:
            self.weight = torch.ones(self.size, dtype=torch.float32, device=env.device)
        else:
            self.weight = weights[self.weight_name].to(torch.float32).contiguous()
            if self.offset != 0.0:
                self.weight = (self.weight + self.offset).contiguous()

    def as_rms(self):
        return self.weight, self.eps

    def forward(self, resid, delta, rows=None, num_rows=None, lazy=False):
        """``lazy``: the rows go to matrix products only, which may then apply the rows'
        scalar factor themselves (the kernel library decides; see its ``add_rmsnorm``)."""
        return self.env.ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.env.dtype,
                                        rows=rows, num_rows=num_rows, **({"lazy": True} if lazy else {}))


class LayerNorm(Norm):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight_name = spec.names["weight"]
        self.weight: Optional[torch.Tensor] = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.weight_name, (self.size,), "ones_normal")]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        self.weight = weights[self.weight_name].to(torch.float32).contiguous()

    def as_layer_norm(self):
        """(weight float32 [size], eps): for an arrangement that norms one row with two such norms
        in one pass."""
        return self.weight, self.eps

    def forward(self, resid, delta, rows=None, num_rows=None):
        deltas = () if delta is None else (delta,)
        return self.env.ops.add_layernorm(resid, deltas, (self.weight,), self.eps, self.env.dtype,
                                          rows=rows, num_rows=num_rows)[0]


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
