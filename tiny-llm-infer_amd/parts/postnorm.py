"""Residual block that norms what a sublayer gives:  x <- x + n1(mixer(x)),  x <- x + n2(ff(x)).
The sublayers read x itself, so nothing stands between the residual and a sublayer's products
but the rounding to the run's type.  One pass over a row norms the sublayer's output (float32),
adds it to the float32 residual and writes the new residual's rows in the run's type for the next
sublayer; those rows are what the block hands on (``ResidualRows``), so that the next block does
not make them again.  Without a feed-forward the block is x <- x + n1(mixer(x)).  The norms are
RMS norms (the kernel has that formula built in); any other kind is refused."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorDecl
from .base import Block, BuildEnv, StepView, register_part, run_norm


class ResidualRows:
    """The residual's rows in the run's type, handed from one block to the next: nothing is owed."""

    def __init__(self, rows: torch.Tensor):
        self.rows = rows


class SublayerPostNormBlock(Block):
    def __init__(self, spec, mixer, ffn, norms):
        super().__init__(spec)
        self.mixer = mixer
        self.ffn = ffn
        self.norm_mixer = norms["mixer"]
        self.norm_ffn = norms["ffn"] if ffn is not None else None
        self.replayable = all(p.replayable for p in self._parts())

    def _parts(self):
        return [p for p in (self.norm_mixer, self.mixer, self.norm_ffn, self.ffn) if p is not None]

    def tensors(self) -> List[TensorDecl]:
        return [d for p in self._parts() for d in p.tensors()]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        for part in self._parts():
            part.load(weights, env)
        self.rms = []
        for norm in (self.norm_mixer, self.norm_ffn):
            rms = norm.as_rms() if norm is not None else None
            if norm is not None and rms is None:
                raise ValueError(f"the norm of a sublayer's output is '{norm.spec.kind}': this arrangement has the RMS norm only")
            self.rms.append(rms)

    def forward(self, resid: torch.Tensor, pending, step: StepView):
        ops = self.env.ops
        if pending is None:
            h = ops.residual_rows(resid, self.env.dtype)
        elif isinstance(pending, ResidualRows):
            h = pending.rows
        else:
            raise TypeError("the block before this one leaves a sum to the residual open; blocks of this arrangement "
                            "follow their own kind only")
        (w1, eps1), second = self.rms[0], self.rms[1]
        h = ops.norm_add(resid, self.mixer.forward(h, step), w1, eps1, self.env.dtype)
        if self.ffn is not None:
            h = ops.norm_add(resid, self.ffn.forward(h, step), second[0], second[1], self.env.dtype)
        return ResidualRows(h)

    def close(self, resid, pending, final_norm, rows=None, num_rows=None):
        return run_norm(final_norm, resid, None, rows=rows, num_rows=num_rows)


register_part("block", "sublayer_postnorm", SublayerPostNormBlock)
