from . import attention, block, conv_attention, delta, differential, latent, lightning, postnorm, sink_attention, embedding, hyper, mlp, moe, norm, parallel, rope  # noqa: F401  (registers the parts)
from .base import (Block, BuildEnv, FeedForward, GroupView, LayerCache, Mixer, Norm, Part,
                   PositionEncoding, RotaryTables, StepView, build_part, register_part)

__all__ = ["Block", "BuildEnv", "FeedForward", "GroupView", "LayerCache", "Mixer", "Norm", "Part",
           "PositionEncoding", "RotaryTables", "StepView", "build_part", "register_part"]
