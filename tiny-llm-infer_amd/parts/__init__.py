from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registers the parts)
from .base import (Block, BuildEnv, FeedForward, GroupView, LayerCache, Mixer, Norm, Part,
                   PositionEncoding, RotaryTables, StepView, build_part, register_part)

__all__ = ["Block", "BuildEnv", "FeedForward", "GroupView", "LayerCache", "Mixer", "Norm", "Part",
           "PositionEncoding", "RotaryTables", "StepView", "build_part", "register_part"]
