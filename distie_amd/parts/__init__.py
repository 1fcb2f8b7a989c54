from . import attention, block, feed_forward, norm, position  # noqa: F401  (registration)
from .base import (Block, FeedForward, FixedState, Mixer, Norm, PagedKV, ParamSpec, Part,
                   PositionEncoding, ResidualStream, StepContext, build_part, register_part)

__all__ = ["Block", "FeedForward", "FixedState", "Mixer", "Norm", "PagedKV", "ParamSpec", "Part",
           "PositionEncoding", "ResidualStream", "StepContext", "build_part", "register_part"]
