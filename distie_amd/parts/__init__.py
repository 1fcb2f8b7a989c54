from . import attention, block, embedding, feed_forward, norm, position  # noqa: F401  (registration)
from .attention import PagedKV
from .base import (PAGE, Block, Embedding, FeedForward, FixedState, Head, Mixer, Norm, PagedTensors, ParamSpec, Part,
                   PositionEncoding, ResidualStream, StepContext, TensorDecl, build_part, register_part)

__all__ = ["PAGE", "Block", "Embedding", "FeedForward", "FixedState", "Head", "Mixer", "Norm", "PagedKV", "PagedTensors",
           "ParamSpec", "Part", "PositionEncoding", "ResidualStream", "StepContext", "TensorDecl", "build_part",
           "register_part"]
