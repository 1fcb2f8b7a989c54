"""What a part is, and the registries that map a `PartSpec.kind` to its class.

A part gets every size and constant from its `PartSpec`; it knows neither the model it
is in nor the layer index. It declares its tensors by local name (`param_specs`), gets
them through `load`, and computes through the kernel surface (`Ops`).

Interfaces, in short:

* `Norm.apply(ops, x_f32, out_dtype)` and `Norm.add_apply(ops, residual_f32, delta, out_dtype)`;
* `PositionEncoding.rotary()` -> inverse frequencies for the fused rotation (or None) and
  `on_embedding(ops, hidden, meta)` for encodings that act on the embeddings;
* `Mixer.cache_requirement()` -> `PagedKV` | `FixedState` | None,
  `Mixer.forward(ops, x, ctx, cache, writes_cache)` with x act [T, C] -> act [T, C];
* `FeedForward.forward(ops, x)`;
* `Block.forward(ops, stream, ctx, cache, writes_cache)`, which owns the arrangement
  (where the norms sit, how the residual is added).
"""

from __future__ import annotations

import abc
from dataclasses import dataclass
from typing import Callable, Dict, Mapping, Optional, Tuple

import torch

from ..config.model_config import PartSpec


@dataclass(frozen=True)
class ParamSpec:
    shape: Tuple[int, ...]
    init: str = "normal"   # "normal" | "ones" | "zeros" | "int"


@dataclass(frozen=True)
class PagedKV:
    """A mixer that keeps keys and values of every token (or of the last `window`)."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class FixedState:
    """A mixer that keeps a state of fixed size for each request: `shape` float32 values."""

    shape: Tuple[int, ...]


class ResidualStream:
    """The residual sum in float32, and a contribution not yet added to it. The next norm
    adds it while it reads the stream, which saves one pass over the activations."""

    def __init__(self, hidden: torch.Tensor) -> None:
        self.hidden = hidden
        self.pending: Optional[torch.Tensor] = None


class StepContext:
    """What one step hands to every part: the batch's addressing and the dtype of
    activations."""

    def __init__(self, meta, act_dtype: torch.dtype, state=None) -> None:
        self.meta = meta
        self.act_dtype = act_dtype
        self.state = state          # float32 [slots+1, ...] state slab of the running layer, or None


class Part(abc.ABC):
    def __init__(self, spec: PartSpec) -> None:
        self.spec = spec

    def param_specs(self) -> Dict[str, ParamSpec]:
        """Local tensor name -> shape; the checkpoint name is `spec.prefix + local`."""
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Take the tensors (by local name, on the device, in the kept dtype)."""

    def prepare(self, ops) -> None:
        """After `load`, once, with the kernel surface the part will run on: announce the weights
        of matrix products (`ops.prepare_linear`)."""


class Norm(Part):
    @abc.abstractmethod
    def apply(self, ops, x: torch.Tensor, out_dtype) -> torch.Tensor: ...

    @abc.abstractmethod
    def add_apply(self, ops, residual: torch.Tensor, delta: torch.Tensor, out_dtype) -> torch.Tensor: ...

    def of_stream(self, ops, stream: ResidualStream, out_dtype) -> torch.Tensor:
        if stream.pending is None:
            return self.apply(ops, stream.hidden, out_dtype)
        delta, stream.pending = stream.pending, None
        return self.add_apply(ops, stream.hidden, delta, out_dtype)


class PositionEncoding(Part):
    def rotary(self) -> Optional[torch.Tensor]:
        """float32 [rotary_dim / 2] inverse frequencies for the rotation fused into the
        cache write, or None if this encoding does not rotate."""
        return None

    def on_embedding(self, ops, hidden: torch.Tensor, meta) -> None:
        """Hook for encodings added to the embeddings."""

    def to_device(self, device) -> None:
        pass


class Mixer(Part):
    def cache_requirement(self):
        return None

    @abc.abstractmethod
    def forward(self, ops, x: torch.Tensor, ctx: StepContext, cache, writes_cache: bool) -> torch.Tensor: ...


class FeedForward(Part):
    @abc.abstractmethod
    def forward(self, ops, x: torch.Tensor, ctx: StepContext) -> torch.Tensor: ...


class Block(Part):
    """An arrangement. Built with its four parts already constructed."""

    def __init__(self, spec: PartSpec, mixer: Mixer, feed_forward: FeedForward,
                 mixer_norm: Norm, feed_forward_norm: Norm) -> None:
        super().__init__(spec)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    @abc.abstractmethod
    def forward(self, ops, stream: ResidualStream, ctx: StepContext, cache, writes_cache: bool) -> None: ...


_REGISTRIES: Dict[str, Dict[str, Callable]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {},
}


def register_part(family: str, kind: str, cls) -> None:
    """Make `PartSpec(kind=kind)` build `cls` wherever a part of `family` is wanted
    (family: mixer | feed_forward | norm | position | block)."""
    if family not in _REGISTRIES:
        raise KeyError(f"no part family {family!r}; families: {sorted(_REGISTRIES)}")
    _REGISTRIES[family][kind] = cls


def build_part(family: str, spec: PartSpec, *args):
    table = _REGISTRIES[family]
    if spec.kind not in table:
        raise KeyError(f"no {family} named {spec.kind!r}; known: {sorted(table)}")
    return table[spec.kind](spec, *args)
