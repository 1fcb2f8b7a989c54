"""What a part is, and the registries that map a `PartSpec.kind` to its class.

A part gets every size and constant from its `PartSpec`; it knows neither the model it
is in nor the layer index. It declares its tensors by local name (`param_specs`), gets
them through `load`, and computes through the kernel surface (`Ops`).

Families and their interfaces, in short:

* `embedding`: `Embedding.forward(ops, ids, meta)` -> float32 [T, C], the start of the residual stream;
* `position`: `PositionEncoding.rotary()` -> inverse frequencies for the fused rotation (or None),
  `head_slopes(num_heads)` -> per-head slopes of a bias by distance inside attention (or None), and
  `on_embedding(ops, hidden, meta)` for encodings that act on the embeddings;
* `norm`: `Norm.apply(ops, x_f32, out_dtype)` and `Norm.add_apply(ops, residual_f32, delta, out_dtype)`;
* `mixer`: `Mixer.cache_requirement()` -> `PagedTensors` | `FixedState` | None,
  `Mixer.forward(ops, x, ctx, cache, writes_cache)` with x act [T, C] -> act [T, C], `cache` being the
  `CacheView` of what the mixer declared;
* `feed_forward`: `FeedForward.forward(ops, x, ctx)`;
* `block`: an arrangement. A block class names the parts it arranges and their families (`CHILDREN`),
  builds them from the layer's specs, and owns where the norms sit and how the residual is added:
  `Block.forward(ops, stream, ctx, cache, writes_cache)`, `cache` being the layer's `LayerCache`, which
  holds one view for each of the block's mixers;
* `head`: `Head.forward(ops, normed)` -> float32 logits [R, vocab].

What a mixer keeps between steps is declared as data: `PagedTensors` names tensors that grow with the
request, a page at a time (per page shape, dtype, and how many of the newest positions must stay readable),
`FixedState` names tensors of fixed size per request. The cache manager allocates what is declared and
knows nothing of what the tensors mean.
"""

from __future__ import annotations

import abc
from dataclasses import dataclass
from typing import Callable, Dict, List, Mapping, Optional, Tuple

import torch

from ..config.model_config import PartSpec


@dataclass(frozen=True)
class ParamSpec:
    shape: Tuple[int, ...]
    init: str = "normal"   # "normal" | "ones" | "zeros" | "int"


PAGE = -1      # stands for the page size in the shape of a paged tensor


@dataclass(frozen=True)
class TensorDecl:
    """One tensor that a mixer keeps: `shape` per page (with `PAGE` where the page size goes) or per
    request; `dtype` None means the cache's own dtype (paged) or float32 (state)."""

    name: str
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None


@dataclass(frozen=True)
class PagedTensors:
    """A mixer that keeps something for every token (or for the last `window` tokens), in pages:
    for each declared tensor the cache holds `[pages + 1, *shape]` per layer, addressed through the
    request's block table of the layer's group. Mixers with equal declarations share a group of pages."""

    tensors: Tuple[TensorDecl, ...]
    window: Optional[int] = None

    def page_shape(self, decl: TensorDecl, block_size: int) -> Tuple[int, ...]:
        return tuple(block_size if s == PAGE else s for s in decl.shape)


@dataclass(frozen=True)
class FixedState:
    """A mixer that keeps tensors of fixed size for each request: the cache holds `[slots + 1, *shape]`
    per layer for each of them, zeroed when a request takes the slot."""

    tensors: Tuple[TensorDecl, ...]

    @classmethod
    def of(cls, shape, name: str = "state") -> "FixedState":
        """One float32 tensor of `shape`."""
        return cls((TensorDecl(name, tuple(shape), torch.float32),))


class ResidualStream:
    """The residual sum in float32, and a contribution not yet added to it. The next norm
    adds it while it reads the stream, which saves one pass over the activations."""

    def __init__(self, hidden: torch.Tensor) -> None:
        self.hidden = hidden
        self.pending: Optional[torch.Tensor] = None


class StepContext:
    """What one step hands to every part: the batch's addressing and the dtype of
    activations."""

    def __init__(self, meta, act_dtype: torch.dtype) -> None:
        self.meta = meta
        self.act_dtype = act_dtype


class Part(abc.ABC):
    # False for a part whose forward cannot be recorded into a device graph (it waits for the device, or
    # its launches depend on values it reads back): a model with such a part runs every step uncaptured
    capturable: bool = True

    def __init__(self, spec: PartSpec) -> None:
        self.spec = spec

    def param_specs(self) -> Dict[str, ParamSpec]:
        """Local tensor name -> shape; the checkpoint name is `spec.prefix + local`."""
        return {}

    def shared_specs(self) -> Dict[str, str]:
        """Local tensor name -> full checkpoint name of a tensor that another part declares and this
        part wants too (a head tied to the embedding); both get the same tensor object."""
        return {}

    def optional_names(self) -> List[str]:
        """Local names that a file may hold although the part does not use them."""
        return []

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Take the tensors (by local name, on the device, in the kept dtype)."""

    def prepare(self, ops) -> None:
        """After `load`, once, with the kernel surface the part will run on: announce the weights
        of matrix products (`ops.prepare_linear`)."""

    def capture_context(self, longest: int, limit: int) -> Optional[int]:
        """For captured decode steps: the one host-side number a captured step may freeze is the longest
        context it is made for. A part whose launches depend on it answers with the length a graph should
        be made for so that it serves a step whose longest request holds `longest` tokens (at most `limit`,
        the engine's own bound); the engine keeps one graph per answer. None: it does not matter."""
        return None

    def parts(self):
        """This part and the parts inside it, children first."""
        yield self


class Embedding(Part):
    @abc.abstractmethod
    def forward(self, ops, ids: torch.Tensor, meta) -> torch.Tensor:
        """ids int32 [T] -> float32 [T, C]."""


class Head(Part):
    @abc.abstractmethod
    def forward(self, ops, normed: torch.Tensor) -> torch.Tensor:
        """act [R, C] (after the final norm) -> float32 logits [R, vocab]."""


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

    def head_slopes(self, num_heads: int) -> Optional[torch.Tensor]:
        """float32 [num_heads] for an encoding that biases every score by the distance to the key,
        score += slope[h] * (key position - query position) (`ScoreExtras.head_slopes`); None otherwise."""
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
    """An arrangement. `CHILDREN` names the parts it arranges and the family of each, in the order in
    which their tensors are declared; the layer's spec must bring exactly these names. Every child is
    built here and becomes an attribute of its name."""

    CHILDREN: Dict[str, str] = {}

    def __init__(self, spec: PartSpec, parts: Mapping[str, PartSpec]) -> None:
        super().__init__(spec)
        missing = [name for name in self.CHILDREN if name not in parts]
        unknown = [name for name in parts if name not in self.CHILDREN]
        if missing or unknown:
            raise ValueError(f"block {spec.kind!r} arranges {sorted(self.CHILDREN)}: "
                             f"missing {missing}, not known to it {unknown}")
        self.children: Dict[str, Part] = {}
        for name, family in self.CHILDREN.items():
            child = build_part(family, parts[name])
            self.children[name] = child
            setattr(self, name, child)

    def parts(self):
        for child in self.children.values():
            yield from child.parts()
        yield self

    def cache_requirements(self) -> Dict[str, object]:
        """What each of the block's mixers keeps, by the mixer's name in the block."""
        return {name: child.cache_requirement() for name, child in self.children.items()
                if self.CHILDREN[name] == "mixer"}

    @abc.abstractmethod
    def forward(self, ops, stream: ResidualStream, ctx: StepContext, cache, writes_cache: bool) -> None: ...


_REGISTRIES: Dict[str, Dict[str, Callable]] = {
    "embedding": {}, "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {}, "head": {},
}


def register_part(family: str, kind: str, cls) -> None:
    """Make `PartSpec(kind=kind)` build `cls` wherever a part of `family` is wanted
    (family: embedding | mixer | feed_forward | norm | position | block | head)."""
    if family not in _REGISTRIES:
        raise KeyError(f"no part family {family!r}; families: {sorted(_REGISTRIES)}")
    _REGISTRIES[family][kind] = cls


def build_part(family: str, spec: PartSpec, *args):
    table = _REGISTRIES[family]
    if spec.kind not in table:
        raise KeyError(f"no {family} named {spec.kind!r}; known: {sorted(table)}")
    return table[spec.kind](spec, *args)
