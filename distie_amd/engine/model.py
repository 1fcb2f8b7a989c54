"""A model put together from parts, as a `ModelSpec` describes it.

`Model` knows no architecture: it builds the embedding, one block per `LayerSpec`, the
final norm and the head from the registries of parts, asks each part for the tensors it
wants, and runs the blocks in the order the spec gives (an order may name a layer twice,
or let a layer use another layer's cache). It computes only through the kernel surface.

The flow of one step is the reference's `forward_batch`
(worker/src/inference/qwen2/model.py:369-380): embed, blocks, select the rows whose
logits are wanted, final norm, head.
"""

from __future__ import annotations

from typing import Callable, Dict, List, Optional

import torch

from ..config.model_config import ModelSpec
from ..parts import ParamSpec, ResidualStream, StepContext, build_part


class Model:
    def __init__(self, spec: ModelSpec) -> None:
        self.spec = spec
        self.blocks = []
        for layer in spec.layers:
            mixer = build_part("mixer", layer.mixer)
            feed_forward = build_part("feed_forward", layer.feed_forward)
            mixer_norm = build_part("norm", layer.mixer_norm)
            feed_forward_norm = build_part("norm", layer.feed_forward_norm)
            self.blocks.append(build_part("block", layer.block, mixer, feed_forward, mixer_norm, feed_forward_norm))
        self.final_norm = build_part("norm", spec.final_norm)
        self.position = build_part("position", spec.position) if spec.position is not None else None
        self.tied_head = bool(spec.head.get("tied", False))
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        for call in spec.order:
            if not 0 <= call.layer < len(self.blocks) or not 0 <= call.cache_layer < len(self.blocks):
                raise ValueError(f"run order names layer {call.layer} / cache of {call.cache_layer}, "
                                 f"the model has {len(self.blocks)} layers")

    # ------------------------------------------------------------ tensors
    def _parts(self):
        """(part, its spec) for every part that owns tensors."""
        for block in self.blocks:
            for part in (block.mixer_norm, block.mixer, block.feed_forward_norm, block.feed_forward, block):
                yield part
        yield self.final_norm
        if self.position is not None:
            yield self.position

    def param_specs(self) -> Dict[str, ParamSpec]:
        """Checkpoint name -> shape, in a fixed order (embedding, layers, final norm, head)."""
        s = self.spec
        out = {s.embedding.prefix + "weight": ParamSpec((s.vocab_size, s.hidden_size))}
        for part in self._parts():
            for local, spec in part.param_specs().items():
                out[part.spec.prefix + local] = spec
        if not self.tied_head:
            out[s.head.prefix + "weight"] = ParamSpec((s.vocab_size, s.hidden_size))
        return out

    @classmethod
    def declare(cls, spec: ModelSpec) -> Dict[str, ParamSpec]:
        return cls(spec).param_specs()

    def ignorable_names(self) -> List[str]:
        """Tensors a file may hold that the model does not use: the head's copy when it is
        tied to the embedding."""
        return [self.spec.head.prefix + "weight"] if self.tied_head else []

    def load_tensors(self, fetch: Callable[[str], torch.Tensor]) -> None:
        """`fetch(name)` gives each declared tensor, on the device, in the kept dtype."""
        s = self.spec
        self.embedding = fetch(s.embedding.prefix + "weight").contiguous()
        for part in self._parts():
            names = part.param_specs()
            if names:
                part.load({local: fetch(part.spec.prefix + local) for local in names})
        # tied: one buffer (worker/src/inference/qwen2/model.py:302-303)
        self.head = self.embedding if self.tied_head else fetch(s.head.prefix + "weight").contiguous()

    def prepare(self, ops) -> None:
        """Once after loading, with the kernel surface the model will run on."""
        for part in self._parts():
            part.prepare(ops)
        ops.prepare_linear(self.head)

    def cache_requirements(self) -> list:
        return [block.mixer.cache_requirement() for block in self.blocks]

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        tensors = [self.embedding, self.head]
        for part in self._parts():
            tensors += [v for v in vars(part).values() if isinstance(v, torch.Tensor)]
        for t in tensors:
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    # ------------------------------------------------------------ the step
    def forward(self, ops, ids: torch.Tensor, meta, cache, act_dtype, want_rows: Optional[torch.Tensor],
                every_row: bool = False):
        """ids int32 [T] -> float32 logits [R, vocab] at `want_rows` (int32 [R]); None if no
        row is wanted (the step then only fills the cache). `every_row`: `want_rows` names every row
        in order (a captured decode step), so nothing needs to be gathered."""
        stream = ResidualStream(ops.embed(ids, self.embedding))
        if self.position is not None:
            self.position.on_embedding(ops, stream.hidden, meta)
        ctx = StepContext(meta, act_dtype)
        for call in self.spec.order:
            view = cache.layer(call.cache_layer)
            ctx.state = view.state
            self.blocks[call.layer].forward(ops, stream, ctx, view, call.writes_cache)
        if want_rows is None:
            return None
        if every_row:
            normed = self.final_norm.of_stream(ops, stream, act_dtype)
            return ops.linear_f32out(normed, self.head)
        hidden = ops.gather_rows(stream.hidden, want_rows)
        if stream.pending is not None:
            normed = self.final_norm.add_apply(ops, hidden, ops.gather_rows(stream.pending, want_rows), act_dtype)
        else:
            normed = self.final_norm.apply(ops, hidden, act_dtype)
        return ops.linear_f32out(normed, self.head)
