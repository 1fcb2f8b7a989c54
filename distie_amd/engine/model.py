"""A model put together from parts, as a `ModelSpec` describes it.

`Model` knows no architecture and no part: it builds the embedding, one block per `LayerSpec` (the
block builds the parts it arranges), the final norm and the head from the registries of parts, asks
every part for the tensors it wants, and runs the blocks in the order the spec gives (an order may name
a layer twice, or let a layer use another layer's cache). It computes only through the parts.

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
        self.embed = build_part("embedding", spec.embedding)
        self.blocks = [build_part("block", layer.block, layer.parts) for layer in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm)
        self.position = build_part("position", spec.position) if spec.position is not None else None
        self.lm_head = build_part("head", spec.head)
        for call in spec.order:
            if not 0 <= call.layer < len(self.blocks) or not 0 <= call.cache_layer < len(self.blocks):
                raise ValueError(f"run order names layer {call.layer} / cache of {call.cache_layer}, "
                                 f"the model has {len(self.blocks)} layers")

    # ------------------------------------------------------------ tensors
    def parts(self):
        """Every part of the model, in the order in which their tensors are declared."""
        yield from self.embed.parts()
        for block in self.blocks:
            yield from block.parts()
        yield from self.final_norm.parts()
        if self.position is not None:
            yield from self.position.parts()
        yield from self.lm_head.parts()

    @property
    def embedding(self) -> Optional[torch.Tensor]:
        return getattr(self.embed, "weight", None)

    @property
    def head(self) -> Optional[torch.Tensor]:
        return getattr(self.lm_head, "weight", None)

    @property
    def capturable(self) -> bool:
        """Every part can be recorded into a device graph."""
        return all(part.capturable for part in self.parts())

    def capture_context(self, longest: int, limit: int) -> int:
        """The context length a captured step should be made for to serve a step whose longest request
        holds `longest` tokens: the largest of the parts' answers, `limit` if no part cares."""
        answers = [a for a in (part.capture_context(longest, limit) for part in self.parts()) if a is not None]
        return max(answers) if answers else limit

    def param_specs(self) -> Dict[str, ParamSpec]:
        """Checkpoint name -> shape, in a fixed order (embedding, layers, final norm, head)."""
        out: Dict[str, ParamSpec] = {}
        for part in self.parts():
            for local, spec in part.param_specs().items():
                name = part.spec.prefix + local
                if name in out and out[name] != spec:
                    raise ValueError(f"two parts declare {name} with different shapes")
                out[name] = spec
        for part in self.parts():
            for local, name in part.shared_specs().items():
                if name not in out:
                    raise ValueError(f"{part.spec.kind} wants to share {name}, which no part declares")
        return out

    @classmethod
    def declare(cls, spec: ModelSpec) -> Dict[str, ParamSpec]:
        return cls(spec).param_specs()

    def ignorable_names(self) -> List[str]:
        """Tensors a file may hold that the model does not use (the head's copy when it is tied to the
        embedding)."""
        return [part.spec.prefix + local for part in self.parts() for local in part.optional_names()]

    def load_tensors(self, fetch: Callable[[str], torch.Tensor]) -> None:
        """`fetch(name)` gives each declared tensor, on the device, in the kept dtype. A tensor that two
        parts use is fetched once: both hold the same object."""
        fetched: Dict[str, torch.Tensor] = {}

        def get(name: str) -> torch.Tensor:
            if name not in fetched:
                fetched[name] = fetch(name).contiguous()
            return fetched[name]

        for part in self.parts():
            wanted = {local: part.spec.prefix + local for local in part.param_specs()}
            wanted.update(part.shared_specs())
            if wanted:
                part.load({local: get(name) for local, name in wanted.items()})

    def prepare(self, ops) -> None:
        """Once after loading, with the kernel surface the model will run on."""
        for part in self.parts():
            part.prepare(ops)

    def cache_requirements(self) -> list:
        """Per layer: what each mixer of the layer's block keeps, by the mixer's name in the block."""
        return [block.cache_requirements() for block in self.blocks]

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        for part in self.parts():
            for t in vars(part).values():
                if isinstance(t, torch.Tensor) and t.data_ptr() not in seen:
                    seen.add(t.data_ptr())
                    total += t.numel() * t.element_size()
        return total

    # ------------------------------------------------------------ the step
    def forward(self, ops, ids: torch.Tensor, meta, cache, act_dtype, want_rows: Optional[torch.Tensor],
                every_row: bool = False):
        """ids int32 [T] -> float32 logits [R, vocab] at `want_rows` (int32 [R]); None if no
        row is wanted (the step then only fills the cache). `every_row`: `want_rows` names every row
        in order (a captured decode step), so nothing needs to be gathered."""
        stream = ResidualStream(self.embed.forward(ops, ids, meta))
        if self.position is not None:
            self.position.on_embedding(ops, stream.hidden, meta)
        ctx = StepContext(meta, act_dtype)
        for call in self.spec.order:
            self.blocks[call.layer].forward(ops, stream, ctx, cache.layer(call.cache_layer), call.writes_cache)
        if want_rows is None:
            return None
        if every_row:
            normed = self.final_norm.of_stream(ops, stream, act_dtype)
            return self.lm_head.forward(ops, normed)
        hidden = ops.gather_rows(stream.hidden, want_rows)
        if stream.pending is not None:
            normed = self.final_norm.add_apply(ops, hidden, ops.gather_rows(stream.pending, want_rows), act_dtype)
        else:
            normed = self.final_norm.apply(ops, hidden, act_dtype)
        return self.lm_head.forward(ops, normed)
