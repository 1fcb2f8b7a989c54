"""Weights by tensor name: from safetensors into the parts, or random.

The reference loads through a library model and copies module to module
(worker/src/inference/qwen2/model.py:382-452); here the model declares the names and
shapes it wants (`Model.param_specs()`), the file says what it has, and the two are
compared before a byte is read.

Precision that is kept: with the engine in bfloat16, a tensor stored in bf16 or fp16
is kept in bfloat16 and a tensor stored in 32-bit (or 64-bit) stays 32-bit; with the
engine in float32 every floating tensor becomes float32. Integer tables become int32.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Iterator, List, Mapping, Tuple

import torch

from .random_init import standard_normal
from .safetensors_io import SafetensorsFile, model_files, write_safetensors


class WeightsError(ValueError):
    """The file's tensors do not fit the model. One error lists everything that is wrong."""

    def __init__(self, missing: List[str], unexpected: List[str],
                 wrong_shape: List[Tuple[str, tuple, tuple]], where: str = "") -> None:
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        lines = [f"weights do not fit the model{' (' + where + ')' if where else ''}:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, want {list(want)}" for n, got, want in self.wrong_shape))
        super().__init__("\n".join(lines))


def kept_dtype(stored: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if engine_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def check_names(wanted: Mapping[str, tuple], found: Mapping[str, tuple], ignorable=(), where: str = "") -> None:
    """Raise one WeightsError for all missing / unexpected / wrongly shaped tensors."""
    missing = [n for n in wanted if n not in found]
    unexpected = [n for n in found if n not in wanted and n not in ignorable]
    wrong = [(n, tuple(found[n]), tuple(wanted[n])) for n in wanted
             if n in found and tuple(found[n]) != tuple(wanted[n])]
    if missing or unexpected or wrong:
        raise WeightsError(missing, unexpected, wrong, where)


def load_into(model, model_dir, device, engine_dtype: torch.dtype) -> None:
    """Read every tensor `model` declares from the folder and hand it to its part."""
    files = model_files(model_dir)
    opened: Dict[Path, SafetensorsFile] = {}
    try:
        for path in set(files.values()):
            opened[path] = SafetensorsFile(path)
        found = {name: opened[path].index[name][1] for name, path in files.items()
                 if name in opened[path].index}
        wanted = {name: spec.shape for name, spec in model.param_specs().items()}
        check_names(wanted, found, model.ignorable_names(), where=str(model_dir))

        def fetch(name: str) -> torch.Tensor:
            source = opened[files[name]]
            tensor = source.read(name)
            return tensor.to(device=device, dtype=kept_dtype(tensor.dtype, engine_dtype))

        model.load_tensors(fetch)
    finally:
        for f in opened.values():
            f.close()


def random_tensor(name: str, spec, seed: int, std: float, device) -> torch.Tensor:
    """Matrices, embeddings and biases ~ N(0, std); norm weights 1; zeros where asked. Always float32, and a
    function of (seed, name, element) alone (`random_init`): the same bits on the CPU and on the device, in
    any order of drawing, so that every user of the random-weights mode sees one model for one seed."""
    if spec.init == "ones":
        return torch.ones(spec.shape, dtype=torch.float32, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=torch.float32, device=device)
    if spec.init == "int":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    count = 1
    for n in spec.shape:
        count *= int(n)
    return torch.mul(standard_normal(seed, name, count, device), std).view(tuple(spec.shape))


def random_into(model, seed: int, device, engine_dtype: torch.dtype, std: float = 0.02) -> None:
    """Random weights straight into the parts, drawn on `device` (no file): tensor for tensor what
    `write_random_model` writes for the same seed, stored in the engine's precision."""
    specs = model.param_specs()
    store = torch.bfloat16 if engine_dtype == torch.bfloat16 else torch.float32

    def fetch(name: str) -> torch.Tensor:
        tensor = random_tensor(name, specs[name], seed, std, device)
        return tensor if not tensor.dtype.is_floating_point else tensor.to(store)

    model.load_tensors(fetch)


def write_random_model(config, out_dir, seed: int, dtype: str = "float32", std: float = 0.02) -> Path:
    """Random-weights mode: write a model folder (config.json, model.safetensors) from a
    typed configuration and a seed. Tensors are drawn in float32 (`random_tensor`), then stored as `dtype`."""
    from ..engine.model import Model  # local import: weights <-> engine

    store = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    config_json = dict(config.to_dict())
    config_json["torch_dtype"] = dtype
    (out_dir / "config.json").write_text(json.dumps(config_json, indent=1))
    specs = Model.declare(config.model_spec())

    def dtype_of(spec) -> torch.dtype:
        return torch.int32 if spec.init == "int" else store

    def tensors() -> Iterator[Tuple[str, torch.Tensor]]:
        for name, spec in specs.items():
            yield name, random_tensor(name, spec, seed, std, "cpu").to(dtype_of(spec))

    write_safetensors(out_dir / "model.safetensors",
                      [(n, dtype_of(s), tuple(s.shape)) for n, s in specs.items()],
                      tensors(), {"format": "pt", "seed": str(seed)})
    return out_dir
