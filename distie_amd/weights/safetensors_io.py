"""Reading and writing safetensors files without any model library.

Format: 8 bytes little-endian length N, N bytes of JSON
(`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`),
then the raw little-endian tensor bytes. Files are memory-mapped, so a tensor is read
only when it is asked for.
"""

from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path
from typing import Dict, Iterable, Iterator, Mapping, Tuple

import torch

DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
NAMES = {v: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped file: `index` maps name -> (dtype, shape); `read(name)` copies
    one tensor out of the mapping."""

    def __init__(self, path) -> None:
        self.path = Path(path)
        self._file = open(self.path, "rb")
        head = self._file.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{self.path}: too short for a safetensors file")
        (n,) = struct.unpack("<Q", head)
        size = self.path.stat().st_size
        if n > size - 8:
            raise SafetensorsError(f"{self.path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._file.read(n))
        except (json.JSONDecodeError, UnicodeDecodeError) as exc:
            raise SafetensorsError(f"{self.path}: header is not JSON") from exc
        self._base = 8 + n
        self.metadata = header.pop("__metadata__", {}) or {}
        self._entries = header
        self.index: Dict[str, Tuple[torch.dtype, Tuple[int, ...]]] = {}
        for name, entry in header.items():
            dtype = DTYPES.get(entry.get("dtype"))
            if dtype is None:
                raise SafetensorsError(f"{self.path}: tensor {name} has unsupported dtype {entry.get('dtype')}")
            begin, end = entry["data_offsets"]
            shape = tuple(int(s) for s in entry["shape"])
            count = 1
            for s in shape:
                count *= s
            if end - begin != count * _itemsize(dtype) or self._base + end > size:
                raise SafetensorsError(f"{self.path}: tensor {name} has inconsistent offsets")
            self.index[name] = (dtype, shape)
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def read(self, name: str) -> torch.Tensor:
        dtype, shape = self.index[name]
        begin, end = self._entries[name]["data_offsets"]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        # one copy out of the mapping; the tensor owns the bytes and outlives the file
        data = bytearray(memoryview(self._map)[self._base + begin:self._base + end])
        if dtype == torch.bool:
            return torch.frombuffer(data, dtype=torch.uint8).bool().reshape(shape)
        return torch.frombuffer(data, dtype=dtype).reshape(shape)

    def close(self) -> None:
        if self._map is not None:
            try:
                self._map.close()
            except BufferError:
                pass
            self._map = None
        self._file.close()


def _itemsize(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


def model_files(model_dir) -> Dict[str, Path]:
    """Tensor name -> file, for `model.safetensors` or a sharded folder with
    `model.safetensors.index.json`."""
    model_dir = Path(model_dir)
    index = model_dir / "model.safetensors.index.json"
    if index.is_file():
        weight_map = json.loads(index.read_text()).get("weight_map", {})
        return {name: model_dir / file for name, file in weight_map.items()}
    single = model_dir / "model.safetensors"
    if not single.is_file():
        raise SafetensorsError(f"no model.safetensors in {model_dir}")
    f = SafetensorsFile(single)
    names = {name: single for name in f.index}
    f.close()
    return names


def write_safetensors(path, entries: Iterable[Tuple[str, torch.dtype, Tuple[int, ...]]],
                      tensors: Iterator[Tuple[str, torch.Tensor]],
                      metadata: Mapping[str, str] = None) -> None:
    """Write `tensors` (an iterator in the order of `entries`) one at a time, so a large
    model never stands in memory twice."""
    entries = list(entries)
    header = {}
    offset = 0
    for name, dtype, shape in entries:
        count = 1
        for s in shape:
            count *= s
        size = count * _itemsize(dtype)
        header[name] = {"dtype": NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + size]}
        offset += size
    if metadata:
        header["__metadata__"] = dict(metadata)
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as out:
        out.write(struct.pack("<Q", len(blob)))
        out.write(blob)
        for (name, dtype, shape), (got_name, tensor) in zip(entries, tensors):
            if got_name != name or tensor.dtype != dtype or tuple(tensor.shape) != tuple(shape):
                raise SafetensorsError(f"tensor {got_name} does not match its header entry {name}")
            data = tensor.detach().cpu().contiguous()
            if dtype == torch.bool:
                data = data.to(torch.uint8)
            out.write(data.reshape(-1).view(torch.uint8).numpy().tobytes())
