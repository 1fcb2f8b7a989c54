"""Random weights as a function of (seed, tensor name, element index), the same bits wherever they are drawn.

The random-weights mode has two users: a model folder written to disk (drawn on the CPU) and weights
put straight into an engine's parts (drawn on the device, where a 32B-shaped model takes seconds
instead of minutes). Both must give one model for one seed, so that a plain implementation reading
the folder can be compared with the engine that never saw it. A library generator cannot promise
that (its CPU and device streams differ), so the values are computed here from operations that
round the same way on both: 64-bit integer mixing, a table lookup, and one float32 multiply and one
float32 add, each as an operation of its own (no fused multiply-add).

element -> splitmix64(base + index * golden ratio); the top 16 bits choose an interval of the standard
normal's inverse distribution function (65,536 intervals of equal probability, the outermost two cut
off at the 2^-20 quantile, 4.9 standard deviations), the next 24 bits a place inside it.
"""

from __future__ import annotations

from statistics import NormalDist
from typing import Dict, Tuple

import torch

_MASK = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_INTERVALS = 1 << 16
CPU_CHUNK = 1 << 22
DEVICE_CHUNK = 1 << 25


def _signed(x: int) -> int:
    x &= _MASK
    return x - (1 << 64) if x >> 63 else x


def _mix(x: int) -> int:
    """The output function of splitmix64 on a Python integer."""
    x &= _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def name_key(name: str) -> int:
    """FNV-1a over the tensor's name: which stream of the seed a tensor draws from does not hang on the
    order in which tensors are declared."""
    h = 0xCBF29CE484222325
    for byte in name.encode("utf-8"):
        h = ((h ^ byte) * 0x100000001B3) & _MASK
    return h


def stream_base(seed: int, name: str) -> int:
    return _mix(_mix(seed & _MASK) ^ name_key(name))


_edges_cpu: Tuple[torch.Tensor, torch.Tensor] = ()
_edges: Dict[torch.device, Tuple[torch.Tensor, torch.Tensor]] = {}


def _tables(device) -> Tuple[torch.Tensor, torch.Tensor]:
    """(lower edge, width) of every interval, float32; computed once in pure Python double arithmetic
    (the same on every machine), rounded to float32, and copied to a device as it is."""
    global _edges_cpu
    device = torch.device(device)
    if not _edges_cpu:
        normal = NormalDist()
        end = normal.inv_cdf(2.0 ** -20)
        edges = [end] + [normal.inv_cdf(j / _INTERVALS) for j in range(1, _INTERVALS)] + [-end]
        edges = torch.tensor(edges, dtype=torch.float64).to(torch.float32)
        _edges_cpu = (edges[:-1].contiguous(), (edges[1:] - edges[:-1]).contiguous())
    if device.type == "cpu":
        return _edges_cpu
    held = _edges.get(device)
    if held is None:
        held = _edges[device] = tuple(t.to(device) for t in _edges_cpu)
    return held


def _logical_shift(x: torch.Tensor, bits: int) -> torch.Tensor:
    return (x >> bits) & ((1 << (64 - bits)) - 1)


def mixed_bits(base: int, start: int, count: int, device) -> torch.Tensor:
    """splitmix64(base + (start + i) * golden) for i < count, as int64 bit patterns."""
    index = torch.arange(start, start + count, dtype=torch.int64, device=device)
    x = index * _signed(_GOLDEN) + _signed(base)
    x = (x ^ _logical_shift(x, 30)) * _signed(0xBF58476D1CE4E5B9)
    x = (x ^ _logical_shift(x, 27)) * _signed(0x94D049BB133111EB)
    return x ^ _logical_shift(x, 31)


def standard_normal(seed: int, name: str, count: int, device) -> torch.Tensor:
    """float32 [count]: the tensor's stream of standard normal values."""
    device = torch.device(device)
    lower, width = _tables(device)
    base = stream_base(seed, name)
    out = torch.empty(count, dtype=torch.float32, device=device)
    chunk = CPU_CHUNK if device.type == "cpu" else DEVICE_CHUNK
    for start in range(0, count, chunk):
        n = min(chunk, count - start)
        bits = mixed_bits(base, start, n, device)
        interval = _logical_shift(bits, 48)
        place = (_logical_shift(bits, 24) & 0xFFFFFF).to(torch.float32) * (2.0 ** -24)     # exact
        step = torch.mul(width[interval], place)           # one rounding
        torch.add(lower[interval], step, out=out[start:start + n])     # one rounding
    return out
