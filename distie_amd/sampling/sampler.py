"""Greedy and temperature sampling: all the reference samples with
(worker/src/inference/model_runner.py:122-130; top-p, top-k and repetition penalty are
fields of its protocol that its server ignores: worker/src/worker/servicer.py:74-80).

Greedy: argmax of the float32 logits, lowest index among equals. Temperature t > 0: one
draw from softmax(logits / t). The reference draws from torch's global generator; here a
request carries a seed and the n-th token of the request uses the uniform number
`uniform_of(seed, n)`, so a run can be repeated and does not depend on what else is in
the batch. The draw inverts the cumulative sum (first index whose cumulative weight
exceeds u * total)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

_MASK = (1 << 64) - 1


def uniform_of(seed: int, counter: int) -> float:
    """The generator of the sampling kernel, in Python: splitmix64 of (seed, counter),
    top 24 bits as a float in [0, 1)."""
    z = (seed * 0x9E3779B97F4A7C15 + counter * 0xD1B54A32D192ED03 + 0x94D049BB133111EB) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z = z ^ (z >> 31)
    return (z >> 40) / 16777216.0


def derive_seed(engine_seed: int, arrival: int) -> int:
    """The seed of the `arrival`-th request of an engine that was not given one: a splitmix64 step of
    the two, so that neighbouring arrivals get unrelated streams."""
    z = ((engine_seed & _MASK) ^ ((arrival * 0x9E3779B97F4A7C15 + 0x632BE59BD9B4E019) & _MASK)) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


@dataclass(frozen=True)
class SamplingParams:
    """`max_new_tokens` and `temperature` are the reference's `max_tokens` and
    `temperature` (proto/inference.proto:17-24); a non-positive `max_new_tokens` means the
    reference's default of 16 (worker/src/inference/engine.py:16-17, 170-173)."""

    max_new_tokens: int = 16
    temperature: float = 0.0
    seed: Optional[int] = None        # None: a stream of the request's own, derived from the engine's seed
    eos_id: Optional[int] = None      # None: the model's own end-of-sequence ids
    ignore_eos: bool = False

    def cap(self) -> int:
        return 16 if self.max_new_tokens <= 0 else self.max_new_tokens


class Sampler:
    def __init__(self, ops) -> None:
        self.ops = ops

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
               counters: Sequence[int]) -> List[int]:
        """logits float32 [R, V] -> R token ids (one device-to-host copy)."""
        return self.sample_device(logits, temperatures, seeds, counters).tolist()

    def sample_device(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
                      counters: Sequence[int]) -> torch.Tensor:
        """As `sample`, but the ids stay on the device (int32 [R]): nothing waits for them."""
        if logits.shape[0] != len(temperatures):
            raise ValueError("one temperature per row of logits")
        if all(t <= 0 for t in temperatures):
            return self.ops.argmax(logits)
        # int64 two's complement carries the unsigned 64-bit seed unchanged
        wrap = lambda v: ((int(v) & _MASK) ^ (1 << 63)) - (1 << 63)
        return self.ops.sample(
            logits,
            self.ops.upload(np.asarray(list(temperatures), dtype=np.float32)),
            self.ops.upload(np.asarray([wrap(s) for s in seeds], dtype=np.int64)),
            self.ops.upload(np.asarray([wrap(c) for c in counters], dtype=np.int64)))
