"""Rotary position encoding: inv_freq[i] = theta^(-2i/D); the angle of pair (j, j + D/2)
at position p is p * inv_freq[j] (worker/src/inference/qwen2/model.py:93-117). The table
of inverse frequencies is all this part owns: angle, cosine and sine are computed in
float32 inside the kernel that also writes the cache."""

from __future__ import annotations

import torch

from .base import PositionEncoding, register_part


_SHARED = {}


class RotaryPosition(PositionEncoding):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.dim = int(spec.params["dim"])
        self.theta = float(spec.params["theta"])
        if self.dim < 2 or self.dim % 2:
            raise ValueError("rotary dimension must be even")
        # the reference builds the exponent as arange(0, D, 2).float() / D in float32 (model.py:98)
        exponent = torch.arange(0, self.dim, 2, dtype=torch.float32) / self.dim
        self.inv_freq = 1.0 / (self.theta ** exponent)

    def to_device(self, device) -> None:
        # layers with the same rotation share one table, so that what a step derives from it
        # (cosines and sines of the step's positions) is derived once
        key = (self.dim, self.theta, str(device))
        if key not in _SHARED:
            _SHARED[key] = self.inv_freq.to(device)
        self.inv_freq = _SHARED[key]

    def rotary(self):
        return self.inv_freq


class NoPosition(PositionEncoding):
    """For mixers whose order comes from elsewhere (a state, a learned table)."""


register_part("position", "rope", RotaryPosition)
register_part("position", "none", NoPosition)
