"""Gated feed-forward: down(silu(gate x) * up x), no biases
(worker/src/inference/qwen2/model.py:228-236). Gate and up are one matrix product:
their weights are stacked at load."""

from __future__ import annotations

import torch

from .base import FeedForward, ParamSpec, register_part


class SwiGLU(FeedForward):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.hidden_size = int(spec.params["hidden_size"])
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.gate_up_weight = self.down_weight = None

    def param_specs(self):
        return {
            "gate_proj.weight": ParamSpec((self.intermediate_size, self.hidden_size)),
            "up_proj.weight": ParamSpec((self.intermediate_size, self.hidden_size)),
            "down_proj.weight": ParamSpec((self.hidden_size, self.intermediate_size)),
        }

    def load(self, tensors) -> None:
        gate, up = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        dtype = torch.float32 if torch.float32 in (gate.dtype, up.dtype) else gate.dtype
        self.gate_up_weight = torch.cat([gate.to(dtype), up.to(dtype)], dim=0).contiguous()
        self.down_weight = tensors["down_proj.weight"].contiguous()

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.gate_up_weight, gated=True, role="gate_up")
        ops.prepare_linear(self.down_weight, role="down")

    def forward(self, ops, x, ctx):
        return ops.linear(ops.linear_silu_mul(x, self.gate_up_weight), self.down_weight)


register_part("feed_forward", "swiglu", SwiGLU)
