"""Grouped-query attention over the paged cache.

q/k/v projections (bias optional), rotation of q and k, the new keys and values written
to the cache before it is read, softmax(q k^T * scale) v over the visible keys, output
projection (worker/src/inference/qwen2/model.py:138-225; the write-then-read order is
worker/src/inference/qwen2/paged_attn.py:389-397). Query head h reads kv head h // G.
On a windowed layer key j is visible to query i iff j <= i and i - j < window (the
reference has no windowed layers: model.py:58-60).

The three projections are one matrix product: their weights are stacked at load.
"""

from __future__ import annotations

import torch

from ..config.model_config import PartSpec
from .base import Mixer, PagedKV, ParamSpec, build_part, register_part


class Attention(Mixer):
    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.num_heads = int(p["num_heads"])
        self.num_kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.qkv_bias = bool(p.get("qkv_bias", False))
        self.out_bias = bool(p.get("out_bias", False))
        self.window = p.get("window")
        self.scale = float(p.get("scale", self.head_dim ** -0.5))
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.position = build_part("position", p.get("position") or PartSpec("none"))
        self.qkv_weight = self.qkv_bias_t = self.out_weight = self.out_bias_t = None

    def cache_requirement(self):
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def param_specs(self):
        q = self.num_heads * self.head_dim
        kv = self.num_kv_heads * self.head_dim
        specs = {
            "q_proj.weight": ParamSpec((q, self.hidden_size)),
            "k_proj.weight": ParamSpec((kv, self.hidden_size)),
            "v_proj.weight": ParamSpec((kv, self.hidden_size)),
            "o_proj.weight": ParamSpec((self.hidden_size, q)),
        }
        if self.qkv_bias:
            specs.update({"q_proj.bias": ParamSpec((q,)), "k_proj.bias": ParamSpec((kv,)),
                          "v_proj.bias": ParamSpec((kv,))})
        if self.out_bias:
            specs["o_proj.bias"] = ParamSpec((self.hidden_size,))
        return specs

    def load(self, tensors) -> None:
        parts = [tensors[f"{n}_proj.weight"] for n in "qkv"]
        dtype = torch.float32 if any(t.dtype == torch.float32 for t in parts) else parts[0].dtype
        self.qkv_weight = torch.cat([t.to(dtype) for t in parts], dim=0).contiguous()
        if self.qkv_bias:
            self.qkv_bias_t = torch.cat([tensors[f"{n}_proj.bias"].float() for n in "qkv"]).contiguous()
        self.out_weight = tensors["o_proj.weight"].contiguous()
        if self.out_bias:
            self.out_bias_t = tensors["o_proj.bias"].float().contiguous()
        self.position.to_device(self.out_weight.device)

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.qkv_weight, rotary=(self.num_heads, self.num_kv_heads, self.head_dim))
        ops.prepare_linear(self.out_weight)

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        qkv = ops.linear_rope_kv_write(x, self.qkv_weight, self.qkv_bias_t, ctx.meta, cache.group, cache.k, cache.v,
                                       self.position.rotary(), self.num_heads, self.num_kv_heads, self.head_dim,
                                       writes_cache)
        mixed = ops.paged_attention(qkv, ctx.meta, cache.group, cache.k, cache.v, self.num_heads,
                                    self.num_kv_heads, self.head_dim, self.scale, self.window)
        return ops.linear(mixed, self.out_weight, self.out_bias_t)


register_part("mixer", "attention", Attention)
