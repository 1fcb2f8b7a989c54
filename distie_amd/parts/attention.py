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

import bisect
from typing import Optional, Tuple

import torch

from ..config.model_config import PartSpec
from ..kernels.interface import ScoreExtras
from .base import PAGE, Mixer, PagedTensors, ParamSpec, TensorDecl, build_part, register_part


def PagedKV(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> PagedTensors:
    """What attention keeps for every token, in the layout its kernels read: keys as
    `[kv_heads, page, head_dim]` per page, values transposed inside a page, `[kv_heads, head_dim, page]`,
    so that the key index is contiguous for the matrix cores."""
    return PagedTensors((TensorDecl("k", (num_kv_heads, PAGE, head_dim)),
                         TensorDecl("v", (num_kv_heads, head_dim, PAGE))), window)


def context_classes(limit: int, first: int = 1024) -> Tuple[int, ...]:
    """(4096) -> 1024, 1536, 2048, 3072, 4096; (700) -> 700: steps of a factor 1.5 or 1.33, so a
    captured step's runs of keys are at most that much longer than the step's own would be."""
    if limit < 1 or first < 1:
        raise ValueError("context lengths must be >= 1")
    out = {limit}
    c = first
    while c < limit:
        out.add(c)
        if c + c // 2 < limit and c >= 2:
            out.add(c + c // 2)
        c *= 2
    return tuple(sorted(out))


class Attention(Mixer):
    FIRST_CONTEXT = 1024        # the shortest class of context length that captured steps are made for

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
        self.score_cap = p.get("score_cap")        # None for this architecture: scores are not bent
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.position = build_part("position", p.get("position") or PartSpec("none"))
        self.qkv_weight = self.qkv_bias_t = self.out_weight = self.out_bias_t = None
        self.extras = None                         # what the position encoding or a cap adds to the scores

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
        slopes = self.position.head_slopes(self.num_heads)
        if slopes is not None or self.score_cap is not None:
            if slopes is not None:
                slopes = slopes.to(device=self.out_weight.device, dtype=torch.float32).contiguous()
            self.extras = ScoreExtras(slopes, None if self.score_cap is None else float(self.score_cap))

    def prepare(self, ops) -> None:
        ops.prepare_linear(self.qkv_weight, rotary=(self.num_heads, self.num_kv_heads, self.head_dim),
                           role="qkv")
        ops.prepare_linear(self.out_weight, role="attn_out")

    def capture_context(self, longest: int, limit: int):
        """Decode attention cuts the keys into runs by the longest context of the step, and that number is
        frozen into a captured step: a graph made for the model's limit would suit a 2,000-token context
        badly. So captured steps are made per class of context length (1,024, 1,536, 2,048, 3,072, ... the
        limit), and a step uses the smallest class that holds its longest request."""
        classes = context_classes(limit, self.FIRST_CONTEXT)
        return classes[min(bisect.bisect_left(classes, longest), len(classes) - 1)]

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        k_cache, v_cache = cache["k"], cache["v"]
        qkv = ops.linear_rope_kv_write(x, self.qkv_weight, self.qkv_bias_t, ctx.meta, cache.group, k_cache, v_cache,
                                       self.position.rotary(), self.num_heads, self.num_kv_heads, self.head_dim,
                                       writes_cache)
        mixed = ops.paged_attention(qkv, ctx.meta, cache.group, k_cache, v_cache, self.num_heads,
                                    self.num_kv_heads, self.head_dim, self.scale, self.window, self.extras)
        return ops.linear(mixed, self.out_weight, self.out_bias_t)


register_part("mixer", "attention", Attention)
