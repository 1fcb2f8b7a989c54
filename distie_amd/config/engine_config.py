"""Options of the engine, typed. The reference reads the same knobs from environment
variables ad hoc (worker/src/inference/torch_engine.py:212-226, worker/src/worker/config.py:22-57):
WORKER_MAX_SEQS (32), WORKER_TOKEN_BUDGET (2048), WORKER_NUM_BLOCKS (1024),
WORKER_DECODE_GRAPHS (1), WORKER_STEP_STATS (0); page size 16 (kv_cache.py:25)."""

from __future__ import annotations

import os
from dataclasses import dataclass, replace
from typing import Optional, Tuple, Union

DTYPE_NAMES = {
    "fp32": "float32", "float32": "float32", "float": "float32",
    "bf16": "bfloat16", "bfloat16": "bfloat16",
}

DEFAULT_BLOCK_SIZE = 16
DEFAULT_NUM_BLOCKS = 1024
DEFAULT_MAX_SEQS = 32
DEFAULT_TOKEN_BUDGET = 2048


def resolve_dtype(name: str) -> str:
    """'auto' is bfloat16, the serving precision on the GPU (the reference's 'auto' is
    half on the GPU: torch_engine.py:60-69). fp16 is not a precision of this engine."""
    key = name.strip().lower()
    if key == "auto":
        return "bfloat16"
    if key not in DTYPE_NAMES:
        raise ValueError("dtype must be one of auto, " + ", ".join(sorted(DTYPE_NAMES)))
    return DTYPE_NAMES[key]


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"
    block_size: int = DEFAULT_BLOCK_SIZE
    num_blocks: Optional[int] = None        # pages of the cache; None = from max_cache_tokens or the default
    max_cache_tokens: Optional[int] = None  # pool made for this many cached tokens
    # with neither of the two: pages until this share of the card's memory is in use (weights and their packed
    # copies included); what stays outside holds a full portion's activations, the library's workspaces and the graphs
    gpu_mem_fraction: Optional[float] = None
    max_seqs: int = DEFAULT_MAX_SEQS
    token_budget: int = DEFAULT_TOKEN_BUDGET
    max_model_len: Optional[int] = None     # None = the model's max positions
    use_graphs: bool = True
    # batch sizes that get a captured decode step of their own; None = 1, 2, 4, 8, then every multiple of 8 up to
    # max_seqs (a step is padded up to the next size; one with more rows than the largest runs uncaptured)
    graph_buckets: Optional[Tuple[int, ...]] = None
    # mixed steps (portions of prompts beside single tokens) of up to so many tokens replay graphs as well, padded
    # to 16, 24, 32, 48, 64, 96, ... tokens: launched kernel by kernel such a step costs the host about as long as
    # the device, replayed a sixth of that. 0: only decode steps are captured. (Up to 96 tokens a step runs on this
    # engine's own kernels alone; every bucket of tokens, requests and context length is a graph of its own.)
    graph_tokens: int = 96
    # a second copy of the weights in the matrix cores' order, for decode: True, False, or the roles that get one.
    # A role is whatever name a part gives its product in `Ops.prepare_linear(role=...)`; the parts of the Qwen2
    # decoder name "qkv", "attn_out", "gate_up", "down" and "head", another part may name others
    packed_weights: Union[bool, Tuple[str, ...]] = True
    lookahead: bool = True                  # launch the next decode step before this step's tokens reach the host
    tune_products: bool = False             # at start, let the library time its kernels for the products of a full portion and of large batches
    step_stats: int = 0
    seed: int = 0

    def __post_init__(self):
        object.__setattr__(self, "dtype", resolve_dtype(self.dtype))
        if self.block_size < 1 or self.max_seqs < 1 or self.token_budget < 1:
            raise ValueError("block_size, max_seqs and token_budget must be >= 1")
        if self.num_blocks is not None and self.num_blocks < 1:
            raise ValueError("num_blocks must be >= 1")
        if self.gpu_mem_fraction is not None and not 0.0 < self.gpu_mem_fraction <= 1.0:
            raise ValueError("gpu_mem_fraction must be in (0, 1]")
        if self.graph_buckets is not None:
            buckets = tuple(sorted({int(b) for b in self.graph_buckets}))
            if not buckets or buckets[0] < 1:
                raise ValueError("graph_buckets must be batch sizes >= 1")
            object.__setattr__(self, "graph_buckets", buckets)
        if self.graph_tokens < 0:
            raise ValueError("graph_tokens must be >= 0")
        if not isinstance(self.packed_weights, bool):
            object.__setattr__(self, "packed_weights", tuple(self.packed_weights))

    def pages(self, page_bytes: Optional[int] = None, free_bytes: Optional[int] = None,
              total_bytes: Optional[int] = None) -> int:
        """Pages of the cache. `page_bytes` (what one more page costs over all layers), `free_bytes` and
        `total_bytes` (of the card, with the weights in place) are needed only for `gpu_mem_fraction`."""
        if self.num_blocks is not None:
            return self.num_blocks
        if self.max_cache_tokens is not None:
            return max(1, -(-self.max_cache_tokens // self.block_size))
        if self.gpu_mem_fraction is not None:
            if not page_bytes or free_bytes is None or total_bytes is None:
                raise ValueError("gpu_mem_fraction needs the card's free and total memory and the bytes of a page")
            room = free_bytes - int((1.0 - self.gpu_mem_fraction) * total_bytes)
            pages = room // page_bytes - 1                    # one page more than the pool hands out is kept
            if pages < 1:
                raise ValueError(
                    f"gpu_mem_fraction={self.gpu_mem_fraction}: {free_bytes / 2**30:.1f} GiB of "
                    f"{total_bytes / 2**30:.1f} GiB are free, which leaves no room for a page of {page_bytes} bytes")
            return int(pages)
        return DEFAULT_NUM_BLOCKS

    @classmethod
    def from_env(cls, **overrides) -> "EngineConfig":
        """Environment variables of the reference's worker, where set."""
        def _int(key):
            raw = os.getenv(key, "").strip()
            if not raw:
                return None
            value = int(raw)
            if value < 1:
                raise ValueError(f"{key} must be >= 1")
            return value
        env = {}
        if _int("WORKER_MAX_SEQS"):
            env["max_seqs"] = _int("WORKER_MAX_SEQS")
        if _int("WORKER_TOKEN_BUDGET"):
            env["token_budget"] = _int("WORKER_TOKEN_BUDGET")
        if _int("WORKER_NUM_BLOCKS"):
            env["num_blocks"] = _int("WORKER_NUM_BLOCKS")
        raw = os.getenv("WORKER_DECODE_GRAPHS", "").strip().lower()
        if raw:
            env["use_graphs"] = raw not in {"0", "false", "no", "off"}
        raw = os.getenv("WORKER_GRAPH_BUCKETS", "").strip()
        if raw:
            env["graph_buckets"] = tuple(int(b) for b in raw.split(","))
        raw = os.getenv("WORKER_GRAPH_TOKENS", "").strip()
        if raw:
            env["graph_tokens"] = int(raw)
        raw = os.getenv("WORKER_GPU_MEM_FRACTION", "").strip()
        if raw:
            env["gpu_mem_fraction"] = float(raw)
        raw = os.getenv("WORKER_STEP_STATS", "").strip()
        if raw:
            env["step_stats"] = int(raw)
        env.update({k: v for k, v in overrides.items() if v is not None})
        return replace(cls(), **env)
