"""The kernel surface: every device operation the parts and the engine use.

The product implementation is `HipOps` (hand-written HIP for gfx950, loaded from
shared libraries built out of `distie_amd/csrc`); there is no other implementation in
this package and no fallback: constructing `HipOps` without a GPU or without the
libraries raises. Parts never touch torch math directly; they call these methods, so
what runs on the device is exactly this list.

Conventions: T = tokens of the step (all requests, flattened), B = requests of the
step, `act` = the engine's activation dtype (bfloat16 or float32). The residual stream
is always float32. Weights may be bfloat16 or float32 whatever `act` is.
"""

from __future__ import annotations

import abc
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np
import torch


@dataclass
class GroupMeta:
    """Addressing of one cache group for one step."""

    block_table: torch.Tensor          # int32 [rows, W]; -1 where a page was given back. Row of request b:
    #                                    BatchMeta.table_rows[b] (the request's state slot: the tables live on the
    #                                    device from step to step), or b itself where table_rows is None
    slots: torch.Tensor                # int32 [T]; block * block_size + offset of each new token


@dataclass
class BatchMeta:
    """Device tensors that describe one flattened step (the reference's BatchMeta,
    worker/src/inference/qwen2/paged_attn.py:310-357, plus what windows, state slots and
    wanted rows need)."""

    num_tokens: int
    num_requests: int
    positions: torch.Tensor            # int32 [T] absolute position of each token
    token_request: torch.Tensor        # int32 [T] index of the request each token belongs to
    cu_q: torch.Tensor                 # int32 [B+1] prefix sums of the new-token counts
    kv_len: torch.Tensor               # int32 [B] tokens cached after this step (past + new)
    state_slots: torch.Tensor          # int32 [B] per-request state slot
    max_q: int                         # host copies, for launch geometry
    max_kv: int
    block_size: int
    groups: List[GroupMeta] = field(default_factory=list)
    # host mirrors (numpy) for parts that run per request on the host side
    host_cu_q: Optional[object] = None
    host_past: Optional[object] = None
    all_decode: bool = False           # every request brings exactly one token
    table_rows: Optional[torch.Tensor] = None    # int32 [B]: each request's row of the groups' block tables
    # In a captured step no launch may depend on how the step's tokens are spread over its requests (that is
    # known on the device only): `max_q` and `max_kv` are then bounds, and so is this, the most requests that
    # bring exactly one token (None: an implementation may count them from `host_cu_q`).
    singles_bound: Optional[int] = None
    scratch: dict = field(default_factory=dict)   # what an implementation computes once per step (cos/sin tables)


@dataclass(frozen=True)
class ScoreExtras:
    """What a variant of attention does to a score beyond scale, causal mask and window; everything None
    for plain attention. An implementation's kernel that does not take a field that is set refuses the call
    (it never ignores it), so a new variant is a kernel added behind this argument, not a changed signature.

    score(i, j) = q_i . k_j * scale; with `score_cap` c: c * tanh(score / c); with `head_slopes` s:
    + s[h] * (j - i), a bias by the distance to the key with a slope of the head's own (a position
    encoding that needs no rotation)."""

    head_slopes: Optional[torch.Tensor] = None      # float32 [H] on the device
    score_cap: Optional[float] = None               # > 0

    def __post_init__(self):
        if self.score_cap is not None and not self.score_cap > 0:
            raise ValueError("score_cap must be positive")

    @property
    def plain(self) -> bool:
        return self.head_slopes is None and self.score_cap is None


class Ops(abc.ABC):
    device: torch.device
    # True while the engine warms or records a captured step: launches then cost the host nothing when the
    # step is replayed, so an implementation may choose kernels by their time on the device alone
    captured: bool = False

    def upload(self, values: np.ndarray) -> torch.Tensor:
        """A small host array (row indexes, sampling parameters) as a device tensor of the same dtype and
        shape. An implementation makes this a copy that does not wait for the work queued before it."""
        return torch.from_numpy(np.ascontiguousarray(values)).to(self.device)

    def scatter_int32(self, table: torch.Tensor, index: torch.Tensor, value: torch.Tensor) -> None:
        """table.view(-1)[index] = value for int32 tensors on the device (distinct indexes): the block tables'
        changed entries of a step."""
        table.view(-1)[index.long()] = value

    @abc.abstractmethod
    def embed(self, ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        """ids int32 [T], table [V, C] -> float32 [T, C]."""

    @abc.abstractmethod
    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
        """float32 [T, C] -> out_dtype [T, C]; statistics in float32.

        As with `linear`, an implementation may return the result in a form of its own that only its own
        operations read (the HIP kernels leave the norm of few rows to the product that reads it: the value
        is then not computed yet, and stays valid only until `x` is next written in place, which the
        implementation finds out and refuses). A part hands the result on to `linear`, `linear_silu_mul`,
        `linear_rope_kv_write`, `linear_f32out` or `gather_rows`; a part that computes on the values itself
        (indexing, `.float()`, any torch operation) calls `ops.dense(result)` first. The same holds for
        `add_rmsnorm`."""

    @abc.abstractmethod
    def add_rmsnorm(self, residual: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor,
                    eps: float, out_dtype) -> torch.Tensor:
        """residual (float32, updated in place) += delta; returns rmsnorm(residual)."""

    @abc.abstractmethod
    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x [T, K] (act) times weight [N, K] transposed, plus bias [N] -> act [T, N].

        An implementation may return the product in a form of its own that only its
        `add_rmsnorm`, `silu_mul`, `rope_kv_write`, `linear`, `paged_attention` and `gather_rows`
        read (the HIP kernels return partial sums over slices of K for small batches, or, for few
        rows, a product not yet computed that adds itself to the residual stream if `add_rmsnorm`
        is what comes next); parts hand the result on to those operations, or as the `delta` of a
        `ResidualStream`, and do nothing else with it. A part that computes on the values itself
        calls `ops.dense(result)` first."""

    def dense(self, x):
        """The plain tensor of a result that `linear`, `rmsnorm` or `add_rmsnorm` returned in a form of
        its own; any other tensor as it is. For parts that compute on the values themselves."""
        return x

    def prepare_linear(self, weight: torch.Tensor, gated: bool = False, rotary=None, role: Optional[str] = None) -> None:
        """Called once for every weight of a `linear` after it is loaded (`gated`: the weight of a
        `linear_silu_mul`; `rotary = (num_heads, num_kv_heads, head_dim)`: the stacked q/k/v weight
        of a `linear_rope_kv_write`; `role`: what the part calls this product, so that a setting
        can name it). An implementation may build what its products need beside
        the tensor (the HIP kernels keep a second copy in the matrix cores' order for small
        batches)."""

    def linear_rope_kv_write(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                             meta: BatchMeta, group: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                             inv_freq: Optional[torch.Tensor], num_heads: int, num_kv_heads: int,
                             head_dim: int, write: bool) -> torch.Tensor:
        """rope_kv_write(linear(x, weight, bias), ...) for the stacked q/k/v weight; an
        implementation may fuse the two."""
        return self.rope_kv_write(self.linear(x, weight, bias), meta, group, k_cache, v_cache, inv_freq,
                                  num_heads, num_kv_heads, head_dim, write)

    def linear_silu_mul(self, x: torch.Tensor, gate_up_weight: torch.Tensor) -> torch.Tensor:
        """silu_mul(linear(x, gate_up_weight)) with gate_up_weight [2I, K] -> act [T, I]; an
        implementation may fuse the two."""
        return self.silu_mul(self.linear(x, gate_up_weight))

    @abc.abstractmethod
    def linear_f32out(self, x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        """As `linear` without bias, result in float32 (the logits)."""

    @abc.abstractmethod
    def rope_kv_write(self, qkv: torch.Tensor, meta: BatchMeta, group: int, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, inv_freq: Optional[torch.Tensor], num_heads: int,
                      num_kv_heads: int, head_dim: int, write: bool) -> torch.Tensor:
        """Rotate q and k of qkv [T, (H+2KH)*D] by each token's position (angles and
        trigonometry in float32; no rotation if inv_freq is None) and, if `write`, store the
        rotated k and v at the token's slot of k_cache [NB, KH, P, D] / v_cache [NB, KH, D, P]. Returns the
        rotated qkv (the argument itself if it was rotated in place)."""

    @abc.abstractmethod
    def paged_attention(self, qkv: torch.Tensor, meta: BatchMeta, group: int, k_cache: torch.Tensor,
                        v_cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                        scale: float, window: Optional[int], extras: Optional[ScoreExtras] = None) -> torch.Tensor:
        """softmax(q k^T * scale) v over the cached keys 0..position of each token (the last
        `window` of them on a windowed layer), read through the block table -> act [T, H*D].
        `extras`: what a variant adds to the scores (`ScoreExtras`); None for plain attention."""

    @abc.abstractmethod
    def silu_mul(self, gate_up: torch.Tensor) -> torch.Tensor:
        """[T, 2I] -> silu(first half) * second half, [T, I]."""

    @abc.abstractmethod
    def gather_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """x [T, C], rows int32 [R] -> x[rows]."""

    @abc.abstractmethod
    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        """float32 [R, V] -> int32 [R], lowest index among equals."""

    @abc.abstractmethod
    def sample(self, logits: torch.Tensor, temperature: torch.Tensor, seeds: torch.Tensor,
               counters: torch.Tensor) -> torch.Tensor:
        """Rows with temperature <= 0: argmax. Others: one draw from softmax(logits / t)
        with the uniform number hash(seed, counter) -> int32 [R]."""
