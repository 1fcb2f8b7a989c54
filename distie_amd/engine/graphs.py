"""Captured decode steps: a step in which every request brings exactly one token replays
a HIP graph of the whole forward instead of launching its kernels one by one.

As in the reference (worker/src/inference/qwen2/batch_decode.py:42-211): batch sizes are
rounded up to a bucket (1, 2, 4, 8, then steps of 8, and the maximum); each bucket has its
own fixed device buffers that the graph reads (tokens, positions, tables, slots) and its own
logits; rows added to fill the bucket write to the sink page; a bucket is captured the first
time it is used, after one ordinary run with the same buffers (so that scratch memory has
its size and the first result is right), and replayed from then on. If capture or replay
fails, graphs are dropped for good and the step runs the ordinary way, which writes the same
cache slots again.

The step's metadata reaches the device with one copy from pinned host memory before the
replay; nothing inside the graph depends on a Python number.
"""

from __future__ import annotations

import bisect
import gc
import logging
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .batch import StepEntry

_log = logging.getLogger(__name__)


def decode_buckets(max_batch: int) -> Tuple[int, ...]:
    """(32) -> 1,2,4,8,16,24,32; (5) -> 1,2,4,5; (1) -> 1
    (worker/tests/test_batch_decode.py:50-56)."""
    if max_batch < 1:
        raise ValueError("max_batch must be >= 1")
    sizes = {b for b in (1, 2, 4, 8) if b < max_batch}
    sizes.update(range(16, max_batch, 8))
    sizes.add(max_batch)
    return tuple(sorted(sizes))


def bucket_for(buckets: Sequence[int], rows: int) -> int:
    """Smallest bucket that holds `rows` (worker/tests/test_batch_decode.py:62)."""
    if rows < 1 or rows > buckets[-1]:
        raise ValueError(f"{rows} rows do not fit the buckets {tuple(buckets)}")
    return buckets[bisect.bisect_left(buckets, rows)]


class _Bucket:
    def __init__(self, size: int, builder, device) -> None:
        self.size = size
        self.offsets = builder.layout(size, size, size)
        words = int(self.offsets[-1])
        self.host = torch.zeros(words, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(words, dtype=torch.int32, device=device)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.copied = torch.cuda.Event()


class DecodeGraphs:
    def __init__(self, runner, max_batch: int) -> None:
        self.runner = runner
        self.buckets = decode_buckets(max_batch)
        self.max_batch = max_batch
        self._made: Dict[int, _Bucket] = {}
        self._pool = None
        self.failed = False
        self.replays = 0

    @property
    def captured(self) -> List[int]:
        return sorted(size for size, b in self._made.items() if b.graph is not None)

    def try_run(self, entries: Sequence[StepEntry], feed: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Logits [wanted, vocab] if this step went through a graph, None if it must run the
        ordinary way (not a pure decode step, too many rows, or graphs have failed)."""
        if self.failed or len(entries) > self.max_batch or any(len(e.tokens) != 1 for e in entries):
            return None
        try:
            return self._run(entries, feed)
        except Exception:  # noqa: BLE001 - the ordinary path rewrites the same slots
            _log.exception("captured decode step failed; all steps run uncaptured from now on")
            self.failed = True
            self._made.clear()
            return None

    def _run(self, entries: Sequence[StepEntry], feed: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        runner = self.runner
        size = bucket_for(self.buckets, len(entries))
        bucket = self._made.get(size)
        if bucket is None:
            bucket = self._made[size] = _Bucket(size, runner.builder, runner.ops.device)
        bucket.copied.synchronize()                      # the previous copy out of the pinned buffer is done
        runner.builder.fill(bucket.host_np, entries, pad_requests=size - len(entries), want_all=True)
        bucket.dev.copy_(bucket.host, non_blocking=True)
        bucket.copied.record()
        if feed is not None:
            bucket.dev[:len(entries)].copy_(feed)        # the token ids lead the packed buffer
        if bucket.graph is None:
            self._capture(bucket)
        else:
            bucket.graph.replay()
            self.replays += 1
        rows = [i for i, e in enumerate(entries) if len(e.want)]
        if not rows:
            return bucket.logits[:0]
        if len(rows) == len(entries):
            return bucket.logits[:len(entries)]
        return bucket.logits[torch.tensor(rows, device=bucket.logits.device)]

    def _forward(self, bucket: _Bucket) -> torch.Tensor:
        runner = self.runner
        n = bucket.size
        ids, meta, want = runner.builder.meta_of(bucket.dev, bucket.offsets, n, n, n, 1, runner.max_model_len)
        return runner.model.forward(runner.ops, ids, meta, runner.cache, runner.act_dtype, want)

    def _capture(self, bucket: _Bucket) -> None:
        # one ordinary run first: sizes scratch buffers and writes this step's keys and values
        torch.cuda.synchronize()
        eager = self._forward(bucket)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        if self._pool is None:
            self._pool = torch.cuda.graph_pool_handle()
        # While a stream captures, calls such as freeing pinned memory or querying an event are errors, and one
        # raised in a destructor ends the process. The garbage collector could run such destructors of
        # objects that died earlier (an engine that was dropped) at any allocation in here: it is held
        # off for the capture, and what other threads do is not this capture's business.
        was_enabled = gc.isenabled()
        gc.collect()
        gc.disable()
        try:
            with torch.cuda.graph(graph, pool=self._pool, capture_error_mode="thread_local"):
                bucket.logits = self._forward(bucket)
        finally:
            if was_enabled:
                gc.enable()
        # capture launches nothing: replay once so that `logits` holds this step's result
        graph.replay()
        bucket.graph = graph
        self.replays += 1
        del eager
