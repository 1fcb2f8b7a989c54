"""Captured steps: a step in which every request brings exactly one token, and a short step that
holds portions of prompts as well, replays a HIP graph of the whole forward instead of launching its
kernels one by one.

As in the reference (worker/src/inference/qwen2/batch_decode.py:42-211): batch sizes are
rounded up to a bucket (1, 2, 4, 8, then steps of 8, and the maximum); each bucket has its
own fixed device buffers that the graph reads (tokens, positions, tables, slots) and its own
logits; rows added to fill the bucket write to the sink page; a bucket is captured the first
time it is used, after one ordinary run with the same buffers (so that scratch memory has
its size and the first result is right), and replayed from then on. If capture or replay
fails, the graphs and the memory pool they share are dropped, the step runs the ordinary way
(which writes the same cache slots again), and so do the next decode steps; later a capture is
tried again, and after a few failures captured steps stay off. Failures are counted and logged.

The step's metadata reaches the device with one copy from pinned host memory before the
replay; nothing inside the graph depends on a Python number.

One number of the step is frozen into a graph all the same: the longest context it is made for
(`BatchMeta.max_kv`). Which lengths deserve a graph of their own is the parts' business
(`Part.capture_context`; attention answers with classes of length, since it cuts the keys into runs
by that number): a bucket keeps one graph per answer of the model, each captured when a step first
needs it.

Short mixed steps (the reference captures decode steps only): a step of at most `mixed_tokens` tokens in
which every request wants the logits of its last token or none is padded to a bucket of tokens and a
bucket of requests; the requests added write to the sink page, and the first of them takes whatever
tokens are left over. Which request brings one token is then a fact of the device's buffers, not of the
graph: the kernels are launched for as many single tokens as there may be (`BatchMeta.singles_bound`).
The logits buffer of such a graph has one row a request.
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


def decode_buckets(max_batch: int, chosen: Optional[Sequence[int]] = None) -> Tuple[int, ...]:
    """Batch sizes that get a captured step of their own. By default the reference's rule
    (worker/src/inference/qwen2/batch_decode.py:43-48, vectors in worker/tests/test_batch_decode.py:50-56):
    (32) -> 1,2,4,8,16,24,32; (5) -> 1,2,4,5; (1) -> 1. `chosen` (`EngineConfig.graph_buckets`) replaces the
    rule: sizes above `max_batch` are dropped, and steps with more rows than the largest left run uncaptured."""
    if max_batch < 1:
        raise ValueError("max_batch must be >= 1")
    if chosen is not None:
        sizes = sorted({int(b) for b in chosen})
        if not sizes or sizes[0] < 1:
            raise ValueError("graph_buckets must be batch sizes >= 1")
        return tuple(b for b in sizes if b <= max_batch) or (max_batch,)
    small = [b for b in (1, 2, 4, 8) if b < max_batch]          # powers of two below the maximum,
    eights = list(range(16, max_batch, 8))                      # then every multiple of 8 below it,
    return tuple(small + eights + [max_batch])                  # and the maximum itself


def bucket_for(buckets: Sequence[int], rows: int) -> int:
    """Smallest bucket that holds `rows` (worker/tests/test_batch_decode.py:62)."""
    if rows < 1 or rows > buckets[-1]:
        raise ValueError(f"{rows} rows do not fit the buckets {tuple(buckets)}")
    return buckets[bisect.bisect_left(buckets, rows)]


class _Bucket:
    def __init__(self, tokens: int, requests: int, builder, device) -> None:
        self.tokens = tokens
        self.requests = requests
        self.mixed = tokens != requests
        self.rows = requests if self.mixed else tokens        # of the logits: one a request, or every token
        self.offsets = builder.layout(tokens, requests, self.rows)
        words = int(self.offsets[-1])
        self.host = torch.zeros(words, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(words, dtype=torch.int32, device=device)
        # per class of context length: (graph, its logits buffer)
        self.graphs: Dict[int, Tuple[torch.cuda.CUDAGraph, torch.Tensor]] = {}
        self.copied = torch.cuda.Event()


def token_buckets(most: int) -> Tuple[int, ...]:
    """Token counts that captured mixed steps are made for: 16, 32, 48, 64, 96, 128, ... up to `most`."""
    sizes, step = [], 16
    while True:
        for k in (2, 3):
            size = step * k // 2
            if size > most:
                return tuple(sizes) if sizes else ((most,) if most > 1 else ())
            sizes.append(size)
        step *= 2


class DecodeGraphs:
    RETRY_AFTER_STEPS = 512     # after a failure, steps run uncaptured for so long before a capture is tried again
    MAX_FAILURES = 3            # ... and after so many failures for good
    MAX_MIXED_GRAPHS = 64       # captured mixed steps kept at most; a shape beyond that runs kernel by kernel

    def __init__(self, runner, max_batch: int, buckets: Optional[Sequence[int]] = None, mixed_tokens: int = 0) -> None:
        self.runner = runner
        self.buckets = decode_buckets(max_batch, buckets)
        self.max_batch = self.buckets[-1]
        # a mixed step that is padded needs a request more than it holds
        self.mixed_tokens = int(mixed_tokens)
        self.token_buckets = token_buckets(self.mixed_tokens) if self.mixed_tokens > 1 else ()
        self.request_buckets = decode_buckets(max_batch + 1, None if buckets is None else list(buckets) + [max_batch + 1])
        self._made: Dict[Tuple[int, int], _Bucket] = {}
        self._pool = None
        self.replays = 0
        self.mixed_replays = 0
        self.failures = 0           # captures or replays that raised
        self._resting = 0           # decode steps still to run uncaptured after a failure

    @property
    def failed(self) -> bool:
        """Captured steps are switched off, for now or for good."""
        return self._resting > 0 or self.failures >= self.MAX_FAILURES

    @property
    def captured(self) -> List[int]:
        """Batch sizes that have a graph of a decode step."""
        return sorted(b.tokens for b in self._made.values() if b.graphs and not b.mixed)

    @property
    def captured_contexts(self) -> List[Tuple[int, int]]:
        """(batch size, context class) of every graph of a decode step."""
        return sorted((b.tokens, limit) for b in self._made.values() if not b.mixed for limit in b.graphs)

    @property
    def captured_mixed(self) -> List[Tuple[int, int, int]]:
        """(tokens, requests, context class) of every graph of a mixed step."""
        return sorted((b.tokens, b.requests, limit) for b in self._made.values() if b.mixed for limit in b.graphs)

    def drop(self) -> None:
        """Forget every graph *and* the memory pool they were captured into. The two go together: graphs
        that are destroyed while their pool lives on leave the allocator with blocks that belong to no
        graph, and the next capture into that pool ends in its internal assertion
        (`use_count > 0`)."""
        self._made.clear()
        self._pool = None

    def _mixed_bucket(self, entries: Sequence[StepEntry]) -> Optional[Tuple[int, int]]:
        """(tokens, requests) of the captured step that takes these entries, or None."""
        tokens = sum(len(e.tokens) for e in entries)
        if not self.token_buckets or tokens > self.token_buckets[-1] or len(entries) > self.max_batch:
            return None
        for e in entries:
            if len(e.want) > 1 or (len(e.want) == 1 and int(e.want[0]) != len(e.tokens) - 1):
                return None
        for size in self.token_buckets:
            if size < tokens:
                continue
            if size == tokens:
                requests = bucket_for(self.request_buckets, len(entries))
            else:
                requests = bucket_for(self.request_buckets, len(entries) + 1)
            # every padding request brings a token; what is left of the bucket goes to the first of them
            if size - tokens >= requests - len(entries) and (size > tokens or requests == len(entries)):
                return size, requests
        return None

    def try_run(self, entries: Sequence[StepEntry], feed: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Logits [wanted, vocab] if this step went through a graph, None if it must run the
        ordinary way (no bucket takes it, or captured steps are switched off).
        What is wrong with the entries themselves (a token id out of range, pages not reserved) raises
        as it does in an ordinary step and switches nothing off."""
        if len(entries) > self.max_batch or self.failures >= self.MAX_FAILURES:
            return None
        if all(len(e.tokens) == 1 for e in entries):
            size = bucket_for(self.buckets, len(entries))
            key = (size, size)
        else:
            key = self._mixed_bucket(entries)
            if key is None:
                return None
        if self._resting > 0:
            self._resting -= 1
            return None
        runner = self.runner
        bucket = self._made.get(key)
        if bucket is None:
            if key[0] != key[1] and sum(len(b.graphs) for b in self._made.values() if b.mixed) >= self.MAX_MIXED_GRAPHS:
                return None
            bucket = self._made[key] = _Bucket(key[0], key[1], runner.builder, runner.ops.device)
        bucket.copied.synchronize()                      # the previous copy out of the pinned buffer is done
        pad_requests = bucket.requests - len(entries)
        pad_tokens = bucket.tokens - sum(len(e.tokens) for e in entries) - pad_requests
        max_kv = runner.builder.fill(bucket.host_np, entries, pad_requests=pad_requests, pad_tokens=pad_tokens,
                                     want_all=not bucket.mixed, want_last=bucket.mixed)[5]
        try:
            return self._run(bucket, entries, feed, max_kv)
        except Exception:  # noqa: BLE001 - the ordinary path rewrites the same slots
            self.failures += 1
            self._resting = self.RETRY_AFTER_STEPS
            self.drop()
            _log.exception("captured step failed (failure %d of %d allowed): graphs and their memory pool "
                           "are dropped, steps run uncaptured %s", self.failures, self.MAX_FAILURES,
                           "from now on" if self.failures >= self.MAX_FAILURES
                           else f"for the next {self.RETRY_AFTER_STEPS} steps that a graph would take")
            return None

    def _run(self, bucket: _Bucket, entries: Sequence[StepEntry], feed: Optional[torch.Tensor],
             max_kv: int) -> Optional[torch.Tensor]:
        runner = self.runner
        runner.builder.flush_tables()                    # outside the graph: the number of changed entries varies
        bucket.dev.copy_(bucket.host, non_blocking=True)
        bucket.copied.record()
        if feed is not None and feed.shape[0]:
            bucket.dev[:feed.shape[0]].copy_(feed)       # the token ids lead the packed buffer
        limit = runner.model.capture_context(max_kv, runner.max_model_len)
        if limit < max_kv:
            raise RuntimeError(f"a part asks for a captured step made for {limit} tokens to serve {max_kv}")
        made = bucket.graphs.get(limit)
        if made is None:
            logits = self._capture(bucket, limit)
        else:
            made[0].replay()
            logits = made[1]
            self.replays += 1
        if bucket.mixed:
            self.mixed_replays += 1
        rows = [i for i, e in enumerate(entries) if len(e.want)]
        if not rows:
            return logits[:0]
        if len(rows) == len(entries):
            return logits[:len(entries)]
        return logits[runner.ops.upload(np.asarray(rows, dtype=np.int64))]

    def _forward(self, bucket: _Bucket, limit: int) -> torch.Tensor:
        runner = self.runner
        T, B = bucket.tokens, bucket.requests
        if bucket.mixed:
            ids, meta, want = runner.builder.meta_of(bucket.dev, bucket.offsets, T, B, B, T, limit, singles_bound=B)
        else:
            ids, meta, want = runner.builder.meta_of(bucket.dev, bucket.offsets, T, T, T, 1, limit)
        runner.ops.captured = True
        try:
            return runner.model.forward(runner.ops, ids, meta, runner.cache, runner.act_dtype, want,
                                        every_row=not bucket.mixed)
        finally:
            runner.ops.captured = False

    def _capture(self, bucket: _Bucket, limit: int) -> torch.Tensor:
        # one ordinary run first: sizes scratch buffers and writes this step's keys and values
        torch.cuda.synchronize()
        eager = self._forward(bucket, limit)
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
                logits = self._forward(bucket, limit)
        finally:
            if was_enabled:
                gc.enable()
        # capture launches nothing: replay once so that `logits` holds this step's result
        graph.replay()
        bucket.graphs[limit] = (graph, logits)
        self.replays += 1
        del eager
        return logits
