"""The step function: a batch of (request, its next tokens) in, logits at the wanted
places out.

It runs only the tokens it is given, as one flattened batch, from the cache that earlier
steps left: portions of prompts beside single decoded tokens, cut anywhere. It samples
nothing (the reference's step also samples: worker/src/inference/model_runner.py:51-62).
Pages for the new tokens are reserved here unless the caller (the scheduler) has done so,
and the cache's counts advance when the step is done.
"""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..cache.manager import CacheManager
from .batch import BatchBuilder, StepEntry
from .model import Model


class ModelRunner:
    def __init__(self, model: Model, cache: CacheManager, ops, act_dtype: torch.dtype,
                 max_model_len: Optional[int] = None) -> None:
        self.model = model
        self.cache = cache
        self.ops = ops
        self.act_dtype = act_dtype
        self.max_model_len = int(max_model_len or model.spec.max_positions)
        self.builder = BatchBuilder(cache, self.max_model_len, ops.device, model.spec.vocab_size, ops)
        self.graphs = None          # set by the engine when captured decode steps are on
        model.prepare(ops)

    def step(self, entries: Sequence[StepEntry], reserve: bool = True,
             feed: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """-> float32 [wanted, vocab] in the order of the entries and of their `want`
        (None if nothing is wanted). A request not yet known to the cache is added.

        `feed` (int32 [F], on the device, F <= len(entries)): each of the first F entries brings one
        token, and the token of entry i is feed[i], which need not have reached the host (those
        entries' own tokens are placeholders)."""
        if feed is not None and (feed.shape[0] > len(entries) or
                                 any(len(e.tokens) != 1 for e in entries[:feed.shape[0]])):
            raise ValueError("a fed step takes one token for each of its first entries")
        if not entries:
            raise ValueError("empty step")
        for entry in entries:
            if entry.request_id not in self.cache:
                self.cache.add(entry.request_id)
        if reserve:
            # if a reservation fails nothing was written yet; pages taken for this step stay with
            # their requests and are returned when those end
            for entry in entries:
                self.cache.reserve(entry.request_id, len(entry.tokens))
        logits, ran = None, False
        if self.graphs is not None:
            logits = self.graphs.try_run(entries, feed)   # a view of the bucket's buffer: use it before the next step
            ran = logits is not None
            if ran and logits.shape[0] == 0:
                logits = None
        if not ran:
            ids, meta, want_rows = self.builder.build(entries)
            if feed is not None and feed.shape[0]:
                ids[:feed.shape[0]].copy_(feed)           # one-token entries lead the step: entry i is token i
            logits = self.model.forward(self.ops, ids, meta, self.cache, self.act_dtype, want_rows)
        for entry in entries:
            self.cache.commit(entry.request_id, len(entry.tokens))
        return logits

    def finish(self, request_id) -> None:
        if request_id in self.cache:
            self.cache.release(request_id)
