"""Continuous batching: which requests run in the next step, and with which tokens.

Bookkeeping only, no tensors. Every step (the order is the reference's,
worker/src/inference/scheduler.py:141-148):

1. requests that were aborted are dropped and what they hold is given back;
2. running requests get their next tokens: one for a request that decodes, the next
   portion for a prompt that is not yet through. If the pages for them are not there,
   the newest running request is preempted (its pages and slot go back, it waits at the
   front of the queue and later recomputes its prompt and the tokens it has produced;
   it never emits a token twice) until they are, or until the needy request itself
   was the newest (scheduler.py:182-194, 213-225);
3. waiting requests are admitted first come first served while there is a seat
   (`max_seqs`), budget, a state slot and pages for the portion they would run now.

Different from the reference: a prompt may be cut. All tokens of a step together stay
within `token_budget`; decoding requests come first, then prompts in flight, then new
admissions, and a prompt gets as many tokens as the budget has left (the reference
never cuts a prompt, so its budget only gates admission: scheduler.py:196-211). Only a
portion that reaches the end of what is known of the request asks for logits and
produces a token.
"""

from __future__ import annotations

import enum
import logging
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence as Seq, Set

from ..cache.block_pool import OutOfBlocks
from ..cache.manager import CacheManager, pages_needed
from ..sampling.sampler import SamplingParams

_log = logging.getLogger(__name__)


class BlockPoolExhausted(OutOfBlocks):
    """A request can never fit the cache (the reference's name: worker/src/inference/engine.py:23)."""


class SeqState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass(eq=False)
class Sequence:
    request_id: Hashable
    prompt_ids: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    eos_ids: Seq[int] = ()
    output_ids: List[int] = field(default_factory=list)
    num_computed: int = 0                 # tokens whose keys and values are in the cache
    state: SeqState = SeqState.WAITING
    preemptions: int = 0
    finish_reason: Optional[str] = None
    error: Optional[BaseException] = None

    @property
    def max_new_tokens(self) -> int:
        return self.params.cap()

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.output_ids)

    def tokens(self, begin: int, end: int) -> List[int]:
        n = len(self.prompt_ids)
        if end <= n:
            return self.prompt_ids[begin:end]
        if begin >= n:
            return self.output_ids[begin - n:end - n]
        return self.prompt_ids[begin:] + self.output_ids[:end - n]


@dataclass(frozen=True)
class ScheduledSeq:
    seq: Sequence
    token_ids: List[int]
    past_len: int
    samples: bool          # this portion ends where the request's known tokens end


@dataclass(frozen=True)
class StepPlan:
    items: tuple
    # For a step planned ahead (`Scheduler.schedule_ahead`): item i continues the request of item
    # `feeds[i]` of the step before, whose sampled token is not known to the host yet.
    feeds: Optional[tuple] = None

    @property
    def num_tokens(self) -> int:
        return sum(len(item.token_ids) for item in self.items)

    @property
    def is_decode(self) -> bool:
        return all(len(item.token_ids) == 1 for item in self.items)


@dataclass(frozen=True)
class Emission:
    seq: Sequence
    token_id: int
    finished: bool


class Scheduler:
    def __init__(self, cache: CacheManager, max_seqs: int = 32, token_budget: int = 2048,
                 max_model_len: Optional[int] = None) -> None:
        if max_seqs < 1 or token_budget < 1:
            raise ValueError("max_seqs and token_budget must be >= 1")
        self.cache = cache
        self.max_seqs = min(int(max_seqs), cache.num_slots)
        self.token_budget = int(token_budget)
        self.max_model_len = max_model_len
        self._waiting: Deque[Sequence] = deque()
        self._running: List[Sequence] = []
        self._aborted: Set[Hashable] = set()
        self._ids: Dict[Hashable, Sequence] = {}

    # ------------------------------------------------------------- queries
    @property
    def num_waiting(self) -> int:
        return len(self._waiting)

    @property
    def num_running(self) -> int:
        return len(self._running)

    def has_work(self) -> bool:
        return bool(self._waiting or self._running or self._aborted)

    # ------------------------------------------------------------- requests
    def submit(self, seq: Sequence) -> None:
        if not seq.prompt_ids:
            raise ValueError("prompt_ids must be non-empty")
        if seq.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")
        if seq.request_id in self._ids:
            raise ValueError(f"duplicate request_id {seq.request_id}")
        total = len(seq.prompt_ids) + seq.max_new_tokens
        if self.max_model_len is not None and total > self.max_model_len:
            raise ValueError(f"request {seq.request_id}: prompt + max_new_tokens = {total} exceeds "
                             f"the model length {self.max_model_len}")
        # worst case the request holds every page it will ever need at once (scheduler.py:125-131)
        need = pages_needed(total, self.cache.block_size)
        if need > self.cache.num_blocks:
            raise BlockPoolExhausted(f"out of KV blocks: request needs {need} pages, pool has {self.cache.num_blocks}")
        seq.state = SeqState.WAITING
        self._waiting.append(seq)
        self._ids[seq.request_id] = seq

    def abort(self, request_id) -> None:
        """Takes effect at the next schedule(); safe while a step is in flight."""
        if request_id in self._ids:
            self._aborted.add(request_id)

    # ------------------------------------------------------------- one step
    def schedule(self) -> StepPlan:
        self._reap_aborted()
        budget = self.token_budget
        preempted = False
        items: List[ScheduledSeq] = []
        # decoding requests first, then prompts in flight; within each, oldest first
        order = sorted(range(len(self._running)),
                       key=lambda i: (self._running[i].num_tokens - self._running[i].num_computed > 1, i))
        for seq in [self._running[i] for i in order]:
            if seq.state is not SeqState.RUNNING:
                continue            # preempted while an older request was served
            pending = seq.num_tokens - seq.num_computed
            n = min(pending, budget)
            if n < 1:
                continue
            while seq.state is SeqState.RUNNING and not self.cache.can_reserve(seq.request_id, n):
                victim = self._running[-1]
                # the victim may already have its tokens in this step's plan: take them out again
                budget += sum(len(it.token_ids) for it in items if it.seq is victim)
                items = [it for it in items if it.seq is not victim]
                self._preempt(victim)
                preempted = True
            if seq.state is not SeqState.RUNNING:
                continue
            self.cache.reserve(seq.request_id, n)
            items.append(self._item(seq, n))
            budget -= n
        # no admission in a step that had to preempt: the victim would come straight back
        while not preempted and self._waiting and len(self._running) < self.max_seqs and budget > 0:
            seq = self._waiting[0]
            n = min(seq.num_tokens, budget)
            # admit by the pages of everything known of the request (scheduler.py:196-211), though
            # only the pages of the portion that runs now are taken
            if self.cache.slots.num_free < 1 or not self.cache.can_reserve(seq.request_id, seq.num_tokens):
                break
            self._waiting.popleft()
            self.cache.add(seq.request_id)
            self.cache.reserve(seq.request_id, n)
            seq.num_computed = 0
            seq.state = SeqState.RUNNING
            self._running.append(seq)
            items.append(self._item(seq, n))
            budget -= n
        return StepPlan(items=tuple(items))

    PENDING = 0        # stands in a planned-ahead item for the token that the step before is still sampling

    def schedule_ahead(self, plan: StepPlan) -> Optional[StepPlan]:
        """The step after `plan` (launched, not yet completed), planned before `plan`'s tokens are
        known, so that it can be launched while the host still waits for them; None where that is not
        plain. Every running request must be in `plan`. The step after then holds, in this order:
        the requests of `plan` that sample, with the pending token as their one token (`feeds` names
        their places in `plan`; those that reach their length with the pending token are left out);
        the next portions of prompts that `plan` has not finished; and waiting requests for which a
        seat, a state slot and pages are free now (the seat of a request that ends with the pending
        token is free one step later). Nobody is preempted for it: if a page is missing the answer is
        None and the plain schedule decides who gives way. A request that turns out to have ended
        with the pending token (end of sequence, abort) has a row of the next step computed for
        nothing; `complete` skips it."""
        self._reap_aborted()
        if not plan.items or len(plan.items) != len(self._running):
            return None
        if any(item.seq.state is not SeqState.RUNNING for item in plan.items):
            return None
        budget = self.token_budget
        items: List[ScheduledSeq] = []
        feeds: List[int] = []
        # called after `plan` was launched and before it is completed: its tokens are the pending ones
        for i, item in enumerate(plan.items):
            if not item.samples:
                continue
            if len(item.seq.output_ids) + 1 >= item.seq.max_new_tokens:
                continue                                  # ends with the pending token, whatever it is
            if budget < 1 or not self.cache.can_reserve(item.seq.request_id, 1):
                # pages run out: the plain schedule decides who gives way. What was taken so far stays
                # with requests that need it for their next token anyway.
                return None
            self.cache.reserve(item.seq.request_id, 1)
            items.append(ScheduledSeq(seq=item.seq, token_ids=[self.PENDING],
                                      past_len=item.past_len + len(item.token_ids), samples=True))
            feeds.append(i)
            budget -= 1
        for item in plan.items:
            if item.samples:
                continue
            seq = item.seq
            begin = item.past_len + len(item.token_ids)
            n = min(seq.num_tokens - begin, budget)
            if n < 1:
                return None                               # every running request is in a step, or the step is not plain
            if not self.cache.can_reserve(seq.request_id, n):
                return None
            self.cache.reserve(seq.request_id, n)
            items.append(ScheduledSeq(seq=seq, token_ids=seq.tokens(begin, begin + n), past_len=begin,
                                      samples=begin + n == seq.num_tokens))
            budget -= n
        while self._waiting and len(self._running) < self.max_seqs and budget > 0:
            seq = self._waiting[0]
            n = min(seq.num_tokens, budget)
            if self.cache.slots.num_free < 1 or not self.cache.can_reserve(seq.request_id, seq.num_tokens):
                break
            self._waiting.popleft()
            self.cache.add(seq.request_id)
            self.cache.reserve(seq.request_id, n)
            seq.num_computed = 0
            seq.state = SeqState.RUNNING
            self._running.append(seq)
            items.append(self._item(seq, n))
            budget -= n
        if not items:
            return None
        return StepPlan(items=tuple(items), feeds=tuple(feeds))

    def _item(self, seq: Sequence, n: int) -> ScheduledSeq:
        begin = seq.num_computed
        return ScheduledSeq(seq=seq, token_ids=seq.tokens(begin, begin + n), past_len=begin,
                            samples=begin + n == seq.num_tokens)

    def complete(self, plan: StepPlan, next_ids: Seq[Optional[int]]) -> List[Emission]:
        """`next_ids[i]` is the token sampled for `plan.items[i]` (ignored where the item does
        not sample). The cache's own counts were advanced by the step function."""
        if len(next_ids) != len(plan.items):
            raise ValueError("one entry per scheduled sequence is required")
        out: List[Emission] = []
        for item, token in zip(plan.items, next_ids):
            seq = item.seq
            if seq.request_id in self._aborted or seq.state is not SeqState.RUNNING:
                continue
            seq.num_computed = item.past_len + len(item.token_ids)
            if not item.samples:
                continue
            token = int(token)
            seq.output_ids.append(token)
            hit_eos = (not seq.params.ignore_eos) and token in seq.eos_ids
            finished = hit_eos or len(seq.output_ids) >= seq.max_new_tokens
            if finished:
                seq.finish_reason = "stop" if hit_eos else "length"
                self._finish(seq)
            out.append(Emission(seq=seq, token_id=token, finished=finished))
        return out

    def fail(self, plan: StepPlan, error: BaseException) -> List[Sequence]:
        """A step raised: every request in it is over, with the error, and what it holds goes
        back (worker/src/inference/batch_loop.py:135-147)."""
        failed = []
        for item in plan.items:
            seq = item.seq
            if seq.state is SeqState.RUNNING:
                seq.error = error
                seq.finish_reason = "error"
                self._finish(seq)
                failed.append(seq)
        return failed

    # ------------------------------------------------------------- internals
    def _reap_aborted(self) -> None:
        for request_id in list(self._aborted):
            seq = self._ids.pop(request_id, None)
            if seq is None:
                continue
            if seq.state is SeqState.WAITING:
                self._waiting.remove(seq)
            elif seq.state is SeqState.RUNNING:
                self._running.remove(seq)
                self._release(seq)
            seq.state = SeqState.FINISHED
            seq.finish_reason = "abort"
            _log.info("sequence aborted request_id=%s", request_id)
        self._aborted.clear()

    def _preempt(self, seq: Sequence) -> None:
        self._running.remove(seq)
        self._release(seq)
        seq.num_computed = 0
        seq.state = SeqState.WAITING
        seq.preemptions += 1
        self._waiting.appendleft(seq)
        _log.info("sequence preempted request_id=%s tokens=%s preemptions=%s",
                  seq.request_id, seq.num_tokens, seq.preemptions)

    def _finish(self, seq: Sequence) -> None:
        self._running.remove(seq)
        self._release(seq)
        seq.state = SeqState.FINISHED
        self._ids.pop(seq.request_id, None)

    def _release(self, seq: Sequence) -> None:
        if seq.request_id in self.cache:
            self.cache.release(seq.request_id)
