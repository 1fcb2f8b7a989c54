"""Continuous batching: which requests run in the next step, and with which of their tokens.

Book-keeping only, no tensors. The cache manager owns pages and slots; the scheduler owns the
*queue* of requests that wait and the *seats* of those that run, and decides, step by step:

1. requests that were cancelled leave, and what they hold goes back;
2. every seated request gets its next *portion*: one token if it decodes, else as much of its
   prompt as the step's token budget has left. If the pages for a portion are not there, the request
   seated last gives way (its pages and slot go back, it returns to the head of the queue and later
   recomputes its prompt and the tokens it has produced; it never emits a token twice), again and
   again until the pages are there or the needy request itself was the one seated last;
3. queued requests are seated first come first served while there is a seat (`max_seqs`), budget,
   a state slot, and pages for everything that is known of them.

The order of these three and the policy of giving way are the reference's
(worker/src/inference/scheduler.py:141-148, 182-225). Different from it: a prompt may be cut. All
tokens of a step together stay within `token_budget`; decoding requests come first, then prompts in
flight, then new arrivals, and a prompt gets as many tokens as the budget has left (the reference
never cuts a prompt, so its budget only gates admission: scheduler.py:196-211). Only a portion that
reaches the end of what is known of the request asks for logits and produces a token.
"""

from __future__ import annotations

import enum
import logging
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, Iterable, List, Optional, Sequence as Seq, Tuple

from ..cache.block_pool import OutOfBlocks
from ..cache.manager import CacheManager, pages_needed
from ..sampling.sampler import SamplingParams

_log = logging.getLogger(__name__)


class BlockPoolExhausted(OutOfBlocks):
    """A request can never fit the cache (the reference's name: worker/src/inference/engine.py:23)."""


class Phase(enum.Enum):
    QUEUED = "queued"       # waits for a seat (new, or gave way and will recompute)
    SEATED = "seated"       # holds a state slot and pages; takes part in steps
    ENDED = "ended"         # length reached, end of sequence, cancelled, or failed


@dataclass(eq=False)
class Request:
    request_id: Hashable
    prompt_ids: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    eos_ids: Seq[int] = ()
    seed: int = 0                         # of this request's draws, fixed when it was submitted
    output_ids: List[int] = field(default_factory=list)
    num_computed: int = 0                 # tokens whose keys and values are in the cache, as far as completed steps go
    phase: Phase = Phase.QUEUED
    preemptions: int = 0
    finish_reason: Optional[str] = None   # "stop" | "length" | "abort" | "error"
    error: Optional[BaseException] = None
    cancelled: bool = False

    @property
    def max_new_tokens(self) -> int:
        return self.params.cap()

    @property
    def num_tokens(self) -> int:
        """Prompt and produced tokens: all that is known of the request."""
        return len(self.prompt_ids) + len(self.output_ids)

    def tokens(self, begin: int, end: int) -> List[int]:
        split = len(self.prompt_ids)
        head = self.prompt_ids[begin:end] if begin < split else []
        tail = self.output_ids[max(begin - split, 0):end - split] if end > split else []
        return head + tail


@dataclass(frozen=True)
class Portion:
    """A request's share of one step: `token_ids` are its tokens `begin .. begin + len - 1`."""

    request: Request
    token_ids: List[int]
    begin: int
    samples: bool          # the portion ends where the request's known tokens end: a token is drawn after it

    @property
    def end(self) -> int:
        return self.begin + len(self.token_ids)


@dataclass(frozen=True)
class StepPlan:
    portions: Tuple[Portion, ...]
    # For a step planned ahead (`Scheduler.schedule_ahead`): portion i continues the request of portion
    # `feeds[i]` of the step before, whose drawn token is not known to the host yet.
    feeds: Optional[Tuple[int, ...]] = None
    gave_way: bool = False     # a request gave way while this step was planned

    @property
    def num_tokens(self) -> int:
        return sum(len(p.token_ids) for p in self.portions)

    @property
    def is_decode(self) -> bool:
        return all(len(p.token_ids) == 1 for p in self.portions)


@dataclass(frozen=True)
class Emission:
    request: Request
    token_id: int
    finished: bool


class _Draft:
    """A step while it is planned: the budget that is left, and the portions chosen so far."""

    def __init__(self, budget: int) -> None:
        self.left = budget
        self.portions: List[Portion] = []
        self.feeds: List[int] = []

    def put(self, request: Request, begin: int, count: int) -> None:
        """The request's known tokens begin .. begin + count - 1."""
        self.portions.append(Portion(request, request.tokens(begin, begin + count), begin,
                                     samples=begin + count == request.num_tokens))
        self.left -= count

    def put_pending(self, request: Request, begin: int, stand_in: int, place: int) -> None:
        """One token that is not known yet: the one drawn after portion `place` of the step before."""
        self.portions.append(Portion(request, [stand_in], begin, samples=True))
        self.feeds.append(place)
        self.left -= 1

    def withdraw(self, request: Request) -> None:
        """A request that gives way may already have its portion in the draft."""
        kept = [p for p in self.portions if p.request is not request]
        self.left += sum(len(p.token_ids) for p in self.portions) - sum(len(p.token_ids) for p in kept)
        self.portions = kept


class Scheduler:
    PENDING = 0        # stands in a step planned ahead for the token that the step before still draws

    def __init__(self, cache: CacheManager, max_seqs: int = 32, token_budget: int = 2048,
                 max_model_len: Optional[int] = None) -> None:
        if max_seqs < 1 or token_budget < 1:
            raise ValueError("max_seqs and token_budget must be >= 1")
        self.cache = cache
        self.max_seqs = min(int(max_seqs), cache.num_slots)
        self.token_budget = int(token_budget)
        self.max_model_len = max_model_len
        self._queue: Deque[Request] = deque()
        self._seated: List[Request] = []            # in the order in which they were seated
        self._known: Dict[Hashable, Request] = {}
        self._to_cancel: List[Request] = []

    # ------------------------------------------------------------- queries
    @property
    def num_waiting(self) -> int:
        return len(self._queue)

    @property
    def num_running(self) -> int:
        return len(self._seated)

    def has_work(self) -> bool:
        return bool(self._queue) or bool(self._seated) or bool(self._to_cancel)

    def request(self, request_id) -> Request:
        return self._known[request_id]

    def queued(self) -> List[Request]:
        return list(self._queue)

    # ------------------------------------------------------------- arrivals and cancellations
    def submit(self, request: Request) -> None:
        """Refuses a request that could never run: empty, a duplicate, longer than the model allows,
        or larger than the whole cache in its worst case (scheduler.py:118-134)."""
        if len(request.prompt_ids) == 0:
            raise ValueError("prompt_ids must be non-empty")
        if request.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")
        if request.request_id in self._known:
            raise ValueError(f"duplicate request_id {request.request_id}")
        longest = len(request.prompt_ids) + request.max_new_tokens
        if self.max_model_len is not None and longest > self.max_model_len:
            raise ValueError(f"request {request.request_id}: prompt + max_new_tokens = {longest} exceeds "
                             f"the model length {self.max_model_len}")
        pages = pages_needed(longest, self.cache.block_size)
        if pages > self.cache.num_blocks:
            raise BlockPoolExhausted(f"out of KV blocks: request needs {pages} pages, pool has {self.cache.num_blocks}")
        request.phase = Phase.QUEUED
        self._known[request.request_id] = request
        self._queue.append(request)

    def abort(self, request_id) -> None:
        """Marks the request; it leaves when the next step is planned, so this is safe while a step
        with the request is in flight (its token is then dropped by `complete`)."""
        request = self._known.get(request_id)
        if request is not None and not request.cancelled:
            request.cancelled = True
            self._to_cancel.append(request)

    # ------------------------------------------------------------- leaving a seat, one way or another
    def _leave(self, request: Request, reason: Optional[str]) -> None:
        """Out of queue or seat; pages and slot back. `reason` None: the request gives way and will be
        recomputed (back to the head of the queue); else it has ended for that reason."""
        if request.phase is Phase.SEATED:
            self._seated.remove(request)
            if request.request_id in self.cache:
                self.cache.release(request.request_id)
        elif request.phase is Phase.QUEUED and reason is not None:
            self._queue.remove(request)
        if reason is None:
            request.num_computed = 0
            request.phase = Phase.QUEUED
            self._queue.appendleft(request)
            return
        request.phase = Phase.ENDED
        request.finish_reason = reason
        self._known.pop(request.request_id, None)

    def _drop_cancelled(self) -> None:
        for request in self._to_cancel:
            if request.phase is not Phase.ENDED:
                self._leave(request, "abort")
                _log.info("request %s cancelled", request.request_id)
        self._to_cancel = []

    def give_way(self, request: Request) -> None:
        """Preemption by recompute."""
        self._leave(request, None)
        request.preemptions += 1
        _log.info("request %s gives way with %d tokens (time %d)", request.request_id, request.num_tokens,
                  request.preemptions)

    def requeue(self, requests: Iterable[Request]) -> None:
        """Seated requests whose cached tokens can no longer be trusted (a step that held them was
        dropped): back to the queue as if they had never run, in their old order, ahead of all others."""
        for request in reversed(list(requests)):
            if request.phase is Phase.SEATED:
                self._leave(request, None)

    # ------------------------------------------------------------- planning a step
    def _seat_arrivals(self, draft: _Draft, spare_each: int = 0) -> None:
        """`spare_each`: pages that must stay free for every request already seated."""
        while self._queue and len(self._seated) < self.max_seqs and draft.left > 0:
            request = self._queue[0]
            # seated by the pages of everything known of it (scheduler.py:196-211), though only the pages
            # of the portion that runs now are taken
            if self.cache.slots.num_free < 1 or not self.cache.can_reserve(
                    request.request_id, request.num_tokens, spare=spare_each * len(self._seated)):
                return
            count = min(request.num_tokens, draft.left)
            self._queue.popleft()
            self.cache.add(request.request_id)
            self.cache.reserve(request.request_id, count)
            request.num_computed = 0
            request.phase = Phase.SEATED
            self._seated.append(request)
            draft.put(request, 0, count)

    def schedule(self) -> StepPlan:
        self._drop_cancelled()
        draft = _Draft(self.token_budget)
        someone_gave_way = False
        decoding = [r for r in self._seated if r.num_tokens - r.num_computed == 1]
        in_prompt = [r for r in self._seated if r.num_tokens - r.num_computed != 1]
        for request in decoding + in_prompt:
            if request.phase is not Phase.SEATED:
                continue                                  # gave way to an older request a moment ago
            count = min(request.num_tokens - request.num_computed, draft.left)
            if count < 1:
                continue
            while request.phase is Phase.SEATED and not self.cache.can_reserve(request.request_id, count):
                last = self._seated[-1]
                draft.withdraw(last)
                self.give_way(last)
                someone_gave_way = True
            if request.phase is Phase.SEATED:
                self.cache.reserve(request.request_id, count)
                draft.put(request, request.num_computed, count)
        if not someone_gave_way:          # else whoever gave way would come straight back
            self._seat_arrivals(draft)
        return StepPlan(tuple(draft.portions), gave_way=someone_gave_way)

    def schedule_ahead(self, plan: StepPlan) -> Optional[StepPlan]:
        """The step after `plan` (launched, not yet completed), planned before `plan`'s tokens are
        known, so that it can be launched while the host still waits for them; None where that is not
        plain. Every seated request must be in `plan`. The step after then holds, in this order:
        the requests of `plan` that sample, with the pending token as their one token (`feeds` names
        their places in `plan`; those that reach their length with the pending token are left out);
        the next portions of prompts that `plan` has not finished; and queued requests for which a
        seat, a state slot and pages are free now (the seat of a request that ends with the pending
        token is free one step later, and a page must stay free for every request already seated, so that
        an arrival does not take the page an older request needs at its next page boundary; none is seated
        behind a step in which somebody gave way, or whoever gave way would come straight back and give way
        again). Nobody gives way for it: if a page is missing the answer is
        None and the plain schedule decides. A request that turns out to have ended with the pending
        token (end of sequence, cancelled) has a row of the next step computed for nothing;
        `complete` skips it."""
        self._drop_cancelled()
        if len(plan.portions) == 0 or len(plan.portions) != len(self._seated):
            return None
        if any(p.request.phase is not Phase.SEATED for p in plan.portions):
            return None
        draft = _Draft(self.token_budget)
        for place, portion in enumerate(plan.portions):
            request = portion.request
            if not portion.samples or len(request.output_ids) + 1 >= request.max_new_tokens:
                continue                  # no token pending, or it is the request's last, whatever it is
            if draft.left < 1 or not self.cache.can_reserve(request.request_id, 1):
                # what was taken so far stays with requests that need it for their next token anyway
                return None
            self.cache.reserve(request.request_id, 1)
            draft.put_pending(request, portion.end, self.PENDING, place)
        for portion in plan.portions:
            if portion.samples:
                continue
            request = portion.request
            count = min(request.num_tokens - portion.end, draft.left)
            if count < 1 or not self.cache.can_reserve(request.request_id, count):
                return None
            self.cache.reserve(request.request_id, count)
            draft.put(request, portion.end, count)
        if not plan.gave_way:
            self._seat_arrivals(draft, spare_each=1)
        if not draft.portions:
            return None
        return StepPlan(tuple(draft.portions), feeds=tuple(draft.feeds))

    # ------------------------------------------------------------- after a step
    def complete(self, plan: StepPlan, drawn: Seq[Optional[int]]) -> List[Emission]:
        """`drawn[i]` is the token drawn after portion i (ignored where the portion does not sample).
        The cache's own counts were advanced by the step function."""
        if len(drawn) != len(plan.portions):
            raise ValueError("one entry per portion of the plan is required")
        emitted: List[Emission] = []
        for portion, token in zip(plan.portions, drawn):
            request = portion.request
            if request.cancelled or request.phase is not Phase.SEATED:
                continue
            request.num_computed = portion.end
            if not portion.samples:
                continue
            token = int(token)
            request.output_ids.append(token)
            reason = None
            if token in request.eos_ids and not request.params.ignore_eos:
                reason = "stop"
            elif len(request.output_ids) >= request.max_new_tokens:
                reason = "length"
            if reason is not None:
                self._leave(request, reason)
            emitted.append(Emission(request, token, reason is not None))
        return emitted

    def fail(self, plan: StepPlan, error: BaseException) -> List[Request]:
        """A step raised: every request in it is over, with the error, and what it holds goes back
        (worker/src/inference/batch_loop.py:135-147)."""
        ended = []
        for portion in plan.portions:
            request = portion.request
            if request.phase is Phase.SEATED:
                request.error = error
                self._leave(request, "error")
                ended.append(request)
        return ended
