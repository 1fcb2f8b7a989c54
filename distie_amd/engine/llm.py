"""The Python entry point: a model folder (or a configuration and a seed) in, generated
tokens out.

`LLM` stands where the reference's `TorchEngine` stands
(worker/src/inference/torch_engine.py:83-164, 295-338): it resolves the precision, loads
the weights, builds cache, step function, scheduler and sampler from the options, and
offers `generate` (continuous batching), `stream`, `trace` (one request step by step,
greedy or teacher-forced, logits kept) and `step` (the bare step function, for replay).
The loop is synchronous: schedule, step, sample, complete
(worker/src/inference/batch_loop.py:81-117 without the asyncio shell).
"""

from __future__ import annotations

import itertools
import logging
import time
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, Hashable, Iterator, List, Optional, Sequence as Seq, Union

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..config import EngineConfig, config_from_dict, load_model_config
from ..sampling import Sampler, SamplingParams, derive_seed
from ..weights import load_into, random_into
from .batch import StepEntry
from .model import Model
from .runner import ModelRunner
from .scheduler import Emission, Phase, Request, Scheduler, StepPlan
from .stats import StepStats

_log = logging.getLogger(__name__)

TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@dataclass
class RequestOutput:
    """What a request produced (the reference streams `TokenEvent`s with the same counts and
    timings: worker/src/inference/engine.py:55-62)."""

    request_id: Hashable
    prompt_token_ids: List[int]
    token_ids: List[int] = field(default_factory=list)
    finished: bool = False
    finish_reason: Optional[str] = None      # "stop" (end-of-sequence), "length", "abort", "error"
    error: Optional[str] = None
    preemptions: int = 0
    time_to_first_token_ms: float = 0.0
    total_latency_ms: float = 0.0
    arrival_time: float = 0.0                # time.perf_counter() at add_request


@dataclass(frozen=True)
class Trace:
    """token_ids[t] is the argmax at step t; logits is float32 [steps, vocab] on the CPU
    (worker/src/inference/torch_engine.py:72-80)."""

    token_ids: List[int]
    logits: torch.Tensor


class LLM:
    def __init__(self, model: Union[str, Path, None] = None, *, config=None, random_weights: bool = False,
                 seed: int = 0, weights_std: float = 0.02, device: str = "cuda:0", ops=None,
                 engine: Optional[EngineConfig] = None, **options) -> None:
        """`model`: a folder with config.json and model.safetensors. Without it, `config` (a typed
        configuration or the dict of a config.json) and `random_weights=True` make a model with
        random weights on the device (drawn from `seed`, which is also the engine's seed for sampling
        unless `options` or `engine` name another, with the spread `weights_std`: the model that
        `write_random_model` writes for the same configuration, seed and spread). `options` are fields of `EngineConfig`. `ops` is the kernel
        surface; by default the HIP kernels, which need the GPU."""
        if engine is None:
            options.setdefault("seed", seed)          # one seed for random weights and for the requests' draws
        self.engine_config = engine or EngineConfig(**options)
        self.dtype = TORCH_DTYPES[self.engine_config.dtype]
        if ops is None:
            from ..kernels.hip_ops import HipOps

            ops = HipOps(device, packed_weights=self.engine_config.packed_weights)
        self.ops = ops
        if model is not None:
            self.model_config = load_model_config(model)
        elif config is not None:
            self.model_config = config_from_dict(config) if isinstance(config, dict) else config
        else:
            raise ValueError("give a model folder, or a config with random_weights=True")
        self.model = Model(self.model_config.model_spec())
        if model is not None and not random_weights:
            load_into(self.model, model, ops.device, self.dtype)
        elif random_weights:
            random_into(self.model, seed, ops.device, self.dtype, std=weights_std)
        else:
            raise ValueError("a config without a model folder needs random_weights=True")
        spec = self.model.spec
        ec = self.engine_config
        self.max_model_len = min(ec.max_model_len or spec.max_positions, spec.max_positions)
        self.model.prepare(ops)                      # packed copies of the weights: in place before memory is counted
        needs = self.model.cache_requirements()
        free = total = None
        if ec.gpu_mem_fraction is not None and ops.device.type == "cuda":
            torch.cuda.empty_cache()
            free, total = torch.cuda.mem_get_info(ops.device)
        self.num_pages = ec.pages(CacheManager.page_bytes(needs, ec.block_size, self.dtype), free, total)
        self.cache = CacheManager(needs, ec.block_size, self.num_pages, ec.max_seqs,
                                  device=ops.device, dtype=self.dtype)
        self.runner = ModelRunner(self.model, self.cache, ops, self.dtype, self.max_model_len)
        self.scheduler = Scheduler(self.cache, ec.max_seqs, ec.token_budget, self.max_model_len)
        self.sampler = Sampler(ops)
        self.stats = StepStats(ec.step_stats, device_events=ops.device.type == "cuda") if ec.step_stats else None
        self.eos_ids = tuple(spec.eos_token_ids)
        self._counter = itertools.count()
        self._ahead = None            # (plan, logits, events) of a step that is launched and not yet completed
        self._picked = None           # pinned host buffer for the sampled ids
        self._ahead_failed = None     # (plan, error) of a step planned ahead whose launch raised
        self.steps_ahead = 0          # steps launched before the tokens of the step before were known
        self.last_logits = None       # of the step completed last: a view that a later step may overwrite (for checks)
        self._outputs: Dict[Hashable, RequestOutput] = {}     # until `generate`, `stream` or `take_output` hands them out
        if ec.use_graphs and hasattr(ops, "graphs_supported") and ops.graphs_supported():
            if self.model.capturable:
                from .graphs import DecodeGraphs

                self.runner.graphs = DecodeGraphs(self.runner, ec.max_seqs, ec.graph_buckets, ec.graph_tokens)
            else:
                names = sorted({type(p).__name__ for p in self.model.parts() if not p.capturable})
                _log.info("decode steps are not captured: %s cannot be recorded into a graph", ", ".join(names))
        if ec.tune_products and hasattr(ops, "tune_library_products"):
            self._tune_products()
        _log.info("engine ready: %s dtype=%s pages=%d x %d tokens, %d cache groups, %.1f MiB cache",
                  spec.architecture, ec.dtype, self.num_pages, ec.block_size, len(self.cache.groups),
                  self.cache.bytes() / 2 ** 20)

    # row counts whose products are timed beside a full portion's: the largest of each class of 32 rows from 96 on,
    # up to this many or the largest batch, whichever is more (a class takes about a second)
    TIMED_ROWS = 192
    TIMED_ROWS_MOST = 512

    def _tune_products(self) -> None:
        """One step with as many tokens as a full portion of a prompt has, while the library is
        allowed to time its candidate kernels for every product shape it meets; afterwards it
        uses what it found for these shapes and its defaults for all others. Then the same for
        the row counts of large decode batches and short portions, class by class, with the
        products going where a captured step sends them."""
        tokens = min(self.engine_config.token_budget, self.max_model_len,
                     self.cache.block_size * self.cache.num_blocks)
        if tokens < 1:
            return
        started = time.perf_counter()
        ids = [i % self.model.spec.vocab_size for i in range(tokens)]
        most = min(tokens, self.TIMED_ROWS_MOST, max(self.TIMED_ROWS, -(-self.engine_config.max_seqs // 32) * 32))
        graphs, self.runner.graphs = self.runner.graphs, None        # (timing a kernel cannot be recorded into a graph)
        self.ops.tune_library_products(True)
        done = False
        try:
            self.step([StepEntry("__tune__", ids, [tokens - 1])])
            self.finish("__tune__")
            # from here on the products of these row counts go where they will go once their kernels are timed
            self.ops.captured, self.ops.library_timed_rows = True, most
            for rows in range(96, most + 1, 32):
                # every row wanted: the head's product has as many rows as a decode step of that batch
                self.step([StepEntry("__tune__", ids[:rows], list(range(rows)))])
                self.finish("__tune__")
            torch.cuda.synchronize()
            done = True
        finally:
            self.ops.captured = False
            if not done:
                self.ops.library_timed_rows = 0
            self.finish("__tune__")
            self.ops.tune_library_products(False)
            self.runner.graphs = graphs
        _log.info("library products tuned for portions of %d tokens and for 65 to %d rows in %.1f s", tokens, most,
                  time.perf_counter() - started)

    # ------------------------------------------------------------ the step function
    def step(self, entries: Seq[StepEntry]) -> Optional[torch.Tensor]:
        """Run the given tokens of the given requests as one batch; float32 logits at the wanted
        places. Requests are created at their first step; `finish` gives back what they hold."""
        return self.runner.step(entries)

    def finish(self, request_id) -> None:
        self.runner.finish(request_id)

    # ------------------------------------------------------------ generation
    def add_request(self, prompt_ids: Seq[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[Hashable] = None) -> Hashable:
        params = params or SamplingParams()
        arrival = next(self._counter)
        if request_id is None:
            request_id = f"req-{arrival}"
        prompt = [int(t) for t in prompt_ids]
        vocab = self.model.spec.vocab_size
        if any(t < 0 or t >= vocab for t in prompt):
            raise ValueError(f"token id outside 0..{vocab - 1}")
        eos = (params.eos_id,) if params.eos_id is not None else self.eos_ids
        # A request without a seed of its own draws from a stream that belongs to it alone: derived from the
        # engine's seed and the request's place in the order of arrival, so that two requests never share
        # their random numbers (the reference draws from one global generator:
        # worker/src/inference/model_runner.py:122-130) and a rerun of the same arrivals repeats.
        seed = params.seed if params.seed is not None else derive_seed(self.engine_config.seed, arrival)
        request = Request(request_id=request_id, prompt_ids=prompt, params=params, eos_ids=tuple(eos), seed=seed)
        self.scheduler.submit(request)
        self._outputs[request_id] = RequestOutput(request_id, prompt, arrival_time=time.perf_counter())
        return request_id

    def abort(self, request_id) -> None:
        self.scheduler.abort(request_id)
        out = self._outputs.get(request_id)
        if out is not None and not out.finished:
            self._close(out, "abort")

    def take_output(self, request_id) -> RequestOutput:
        """The record of a request, which the engine then forgets. `generate` and `stream` do this for their
        own requests; who drives `add_request` and `run_step` takes the records of finished requests here."""
        return self._outputs.pop(request_id)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    @staticmethod
    def _close(out: RequestOutput, reason: str, error: Optional[str] = None) -> None:
        out.finished, out.finish_reason, out.error = True, reason, error
        out.total_latency_ms = (time.perf_counter() - out.arrival_time) * 1e3

    def _fail(self, plan: StepPlan, exc: BaseException) -> None:
        for request in self.scheduler.fail(plan, exc):
            self._close(self._outputs[request.request_id], "error", repr(exc))

    def run_step(self) -> List[Emission]:
        """One turn of the loop: schedule, step, sample, complete.

        With `lookahead`, a step of decoding requests is followed at once by the next one, planned
        before the host has seen this step's tokens (`Scheduler.schedule_ahead`) and fed with them
        on the device; the host then waits for this step's tokens while the next step runs, and the
        next turn starts with that step already launched."""
        t0 = time.perf_counter()
        plan, logits, timing = None, None, None
        if self._ahead is not None:
            plan, logits, timing = self._ahead
            self._ahead = None
            if not any(p.request.phase is Phase.SEATED for p in plan.portions):
                plan, logits = None, None        # every request of it has ended meanwhile: nothing to take from it
        launched = plan is not None
        if plan is None:
            plan = self.scheduler.schedule()
            if not plan.portions:
                if self.scheduler.num_waiting and not self.scheduler.num_running:
                    raise RuntimeError("the scheduler cannot place the waiting requests: cache too small")
                return []
        t1 = time.perf_counter()
        try:
            if not launched:
                logits, timing = self._launch(plan, None)
            t2 = time.perf_counter()
            sampling = [p for p in plan.portions if p.samples]
            drawn: List[Optional[int]] = [None] * len(plan.portions)
            self.last_logits = logits
            if sampling:
                chosen = self.sampler.sample_device(
                    logits, [p.request.params.temperature for p in sampling], [p.request.seed for p in sampling],
                    [len(p.request.output_ids) for p in sampling])
                fetch = self._to_host(chosen)
                if self.engine_config.lookahead:
                    self._launch_ahead(plan, chosen)
                tokens = iter(fetch())
                drawn = [next(tokens) if p.samples else None for p in plan.portions]
        except Exception as exc:  # noqa: BLE001 - every request of the step learns of it
            _log.exception("step failed; its %d requests end with the error", len(plan.portions))
            self._fail(plan, exc)
            self._drop_ahead()
            return []
        emissions = self.scheduler.complete(plan, drawn)
        if self._ahead_failed is not None:
            failed_plan, exc = self._ahead_failed
            self._ahead_failed = None
            self._fail(failed_plan, exc)
        now = time.perf_counter()
        for e in emissions:
            out = self._outputs[e.request.request_id]
            if out.finished:
                continue                         # aborted meanwhile
            if not out.token_ids:
                out.time_to_first_token_ms = (now - out.arrival_time) * 1e3
            out.token_ids.append(e.token_id)
            out.preemptions = e.request.preemptions
            if e.finished:
                self._close(out, e.request.finish_reason)
        if self.stats is not None:
            # `launch` is the host's time inside the step function when this turn launched the step (0 when it
            # was launched a turn earlier, behind the step before); `device` is the step's own time on the GPU,
            # between two events, read when the step after has been queued, so that nothing waits for it
            self.stats.record("decode" if plan.is_decode else "prefill", len(plan.portions), plan.num_tokens,
                              timing, sched=(t1 - t0) * 1e3, launch=(t2 - t1) * 1e3, emit=(now - t2) * 1e3)
        return emissions

    def _launch(self, plan: StepPlan, feed):
        """-> (logits, the step's pair of events or None)"""
        entries = [StepEntry(p.request.request_id, p.token_ids, [len(p.token_ids) - 1] if p.samples else [])
                   for p in plan.portions]
        timing = self.stats.events() if self.stats is not None else None
        if timing is not None:
            timing[0].record()
        logits = self.runner.step(entries, reserve=False, feed=feed)
        if timing is not None:
            timing[1].record()
        return logits, timing

    def _drop_ahead(self) -> None:
        """The step in flight failed with a step already launched behind it. That step's results are worth
        nothing, but it has advanced the cache's counts of its requests: those of them that are still
        seated (requests that it seated itself) go back to the queue and start over."""
        if self._ahead is None:
            return
        ahead_plan = self._ahead[0]
        self._ahead = None
        self.scheduler.requeue(p.request for p in ahead_plan.portions)

    def _forget_ahead(self) -> None:
        """When every request ended in the step that was being completed, the step launched behind it is
        worth nothing, and the loop ends without another turn that would drop it: let go of its plan, its
        requests and its view of a captured step's logits here. (If one of its requests is still seated
        the step is needed and stays.)"""
        if self._ahead is not None and not any(p.request.phase is Phase.SEATED for p in self._ahead[0].portions):
            self._ahead = None
        if self._ahead_failed is not None and not self.scheduler.has_work():
            self._ahead_failed = None

    def _to_host(self, chosen: torch.Tensor):
        """Start the copy of the sampled ids to the host; the returned function waits for it."""
        if chosen.device.type != "cuda":
            return chosen.tolist
        n = chosen.shape[0]
        if self._picked is None or self._picked.shape[0] < n:
            self._picked = torch.empty(max(n, self.engine_config.max_seqs), dtype=torch.int32, pin_memory=True)
        self._picked[:n].copy_(chosen, non_blocking=True)
        arrived = torch.cuda.Event()
        arrived.record()

        def fetch():
            arrived.synchronize()
            return self._picked[:n].tolist()
        return fetch

    def _launch_ahead(self, plan: StepPlan, chosen: torch.Tensor) -> None:
        """Launch the step after `plan`, if it can be planned without `plan`'s tokens: they are taken
        from `chosen` (row i of the sampled rows of `plan`) on the device."""
        ahead = self.scheduler.schedule_ahead(plan)
        if ahead is None:
            return
        try:
            sampled_row = {}
            for i, p in enumerate(plan.portions):
                if p.samples:
                    sampled_row[i] = len(sampled_row)
            rows = [sampled_row[i] for i in ahead.feeds]
            feed = chosen
            if not rows:
                feed = None                              # nothing of it hangs on a pending token
            elif rows != list(range(chosen.shape[0])):
                index = self.ops.upload(np.asarray(rows, dtype=np.int32))
                feed = self.ops.gather_rows(chosen.view(-1, 1), index).view(-1)
            self._ahead = (ahead,) + self._launch(ahead, feed)
            self.steps_ahead += 1
        except Exception as exc:  # noqa: BLE001 - its requests learn of it once the running step is completed
            _log.exception("the step planned ahead failed; its %d requests end with the error", len(ahead.portions))
            self._ahead = None
            self._ahead_failed = (ahead, exc)

    def stream(self, prompts: Seq[Seq[int]], params=None) -> Iterator[Emission]:
        """Yield (request, token, finished) as tokens are produced."""
        mine = set(self._submit_all(prompts, params))
        while self.scheduler.has_work():
            for emission in self.run_step():
                yield emission
            for rid in [r for r in mine if self._outputs[r].finished]:
                mine.discard(rid)
                del self._outputs[rid]
        for rid in mine:
            self._outputs.pop(rid, None)
        self._forget_ahead()

    def generate(self, prompts: Seq[Seq[int]], params=None) -> List[RequestOutput]:
        """Token ids in, `RequestOutput`s out, in the order of the prompts. `params`: one
        `SamplingParams` for all, or one per prompt."""
        ids = self._submit_all(prompts, params)
        while self.scheduler.has_work():
            self.run_step()
        self._forget_ahead()
        if self.stats is not None:
            self.stats.flush()
        return [self._outputs.pop(i) for i in ids]

    def _submit_all(self, prompts, params) -> List[Hashable]:
        if params is None or isinstance(params, SamplingParams):
            params = [params] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt (or one for all)")
        return [self.add_request(p, sp) for p, sp in zip(prompts, params)]

    # ------------------------------------------------------------ trace
    def trace(self, prompt_ids: Seq[int], max_new_tokens: int, forced_ids: Optional[Seq[int]] = None) -> Trace:
        """One request through the step function: the whole prompt in one step, then a token a step,
        keeping the logits at the last position of every step. Without `forced_ids` each step is fed
        the greedy pick of the one before and the run ends after an end-of-sequence token; with them,
        step t is fed `forced_ids[t - 1]` whatever was picked, so that the logits can be compared with
        those of another implementation that saw the same tokens
        (worker/src/inference/torch_engine.py:295-338)."""
        prompt = [int(t) for t in prompt_ids]
        forced = None if forced_ids is None else [int(t) for t in forced_ids]
        if len(prompt) == 0:
            raise ValueError("a trace needs at least one prompt token")
        if max_new_tokens < 1:
            raise ValueError("a trace needs max_new_tokens >= 1")
        if forced is not None and len(forced) < max_new_tokens:
            raise ValueError(f"{len(forced)} forced ids for {max_new_tokens} steps")
        name = f"trace-{next(self._counter)}"
        kept = torch.empty((max_new_tokens, self.model.spec.vocab_size), dtype=torch.float32)
        chosen: List[int] = []
        feed = prompt
        try:
            while len(chosen) < max_new_tokens:
                row = self.runner.step([StepEntry(name, feed, [len(feed) - 1])])
                greedy = int(self.ops.argmax(row)[0])
                kept[len(chosen)].copy_(row[0])
                chosen.append(greedy)
                if forced is None and greedy in self.eos_ids:
                    break
                feed = [greedy if forced is None else forced[len(chosen) - 1]]
        finally:
            self.runner.finish(name)
        return Trace(token_ids=chosen, logits=kept[:len(chosen)].clone())

    def close(self) -> None:
        self.last_logits = None
        self._ahead = None
        self._ahead_failed = None
        self.runner.graphs = None
