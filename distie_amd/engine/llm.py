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
from ..sampling import Sampler, SamplingParams
from ..weights import load_into, random_into
from .batch import StepEntry
from .model import Model
from .runner import ModelRunner
from .scheduler import Emission, Scheduler, Sequence, SeqState, StepPlan
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


@dataclass(frozen=True)
class Trace:
    """token_ids[t] is the argmax at step t; logits is float32 [steps, vocab] on the CPU
    (worker/src/inference/torch_engine.py:72-80)."""

    token_ids: List[int]
    logits: torch.Tensor


class LLM:
    def __init__(self, model: Union[str, Path, None] = None, *, config=None, random_weights: bool = False,
                 seed: int = 0, device: str = "cuda:0", ops=None, engine: Optional[EngineConfig] = None,
                 **options) -> None:
        """`model`: a folder with config.json and model.safetensors. Without it, `config` (a typed
        configuration or the dict of a config.json) and `random_weights=True` make a model with
        random weights on the device. `options` are fields of `EngineConfig`. `ops` is the kernel
        surface; by default the HIP kernels, which need the GPU."""
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
            random_into(self.model, seed, ops.device, self.dtype)
        else:
            raise ValueError("a config without a model folder needs random_weights=True")
        spec = self.model.spec
        ec = self.engine_config
        self.max_model_len = min(ec.max_model_len or spec.max_positions, spec.max_positions)
        self.cache = CacheManager(self.model.cache_requirements(), ec.block_size, ec.pages(), ec.max_seqs,
                                  device=ops.device, dtype=self.dtype)
        self.runner = ModelRunner(self.model, self.cache, ops, self.dtype, self.max_model_len)
        self.scheduler = Scheduler(self.cache, ec.max_seqs, ec.token_budget, self.max_model_len)
        self.sampler = Sampler(ops)
        self.stats = StepStats(ec.step_stats) if ec.step_stats else None
        self.eos_ids = tuple(spec.eos_token_ids)
        self._counter = itertools.count()
        self._ahead = None            # (plan, logits) of a step that is launched and not yet completed
        self._picked = None           # pinned host buffer for the sampled ids
        self._ahead_failed = None     # (plan, error) of a step planned ahead whose launch raised
        self.steps_ahead = 0          # steps launched before the tokens of the step before were known
        self._outputs: Dict[Hashable, RequestOutput] = {}
        self._started: Dict[Hashable, float] = {}
        if ec.use_graphs and hasattr(ops, "graphs_supported") and ops.graphs_supported():
            from .graphs import DecodeGraphs

            self.runner.graphs = DecodeGraphs(self.runner, ec.max_seqs)
        if ec.tune_products and hasattr(ops, "tune_library_products"):
            self._tune_products()
        _log.info("engine ready: %s dtype=%s pages=%d x %d tokens, %d cache groups, %.1f MiB cache",
                  spec.architecture, ec.dtype, ec.pages(), ec.block_size, len(self.cache.groups),
                  self.cache.bytes() / 2 ** 20)

    def _tune_products(self) -> None:
        """One step with as many tokens as a full portion of a prompt has, while the library is
        allowed to time its candidate kernels for every product shape it meets; afterwards it
        uses what it found for these shapes and its defaults for all others."""
        tokens = min(self.engine_config.token_budget, self.max_model_len,
                     self.cache.block_size * self.cache.num_blocks)
        if tokens < 1:
            return
        started = time.perf_counter()
        self.ops.tune_library_products(True)
        try:
            ids = [i % self.model.spec.vocab_size for i in range(tokens)]
            self.step([StepEntry("__tune__", ids, [tokens - 1])])
            torch.cuda.synchronize()
        finally:
            self.finish("__tune__")
            self.ops.tune_library_products(False)
        _log.info("library products tuned for portions of %d tokens in %.1f s", tokens, time.perf_counter() - started)

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
        if request_id is None:
            request_id = f"req-{next(self._counter)}"
        prompt = [int(t) for t in prompt_ids]
        vocab = self.model.spec.vocab_size
        if any(t < 0 or t >= vocab for t in prompt):
            raise ValueError(f"token id outside 0..{vocab - 1}")
        eos = (params.eos_id,) if params.eos_id is not None else self.eos_ids
        seq = Sequence(request_id=request_id, prompt_ids=prompt, params=params, eos_ids=tuple(eos))
        self.scheduler.submit(seq)
        self._outputs[request_id] = RequestOutput(request_id, prompt)
        self._started[request_id] = time.perf_counter()
        return request_id

    def abort(self, request_id) -> None:
        self.scheduler.abort(request_id)
        out = self._outputs.get(request_id)
        if out is not None and not out.finished:
            out.finished, out.finish_reason = True, "abort"

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def run_step(self) -> List[Emission]:
        """One turn of the loop: schedule, step, sample, complete.

        With `lookahead`, a step of decoding requests is followed at once by the next one, planned
        before the host has seen this step's tokens (`Scheduler.schedule_ahead`) and fed with them
        on the device; the host then waits for this step's tokens while the next step runs, and the
        next turn starts with that step already launched."""
        t0 = time.perf_counter()
        plan, logits = None, None
        if self._ahead is not None:
            plan, logits = self._ahead
            self._ahead = None
            if not any(it.seq.state is SeqState.RUNNING for it in plan.items):
                plan, logits = None, None        # every request of it has ended meanwhile: nothing to take from it
        launched = plan is not None
        if plan is None:
            plan = self.scheduler.schedule()
            if not plan.items:
                if self.scheduler.num_waiting and not self.scheduler.num_running:
                    raise RuntimeError("the scheduler cannot place the waiting requests: cache too small")
                return []
        t1 = time.perf_counter()
        try:
            if not launched:
                logits = self.runner.step(self._entries(plan), reserve=False)
            t2 = time.perf_counter()
            sampling = [it for it in plan.items if it.samples]
            picks: List[Optional[int]] = [None] * len(plan.items)
            if sampling:
                seeds = [it.seq.params.seed if it.seq.params.seed is not None else self.engine_config.seed
                         for it in sampling]
                chosen = self.sampler.sample_device(
                    logits, [it.seq.params.temperature for it in sampling], seeds,
                    [len(it.seq.output_ids) for it in sampling])
                fetch = self._to_host(chosen)
                if self.engine_config.lookahead:
                    self._launch_ahead(plan, chosen)
                tokens = iter(fetch())
                picks = [next(tokens) if it.samples else None for it in plan.items]
        except Exception as exc:  # noqa: BLE001 - every request of the step learns of it
            _log.exception("step failed; its %d requests end with the error", len(plan.items))
            self._ahead = None
            for seq in self.scheduler.fail(plan, exc):
                out = self._outputs[seq.request_id]
                out.finished, out.finish_reason, out.error = True, "error", repr(exc)
            return []
        emissions = self.scheduler.complete(plan, picks)
        if self._ahead_failed is not None:
            failed_plan, exc = self._ahead_failed
            self._ahead_failed = None
            for seq in self.scheduler.fail(failed_plan, exc):
                out = self._outputs[seq.request_id]
                out.finished, out.finish_reason, out.error = True, "error", repr(exc)
        now = time.perf_counter()
        for e in emissions:
            out = self._outputs[e.seq.request_id]
            if out.finished:
                continue                         # aborted meanwhile
            if not out.token_ids:
                out.time_to_first_token_ms = (now - self._started[e.seq.request_id]) * 1e3
            out.token_ids.append(e.token_id)
            out.preemptions = e.seq.preemptions
            if e.finished:
                out.finished, out.finish_reason = True, e.seq.finish_reason
                out.total_latency_ms = (now - self._started[e.seq.request_id]) * 1e3
        if self.stats is not None:
            self.stats.record("decode" if plan.is_decode else "prefill", len(plan.items), plan.num_tokens,
                              sched=(t1 - t0) * 1e3, gpu=(t2 - t1) * 1e3, emit=(now - t2) * 1e3)
        return emissions

    @staticmethod
    def _entries(plan: StepPlan) -> List[StepEntry]:
        return [StepEntry(it.seq.request_id, it.token_ids, [len(it.token_ids) - 1] if it.samples else [])
                for it in plan.items]

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
            for i, it in enumerate(plan.items):
                if it.samples:
                    sampled_row[i] = len(sampled_row)
            rows = [sampled_row[i] for i in ahead.feeds]
            feed = chosen
            if not rows:
                feed = None                              # nothing of it hangs on a pending token
            elif rows != list(range(chosen.shape[0])):
                index = self.ops.upload(np.asarray(rows, dtype=np.int32))
                feed = self.ops.gather_rows(chosen.view(-1, 1), index).view(-1)
            self._ahead = (ahead, self.runner.step(self._entries(ahead), reserve=False, feed=feed))
            self.steps_ahead += 1
        except Exception as exc:  # noqa: BLE001 - its requests learn of it once the running step is completed
            _log.exception("the step planned ahead failed; its %d requests end with the error", len(ahead.items))
            self._ahead = None
            self._ahead_failed = (ahead, exc)

    def stream(self, prompts: Seq[Seq[int]], params=None) -> Iterator[Emission]:
        """Yield (request, token, finished) as tokens are produced."""
        self._submit_all(prompts, params)
        while self.scheduler.has_work():
            yield from self.run_step()

    def generate(self, prompts: Seq[Seq[int]], params=None) -> List[RequestOutput]:
        """Token ids in, `RequestOutput`s out, in the order of the prompts. `params`: one
        `SamplingParams` for all, or one per prompt."""
        ids = self._submit_all(prompts, params)
        while self.scheduler.has_work():
            self.run_step()
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
        """One request through the step function: the whole prompt, then one token a step.
        Free-running feeds back the greedy pick and stops after an end-of-sequence token;
        teacher-forced feeds `forced_ids`. Last-position logits of every step are kept
        (worker/src/inference/torch_engine.py:295-338)."""
        if not prompt_ids:
            raise ValueError("prompt_ids must be non-empty")
        if max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")
        if forced_ids is not None and len(forced_ids) < max_new_tokens:
            raise ValueError("forced_ids shorter than max_new_tokens")
        rid = f"trace-{next(self._counter)}"
        picks: List[int] = []
        rows: List[torch.Tensor] = []
        current = [int(t) for t in prompt_ids]
        try:
            for step in range(max_new_tokens):
                logits = self.runner.step([StepEntry(rid, current, [len(current) - 1])])
                pick = int(self.ops.argmax(logits)[0])
                picks.append(pick)
                rows.append(logits[0].float().cpu())
                if forced_ids is None:
                    if pick in self.eos_ids:
                        break
                    current = [pick]
                else:
                    current = [int(forced_ids[step])]
        finally:
            self.runner.finish(rid)
        return Trace(token_ids=picks, logits=torch.stack(rows))

    def close(self) -> None:
        self.runner.graphs = None
