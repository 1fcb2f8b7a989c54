"""Where a step's time goes, averaged over steps and logged every N steps.

The split follows the reference (worker/src/inference/step_stats.py:1-19, 56-100;
worker/src/inference/model_runner.py:92-119): the host's time in the scheduler (`sched`), in the
step function while it queues the step's work (`launch`), and in sampling, waiting for the ids and
delivery (`emit`); and the step's own time on the GPU (`device`), taken between two events that
bracket the step on its stream. The events of a step are read when a later step is recorded, by
which time they have long passed, so measuring makes nothing wait. Kinds: "decode" (every row
brings one token) and "prefill" (any row brings more).
"""

from __future__ import annotations

import logging
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Optional, Tuple

_log = logging.getLogger("distie_amd.steps")

HOST_PARTS = ("sched", "launch", "emit")


@dataclass
class _Kind:
    steps: int = 0
    rows: int = 0
    tokens: int = 0
    ms: Dict[str, float] = field(default_factory=lambda: {p: 0.0 for p in HOST_PARTS})
    device_ms: float = 0.0
    device_steps: int = 0


class StepStats:
    def __init__(self, every: int, device_events: bool = False) -> None:
        if every < 0:
            raise ValueError("every must be >= 0")
        self.every = every
        self.device_events = device_events
        self.total_steps = 0
        self._kinds: Dict[str, _Kind] = {}
        self._unread: Deque[Tuple[str, object, object]] = deque()     # (kind, first event, second event)
        self._spare: list = []

    def events(self) -> Optional[tuple]:
        """A pair of timing events for the step that is about to be launched (None without a GPU)."""
        if not self.device_events:
            return None
        if self._spare:
            return self._spare.pop()
        import torch

        return (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))

    def record(self, kind: str, rows: int, tokens: int, timing: Optional[tuple] = None, **ms: float) -> None:
        k = self._kinds.setdefault(kind, _Kind())
        k.steps += 1
        k.rows += rows
        k.tokens += tokens
        for part in HOST_PARTS:
            k.ms[part] += ms.get(part, 0.0)
        if timing is not None:
            self._unread.append((kind, timing[0], timing[1]))
        self._read(keep=1)
        self.total_steps += 1
        if self.every and self.total_steps % self.every == 0:
            self.flush()

    def _read(self, keep: int) -> None:
        """Take the device times of all steps but the newest `keep` (theirs may not have passed yet)."""
        while len(self._unread) > keep:
            kind, first, second = self._unread.popleft()
            if keep:
                if not second.query():
                    self._unread.appendleft((kind, first, second))
                    return
            else:
                second.synchronize()
            k = self._kinds.setdefault(kind, _Kind())
            k.device_ms += first.elapsed_time(second)
            k.device_steps += 1
            self._spare.append((first, second))

    def summary(self) -> Dict[str, Dict[str, float]]:
        """Per kind: steps, rows and tokens a step, mean milliseconds of every part."""
        out = {}
        for kind, k in sorted(self._kinds.items()):
            if not k.steps:
                continue
            row = {"steps": k.steps, "rows": k.rows / k.steps, "tokens": k.tokens / k.steps}
            row.update({p: k.ms[p] / k.steps for p in HOST_PARTS})
            row["host"] = sum(k.ms.values()) / k.steps
            if k.device_steps:
                row["device"] = k.device_ms / k.device_steps
            out[kind] = row
        return out

    def format(self) -> str:
        lines = []
        for kind, row in self.summary().items():
            parts = " ".join(f"{p}={row[p]:.2f}ms" for p in HOST_PARTS)
            device = f" device={row['device']:.2f}ms" if "device" in row else ""
            lines.append(f"{kind}: steps={row['steps']} rows/step={row['rows']:.1f} "
                         f"tokens/step={row['tokens']:.1f} host={row['host']:.2f}ms ({parts}){device}")
        return "; ".join(lines)

    def flush(self) -> None:
        self._read(keep=0)
        if self._kinds:
            _log.info("step stats %s", self.format())
            self._kinds.clear()


def distribution_ms(seconds) -> dict:
    """Mean, median, 90th and 99th percentile and maximum of times given in seconds, in milliseconds; a
    percentile between two samples is interpolated linearly (the reference's load generator reports
    latencies this way: benchmarks/load/stats.py:42-64)."""
    samples = sorted(1e3 * float(s) for s in seconds)
    if not samples:
        return {}

    def at(share: float) -> float:
        place = share * (len(samples) - 1)
        below = int(place)
        above = min(below + 1, len(samples) - 1)
        return samples[below] + (place - below) * (samples[above] - samples[below])

    return {"mean": sum(samples) / len(samples), "p50": at(0.5), "p90": at(0.9), "p99": at(0.99), "max": samples[-1]}
