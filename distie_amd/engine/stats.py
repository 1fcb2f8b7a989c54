"""Where a step's time goes, averaged over steps and logged every N steps.

The split is the reference's (worker/src/inference/step_stats.py:1-19, 56-100): time in the
scheduler, in the step function (host view), in sampling and delivery; kinds "decode" (every
row brings one token) and "prefill" (any row brings more)."""

from __future__ import annotations

import logging
from dataclasses import dataclass, field
from typing import Dict

_log = logging.getLogger("distie_amd.steps")

PARTS = ("sched", "gpu", "emit")


@dataclass
class _Group:
    steps: int = 0
    rows: int = 0
    tokens: int = 0
    ms: Dict[str, float] = field(default_factory=lambda: {p: 0.0 for p in PARTS})


class StepStats:
    def __init__(self, every: int) -> None:
        if every < 0:
            raise ValueError("every must be >= 0")
        self.every = every
        self.total_steps = 0
        self._groups: Dict[str, _Group] = {}

    def record(self, kind: str, rows: int, tokens: int, **ms: float) -> None:
        g = self._groups.setdefault(kind, _Group())
        g.steps += 1
        g.rows += rows
        g.tokens += tokens
        for part in PARTS:
            g.ms[part] += ms.get(part, 0.0)
        self.total_steps += 1
        if self.every and self.total_steps % self.every == 0:
            self.flush()

    def format(self) -> str:
        lines = []
        for kind, g in sorted(self._groups.items()):
            parts = " ".join(f"{p}={g.ms[p] / g.steps:.2f}ms" for p in PARTS)
            lines.append(f"{kind}: steps={g.steps} rows/step={g.rows / g.steps:.1f} "
                         f"tokens/step={g.tokens / g.steps:.1f} {parts}")
        return "; ".join(lines)

    def flush(self) -> None:
        if self._groups:
            _log.info("step stats %s", self.format())
            self._groups.clear()
