"""Counters and histograms of the step function and of the scheduler.

The reference registers handles with a metrics recorder: per phase (prefill, decode)
steps, input tokens, step wall time and host submit time, failed steps, batch size and
duration, readback time (rust/engine/src/runner/model/qwen2/metrics.rs:50-113); per
request received / failed / in flight, duration by outcome, time to first text,
generated tokens, tokens per second (rust/engine/src/scheduler/observer.rs:122-170).
Here the same quantities are plain objects of the engine: ``snapshot()`` gives them as
one dictionary of numbers (what ``Engine.metrics()`` returns and ``--trace-steps``
prints).  Request and session ids are never part of a metric's name.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional


class Histogram:
    """Count, sum, extremes and a quantile estimate from buckets whose bounds grow by a
    fixed factor (``per_decade`` buckets for every factor of ten above ``lowest``)."""

    def __init__(self, lowest: float = 1e-6, per_decade: int = 8, decades: int = 9):
        self.lowest = float(lowest)
        self.per_decade = int(per_decade)
        self.buckets: List[int] = [0] * (per_decade * decades + 2)
        self.count = 0
        self.total = 0.0
        self.smallest = math.inf
        self.largest = -math.inf

    def _bucket(self, value: float) -> int:
        if value <= self.lowest:
            return 0
        i = 1 + int(math.log10(value / self.lowest) * self.per_decade)
        return min(i, len(self.buckets) - 1)

    def record(self, value: float) -> None:
        value = float(value)
        self.buckets[self._bucket(value)] += 1
        self.count += 1
        self.total += value
        if value < self.smallest:
            self.smallest = value
        if value > self.largest:
            self.largest = value

    def quantile(self, q: float) -> Optional[float]:
        """Upper bound of the bucket that holds the q-quantile (within one bucket's
        factor, 10^(1/per_decade), of the true value), clipped to the extremes."""
        if self.count == 0:
            return None
        need = q * self.count
        run = 0
        for i, n in enumerate(self.buckets):
            run += n
            if run >= need and n:
                bound = self.lowest * 10.0 ** (i / self.per_decade)
                return min(max(bound, self.smallest), self.largest)
        return self.largest

    def snapshot(self) -> Dict[str, Optional[float]]:
        if self.count == 0:
            return {"count": 0}
        return {"count": self.count, "sum": self.total, "mean": self.total / self.count,
                "min": self.smallest, "max": self.largest,
                "p50": self.quantile(0.5), "p95": self.quantile(0.95)}


class PhaseInstruments:
    def __init__(self):
        self.steps = 0
        self.input_tokens = 0
        self.host_submit_seconds = Histogram()     # from the step's call to its last kernel queued
        self.step_wall_seconds = Histogram()       # from the step's call until its tokens were read

    def snapshot(self):
        return {"steps": self.steps, "input_tokens": self.input_tokens,
                "host_submit_seconds": self.host_submit_seconds.snapshot(),
                "step_wall_seconds": self.step_wall_seconds.snapshot()}


class StepInstruments:
    """Of the step function: a step is prefill if any request in it has nothing cached yet
    or brings more than one token, else decode (metrics.rs:96-113, engine.rs:1954-1956)."""

    def __init__(self):
        self.prefill = PhaseInstruments()
        self.decode = PhaseInstruments()
        self.failed_steps = 0
        self.batch_size = Histogram(lowest=1.0, per_decade=16, decades=5)
        self.readback_seconds = Histogram()        # waiting for a step's chosen tokens
        self.last_phase = "decode"

    def step(self, prefill: bool, rows: int, requests: int, submit_seconds: float) -> None:
        phase = self.prefill if prefill else self.decode
        self.last_phase = "prefill" if prefill else "decode"
        phase.steps += 1
        phase.input_tokens += int(rows)
        phase.host_submit_seconds.record(submit_seconds)
        self.batch_size.record(requests)

    def wall(self, phase: str, seconds: float) -> None:
        (self.prefill if phase == "prefill" else self.decode).step_wall_seconds.record(seconds)

    def snapshot(self):
        return {"prefill": self.prefill.snapshot(), "decode": self.decode.snapshot(),
                "failed_steps": self.failed_steps, "batch_size": self.batch_size.snapshot(),
                "readback_seconds": self.readback_seconds.snapshot()}


class RequestInstruments:
    """Of the scheduler (observer.rs:122-170), with the time a request waited for
    admission beside them."""

    def __init__(self):
        self.requests = 0
        self.failures = 0
        self.cancelled = 0
        self.in_flight = 0
        self.generated_tokens = 0
        self.duration_seconds = {"success": Histogram(), "error": Histogram()}
        self.queue_wait_seconds = Histogram()
        self.first_token_seconds = Histogram()
        self.output_tokens_per_second = Histogram(lowest=1e-2, per_decade=8, decades=9)

    def received(self) -> None:
        self.requests += 1
        self.in_flight += 1

    def admitted(self, waited: float) -> None:
        self.queue_wait_seconds.record(waited)

    def first_token(self, seconds: float) -> None:
        self.first_token_seconds.record(seconds)

    def finished(self, ok: bool, seconds: float, generated: int, cancelled: bool = False) -> None:
        self.in_flight -= 1
        self.generated_tokens += int(generated)
        if cancelled:
            self.cancelled += 1         # neither a success nor a failure: no duration is recorded
            return
        self.duration_seconds["success" if ok else "error"].record(seconds)
        if not ok:
            self.failures += 1
        elif generated > 0 and seconds > 0:
            self.output_tokens_per_second.record(generated / seconds)

    def snapshot(self):
        return {"requests": self.requests, "failures": self.failures, "cancelled": self.cancelled,
                "in_flight": self.in_flight,
                "generated_tokens": self.generated_tokens,
                "duration_seconds": {k: h.snapshot() for k, h in self.duration_seconds.items()},
                "queue_wait_seconds": self.queue_wait_seconds.snapshot(),
                "first_token_seconds": self.first_token_seconds.snapshot(),
                "output_tokens_per_second": self.output_tokens_per_second.snapshot()}
