"""The scheduler: admits requests, cuts prompts into portions under a token
budget, decodes, finishes and frees.

Decisions, all taken from the reference's Runner and its batch policy:

* Admission (rust/engine/src/runner/model_runner.rs:577-694): a request is
  refused if its prompt is empty, a token id is outside the vocabulary, or
  ``prompt + max_new_tokens - 1`` exceeds the longest sequence the cache takes.
  Otherwise it is admitted when a request row is free and every cache group has
  pages for the WHOLE turn (prompt and all generated tokens but the last) on top
  of what the active requests are still promised.  So pages never run out in the
  middle of a request.
* When pages are short (model_runner.rs:745-756): the request waits while others
  are active and is tried again every step; requests behind it that fit are
  admitted meanwhile.  If nothing is active and it still does not fit, it fails
  with ``CapacityExhausted``.  No preemption, no swapping, no recomputation.
* The step's plan (rust/engine/src/runner/model_runner/batch_policy.rs:36-88):
  every decoding request gets one token first (at most ``max_batch_tokens`` of
  them); what is left of the budget goes to prompts in order of admission, each
  ``min(rest of the prompt, budget left)``; a request that gets nothing sits
  the step out.  A request decodes once it has produced a token; the last
  portion of a prompt, however short, is still prefill.
* Only a portion that ends the prompt yields a token (model_runner.rs:825);
  the end-of-sequence token counts as generated and is kept
  (model_runner.rs:280-321); a request ends at end-of-sequence or at its budget
  and gives its pages and its row back before the next step.
* Overlap (model_runner.rs:839-896; the reference's ``--disable-overlap`` turns it
  off): step N+1 is put on the GPU before the tokens of step N are read; a request
  whose token is still on its way takes it from the GPU's memory as its next input.
  What the host does between two steps then hides behind the GPU's work.  A request
  that turns out to have ended at step N (end of sequence) has by then been given
  one more token in step N+1; that token is dropped.  The tokens are the same as
  without overlap.
"""
from __future__ import annotations

import array
import collections
import dataclasses
import time
from typing import Callable, Deque, Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..sampling.params import SamplingConfig
from .instruments import RequestInstruments
from .step import StepEntry, StepResult


def _token_array(tokens: Sequence[int]):
    """The token ids as an array of 64-bit integers: a list of a long prompt is a hundred
    thousand references that Python's cyclic collector walks at every full pass (2 M tokens
    of 256 live requests: 23 ms a pass, a third of a millisecond on every decode step of
    that batch), an array is one object that it does not look into.  Ids that no such
    array holds stay a list; the admission check reports them."""
    try:
        return array.array("q", [int(t) for t in tokens])
    except (OverflowError, TypeError, ValueError):
        return [t for t in tokens]


class CapacityExhausted(RuntimeError):
    """The cache cannot hold the request even with nothing else running."""


@dataclasses.dataclass(eq=False)      # a request is itself, not its fields: compared and hashed by identity
class Request:
    request_id: int
    prompt: Sequence[int]                      # (an array of integers: see _token_array)
    sampling: SamplingConfig
    tokens: Sequence[int] = dataclasses.field(default_factory=list)     # prompt + generated
    generated: List[int] = dataclasses.field(default_factory=list)
    cache: object = None
    remaining: int = 0
    promised_pages: List[int] = dataclasses.field(default_factory=list)
    error: Optional[Exception] = None
    finish_reason: Optional[str] = None        # "eos", "length", "error", "cancelled"
    in_flight: bool = False                    # a token of this request is chosen but not read yet
    eos: Tuple[int, ...] = ()                  # end-of-sequence ids, temperature and seed: worked out once
    temperature: float = 0.0
    seed: int = 0
    arrival: float = 0.0
    admit_time: Optional[float] = None
    first_token_time: Optional[float] = None
    finish_time: Optional[float] = None

    @property
    def finished(self) -> bool:
        return self.finish_reason is not None

    @property
    def decoding(self) -> bool:
        return len(self.generated) > 0 or self.in_flight

    @property
    def budget_left(self) -> int:
        """Tokens this request may still be given (one is taken by a token in flight)."""
        return self.remaining - (1 if self.in_flight else 0)

    @property
    def known_len(self) -> int:
        """Tokens of the sequence, the one in flight included."""
        return len(self.tokens) + (1 if self.in_flight else 0)

    @property
    def computed(self) -> int:
        return self.cache.computed_len if self.cache is not None else 0


@dataclasses.dataclass(slots=True)
class Planned:
    request: Request
    count: int              # tokens of this step
    yields_token: bool      # the portion ends the request's known tokens


def plan_step(active: Sequence[Request], max_batch_tokens: int) -> List[Planned]:
    """Decode first, then prompts in order, under one token budget."""
    # (plain attribute reads instead of the properties: this loop runs per request and step)
    runnable, decoding = [], 0
    for r in active:
        if r.finish_reason is None and r.remaining - (1 if r.in_flight else 0) > 0:
            runnable.append(r)
            if r.in_flight or r.generated:
                decoding += 1
    decode_budget = min(decoding, max_batch_tokens)
    prefill_budget = max_batch_tokens - decode_budget
    plan: List[Planned] = []
    for r in runnable:
        ready = r.cache.computed_len if r.cache is not None else 0
        known = len(r.tokens) + (1 if r.in_flight else 0)
        if r.in_flight or r.generated:
            if decode_budget == 0:
                continue
            decode_budget -= 1
            count = 1
        else:
            if prefill_budget == 0:
                continue
            count = min(len(r.tokens) - ready, prefill_budget)
            prefill_budget -= count
        plan.append(Planned(r, count, ready + count == known))
    return plan


class Scheduler:
    """Continuous batching over an engine's step function.

    ``engine`` needs: ``step(entries) -> logits``, ``cache`` (a ``CacheManager``),
    ``open(id)``, ``close(request_cache)``, ``spec`` (vocab_size, eos_token_ids),
    ``max_seq_len``, and optionally ``eos_token_ids`` (goes before the spec's).  ``sampler.sample(logits, temperatures, seeds, counters)``
    picks the tokens."""

    def __init__(self, engine, sampler, max_batch_tokens: Optional[int] = None,
                 on_token: Optional[Callable[[Request, int], None]] = None,
                 trace: Optional[Callable[[dict], None]] = None, overlap: bool = True):
        self.engine = engine
        self.sampler = sampler
        self.max_batch_tokens = int(max_batch_tokens or engine.max_batch_tokens)
        if self.max_batch_tokens <= 0:
            raise ValueError("max_batch_tokens must be positive")
        self.waiting: Deque[Request] = collections.deque()
        self.active: List[Request] = []
        self.finished: Dict[int, Request] = {}
        self._next_id = 0
        self.on_token = on_token
        self.trace = trace
        self.overlap = bool(overlap)
        model_eos = getattr(engine, "eos_token_ids", None)
        self._model_eos = tuple(model_eos if model_eos is not None else engine.spec.eos_token_ids)
        self._pending = None            # (requests, PendingTokens) of the step whose tokens are unread
        self.steps = 0
        self.instruments = getattr(engine, "request_instruments", None) or RequestInstruments()
        self.step_log: List[List[Tuple[int, int]]] = []     # per step: (request id, tokens)
        self.keep_step_log = False

    # ---------------------------------------------------------------- ingress
    def add_request(self, prompt: Sequence[int], sampling: Optional[SamplingConfig] = None) -> int:
        request = Request(self._next_id, _token_array(prompt), sampling or SamplingConfig(),
                          arrival=time.perf_counter())
        self._next_id += 1
        request.tokens = request.prompt[:]
        request.remaining = request.sampling.new_tokens
        request.eos = tuple(request.sampling.eos_ids(self._model_eos))
        request.temperature, request.seed = request.sampling.effective_temperature, request.sampling.seed
        self.waiting.append(request)
        self.instruments.received()
        return request.request_id

    # -------------------------------------------------------------- admission
    def _promised(self) -> List[int]:
        """Pages per group that active requests may still take."""
        cache = self.engine.cache
        owed = [0] * len(cache.groups)
        for r in self.active:
            for g in range(len(cache.groups)):
                held = sum(1 for p in r.cache.pages[g] if p >= 0)
                owed[g] += max(0, r.promised_pages[g] - held)
        return owed

    def _refusal(self, r: Request) -> Optional[Exception]:
        try:
            r.sampling.validate()
        except ValueError as e:
            return e
        if not r.prompt:
            return ValueError("empty prompt")
        vocab = self.engine.spec.vocab_size
        if isinstance(r.prompt, array.array):          # (one pass in numpy, not a Python loop over a long prompt)
            ids = np.frombuffer(r.prompt, dtype=np.int64)
            lowest, highest = int(ids.min()), int(ids.max())
            if lowest < 0 or highest >= vocab:
                return ValueError(f"token id {lowest if lowest < 0 else highest} is outside the vocabulary of {vocab}")
        else:
            for t in r.prompt:
                if not 0 <= t < vocab:
                    return ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        end = len(r.prompt) + max(0, r.remaining - 1)
        if end > self.engine.max_seq_len:
            return ValueError(f"generation to {end} tokens exceeds the cache's longest "
                              f"sequence {self.engine.max_seq_len}")
        return None

    def _fits(self, r: Request) -> Tuple[bool, List[int]]:
        cache = self.engine.cache
        end = len(r.prompt) + max(0, r.remaining - 1)
        need = cache.page_need(end, self.max_batch_tokens)
        if cache.free_rows == 0:
            return False, need
        owed = self._promised()
        for g in range(len(cache.groups)):
            if need[g] > cache.free_pages(g) - owed[g]:
                return False, need
        return True, need

    def _admit(self) -> None:
        still_waiting: Deque[Request] = collections.deque()
        while self.waiting:
            r = self.waiting.popleft()
            refusal = self._refusal(r)
            if refusal is not None:
                self._finish(r, "error", refusal)
                continue
            if r.remaining == 0:
                self._finish(r, "length")
                continue
            fits, need = self._fits(r)
            if fits:
                r.cache = self.engine.open(("request", r.request_id))
                r.promised_pages = need
                r.admit_time = time.perf_counter()
                self.instruments.admitted(r.admit_time - r.arrival)
                self.active.append(r)
            elif self.active:
                still_waiting.append(r)
            else:
                self._finish(r, "error", CapacityExhausted(
                    f"insufficient cache capacity for request {r.request_id}: it needs {need} "
                    f"pages per group"))
        self.waiting = still_waiting

    # ------------------------------------------------------------------- step
    def _run(self, entries: List[StepEntry]) -> StepResult:
        """One step of the engine with a result for every entry.  Whatever the engine
        raises for the step as a whole becomes every entry's error."""
        run = getattr(self.engine, "run_step", None)
        try:
            if run is not None:
                return run(entries)
            logits = self.engine.step(entries)
        except Exception as err:            # the batch failed as one (engine.rs:2041-2045)
            return StepResult(None, [err] * len(entries), [None] * len(entries), shared_failure=err)
        rows, at = [], 0
        for e in entries:
            rows.append(range(at, at + len(e.want)))
            at += len(e.want)
        return StepResult(logits, [None] * len(entries), rows)

    def step(self) -> List[Request]:
        """Admit, plan, run one step, choose tokens, finish.  Returns the requests that
        finished in this call.  With overlap the tokens read in this call are those of
        the step before the one it starts.

        A request whose entry the engine refuses ends with that error and its peers run
        on; if the step fails as a whole every request in it ends with the error; a
        request whose logits row held no finite value ends alone (engine.rs:844-851).
        Each gives its pages and its row back like any finished request."""
        before = set(self.finished)
        self._admit()
        plan = plan_step(self.active, self.max_batch_tokens)
        started = None
        if plan:
            entries = []
            # where the token of a request in flight lies among those chosen in the step before
            place = {id(r): i for i, r in enumerate(self._pending[0])} if self._pending is not None else {}
            for p in plan:
                r = p.request
                start = r.computed
                if r.in_flight:       # its input token is still on the GPU
                    source = (self._pending[1].device_tokens, place[id(r)])
                    entries.append(StepEntry(r.cache, [0], [0] if p.yields_token else [], source))
                else:
                    entries.append(StepEntry(r.cache, r.tokens[start:start + p.count],
                                             [p.count - 1] if p.yields_token else []))
            t0 = time.perf_counter()
            result = self._run(entries)
            ran = []
            for p, err in zip(plan, result.errors):
                if err is None:
                    ran.append(p)
                else:
                    self._fail(p.request, err)
            yielding = [p.request for p in ran if p.yields_token]
            phase = "decode" if all(p.count == 1 and (p.request.in_flight or p.request.generated) for p in plan) else "prefill"
            if yielding:
                counters = [len(r.generated) + (1 if r.in_flight else 0) for r in yielding]
                try:
                    handle = self.sampler.sample_async(
                        result.logits, [r.temperature for r in yielding], [r.seed for r in yielding], counters)
                    started = (yielding, handle, t0, phase)
                except Exception as err:
                    for r in yielding:
                        self._fail(r, err)
            self.steps += 1
            if self.keep_step_log:
                self.step_log.append([(p.request.request_id, p.count) for p in plan])
            if self.trace is not None:
                self.trace({"event": "step_submitted", "step": self.steps, "phase": phase,
                            "requests": len(plan), "tokens": sum(p.count for p in plan),
                            "failed": len(plan) - len(ran),
                            "submit_seconds": time.perf_counter() - t0})
        # the tokens of the step before (with overlap), or of this one
        self._collect()
        if started is not None:
            self._pending = started
            for r in started[0]:
                r.in_flight = True
            if not self.overlap:
                self._collect()
        for r in [r for r in self.active if r.finished]:
            self._release(r)
        return [self.finished[i] for i in self.finished if i not in before]

    def _collect(self) -> None:
        """Read the tokens of the pending step and give them to their requests."""
        if self._pending is None:
            return
        requests, handle, submitted, phase = self._pending
        self._pending = None
        wait_from = time.perf_counter()
        try:
            tokens = handle.tokens() if hasattr(handle, "tokens") else handle.result()
        except Exception as err:
            for r in requests:
                r.in_flight = False
                if not r.finished:
                    self._fail(r, err)
            return
        now = time.perf_counter()
        step_metrics = getattr(self.engine, "step_instruments", None)
        if step_metrics is not None:
            step_metrics.readback_seconds.record(now - wait_from)
            step_metrics.wall(phase, now - submitted)
        for r, token in zip(requests, tokens):
            r.in_flight = False
            if r.finished:
                continue            # it ended a step earlier; this token was one too many
            if token < 0:
                self._fail(r, FloatingPointError(
                    f"request {r.request_id}: non-finite logits, no token can be chosen"))
                continue
            self._accept(r, token, now)

    def _fail(self, r: Request, error: Exception) -> None:
        """The request ends here with an error; ``step`` releases what it holds."""
        if not r.finished:
            r.finish_reason, r.error, r.remaining = "error", error, 0

    def _accept(self, r: Request, token: int, now: float) -> None:
        r.generated.append(token)
        r.tokens.append(token)
        r.remaining -= 1
        if r.first_token_time is None:
            r.first_token_time = now
            self.instruments.first_token(now - r.arrival)
        if self.on_token is not None:
            self.on_token(r, token)
        if token in r.eos:
            r.remaining = 0
            r.finish_reason = "eos"
        elif r.remaining == 0:
            r.finish_reason = "length"

    def _release(self, r: Request) -> None:
        self.active.remove(r)
        if r.cache is not None:
            self.engine.close(r.cache)
            r.cache = None
        r.finish_time = time.perf_counter()
        self.finished[r.request_id] = r
        self.instruments.finished(r.error is None, r.finish_time - r.arrival, len(r.generated),
                                  cancelled=r.finish_reason == "cancelled")

    def _finish(self, r: Request, reason: str, error: Optional[Exception] = None) -> None:
        r.finish_reason, r.error, r.remaining = reason, error, 0
        r.finish_time = time.perf_counter()
        self.finished[r.request_id] = r
        self.instruments.finished(error is None, r.finish_time - r.arrival, 0)

    def cancel(self, request_id: int) -> bool:
        """End a waiting or running request now, between two steps: it leaves its queue,
        gives its pages and its row back at once (what the GPU still writes there is
        ordered before the next step's work on the same stream) and is reported as
        finished with ``finish_reason="cancelled"`` and the tokens it had been given.  A
        token of it that is still on its way is dropped when it arrives.  Returns False
        if no such request is waiting or running.  The reference cancels the runner as a
        whole, which drops every active and waiting turn
        (rust/engine/src/runner/model_runner.rs:899-910, test 1796-1827); ``cancel_all``
        is that."""
        for r in self.waiting:
            if r.request_id == request_id:
                self.waiting.remove(r)
                r.finish_reason, r.remaining = "cancelled", 0
                r.finish_time = time.perf_counter()
                self.finished[r.request_id] = r
                self.instruments.finished(True, r.finish_time - r.arrival, 0, cancelled=True)
                return True
        for r in self.active:
            if r.request_id == request_id:
                if not r.finished:
                    r.finish_reason, r.remaining = "cancelled", 0
                self._release(r)
                return True
        return False

    def cancel_all(self) -> List[int]:
        """Cancel everything that waits or runs; returns the ids."""
        ids = [r.request_id for r in list(self.waiting) + list(self.active)]
        for i in ids:
            self.cancel(i)
        return ids

    @property
    def idle(self) -> bool:
        return not self.waiting and not self.active and self._pending is None

    def run(self) -> Dict[int, Request]:
        """Step until every request has finished."""
        while not self.idle:
            self.step()
        return self.finished
