"""The step function: one packed, ragged batch from the cache to logits.

A step takes, for each request in it, the request's next tokens (a portion of
its prompt, cut anywhere, or one decoded token) and the places among those
tokens whose logits are wanted.  All rows of all requests run as one batch;
keys and values of the new positions go to the request's pages; earlier
positions are read from there.  Only the given tokens are computed.

The reference's counterpart is ``CausalModel::forward`` over
``ModelInput{token_ids, kv}`` (rust/engine/src/runner/model/api.rs:11-16,
203-207): rows packed in input order with per-row (context row, position)
metadata and per-request last-row indices
(rust/engine/src/runner/model/qwen2/engine.rs:936-969, 1794-1851).  It returns
one prediction per request; this one returns logits at the wanted places.
"""
from __future__ import annotations

import collections
import dataclasses
import time
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager, RequestCache
from .instruments import StepInstruments
from .model import CausalLM


@dataclasses.dataclass
class StepEntry:
    """One request's share of a step."""

    request: RequestCache
    tokens: Sequence[int]
    want: Sequence[int] = ()        # indices into ``tokens`` whose logits are returned
    # The one token of this entry is not known to the host yet: it is element
    # ``source[1]`` of the int32 device tensor ``source[0]`` (what the sampler wrote
    # for the previous step).  ``tokens`` then holds one placeholder.
    source: Optional[Tuple[torch.Tensor, int]] = None


@dataclasses.dataclass
class GroupView:
    block_table: torch.Tensor       # int32 [max_requests, max_pages_per_request], row b = b-th request of the step
    page_size: int
    window: Optional[int]


class ScratchExhausted(RuntimeError):
    """A step needs more scratch memory than the weights and the cache left free."""


@dataclasses.dataclass
class StepResult:
    """What a step gives back.  ``errors[i]`` is None if entry i ran; ``rows[i]`` are then
    the rows of ``logits`` that hold its wanted places (``logits`` has the wanted places of
    the entries that ran, in their order).  ``shared_failure``: the batch as a whole
    failed, every entry that was in it carries this error."""

    logits: Optional[torch.Tensor]
    errors: List[Optional[Exception]]
    rows: List[Optional[range]]
    shared_failure: Optional[Exception] = None


class StepContext:
    """What the parts see of a step.  Device tensors (int32):

    ``token_ids [rows]``, ``positions [rows]`` (absolute position of each row in
    its request), ``row_req [rows]`` (which request of the step a row belongs
    to), ``q_start [reqs + 1]`` (first row of each request; rows of a request are
    adjacent), ``start_pos [reqs]`` (tokens already cached before this step),
    ``req_rows [reqs]`` (the request's row in the state slots), ``want_rows
    [wanted]``.  Host-side: ``n_rows``, ``n_reqs``, ``n_want``, ``max_q_len``,
    ``max_ctx_len``, ``host_q_start``, ``host_start_pos``, ``host_req_rows``, and ``memo``,
    a dictionary for what a part works out once per step and its other layers use again."""

    def __init__(self, ops, device, max_rows: int, max_reqs: int, groups: List[Tuple[int, Optional[int]]],
                 max_pages_per_request: int):
        self.ops = ops
        self.device = device
        self.max_rows, self.max_reqs = int(max_rows), int(max_reqs)
        self.max_pages = int(max_pages_per_request)
        r, b = self.max_rows, self.max_reqs
        # One int32 buffer, fixed offsets: the addresses never change, so a
        # captured graph of a step stays valid while only the contents move.
        sizes = [("token_ids", r), ("positions", r), ("row_req", r), ("q_start", b + 1),
                 ("start_pos", b), ("req_rows", b), ("want_rows", r), ("feed_dst", b), ("feed_src", b)]
        self._offsets: Dict[str, Tuple[int, int]] = {}
        at = 0
        for name, n in sizes:
            self._offsets[name] = (at, n)
            at += n
        self._meta_len = at
        self._table_at = []
        for _ in groups:
            self._table_at.append(at)
            at += b * self.max_pages
        pin = (torch.device(device).type == "cuda")
        self._host = torch.zeros(at, dtype=torch.int32, pin_memory=pin)
        self._host_np = self._host.numpy()
        self._counting = np.arange(max(r, b) + 1, dtype=np.int32)
        self._dev = torch.zeros(at, dtype=torch.int32, device=device)
        self._groups = [
            GroupView(self._dev[t:t + b * self.max_pages].view(b, self.max_pages), page_size, window)
            for t, (page_size, window) in zip(self._table_at, groups)]
        self._uploaded = torch.cuda.Event() if pin else None
        self._scratch: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self._views: Dict[tuple, torch.Tensor] = {}     # views of the scratch buffers handed out so far
        self._step_views: Dict[tuple, tuple] = {}       # views of the step's description by (rows, requests, wanted)
        self.scratch_version = 0
        self.scratch_bytes = 0
        self.scratch_allocations = 0
        self.n_rows = self.n_reqs = self.n_want = 0
        self.max_q_len = self.max_ctx_len = 0
        self.memo: Dict[object, object] = {}     # notes of the parts about this step, emptied by fill()
        self.pending = None            # PendingSums owed to the residual stream, within a forward
        self.host_q_start: List[int] = []
        self.host_start_pos: List[int] = []
        self.host_req_rows: List[int] = []
        # (the whole arrays behind ``q_start`` and ``start_pos``, for a caller that checks once
        # what it will use for steps of any number of requests)
        self.all_q_start, self.all_start_pos = self._view("q_start", b + 1), self._view("start_pos", b)
        self._set_views()

    def _view(self, name: str, count: int) -> torch.Tensor:
        at, cap = self._offsets[name]
        return self._dev[at:at + count]

    def _set_views(self) -> None:
        key = (self.n_rows, self.n_reqs, self.n_want)
        views = self._step_views.get(key)          # (slicing seven tensors anew costs 10 us a step)
        if views is None:
            views = (self._view("token_ids", self.n_rows), self._view("positions", self.n_rows),
                     self._view("row_req", self.n_rows), self._view("q_start", self.n_reqs + 1),
                     self._view("start_pos", self.n_reqs), self._view("req_rows", self.n_reqs),
                     self._view("want_rows", self.n_want))
            if len(self._step_views) < 1024:
                self._step_views[key] = views
        (self.token_ids, self.positions, self.row_req, self.q_start, self.start_pos, self.req_rows,
         self.want_rows) = views

    def group(self, index: int) -> GroupView:
        return self._groups[index]

    def scratch(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        """A reusable buffer: the same name and dtype give the same memory on
        every step, grown when a larger shape is asked for.  Before it grows it asks
        whether the GPU still has the memory (what is free, and what the allocator holds
        unused): the page pool takes most of what the weights left, and a step that needs
        more scratch than remains fails with ``ScratchExhausted`` instead of somewhere in
        the allocator (rust/engine/src/runner/model/qwen2/workspace.rs:348-373)."""
        hit = self._views.get((name, dtype, shape))      # (slicing and viewing anew costs microseconds a call)
        if hit is not None:
            return hit
        count = 1
        for s in shape:
            count *= int(s)
        key = (name, dtype)
        buf = self._scratch.get(key)
        if buf is None or buf.numel() < count:
            width = torch.empty((), dtype=dtype).element_size()
            need = max(count, 1) * width
            have = self._memory_available()
            if have is not None and need > have:
                raise ScratchExhausted(f"scratch buffer '{name}' needs {need} bytes; {have} bytes are "
                                       f"available after the weights and the cache")
            self.scratch_bytes += need - (0 if buf is None else buf.numel() * width)
            self.scratch_allocations += 1
            buf = None                      # give the old one back before taking the new
            self._scratch.pop(key, None)
            buf = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._scratch[key] = buf
            self.scratch_version += 1
            self._views = {k: v for k, v in self._views.items() if (k[0], k[1]) != key}
        view = buf[:count].view(shape)
        if len(self._views) < 4096 and isinstance(shape, tuple):
            self._views[(name, dtype, shape)] = view
        return view

    def _memory_available(self) -> Optional[int]:
        if torch.device(self.device).type != "cuda":
            return None
        free, _ = torch.cuda.mem_get_info(self.device)
        stats = torch.cuda.memory_stats(self.device)
        reusable = stats.get("reserved_bytes.all.current", 0) - stats.get("allocated_bytes.all.current", 0)
        return int(free) + max(0, int(reusable))

    # ------------------------------------------------------------------ fill
    def fill(self, entries: Sequence[StepEntry], cache: CacheManager) -> None:
        n_rows = sum(len(e.tokens) for e in entries)
        n_reqs = len(entries)
        if n_rows > self.max_rows:
            raise ValueError(f"a step of {n_rows} tokens exceeds max_batch_tokens {self.max_rows}")
        if n_reqs > self.max_reqs:
            raise ValueError(f"a step of {n_reqs} requests exceeds max_requests {self.max_reqs}")
        if self._uploaded is not None:
            self._uploaded.synchronize()      # the staging buffer is free again
        h = self._host_np
        o = {k: v[0] for k, v in self._offsets.items()}
        row = 0
        want: List[int] = []
        feeds: List[Tuple[int, int]] = []
        feed_tensor = None
        self.host_q_start, self.host_start_pos, self.host_req_rows = [], [], []
        self.memo = {}
        max_q = max_ctx = 0
        one_token_each = n_rows == n_reqs and all(len(e.tokens) == 1 for e in entries)
        if one_token_each:
            # a decode step: every array in one piece (a numpy store per number costs as much
            # as the rest of the host's work on a request)
            n = n_reqs
            starts = [e.request.computed_len for e in entries]
            slots = [e.request.row for e in entries]
            count = self._counting[:n + 1]
            h[o["token_ids"]:o["token_ids"] + n] = [e.tokens[0] for e in entries]
            h[o["positions"]:o["positions"] + n] = starts
            h[o["row_req"]:o["row_req"] + n] = count[:n]
            h[o["q_start"]:o["q_start"] + n] = count[:n]
            h[o["start_pos"]:o["start_pos"] + n] = starts
            h[o["req_rows"]:o["req_rows"] + n] = slots
            for b, e in enumerate(entries):
                if e.source is not None:
                    if feed_tensor is not None and feed_tensor is not e.source[0]:
                        raise ValueError("all device-fed entries of a step share one source tensor")
                    feed_tensor = e.source[0]
                    feeds.append((b, int(e.source[1])))
                for w in e.want:
                    if w != 0:
                        raise ValueError(f"request {e.request.request_id!r}: wanted place {w} is not "
                                         f"among its 1 tokens of this step")
                    want.append(b)
            self.host_q_start, self.host_start_pos, self.host_req_rows = list(range(n)), starts, slots
            max_q, max_ctx, row = 1, max(starts) + 1, n
        for b, e in enumerate(() if one_token_each else entries):
            n = len(e.tokens)
            start = e.request.computed_len
            if n == 1:          # (a decoding request: no arrays for one number)
                h[o["token_ids"] + row] = e.tokens[0]
                h[o["positions"] + row] = start
                h[o["row_req"] + row] = b
            else:
                h[o["token_ids"] + row:o["token_ids"] + row + n] = np.asarray(e.tokens, dtype=np.int32)
                h[o["positions"] + row:o["positions"] + row + n] = np.arange(start, start + n, dtype=np.int32)
                h[o["row_req"] + row:o["row_req"] + row + n] = b
            h[o["q_start"] + b] = row
            h[o["start_pos"] + b] = start
            h[o["req_rows"] + b] = e.request.row
            if e.source is not None:
                if n != 1:
                    raise ValueError("an entry fed from the device brings exactly one token")
                if feed_tensor is not None and feed_tensor is not e.source[0]:
                    raise ValueError("all device-fed entries of a step share one source tensor")
                feed_tensor = e.source[0]
                feeds.append((row, int(e.source[1])))
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.request.request_id!r}: wanted place {w} is not "
                                     f"among its {n} tokens of this step")
                want.append(row + int(w))
            self.host_q_start.append(row)
            self.host_start_pos.append(start)
            self.host_req_rows.append(e.request.row)
            max_q = max(max_q, n)
            max_ctx = max(max_ctx, start + n)
            row += n
        h[o["q_start"] + n_reqs] = row
        self.host_q_start.append(row)
        if want:
            h[o["want_rows"]:o["want_rows"] + len(want)] = np.asarray(want, dtype=np.int32)
        self.n_rows, self.n_reqs, self.n_want = n_rows, n_reqs, len(want)
        self.max_q_len, self.max_ctx_len = max_q, max_ctx
        used_pages = (max_ctx + cache.page_size - 1) // cache.page_size
        cache_rows = self.host_req_rows
        for gi, at in enumerate(self._table_at):
            table = h[at:at + self.max_reqs * self.max_pages].reshape(self.max_reqs, self.max_pages)
            table[:n_reqs, :used_pages] = cache.tables[gi][cache_rows, :used_pages]
        if feeds:
            h[o["feed_dst"]:o["feed_dst"] + len(feeds)] = [dst for dst, _ in feeds]
            h[o["feed_src"]:o["feed_src"] + len(feeds)] = [src for _, src in feeds]
        self._upload(n_reqs)
        self._set_views()
        if feeds:
            self.ops.gather_tokens(self._view("token_ids", self.max_rows), self._view("feed_dst", len(feeds)),
                                   feed_tensor, self._view("feed_src", len(feeds)), len(feeds))

    ONE_COPY_INTS = 64 * 1024      # up to here the description and the block tables go in one copy

    def _upload(self, n_reqs: int) -> None:
        n = n_reqs * self.max_pages
        end = self._table_at[-1] + n if self._table_at else self._meta_len
        if end <= self.ONE_COPY_INTS:
            # (the rows between the groups' tables that no request of this step uses go along:
            # a copy more would cost more than their bytes)
            self._dev[:end].copy_(self._host[:end], non_blocking=True)
        else:
            self._dev[:self._meta_len].copy_(self._host[:self._meta_len], non_blocking=True)
            for at in self._table_at:
                self._dev[at:at + n].copy_(self._host[at:at + n], non_blocking=True)
        if self._uploaded is not None:
            self._uploaded.record()


class StepFunction:
    """Owns the step's buffers; ``__call__`` runs one step."""

    MAX_GRAPHS = 16
    CAPTURE_AT = 2           # a decode graph is captured when its key comes this many times ...
    CAPTURE_WINDOW = 32      # ... within so many decode steps

    def __init__(self, model: CausalLM, cache: CacheManager, ops, max_batch_tokens: int,
                 graph=False):
        self.model = model
        self.cache = cache
        self.ops = ops
        self.max_batch_tokens = int(max_batch_tokens)
        # Pure decode steps (one token and one wanted place per request) can be
        # replayed from a captured HIP graph: buffers have fixed addresses and
        # everything that changes from step to step (tokens, positions, block
        # tables) lives in device memory that is rewritten before the replay.
        # A model with a part that cannot be captured (``graph_safe`` False) runs
        # eagerly whatever is asked for here.  ``graph="auto"``: the first decode step
        # runs eagerly and the calls into the kernel libraries that it makes are counted;
        # from then on every decode step is replayed or launched call by call as the
        # kernel set's rules say for that many calls, the model's weights and the cache
        # that the step's requests hold (``ops.rules.graph_pays``).
        self.use_graph = graph if graph == "auto" else bool(graph)
        self.auto_graph = graph == "auto"
        self._graphs: "collections.OrderedDict" = collections.OrderedDict()
        self._seen: Dict[tuple, tuple] = {}       # key without a graph -> (times it has come, at which step last)
        self._decode_steps = 0                    # decode steps that asked for a graph
        self.graph_replays = 0
        self.graph_captures = 0
        self.graph_evictions = 0
        self.decode_calls: Optional[int] = None    # library calls of one decode step (measured)
        self.ctx = StepContext(
            ops, cache.device, self.max_batch_tokens, cache.max_requests,
            [(cache.page_size, g.window) for g in cache.groups], cache.max_pages_per_request)
        self.steps = 0
        self.rows_total = 0
        self.failed_steps = 0
        self.instruments = StepInstruments()

    def cache_bytes_of_step(self) -> int:
        """Bytes of cache that the step in ``ctx`` reads: for every group what its layers
        keep per token, times the positions of each request that they still see."""
        ctx, total = self.ctx, 0
        seen_all = sum(ctx.host_start_pos[:ctx.n_reqs]) + ctx.n_rows      # (without a window: one sum for all requests)
        for g in self.cache.groups:
            per_token = len(g.entries) * g.spec.bytes_per_token(self.cache.dtype)
            if not g.window:
                total += per_token * seen_all
                continue
            for b in range(ctx.n_reqs):
                seen = ctx.host_start_pos[b] + ctx.host_q_start[b + 1] - ctx.host_q_start[b]
                total += per_token * min(seen, g.window)
        return total

    def _decode_auto(self) -> torch.Tensor:
        """``graph="auto"``: the first decode step runs eagerly and its calls are counted;
        then the rules decide, step by step."""
        rules = getattr(self.ops, "rules", None)
        counted = getattr(self.ops, "calls_made", None)
        if counted is None or not hasattr(rules, "graph_pays"):
            self.use_graph = self.auto_graph = False       # a kernel set that does not count
            return self.model.forward(self.ctx)
        if self.decode_calls is None:
            logits = self.model.forward(self.ctx)
            self.decode_calls = self.ops.calls_made - counted
            self.use_graph = rules.graph_pays(self.decode_calls, self.model.weight_bytes_per_step(),
                                              self.cache_bytes_of_step())
            return logits
        self.use_graph = rules.graph_pays(self.decode_calls, self.model.weight_bytes_per_step(),
                                          self.cache_bytes_of_step())
        return self._decode_with_graph() if self.use_graph else self.model.forward(self.ctx)

    def _decode_with_graph(self) -> torch.Tensor:
        ctx = self.ctx
        # Grid sizes and split counts are frozen into a graph: take them from a
        # bucket of the context length, so one graph serves while contexts grow.
        bucket = 128
        while bucket < ctx.max_ctx_len:
            bucket *= 2
        ctx.max_ctx_len = min(bucket, self.cache.max_pages_per_request * self.cache.page_size)
        key = (ctx.n_reqs, ctx.max_ctx_len, ctx.scratch_version)
        self._decode_steps += 1
        hit = self._graphs.get(key)
        if hit is not None:
            self._graphs.move_to_end(key)
            graph, logits = hit
            graph.replay()
            self.graph_replays += 1
            return logits
        logits = self.model.forward(ctx)       # this step's result; also sizes every scratch buffer
        if key[2] != ctx.scratch_version:
            return logits                      # buffers moved: capture at the next step
        # A capture costs milliseconds (a second forward and the making of the graph): it is
        # made when a key comes the second time within a few decode steps.  While requests
        # end one after the other (the tail of a run) every key comes once, and again once
        # in the next run's tail: capturing each made those steps twice as slow as launching
        # them from the kept sequences, and pushed the graphs of the steady state out.
        count, last = self._seen.pop(key, (0, -self.CAPTURE_WINDOW))
        count = count + 1 if self._decode_steps - last <= self.CAPTURE_WINDOW else 1
        self._seen[key] = (count, self._decode_steps)
        if len(self._seen) > 4 * self.MAX_GRAPHS:
            self._seen.pop(next(iter(self._seen)))
        if count < self.CAPTURE_AT:
            return logits
        self._seen.pop(key, None)
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize(ctx.device)
        with torch.cuda.graph(graph):
            captured = self.model.forward(ctx)
        self._graphs[key] = (graph, captured)
        self.graph_captures += 1
        while len(self._graphs) > self.MAX_GRAPHS:
            self._graphs.popitem(last=False)
            self.graph_evictions += 1
        return logits

    # ------------------------------------------------------------- validation
    def _refusal(self, e: StepEntry, seen: set) -> Optional[Exception]:
        """Why this entry cannot be part of a step, or None (the reference checks the
        same per input: rust/engine/src/runner/model/qwen2/engine.rs:811-842)."""
        vocab, max_pos = self.model.spec.vocab_size, self.model.spec.max_positions
        rid = e.request.request_id
        if id(e.request) in seen:
            return ValueError(f"request {rid!r} appears twice in one step")
        if e.request.released:
            return ValueError(f"request {rid!r} was released")
        if e.request.invalid:
            return ValueError(f"request {rid!r} was in a step that failed: its cache is not "
                              f"to be trusted any more, release it")
        if e.request.reserved_len != e.request.computed_len:
            return ValueError(f"request {rid!r} has a step pending")
        n = len(e.tokens)
        if n == 0:
            return ValueError(f"request {rid!r} brings no token")
        if e.source is None:
            if n > 8:       # (a portion of a prompt: one pass in numpy instead of a Python loop)
                ids = np.asarray(e.tokens)
                lowest, highest = int(ids.min()), int(ids.max())
                if lowest < 0 or highest >= vocab:
                    return ValueError(f"token id {lowest if lowest < 0 else highest} is outside the "
                                      f"vocabulary of {vocab}")
            else:
                for t in e.tokens:
                    if not 0 <= int(t) < vocab:
                        return ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        elif n != 1:
            return ValueError("an entry fed from the device brings exactly one token")
        end = e.request.computed_len + n
        if end > max_pos:
            return ValueError(f"request {rid!r}: position {end - 1} exceeds "
                              f"max_position_embeddings {max_pos}")
        if end > self.cache.max_seq_len:
            return ValueError(f"request {rid!r}: {end} tokens exceed the cache's maximum "
                              f"sequence length {self.cache.max_seq_len}")
        for w in e.want:
            if not 0 <= int(w) < n:
                return ValueError(f"request {rid!r}: wanted place {w} is not among its {n} "
                                  f"tokens of this step")
        return None

    def run(self, entries: Sequence[StepEntry], strict: bool = False) -> "StepResult":
        """One step with a result for every entry.  An entry that cannot run (a token id
        outside the vocabulary, a position beyond the longest sequence, no page left for
        it) gets its error and is left out; the others still run as one batch
        (rust/engine/src/runner/model/qwen2/engine.rs:1943-2003).  If the batch itself
        fails (a kernel refuses a size, a launch fails), every entry that was in it gets
        that error (engine.rs:2041-2045), their reservations are dropped and their caches
        are marked invalid (rust/engine/src/runner/kv_pool/api.rs:257-262): what the step
        half wrote is not to be read, such a request can only be released.

        ``strict``: all or nothing.  The first entry that cannot run (also one that finds
        no page) raises its error before anything has run, and every reservation this
        call made is given back: lengths and pages of all entries are as before."""
        errors: List[Optional[Exception]] = [None] * len(entries)
        seen: set = set()
        for i, e in enumerate(entries):
            errors[i] = self._refusal(e, seen)
            if errors[i] is None:
                seen.add(id(e.request))
            elif strict:
                raise errors[i]
        # what is wrong with the step as a whole is the caller's mistake: nothing runs
        n_rows = sum(len(e.tokens) for e, err in zip(entries, errors) if err is None)
        if n_rows > self.max_batch_tokens:
            raise ValueError(f"a step of {n_rows} tokens exceeds max_batch_tokens {self.max_batch_tokens}")
        if sum(1 for err in errors if err is None) > self.cache.max_requests:
            raise ValueError(f"a step of more than {self.cache.max_requests} requests (max_requests)")
        for i, e in enumerate(entries):
            if errors[i] is None:
                try:
                    self.cache.reserve(e.request, len(e.tokens))
                except Exception as err:            # no page left: this entry sits out, with its reason
                    if strict:
                        for earlier in entries[:i]:
                            self.cache.cancel_reservation(earlier.request)
                        raise
                    errors[i] = err
        valid = [e for e, err in zip(entries, errors) if err is None]
        rows: List[Optional[range]] = []
        at = 0
        for e, err in zip(entries, errors):
            rows.append(None if err is not None else range(at, at + len(e.want)))
            at += 0 if err is not None else len(e.want)
        if not valid:
            return StepResult(None, errors, rows)
        started = time.perf_counter()
        try:
            self.ctx.fill(valid, self.cache)
            if ((self.use_graph or self.auto_graph) and self.model.graph_safe
                    and all(len(e.tokens) == 1 and len(e.want) == 1 for e in valid)):
                logits = self._decode_auto() if self.auto_graph else self._decode_with_graph()
            else:
                logits = self.model.forward(self.ctx)
        except Exception as err:
            for e in valid:
                self.cache.cancel_reservation(e.request)
                e.request.invalid = True
            for i, had in enumerate(errors):
                if had is None:
                    errors[i] = err
            self.failed_steps += 1
            return StepResult(None, errors, [None] * len(entries), shared_failure=err)
        for e in valid:
            self.cache.commit(e.request)
        self.steps += 1
        self.rows_total += self.ctx.n_rows
        self.instruments.step(
            prefill=any(e.request.computed_len == len(e.tokens) or len(e.tokens) > 1 for e in valid),
            rows=self.ctx.n_rows, requests=len(valid), submit_seconds=time.perf_counter() - started)
        return StepResult(logits, errors, rows)

    def __call__(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Reserve pages, run the rows, commit.  Returns float32 logits
        ``[wanted, vocab]`` in the order of the entries and of their ``want``
        (None when nothing is wanted).  The tensor is reused by the next step.
        All or nothing: an entry that cannot run (an invalid token, a position too far, no
        page left for it) raises here before anything has run, with the lengths and the
        pages of every entry as they were, so the caller may try again with other entries.
        A batch that fails while it runs raises too; its requests are then invalid."""
        if not entries:
            return None
        result = self.run(entries, strict=True)
        for err in result.errors:
            if err is not None:
                raise err
        return result.logits
