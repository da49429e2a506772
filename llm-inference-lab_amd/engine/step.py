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
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager, RequestCache
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


class StepContext:
    """What the parts see of a step.  Device tensors (int32):

    ``token_ids [rows]``, ``positions [rows]`` (absolute position of each row in
    its request), ``row_req [rows]`` (which request of the step a row belongs
    to), ``q_start [reqs + 1]`` (first row of each request; rows of a request are
    adjacent), ``start_pos [reqs]`` (tokens already cached before this step),
    ``req_rows [reqs]`` (the request's row in the state slots), ``want_rows
    [wanted]``.  Host-side: ``n_rows``, ``n_reqs``, ``n_want``, ``max_q_len``,
    ``max_ctx_len``, ``host_q_start``, ``host_start_pos``, ``host_req_rows``."""

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
        self._dev = torch.zeros(at, dtype=torch.int32, device=device)
        self._groups = [
            GroupView(self._dev[t:t + b * self.max_pages].view(b, self.max_pages), page_size, window)
            for t, (page_size, window) in zip(self._table_at, groups)]
        self._uploaded = torch.cuda.Event() if pin else None
        self._scratch: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self.scratch_version = 0
        self.n_rows = self.n_reqs = self.n_want = 0
        self.max_q_len = self.max_ctx_len = 0
        self._short = {}
        self.pending = None            # PendingSums owed to the residual stream, within a forward
        self.host_q_start: List[int] = []
        self.host_start_pos: List[int] = []
        self.host_req_rows: List[int] = []
        self._set_views()

    def _view(self, name: str, count: int) -> torch.Tensor:
        at, cap = self._offsets[name]
        return self._dev[at:at + count]

    def _set_views(self) -> None:
        self.token_ids = self._view("token_ids", self.n_rows)
        self.positions = self._view("positions", self.n_rows)
        self.row_req = self._view("row_req", self.n_rows)
        self.q_start = self._view("q_start", self.n_reqs + 1)
        self.start_pos = self._view("start_pos", self.n_reqs)
        self.req_rows = self._view("req_rows", self.n_reqs)
        self.want_rows = self._view("want_rows", self.n_want)

    def group(self, index: int) -> GroupView:
        return self._groups[index]

    def scratch(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        """A reusable buffer: the same name and dtype give the same memory on
        every step, grown when a larger shape is asked for."""
        count = 1
        for s in shape:
            count *= int(s)
        key = (name, dtype)
        buf = self._scratch.get(key)
        if buf is None or buf.numel() < count:
            buf = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._scratch[key] = buf
            self.scratch_version += 1
        return buf[:count].view(shape)

    def short_requests(self, limit: int) -> Tuple[int, int]:
        """How many of this step's requests bring at most ``limit`` tokens, and the
        longest context among those (0 if none)."""
        hit = self._short.get(limit)
        if hit is None:
            count = longest = 0
            for b in range(self.n_reqs):
                n = self.host_q_start[b + 1] - self.host_q_start[b]
                if n <= limit:
                    count += 1
                    longest = max(longest, self.host_start_pos[b] + n)
            hit = self._short[limit] = (count, longest)
        return hit

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
        self._short = {}
        max_q = max_ctx = 0
        for b, e in enumerate(entries):
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
        for i, (dst, src) in enumerate(feeds):
            h[o["feed_dst"] + i] = dst
            h[o["feed_src"] + i] = src
        self._upload(n_reqs)
        self._set_views()
        if feeds:
            self.ops.gather_tokens(self._view("token_ids", self.max_rows), self._view("feed_dst", len(feeds)),
                                   feed_tensor, self._view("feed_src", len(feeds)), len(feeds))

    def _upload(self, n_reqs: int) -> None:
        self._dev[:self._meta_len].copy_(self._host[:self._meta_len], non_blocking=True)
        for at in self._table_at:
            n = n_reqs * self.max_pages
            self._dev[at:at + n].copy_(self._host[at:at + n], non_blocking=True)
        if self._uploaded is not None:
            self._uploaded.record()


class StepFunction:
    """Owns the step's buffers; ``__call__`` runs one step."""

    MAX_GRAPHS = 16

    def __init__(self, model: CausalLM, cache: CacheManager, ops, max_batch_tokens: int,
                 graph: bool = False):
        self.model = model
        self.cache = cache
        self.ops = ops
        self.max_batch_tokens = int(max_batch_tokens)
        # Pure decode steps (one token and one wanted place per request) can be
        # replayed from a captured HIP graph: buffers have fixed addresses and
        # everything that changes from step to step (tokens, positions, block
        # tables) lives in device memory that is rewritten before the replay.
        self.use_graph = bool(graph)
        self._graphs: "collections.OrderedDict" = collections.OrderedDict()
        self.graph_replays = 0
        self.graph_captures = 0
        self.ctx = StepContext(
            ops, cache.device, self.max_batch_tokens, cache.max_requests,
            [(cache.page_size, g.window) for g in cache.groups], cache.max_pages_per_request)
        self.steps = 0
        self.rows_total = 0

    def _decode_with_graph(self) -> torch.Tensor:
        ctx = self.ctx
        # Grid sizes and split counts are frozen into a graph: take them from a
        # bucket of the context length, so one graph serves while contexts grow.
        bucket = 128
        while bucket < ctx.max_ctx_len:
            bucket *= 2
        ctx.max_ctx_len = min(bucket, self.cache.max_pages_per_request * self.cache.page_size)
        key = (ctx.n_reqs, ctx.max_ctx_len, ctx.scratch_version)
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
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize(ctx.device)
        with torch.cuda.graph(graph):
            captured = self.model.forward(ctx)
        self._graphs[key] = (graph, captured)
        self.graph_captures += 1
        while len(self._graphs) > self.MAX_GRAPHS:
            self._graphs.popitem(last=False)
        return logits

    def __call__(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Reserve pages, run the rows, commit.  Returns float32 logits
        ``[wanted, vocab]`` in the order of the entries and of their ``want``
        (None when nothing is wanted).  The tensor is reused by the next step."""
        if not entries:
            return None
        vocab, max_pos = self.model.spec.vocab_size, self.model.spec.max_positions
        seen = set()
        for e in entries:
            if id(e.request) in seen:
                raise ValueError(f"request {e.request.request_id!r} appears twice in one step")
            seen.add(id(e.request))
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.request.request_id!r} brings no token")
            for t in (e.tokens if e.source is None else ()):
                if not 0 <= int(t) < vocab:
                    raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
            if e.request.computed_len + len(e.tokens) > max_pos:
                raise ValueError(
                    f"request {e.request.request_id!r}: position "
                    f"{e.request.computed_len + len(e.tokens) - 1} exceeds max_position_embeddings {max_pos}")
        reserved: List[RequestCache] = []
        try:
            for e in entries:
                self.cache.reserve(e.request, len(e.tokens))
                reserved.append(e.request)
            self.ctx.fill(entries, self.cache)
        except Exception:
            for r in reserved:
                self.cache.cancel_reservation(r)
            raise
        if self.use_graph and all(len(e.tokens) == 1 and len(e.want) == 1 and e.want[0] == 0 for e in entries):
            logits = self._decode_with_graph()
        else:
            logits = self.model.forward(self.ctx)
        for e in entries:
            self.cache.commit(e.request)
        self.steps += 1
        self.rows_total += self.ctx.n_rows
        return logits
