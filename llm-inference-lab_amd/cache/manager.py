"""The cache manager: pages of keys and values with a block table for each
request, one page pool per group of layers with the same need, and slots for
per-request state of fixed size.

Storage of one group (``S`` cache-owning runs of layers, ``N`` pages of ``P``
tokens): one tensor ``[S, N, *page_shape]`` for every named tensor of the group's
``CacheSpec``.  For attention (``G`` kv heads of width ``d``), in the compute dtype::

    k   [S, N, G, P, d]     a page holds, per kv head, P keys of d numbers
    v   [S, N, G, d, P]     and as many values

A page number addresses the same page in every run of the group and in every one
of its tensors, so the group needs one block table.  Position ``p`` of a request lives in page
``table[p // P]`` at offset ``p % P``.  Inside a (page, kv head) pair the
``P * d`` numbers lie in the order of the attention kernels' matrix-core
fragments, not row by row (``cache/layout.py`` has the index maps); the manager
itself never looks inside a page.

The reference's pool has pages of one token, one group, and a slot table
``[rows, max_seq_len]`` (rust/engine/src/runner/kv_pool/naive_kvpool.rs:55-81);
progress per request is split into committed and reserved lengths as in
rust/engine/src/runner/kv_pool/api.rs:193-203.  Windows and groups are not in
the reference.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import CacheSpec
from .pages import OutOfPages, PagePool

NO_PAGE = -1


@dataclasses.dataclass
class GroupLayout:
    """Layers (schedule entries) with one cache need."""

    spec: CacheSpec
    entries: List[int]                     # schedule entries that own a cache in this group
    num_pages: int = 0

    @property
    def window(self) -> Optional[int]:
        return self.spec.window


def pages_for_tokens(tokens: int, page_size: int) -> int:
    return (tokens + page_size - 1) // page_size


def group_page_need(window: Optional[int], page_size: int, total_tokens: int, max_step_tokens: int) -> int:
    """Most pages of one group a request holds at any time when it grows to
    ``total_tokens`` in steps of at most ``max_step_tokens``."""
    full = pages_for_tokens(total_tokens, page_size)
    if window is None:
        return full
    # Before a step of n tokens is committed the request holds the pages of the
    # positions [computed - window + 1, computed + n); that span touches at most
    # ceil((window - 1 + n) / P) + 1 pages.
    span = window - 1 + max(1, max_step_tokens)
    return min(full, pages_for_tokens(span, page_size) + 1)


class RequestCache:
    """What one live request holds: a row (its index in the block tables and
    the state slots), its pages in every group, and how far it has come."""

    def __init__(self, request_id, row: int, num_groups: int):
        self.request_id = request_id
        self.row = row
        self.computed_len = 0          # positions whose keys and values are final
        self.reserved_len = 0          # positions that have pages (>= computed_len)
        self.pages: List[List[int]] = [[] for _ in range(num_groups)]   # logical page -> page or NO_PAGE
        self.first_live: List[int] = [0] * num_groups                   # first logical page still held
        self.released = False
        self.invalid = False           # a step that wrote to it failed: it can only be released


class CacheManager:
    def __init__(self, groups: Sequence[GroupLayout], page_size: int, max_requests: int,
                 max_seq_len: int, state_specs: Dict[int, Dict[str, Tuple[Tuple[int, ...], torch.dtype]]],
                 dtype: torch.dtype, device):
        if page_size < 16 or page_size & (page_size - 1):
            raise ValueError(f"page_size must be a power of two >= 16, got {page_size}")
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.max_seq_len = int(max_seq_len)
        self.max_pages_per_request = pages_for_tokens(self.max_seq_len, self.page_size)
        self.groups = list(groups)
        self.dtype = dtype
        self.device = device
        self.pools = [PagePool(g.num_pages) for g in self.groups]
        self._free_rows = list(range(self.max_requests - 1, -1, -1))
        self._live: Dict[object, RequestCache] = {}
        # host mirror of the block tables; rows of dead requests are NO_PAGE
        self.tables = [np.full((self.max_requests, self.max_pages_per_request), NO_PAGE, dtype=np.int32)
                       for _ in self.groups]
        # per group: name -> [runs, pages, *page_shape].  Zeroed once: a masked position
        # must never meet a NaN bit pattern.
        self.storage: List[Dict[str, torch.Tensor]] = []
        for g in self.groups:
            if not isinstance(g.spec, CacheSpec):
                raise TypeError(f"a cache group is described by a CacheSpec, got {type(g.spec).__name__}")
            self.storage.append({
                name: torch.zeros((len(g.entries), g.num_pages) + t.page_shape(self.page_size),
                                  dtype=t.dtype or dtype, device=device)
                for name, t in g.spec.tensors})
        self.entry_group: Dict[int, Tuple[int, int]] = {}
        for gi, g in enumerate(self.groups):
            for si, e in enumerate(g.entries):
                self.entry_group[e] = (gi, si)
        # per-request state of fixed size: entry -> name -> [max_requests, *shape]
        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        for entry, spec in state_specs.items():
            self.state[entry] = {
                name: torch.zeros((self.max_requests,) + tuple(shape), dtype=dt, device=device)
                for name, (shape, dt) in spec.items()}

    # ------------------------------------------------------------ accounting
    @property
    def live_requests(self) -> int:
        return len(self._live)

    @property
    def free_rows(self) -> int:
        return len(self._free_rows)

    def free_pages(self, group: int) -> int:
        return self.pools[group].free_count

    def metrics(self) -> Dict[str, object]:
        return {
            "page_size": self.page_size,
            "rows_total": self.max_requests, "rows_used": self.live_requests,
            "groups": [{"window": g.window, "layers": len(g.entries), "pages_total": p.num_pages,
                        "pages_free": p.free_count, "pages_used": p.used_count,
                        "pages_high_water": p.high_water}
                       for g, p in zip(self.groups, self.pools)],
        }

    def bytes_per_token(self) -> int:
        """Cache bytes one token takes in all groups (a windowed group holds them for the
        latest ``window`` tokens only)."""
        return sum(len(g.entries) * g.spec.bytes_per_token(self.dtype) for g in self.groups)

    @property
    def keys(self) -> List[torch.Tensor]:
        """Per group the tensor named ``k`` (attention's keys; None for a group without)."""
        return [st.get("k") for st in self.storage]

    @property
    def values(self) -> List[torch.Tensor]:
        return [st.get("v") for st in self.storage]

    def page_need(self, total_tokens: int, max_step_tokens: int) -> List[int]:
        return [group_page_need(g.window, self.page_size, total_tokens, max_step_tokens)
                for g in self.groups]

    # -------------------------------------------------------------- lifecycle
    def get(self, request_id) -> Optional[RequestCache]:
        return self._live.get(request_id)

    def admit(self, request_id) -> RequestCache:
        """Give a request a row; its state slots start at zero."""
        if request_id in self._live:
            raise ValueError(f"request {request_id!r} is already live")
        if not self._free_rows:
            raise OutOfPages(f"all {self.max_requests} request rows are in use")
        row = self._free_rows.pop()
        req = RequestCache(request_id, row, len(self.groups))
        self._live[request_id] = req
        for tensors in self.state.values():
            for t in tensors.values():
                t[row].zero_()
        return req

    def reserve(self, req: RequestCache, new_tokens: int) -> None:
        """Make sure the positions ``[computed_len, computed_len + new_tokens)``
        have pages in every group.  If a group runs out, the pages taken by this
        call are given back and ``OutOfPages`` is raised; the request keeps what
        it had."""
        if req.released:
            raise ValueError(f"request {req.request_id!r} was released")
        if req.invalid:
            raise ValueError(f"request {req.request_id!r} was in a step that failed; release it")
        if new_tokens <= 0:
            raise ValueError("a step brings at least one token for each request in it")
        if req.reserved_len != req.computed_len:
            raise AssertionError("a reservation is already pending")
        end = req.computed_len + new_tokens
        if end > self.max_seq_len:
            raise ValueError(f"request {req.request_id!r}: {end} tokens exceed the cache's "
                             f"maximum sequence length {self.max_seq_len}")
        last_page = (end - 1) // self.page_size
        taken: List[Tuple[int, int]] = []
        try:
            for gi, pool in enumerate(self.pools):
                pages = req.pages[gi]
                while len(pages) <= last_page:
                    page = pool.alloc(req.row)
                    taken.append((gi, page))
                    pages.append(page)
                    self.tables[gi][req.row, len(pages) - 1] = page
        except OutOfPages:
            for gi, page in reversed(taken):
                popped = req.pages[gi].pop()
                assert popped == page
                self.tables[gi][req.row, len(req.pages[gi])] = NO_PAGE
                self.pools[gi].free(page, req.row)
            raise
        req.reserved_len = end

    def commit(self, req: RequestCache) -> None:
        """The step that wrote the reserved positions is done: they count, and
        pages that every later query's window has passed are given back."""
        req.computed_len = req.reserved_len
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            # A later query sits at position >= computed_len and reads keys from
            # position - window + 1 on: nothing below this bound is read again.
            lowest_needed = max(0, req.computed_len - g.window + 1)
            first_needed_page = lowest_needed // self.page_size
            pages = req.pages[gi]
            for lp in range(req.first_live[gi], min(first_needed_page, len(pages))):
                if pages[lp] != NO_PAGE:
                    self.pools[gi].free(pages[lp], req.row)
                    pages[lp] = NO_PAGE
                    self.tables[gi][req.row, lp] = NO_PAGE
            req.first_live[gi] = max(req.first_live[gi], min(first_needed_page, len(pages)))

    def cancel_reservation(self, req: RequestCache) -> None:
        """Drop pages reserved for a step that did not run."""
        keep = pages_for_tokens(req.computed_len, self.page_size)
        for gi, pool in enumerate(self.pools):
            pages = req.pages[gi]
            while len(pages) > keep:
                page = pages.pop()
                if page != NO_PAGE:
                    pool.free(page, req.row)
                self.tables[gi][req.row, len(pages)] = NO_PAGE
        req.reserved_len = req.computed_len

    def release(self, req: RequestCache) -> None:
        """The request has ended: its pages in every group and its row go back."""
        if req.released:
            raise AssertionError(f"request {req.request_id!r} released twice")
        for gi, pool in enumerate(self.pools):
            for page in req.pages[gi]:
                if page != NO_PAGE:
                    pool.free(page, req.row)
            req.pages[gi] = []
            self.tables[gi][req.row, :] = NO_PAGE
        req.released = True
        del self._live[req.request_id]
        self._free_rows.append(req.row)

    def release_all(self) -> None:
        for req in list(self._live.values()):
            self.release(req)

    def check(self) -> None:
        """Invariants: no page lost, none held twice, tables agree with the lists."""
        for gi, pool in enumerate(self.pools):
            pool.check()
            held = {}
            for req in self._live.values():
                for lp, page in enumerate(req.pages[gi]):
                    if page == NO_PAGE:
                        continue
                    if page in held:
                        raise AssertionError(f"page {page} of group {gi} is held twice")
                    held[page] = req.row
                    if pool.owner_of(page) != req.row:
                        raise AssertionError(f"page {page} of group {gi}: owner mismatch")
                    if self.tables[gi][req.row, lp] != page:
                        raise AssertionError("block table disagrees with the page list")
            if len(held) != pool.used_count:
                raise AssertionError(f"group {gi}: {pool.used_count} pages are taken but "
                                     f"{len(held)} are held by live requests")
        rows = [r.row for r in self._live.values()]
        if len(set(rows)) != len(rows) or set(rows) & set(self._free_rows):
            raise AssertionError("a request row is used twice")
        if len(rows) + len(self._free_rows) != self.max_requests:
            raise AssertionError("a request row is lost")
