"""Page allocator of one cache group: a stack of free page numbers plus an
owner table that makes every misuse (a page handed out twice, freed twice, or
freed by someone who does not hold it) an immediate error.

The reference keeps free slot numbers in a vector and pops from its tail
(rust/engine/src/runner/kv_pool/naive_kvpool.rs:159-163, 449-460); its slots
hold one token each, ours hold ``page_size`` tokens.
"""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """A request needs more pages than its group has free."""


FREE = -1


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        # Low page numbers are handed out first.
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))
        self._owner: List[int] = [FREE] * self.num_pages
        self.high_water = 0

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def used_count(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self, owner: int) -> int:
        if owner < 0:
            raise ValueError("owner ids are non-negative")
        if not self._free:
            raise OutOfPages(f"no free page among {self.num_pages}")
        page = self._free.pop()
        if self._owner[page] != FREE:
            raise AssertionError(f"page {page} on the free stack is held by {self._owner[page]}")
        self._owner[page] = owner
        self.high_water = max(self.high_water, self.used_count)
        return page

    def free(self, page: int, owner: int) -> None:
        if not 0 <= page < self.num_pages:
            raise ValueError(f"page {page} is not in the pool")
        if self._owner[page] == FREE:
            raise AssertionError(f"page {page} freed twice")
        if self._owner[page] != owner:
            raise AssertionError(f"page {page} is held by {self._owner[page]}, not by {owner}")
        self._owner[page] = FREE
        self._free.append(page)

    def owner_of(self, page: int) -> int:
        return self._owner[page]

    def check(self) -> None:
        """Every page is either on the free stack once or held by one owner."""
        seen = set()
        for page in self._free:
            if page in seen:
                raise AssertionError(f"page {page} is on the free stack twice")
            seen.add(page)
            if self._owner[page] != FREE:
                raise AssertionError(f"free page {page} has owner {self._owner[page]}")
        held = sum(1 for o in self._owner if o != FREE)
        if held + len(self._free) != self.num_pages:
            raise AssertionError("a page is lost: neither free nor held")
