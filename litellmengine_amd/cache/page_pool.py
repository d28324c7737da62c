"""The free list of one group's pages.

Behaviour pinned by the reference's tests (src/engine/block_table_manager.cpp:213-253,
tests/test_block_table_manager.cpp:279-326): the first pages handed out are
0, 1, 2, ...; pages given back are stacked in the order given, so the last one
given back is the first one used again; asking for more than is free changes
nothing; giving a page back twice is an error.
"""
from __future__ import annotations

from typing import Iterable, List


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was taken."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._held = bytearray(num_pages)

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self, n: int) -> List[int]:
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        if n > len(self._free):
            raise OutOfPages(f"not enough free physical blocks: {n} wanted, {len(self._free)} free")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._held[p] = 1
        return pages

    def release(self, pages: Iterable[int]) -> None:
        pages = list(pages)
        seen = set()
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} does not exist")
            if not self._held[p] or p in seen:
                raise ValueError(f"page {p} is given back twice")
            seen.add(p)
        for p in pages:
            self._held[p] = 0
            self._free.append(p)

    def is_held(self, page: int) -> bool:
        return bool(self._held[page])
