"""The pages of one cache group: the free list and the block tables, kept by the
native host library (csrc/host.cpp); this module is its Python face.

Behaviour pinned by the reference's tests (src/engine/block_table_manager.cpp:213-253,
tests/test_block_table_manager.cpp:279-326): the first pages handed out are
0, 1, 2, ...; pages given back are stacked in the order given, so the last one
given back is the first one used again; asking for more than is free changes
nothing; giving a page back twice is an error.
"""
from __future__ import annotations

import ctypes
from typing import Iterable, List, Optional

from ..csrc import build

OK, OUT_OF_PAGES, NO_SUCH_PAGE, FREED_TWICE, TOO_MANY_PAGES, BAD_TOKEN, NO_PAGE_AT_POSITION, BAD_ARGUMENT = range(8)

_I, _P, _L = ctypes.c_int, ctypes.c_void_p, ctypes.c_int64
_SIGNATURES = {
    "lle_pt_create": ([_I, _I, _I, _I, _I], _P),
    "lle_pt_destroy": ([_P], None),
    "lle_pt_num_pages": ([_P], _I),
    "lle_pt_num_free": ([_P], _I),
    "lle_pt_is_held": ([_P, _I], _I),
    "lle_pt_allocate": ([_P, _I, _P], _I),
    "lle_pt_release": ([_P, _P, _I, _P], _I),
    "lle_pt_table_len": ([_P, _I], _I),
    "lle_pt_table_copy": ([_P, _I, _P], None),
    "lle_pt_first_live": ([_P, _I], _I),
    "lle_pt_new_pages_needed": ([_P, _I, _I], _I),
    "lle_pt_grow": ([_P, _I, _I], _I),
    "lle_pt_pages_needed_many": ([_P, _I, _P, _P], _I),
    "lle_pt_grow_many": ([_P, _I, _P, _P], _I),
    "lle_pt_shrink": ([_P, _I, _I], None),
    "lle_pt_shrink_many": ([_P, _I, _P, _P], None),
    "lle_pt_trim": ([_P, _I, _I], None),
    "lle_pt_trim_many": ([_P, _I, _P, _P], None),
    "lle_pt_release_slot": ([_P, _I], None),
    "lle_pt_token_slot": ([_P, _I, _I], _L),
    "lle_pt_num_pending": ([_P], _I),
    "lle_pt_take_pending": ([_P, _P, _P], None),
    "lle_layout_step": ([_I, _P, _P, _P, _P, _I, _I, _I, _P, _I, _P, _I, _I, _P, _P], _I),
}
_lib = None


def host_library():
    """The loaded host library with its signatures declared (built at first use)."""
    global _lib
    if _lib is None:
        lib = build.load_library("host")
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, restype
        _lib = lib
    return _lib


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was taken."""


class PageTables:
    """Owner of one native table set: `num_pages` pages of `page_size` tokens and the block
    tables of `max_requests` request slots."""

    def __init__(self, num_pages: int, page_size: int = 1, max_requests: int = 0, max_pages_per_request: int = 0,
                 window: Optional[int] = None):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.lib = host_library()
        self.handle = self.lib.lle_pt_create(num_pages, page_size, max_requests, max_pages_per_request,
                                             -1 if window is None else int(window))
        if not self.handle:
            raise ValueError("page tables need positive sizes")

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            self.lib.lle_pt_destroy(handle)


class PagePool:
    """The free list of a group's pages."""

    def __init__(self, num_pages: int, tables: Optional[PageTables] = None):
        self._tables = tables or PageTables(num_pages)
        self._lib, self._h = self._tables.lib, self._tables.handle
        self.num_pages = num_pages

    @property
    def num_free(self) -> int:
        return self._lib.lle_pt_num_free(self._h)

    @property
    def num_held(self) -> int:
        return self.num_pages - self.num_free

    def allocate(self, n: int) -> List[int]:
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        out = (ctypes.c_int32 * max(1, n))()
        if self._lib.lle_pt_allocate(self._h, n, out) != OK:
            raise OutOfPages(f"not enough free physical blocks: {n} wanted, {self.num_free} free")
        return list(out[:n])

    def release(self, pages: Iterable[int]) -> None:
        pages = [int(p) for p in pages]
        arr = (ctypes.c_int32 * max(1, len(pages)))(*pages)
        bad = ctypes.c_int32(0)
        code = self._lib.lle_pt_release(self._h, arr, len(pages), ctypes.byref(bad))
        if code == NO_SUCH_PAGE:
            raise ValueError(f"page {bad.value} does not exist")
        if code != OK:
            raise ValueError(f"page {bad.value} is given back twice")

    def is_held(self, page: int) -> bool:
        return bool(self._lib.lle_pt_is_held(self._h, int(page)))
