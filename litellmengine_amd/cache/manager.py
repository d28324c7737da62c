"""The cache manager: pages of keys and values with a block table per request,
in groups, and slots of fixed-size per-request state.

Reference: ModelPagedKVCache (src/engine/paged_kv_cache.cpp:18-105),
BlockTableManager (src/engine/block_table_manager.cpp:17-274) and
PagedKVCacheManager (src/engine/paged_kv_cache_manager.cpp:9-140).  Kept from
it: one page id serves every layer of its group, all-or-nothing growth
(:60-89), LIFO reuse, `token slot = table[pos / P] * P + pos % P` (:91-122),
no zero-filling of reused pages (lengths say what is valid).  Different:
 * block tables live on the device as one int32 matrix per group, row = request
   slot; only new entries travel (the reference packs and uploads the whole
   table per layer per step, src/ops/attention.cu:959-1020);
 * cache layers with the same needs form a group with pages and tables of its
   own; a group with a window gives pages back as soon as the window has
   passed them;
 * mixers may ask for fixed-size state rows, zeroed at admission.

Pool layout of a group: [layer, page, elements of a page]; a page holds the fields of
the mixers' per-token record one after the other (parts.base.CacheSpec).  For keys and
values that is [layer, page, 2 (K, V), kv_head, page_size, head_dim], V transposed.
"""
from __future__ import annotations

import ctypes
import dataclasses
from array import array
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import CacheSpec, StateSpec
from .page_pool import OK, TOO_MANY_PAGES, OutOfPages, PagePool, PageTables


class _TableView:
    """`group.tables[slot]`: a request slot's block table as a list (a copy of the native one)."""

    def __init__(self, group: "CacheGroup"):
        self._group = group

    def __len__(self) -> int:
        return self._group.max_requests

    def __getitem__(self, slot: int) -> List[int]:
        g = self._group
        if not 0 <= slot < g.max_requests:
            raise IndexError(slot)
        n = g._lib.lle_pt_table_len(g._h, slot)
        out = (ctypes.c_int32 * max(1, n))()
        g._lib.lle_pt_table_copy(g._h, slot, out)
        return list(out[:n])

    def __iter__(self):
        return (self[slot] for slot in range(len(self)))


class CacheGroup:
    """Pages, pool and block tables of the cache layers that share one CacheSpec.  The
    bookkeeping (free list, tables, what has not reached the device table yet) is the native
    host library's; the pool and the device table are tensors held here."""

    def __init__(self, index: int, spec: CacheSpec, cache_ids: Sequence[int], page_size: int, num_pages: int,
                 max_requests: int, max_pages_per_request: int, dtype: torch.dtype, device: torch.device):
        self.index = index
        self.spec = spec
        self.cache_ids = list(cache_ids)
        self.page_size = page_size
        self.window = spec.window
        self.max_requests = max_requests
        self.max_pages_per_request = max_pages_per_request
        self.native = PageTables(num_pages, page_size, max_requests, max_pages_per_request, spec.window)
        self._lib, self._h = self.native.lib, self.native.handle
        self.pool = PagePool(num_pages, self.native)
        # One page more than the pool hands out: page `num_pages` is never written (it stays zero)
        # and is what the spare table row below points at.  A page is flat: the record's fields
        # one after the other, each for all tokens of the page.
        self.page_elems = page_size * spec.elems_per_token
        self.data = torch.zeros((len(self.cache_ids), num_pages + 1, self.page_elems), dtype=dtype, device=device)
        # keys and values in the attention kernels' layout: the same memory as
        # [layer, page, 2 (K, V), kv_head, page_size, head_dim]
        pair = spec.keys_and_values()
        self.kv = None if pair is None else self.data.view(
            len(self.cache_ids), num_pages + 1, 2, pair[0], page_size, pair[1])
        # per request slot: logical page -> physical page (-1 once the window has passed it);
        # row `max_requests` belongs to no request: rows that pad a batch read one key through it
        self.tables = _TableView(self)
        self.block_table = torch.full((max_requests + 1, max_pages_per_request), -1, dtype=torch.int32, device=device)
        self.block_table[max_requests, 0] = num_pages
        self.slot_mapping: Optional[torch.Tensor] = None  # int32 [N] of the step being run

    def pages_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size

    def table_len(self, slot: int) -> int:
        return self._lib.lle_pt_table_len(self._h, slot)

    def new_pages_needed(self, slot: int, new_len: int) -> int:
        return self._lib.lle_pt_new_pages_needed(self._h, slot, new_len)

    def grow(self, slot: int, new_len: int) -> None:
        code = self._lib.lle_pt_grow(self._h, slot, new_len)
        if code == TOO_MANY_PAGES:
            raise OutOfPages(
                f"a request may hold {self.max_pages_per_request} pages of {self.page_size} tokens; "
                f"{new_len} tokens need {self.pages_for(new_len)}"
            )
        if code != OK:
            raise OutOfPages(f"not enough free physical blocks: {self.pool.num_free} free")

    def trim(self, slot: int, length: int) -> None:
        """Give back the pages that no later query can see: with a window w the
        next query (position `length`) sees keys >= length - w + 1."""
        self._lib.lle_pt_trim(self._h, slot, length)

    def release(self, slot: int) -> None:
        self._lib.lle_pt_release_slot(self._h, slot)

    def token_slot(self, slot: int, pos: int) -> int:
        where = self._lib.lle_pt_token_slot(self._h, slot, pos)
        if where == -2:
            raise IndexError(f"position {pos} lies in a page that was given back")
        if where < 0:
            raise IndexError(f"position {pos} has no page")
        return where

    def take_pending(self) -> Tuple[List[int], List[int]]:
        """(flat indices into the device table, pages) of entries made since the last call."""
        n = self._lib.lle_pt_num_pending(self._h)
        if n == 0:
            return [], []
        index, pages = (ctypes.c_int32 * n)(), (ctypes.c_int32 * n)()
        self._lib.lle_pt_take_pending(self._h, index, pages)
        latest = dict(zip(index, pages))  # an entry made twice (a slot given back and used again): the later one
        return list(latest.keys()), list(latest.values())

    def apply_table_updates(self, flat_index: torch.Tensor, pages: torch.Tensor) -> None:
        """Write new table entries (int32 device arrays) into the device table."""
        self.block_table.view(-1).index_copy_(0, flat_index.long(), pages)

    def held_pages(self, slot: int) -> List[int]:
        return [p for p in self.tables[slot] if p >= 0]


@dataclasses.dataclass
class LayerCache:
    """What the mixer of one plan entry gets: the pages of its cache layer (`pages`,
    flat [page, elements]; `kv`, the same memory as [page, 2, kv_head, page_size,
    head_dim] when the record is a key/value pair; `field(name)` for any record), its
    group (block table and the step's slot mapping), whether it writes, and its state
    rows [slot, ...]."""

    group: Optional[CacheGroup]
    kv: Optional[torch.Tensor]
    writes: bool
    state: Optional[torch.Tensor]
    pages: Optional[torch.Tensor] = None

    def field(self, name: str) -> torch.Tensor:
        """The pages' share of one field of the record: [page, head, page_size, width], or
        [page, head, width, page_size] for a transposed field (a view, no copy)."""
        group = self.group
        at = 0
        for f in group.spec.fields:
            n = f.elems_per_token * group.page_size
            if f.name == name:
                shape = (f.num_heads, f.width, group.page_size) if f.transposed else (f.num_heads, group.page_size, f.width)
                return self.pages[:, at : at + n].unflatten(1, shape)
            at += n
        raise KeyError(f"the cache record has no field {name!r}")


@dataclasses.dataclass(frozen=True)
class GroupSizes:
    """Page size and pool of one cache group, where the caller wants to set them."""

    page_size: Optional[int] = None
    num_pages: Optional[int] = None


class CacheManager:
    def __init__(self, model, *, page_size: int, num_pages: int, max_requests: int,
                 max_pages_per_request: Optional[int] = None, dtype: torch.dtype, device,
                 max_tokens_per_step: Optional[int] = None,
                 group_sizes: Optional[Dict[CacheSpec, GroupSizes]] = None):
        """`model` is a models.decoder.DecoderLM (its plan and mixers say what is needed).
        `page_size` and `num_pages` give the page size and the capacity (num_pages * page_size
        tokens) of a group that asks for nothing else; every group has a page size and a pool
        of its own:
          * page size: `group_sizes[spec].page_size`, else the spec's own, else `page_size`;
          * pool: `group_sizes[spec].num_pages`, else pages for the same number of tokens; a
            group with a window needs no more than the window and one step's tokens per
            request, and is sized so when `max_tokens_per_step` says how long a step may be
            (the reference has one geometry and one pool for all layers,
            src/engine/paged_kv_cache.cpp:26-52).
        `max_pages_per_request` counts pages of `page_size` tokens: the longest request."""
        if page_size <= 0:
            raise ValueError("--page-size must be positive")  # src/main.cpp:62-64
        device = torch.device(device)
        self.page_size = page_size
        self.max_requests = max_requests
        self.pad_slot = max_requests  # the table row (of every group) that padding rows of a batch read
        self.device = device
        self.dtype = dtype
        max_pages_per_request = max_pages_per_request or num_pages
        capacity, longest = num_pages * page_size, max_pages_per_request * page_size

        by_spec: Dict[CacheSpec, List[int]] = {}
        for cache_id, mixer in sorted(model.cache_layers().items()):
            spec = mixer.cache_spec()
            if spec is not None:
                by_spec.setdefault(spec, []).append(cache_id)
        self.groups: List[CacheGroup] = []
        for g, (spec, ids) in enumerate(by_spec.items()):
            asked = (group_sizes or {}).get(spec, GroupSizes())
            P = asked.page_size or spec.page_size or page_size
            if P <= 0:
                raise ValueError("a group's page size must be positive")
            pages = asked.num_pages
            if pages is None:
                pages = -(-capacity // P)
                if spec.window is not None and max_tokens_per_step is not None:
                    # positions past - window + 1 .. past + step - 1 of a request, wherever they start in a page
                    each = -(-(spec.window - 1 + max_tokens_per_step) // P) + 1
                    pages = min(pages, max_requests * each)
            self.groups.append(CacheGroup(g, spec, ids, P, pages, max_requests, -(-longest // P), dtype, device))
        where: Dict[int, Tuple[CacheGroup, int]] = {}
        for group in self.groups:
            for n, cache_id in enumerate(group.cache_ids):
                where[cache_id] = (group, n)

        # state rows belong to a cache id too: every entry that names it shares them; row `pad_slot`
        # (one more than there are request slots) belongs to nobody: the rows that pad a batch use it
        self.states: Dict[int, torch.Tensor] = {}
        self._layers: List[LayerCache] = []
        for entry in model.plan:
            mixer = model.blocks[entry.block].mixer
            sspec: Optional[StateSpec] = mixer.state_spec()
            if sspec is not None and entry.cache not in self.states:
                self.states[entry.cache] = torch.zeros((max_requests + 1,) + tuple(sspec.shape), dtype=sspec.dtype, device=device)
            group, n = where.get(entry.cache, (None, 0))
            self._layers.append(
                LayerCache(group, None if group is None or group.kv is None else group.kv[n], entry.writes,
                           self.states.get(entry.cache), None if group is None else group.data[n])
            )

        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        self._live = bytearray(max_requests)
        self._length: List[int] = [0] * max_requests

    # -- request slots -----------------------------------------------------------
    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self) -> int:
        """A slot for a new request: empty tables, length 0, state rows zeroed."""
        if not self._free_slots:
            raise OutOfPages("no free request slot")
        slot = self._free_slots.pop()
        self._live[slot] = 1
        self._length[slot] = 0
        for state in self.states.values():
            state[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        """Give back everything the request holds (pages of every group, its slot)."""
        self._check_live(slot)
        for group in self.groups:
            group.release(slot)
        self._live[slot] = 0
        self._length[slot] = 0
        self._free_slots.append(slot)

    def is_live(self, slot: int) -> bool:
        return 0 <= slot < self.max_requests and bool(self._live[slot])

    def length(self, slot: int) -> int:
        self._check_live(slot)
        return self._length[slot]

    def lengths_of(self, slots: Sequence[int]) -> List[int]:
        """length() of every slot in `slots` (all must be in use)."""
        live, length, most = self._live, self._length, self.max_requests
        for slot in slots:
            if not (0 <= slot < most and live[slot]):
                raise ValueError(f"request slot {slot} is not in use")
        return [length[slot] for slot in slots]

    def _check_live(self, slot: int) -> None:
        if not self.is_live(slot):
            raise ValueError(f"request slot {slot} is not in use")

    # -- pages -----------------------------------------------------------------------
    @staticmethod
    def _arrays(wants: Sequence[Tuple[int, int]]):
        slots, lens = array("i", (w[0] for w in wants)), array("i", (w[1] for w in wants))
        return len(wants), slots.buffer_info()[0], lens.buffer_info()[0], (slots, lens)

    def _can_extend(self, n: int, slots: int, lens: int) -> bool:
        for group in self.groups:
            need = group._lib.lle_pt_pages_needed_many(group._h, n, slots, lens)
            if need < 0 or need > group.pool.num_free:
                return False
        return True

    def can_extend(self, wants: Sequence[Tuple[int, int]]) -> bool:
        """Would `extend_many(wants)` succeed?  wants = [(slot, new_len), ...]."""
        n, slots, lens, keep = self._arrays(wants)
        return self._can_extend(n, slots, lens)

    def extend_many(self, wants: Sequence[Tuple[int, int]]) -> None:
        """Make room for positions < new_len of every (slot, new_len): all or nothing."""
        for slot, new_len in wants:
            self._check_live(slot)
            if new_len < self._length[slot]:
                raise ValueError("a request cannot shrink")
        n, slots, lens, keep = self._arrays(wants)
        if not self._can_extend(n, slots, lens):
            free = ", ".join(f"group {g.index}: {g.pool.num_free}" for g in self.groups)
            raise OutOfPages(f"not enough free physical blocks for this step (free pages: {free})")
        for group in self.groups:
            if group._lib.lle_pt_grow_many(group._h, n, slots, lens) != OK:
                raise RuntimeError("the pages of a group changed between the check and the growth")

    def extend(self, slot: int, new_len: int) -> None:
        self.extend_many([(slot, new_len)])

    def shrink_many(self, wants: Sequence[Tuple[int, int]]) -> None:
        """Undo an extend_many whose step did not happen: wants = [(slot, the length that is
        committed), ...]; the pages beyond those lengths go back, last taken first."""
        for slot, length in wants:
            self._check_live(slot)
            if length != self._length[slot]:
                raise ValueError("a request shrinks back to its committed length only")
        n, slots, lens, keep = self._arrays(wants)
        for group in self.groups:
            group._lib.lle_pt_shrink_many(group._h, n, slots, lens)

    def commit(self, slot: int, new_len: int) -> None:
        """The positions < new_len are now written; windows move on."""
        self._check_live(slot)
        self._length[slot] = new_len
        for group in self.groups:
            if group.window is not None:
                group.trim(slot, new_len)

    def commit_many(self, wants: Sequence[Tuple[int, int]]) -> None:
        """commit() for every (slot, new_len) of a step."""
        for slot, new_len in wants:
            self._check_live(slot)
            self._length[slot] = new_len
        if any(group.window is not None for group in self.groups):
            n, slots, lens, keep = self._arrays(wants)
            for group in self.groups:
                group._lib.lle_pt_trim_many(group._h, n, slots, lens)

    def shortfall(self, wants: Sequence[Tuple[int, int]]) -> List[int]:
        """Per group: pages that `extend_many(wants)` needs minus the free ones (<= 0: they are there)."""
        n, slots, lens, keep = self._arrays(wants)
        out = []
        for group in self.groups:
            need = group._lib.lle_pt_pages_needed_many(group._h, n, slots, lens) if n else 0
            out.append((group.pool.num_pages + 1 if need < 0 else need) - group.pool.num_free)
        return out

    def pages_held(self, slot: int) -> List[int]:
        """Pages per group that the request in `slot` holds."""
        self._check_live(slot)
        return [len(g.held_pages(slot)) for g in self.groups]

    def free_pages(self) -> List[int]:
        return [g.pool.num_free for g in self.groups]

    def pages_needed(self, slot: Optional[int], new_len: int) -> List[int]:
        """New pages per group that growing `slot` (None: a fresh request) to new_len takes."""
        return [
            g.pages_for(new_len) if slot is None else g.new_pages_needed(slot, new_len) for g in self.groups
        ]

    # -- what a step needs ---------------------------------------------------------------
    def layer(self, plan_index: int) -> LayerCache:
        return self._layers[plan_index]

    def take_table_updates(self):
        """[(group index, flat indices, pages)] of table entries not yet on the device."""
        out = []
        for g in self.groups:
            index, pages = g.take_pending()
            if index:
                out.append((g.index, index, pages))
        return out
