"""The batch of one step, as the kernels see it.

One step runs a flat list of tokens: for each request its next tokens (a
portion of its prompt, or one decoded token), cut anywhere.  The reference
splits this into two forwards that cannot be mixed (one request with T tokens
and no past, or B single tokens; include/runtime/forward_context.hpp:16-48);
here one description covers both.  All integer arrays of a step travel to the
device in ONE copy and are views of that buffer.
"""
from __future__ import annotations

import ctypes
import dataclasses
from array import array
from typing import List, NamedTuple, Optional, Sequence, Tuple

import torch

from ..cache.page_pool import BAD_TOKEN, NO_PAGE_AT_POSITION, host_library


class StepEntry(NamedTuple):
    """A request's share of a step: its cache slot, its next tokens and the
    places among them (0-based) whose logits are wanted."""

    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


class SeqInfo(NamedTuple):
    slot: int
    q_start: int  # first row of the request in the flat batch
    q_len: int
    past_len: int  # tokens already in the cache before this step


@dataclasses.dataclass
class StepState:
    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor  # int32 [N]
    positions: torch.Tensor  # int32 [N] position of each token in its request
    token_seq: torch.Tensor  # int32 [N] index of the token's request in this batch
    seq_slots: torch.Tensor  # int32 [S] cache slot (block-table row) of each request
    cu_tokens: torch.Tensor  # int32 [S + 1] first row of each request, then N
    kv_lens: torch.Tensor  # int32 [S] cached length of each request after this step
    logit_rows: torch.Tensor  # int32 [R] rows whose logits are wanted
    every_row_wanted: bool  # logit_rows is 0 .. N - 1 in order (known on the host)
    min_q_len: int
    max_q_len: int
    max_kv_len: int  # host-side bounds; they choose kernels, never results
    seqs: Optional[List[SeqInfo]]  # the same on the host (None inside a captured graph)
    scratch: dict = dataclasses.field(default_factory=dict)  # what parts make once per step and share
    # int32, indexed by request slot: the token that the step before picked for a request, left on the
    # device; a token id of -1 in `token_ids` stands for it (None: every id of the step is given)
    token_feedback: Optional[torch.Tensor] = None


@dataclasses.dataclass
class StepLayout:
    """The host side of a step: one flat int32 tensor and where its parts lie."""

    host: torch.Tensor  # int32, on the host (pinned when the step runs on a GPU)
    num_tokens: int
    num_seqs: int
    num_logit_rows: int
    num_groups: int
    seqs: Optional[List[SeqInfo]]  # None when the caller asked for none
    max_kv_len: int
    q_lens: Tuple[int, int] = (1, 1)  # fewest and most tokens of a request in this step
    every_row_wanted: bool = False  # the wanted rows are all rows, in order

    def sizes(self) -> List[int]:
        N, S, R = self.num_tokens, self.num_seqs, self.num_logit_rows
        return [N, N, N, S, S + 1, S, R] + [N] * self.num_groups


class _Staging:
    """Host buffers that the native layout writes into: pinned (page-locked) when a GPU will
    read them, grown as needed and used again.  Three take turns: a step may be laid out while
    the copy of the step before it to the device has not run yet (steps that are launched
    ahead of the host's reading of their predecessor), and whoever launches ahead waits for
    step k before laying out step k + 2."""

    TURNS = 3

    def __init__(self):
        self.buffers = {}
        self.copied = {}  # buffer -> event after the last copy out of it that was put on a stream
        self.turn = 0
        self.key = None

    def get(self, n: int, pinned: bool) -> torch.Tensor:
        self.turn = (self.turn + 1) % self.TURNS
        key = self.key = (pinned, self.turn)
        done = self.copied.pop(key, None)
        if done is not None:
            done.synchronize()  # (long past, unless the caller put three steps on the stream without ever waiting)
        buf = self.buffers.get(key)
        if buf is None or buf.numel() < n:
            size = max(1024, 1 << (max(1, n) - 1).bit_length())
            buf = torch.empty(size, dtype=torch.int32, pin_memory=pinned)
            self.buffers[key] = buf
        return buf[:n]

    def copy_enqueued(self) -> None:
        """The buffer handed out last has a copy to the device waiting on the current stream."""
        if self.key is not None and self.key[0]:
            event = torch.cuda.Event()
            event.record()
            self.copied[self.key] = event


_staging = _Staging()
_update_staging = _Staging()


def layout_step(entries: Sequence[StepEntry], cache, all_rows: bool = False, vocab_size: int = 0,
                device=None, pad_to: int = 0, with_seqs: bool = True, allow_deferred: bool = False) -> StepLayout:
    """Lay the entries out flat and compute every token's page slot in every cache
    group (csrc/host.cpp does both).  Pages for the new lengths must already be there.
    `all_rows` asks for the logits of every row whatever the entries want; with
    `vocab_size` token ids outside [0, vocab_size) are refused.  `pad_to` fills the batch
    up to that many requests with single tokens that stand for nobody: they read the
    cache's spare table row and page (`cache.pad_slot`) and write nothing.  Without
    `with_seqs` the host-side list of the requests is left out (a step that runs as a graph
    has no use for it, and it costs as much as everything else here).  With `allow_deferred` a
    token id of -1 is let through: it stands for the token that is still on the device
    (StepState.token_feedback)."""
    S = len(entries)
    pad = max(0, pad_to - S)
    slots = array("i", [e.slot for e in entries])
    lengths = cache.lengths_of(slots)
    past = array("i", lengths)
    q_len = array("i", [len(e.tokens) for e in entries])
    tokens = array("i")
    rows = array("i")
    seqs: Optional[List[SeqInfo]] = [] if with_seqs else None
    start = 0
    if all_rows and max(q_len, default=1) == 1:  # single tokens: row i is request i's
        for e in entries:
            tokens.extend(e.tokens if isinstance(e.tokens, (list, array)) else [int(t) for t in e.tokens])
        start = S
        rows.extend(range(S))
        if with_seqs:
            seqs.extend(SeqInfo(e.slot, i, 1, p) for i, (e, p) in enumerate(zip(entries, past)))
    else:
        for e, p, n in zip(entries, past, q_len):
            tokens.extend(e.tokens if isinstance(e.tokens, (list, array)) else [int(t) for t in e.tokens])
            if all_rows:
                rows.extend(range(start, start + n))
            else:
                rows.extend(start + int(w) for w in e.want)
            if with_seqs:
                seqs.append(SeqInfo(e.slot, start, n, p))
            start += n
    N, G = start, len(cache.groups)
    if pad:
        if all_rows:
            rows.extend(range(N, N + pad))
        if with_seqs:
            seqs.extend(SeqInfo(cache.pad_slot, N + i, 1, 0) for i in range(pad))
    R = len(rows)
    every_row = all_rows or (R == N + pad and all(r == i for i, r in enumerate(rows)))
    pinned = device is not None and torch.device(device).type == "cuda"
    host = _staging.get(3 * (N + pad) + 3 * (S + pad) + 1 + R + G * (N + pad), pinned)
    lib = host_library()
    handles = (ctypes.c_void_p * max(1, G))(*[g.native.handle for g in cache.groups])
    info = ctypes.c_int64(0)
    address = lambda a: a.buffer_info()[0]
    code = lib.lle_layout_step(S, address(slots), address(past), address(q_len), address(tokens), int(vocab_size),
                               int(allow_deferred), R, address(rows), G, handles, pad, cache.pad_slot if pad else 0,
                               host.data_ptr(), ctypes.byref(info))
    if code == BAD_TOKEN:
        raise ValueError(f"token id {tokens[info.value]} outside [0, {vocab_size})")
    if code == NO_PAGE_AT_POSITION:
        raise IndexError(f"position {info.value} has no page: the cache was not extended for this step")
    if code != 0:
        raise ValueError(f"the step cannot be laid out: {lib.lle_error_string(code).decode()} (at {info.value})")
    q_lens = (min(q_len, default=1) if not pad else 1, max(q_len, default=1))
    return StepLayout(host, N + pad, S + pad, R, G, seqs, max((p + n for p, n in zip(past, q_len)), default=1), q_lens,
                      every_row)


def views_of(buf: torch.Tensor, sizes: Sequence[int]) -> List[torch.Tensor]:
    out, off = [], 0
    for n in sizes:
        out.append(buf[off : off + n])
        off += n
    return out


def apply_table_updates(cache, device) -> None:
    """Send the block-table entries made since the last step to the device tables (through a
    pinned buffer and a copy that does not wait for the work already on the stream)."""
    updates = cache.take_table_updates()
    if not updates:
        return
    flat: List[int] = []
    for _, idx, pages in updates:
        flat += idx
        flat += pages
    if torch.device(device).type == "cuda":
        host = _update_staging.get(len(flat), True)
        host.copy_(torch.tensor(flat, dtype=torch.int32))
        buf = host.to(device, non_blocking=True)  # a few entries a step
        _update_staging.copy_enqueued()
    else:
        buf = torch.tensor(flat, dtype=torch.int32)
    off = 0
    for g, idx, pages in updates:
        n = len(idx)
        cache.groups[g].apply_table_updates(buf[off : off + n], buf[off + n : off + 2 * n])
        off += 2 * n


def state_on(buf: torch.Tensor, layout: StepLayout, cache, max_kv_len: Optional[int] = None,
             with_seqs: bool = True, token_feedback: Optional[torch.Tensor] = None) -> StepState:
    """A StepState whose arrays are views of `buf` (which holds, or will hold,
    layout.flat); also points every cache group's slot mapping into it."""
    v = views_of(buf, layout.sizes())
    for group, mapping in zip(cache.groups, v[7:]):
        group.slot_mapping = mapping
    return StepState(
        num_tokens=layout.num_tokens, num_seqs=layout.num_seqs, token_ids=v[0], positions=v[1], token_seq=v[2],
        seq_slots=v[3], cu_tokens=v[4], kv_lens=v[5], logit_rows=v[6],
        every_row_wanted=layout.every_row_wanted,
        min_q_len=layout.q_lens[0], max_q_len=layout.q_lens[1],
        max_kv_len=max_kv_len or layout.max_kv_len, seqs=layout.seqs if with_seqs else None,
        token_feedback=token_feedback,
    )


def build_step(entries: Sequence[StepEntry], cache, device, vocab_size: int = 0, all_rows: bool = False,
               token_feedback: Optional[torch.Tensor] = None) -> StepState:
    """Layout, one upload, views; also sends new block-table entries."""
    layout = layout_step(entries, cache, all_rows=all_rows, vocab_size=vocab_size, device=device,
                         allow_deferred=token_feedback is not None)
    apply_table_updates(cache, device)
    on_gpu = torch.device(device).type != "cpu"
    buf = layout.host.to(device, non_blocking=True) if on_gpu else layout.host.clone()
    if on_gpu:
        _staging.copy_enqueued()
    return state_on(buf, layout, cache, token_feedback=token_feedback)
