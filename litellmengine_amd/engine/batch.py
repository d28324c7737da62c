"""The batch of one step, as the kernels see it.

One step runs a flat list of tokens: for each request its next tokens (a
portion of its prompt, or one decoded token), cut anywhere.  The reference
splits this into two forwards that cannot be mixed (one request with T tokens
and no past, or B single tokens; include/runtime/forward_context.hpp:16-48);
here one description covers both.  All integer arrays of a step travel to the
device in ONE copy and are views of that buffer.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence, Tuple

import torch


@dataclasses.dataclass(frozen=True)
class StepEntry:
    """A request's share of a step: its cache slot, its next tokens and the
    places among them (0-based) whose logits are wanted."""

    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclasses.dataclass(frozen=True)
class SeqInfo:
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
    min_q_len: int
    max_q_len: int
    max_kv_len: int  # host-side bounds; they choose kernels, never results
    seqs: Optional[List[SeqInfo]]  # the same on the host (None inside a captured graph)
    scratch: dict = dataclasses.field(default_factory=dict)  # what parts make once per step and share


@dataclasses.dataclass
class StepLayout:
    """The host side of a step: one flat int32 list and where its parts lie."""

    flat: List[int]
    num_tokens: int
    num_seqs: int
    num_logit_rows: int
    num_groups: int
    seqs: List[SeqInfo]
    max_kv_len: int

    def sizes(self) -> List[int]:
        N, S, R = self.num_tokens, self.num_seqs, self.num_logit_rows
        return [N, N, N, S, S + 1, S, R] + [N] * self.num_groups


def layout_step(entries: Sequence[StepEntry], cache, all_rows: bool = False) -> StepLayout:
    """Lay the entries out flat and compute every token's page slot in every cache
    group.  Pages for the new lengths must already be there.  `all_rows` asks for
    the logits of every row whatever the entries want."""
    token_ids: List[int] = []
    positions: List[int] = []
    token_seq: List[int] = []
    seq_slots: List[int] = []
    cu_tokens: List[int] = [0]
    kv_lens: List[int] = []
    logit_rows: List[int] = []
    seqs: List[SeqInfo] = []
    for s, e in enumerate(entries):
        past = cache.length(e.slot)
        n = len(e.tokens)
        start = len(token_ids)
        token_ids.extend(int(t) for t in e.tokens)
        positions.extend(range(past, past + n))
        token_seq.extend([s] * n)
        seq_slots.append(e.slot)
        cu_tokens.append(start + n)
        kv_lens.append(past + n)
        if all_rows:
            logit_rows.extend(range(start, start + n))
        else:
            logit_rows.extend(start + int(w) for w in e.want)
        seqs.append(SeqInfo(e.slot, start, n, past))
    flat: List[int] = token_ids + positions + token_seq + seq_slots + cu_tokens + kv_lens + logit_rows
    for group in cache.groups:
        P = group.page_size
        for q in seqs:
            table = group.tables[q.slot]
            flat.extend(table[pos // P] * P + pos % P for pos in range(q.past_len, q.past_len + q.q_len))
    return StepLayout(flat, len(token_ids), len(seqs), len(logit_rows), len(cache.groups), seqs, max(kv_lens))


def views_of(buf: torch.Tensor, sizes: Sequence[int]) -> List[torch.Tensor]:
    out, off = [], 0
    for n in sizes:
        out.append(buf[off : off + n])
        off += n
    return out


def apply_table_updates(cache, device) -> None:
    """Send the block-table entries made since the last step to the device tables."""
    updates = cache.take_table_updates()
    if not updates:
        return
    flat: List[int] = []
    for _, idx, pages in updates:
        flat += idx
        flat += pages
    buf = torch.tensor(flat, dtype=torch.int32).to(device)
    off = 0
    for g, idx, pages in updates:
        n = len(idx)
        cache.groups[g].apply_table_updates(buf[off : off + n], buf[off + n : off + 2 * n])
        off += 2 * n


def state_on(buf: torch.Tensor, layout: StepLayout, cache, max_kv_len: Optional[int] = None,
             with_seqs: bool = True) -> StepState:
    """A StepState whose arrays are views of `buf` (which holds, or will hold,
    layout.flat); also points every cache group's slot mapping into it."""
    v = views_of(buf, layout.sizes())
    for group, mapping in zip(cache.groups, v[7:]):
        group.slot_mapping = mapping
    return StepState(
        num_tokens=layout.num_tokens, num_seqs=layout.num_seqs, token_ids=v[0], positions=v[1], token_seq=v[2],
        seq_slots=v[3], cu_tokens=v[4], kv_lens=v[5], logit_rows=v[6],
        min_q_len=min(q.q_len for q in layout.seqs), max_q_len=max(q.q_len for q in layout.seqs),
        max_kv_len=max_kv_len or layout.max_kv_len, seqs=layout.seqs if with_seqs else None,
    )


def build_step(entries: Sequence[StepEntry], cache, device) -> StepState:
    """Layout, one upload, views; also sends new block-table entries."""
    layout = layout_step(entries, cache)
    apply_table_updates(cache, device)
    buf = torch.tensor(layout.flat, dtype=torch.int32).to(device)
    return state_on(buf, layout, cache)
