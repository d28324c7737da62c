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
from typing import List, Optional, Sequence

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
    max_kv_len: int
    seqs: List[SeqInfo]  # the same on the host


def build_step(entries: Sequence[StepEntry], cache, vocab_size: int, device) -> StepState:
    """Lay the entries out flat, compute every token's page slot in every cache
    group, upload, and apply the new block-table entries.  `cache` is the
    CacheManager; pages for the new lengths must already be there."""
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
        logit_rows.extend(start + int(w) for w in e.want)
        seqs.append(SeqInfo(e.slot, start, n, past))
    N, S, R = len(token_ids), len(seqs), len(logit_rows)

    mappings = []
    for group in cache.groups:
        m: List[int] = []
        P = group.page_size
        for q in seqs:
            table = group.tables[q.slot]
            for pos in range(q.past_len, q.past_len + q.q_len):
                m.append(table[pos // P] * P + pos % P)
        mappings.append(m)
    updates = cache.take_table_updates()

    flat: List[int] = token_ids + positions + token_seq + seq_slots + cu_tokens + kv_lens + logit_rows
    for m in mappings:
        flat += m
    for _, idx, pages in updates:
        flat += idx
        flat += pages
    buf = torch.tensor(flat, dtype=torch.int32).to(device)

    off = 0

    def take(n: int) -> torch.Tensor:
        nonlocal off
        v = buf[off : off + n]
        off += n
        return v

    state = StepState(
        num_tokens=N,
        num_seqs=S,
        token_ids=take(N),
        positions=take(N),
        token_seq=take(N),
        seq_slots=take(S),
        cu_tokens=take(S + 1),
        kv_lens=take(S),
        logit_rows=take(R),
        min_q_len=min(q.q_len for q in seqs),
        max_q_len=max(q.q_len for q in seqs),
        max_kv_len=max(kv_lens),
        seqs=seqs,
    )
    for group in cache.groups:
        group.slot_mapping = take(N)
    for g, idx, pages in updates:
        i, p = take(len(idx)), take(len(pages))
        cache.groups[g].apply_table_updates(i, p)
    return state
