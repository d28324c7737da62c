"""The step function: one batch of (request, its next tokens) through the model.

The reference's nearest piece is `forward_uncached_chunk_and_sample`
(src/engine/paged_generate_engine.cpp:475-598) for one request and
`decode_batch` (:182-341) for single tokens of several; both return logits of
every row.  `ModelRunner.step` takes any mix, runs only the tokens it is given
from the cache that earlier steps left, and returns float32 logits at the
wanted places only.  Order inside a step as in the reference: the step's K/V
are written to their pages first, then every token attends through the block
table (src/model/qwen3.cpp:464-481 before :498-557).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..cache import CacheManager
from .batch import StepEntry, StepState, build_step


class ModelRunner:
    def __init__(self, model, cache: CacheManager):
        self.model = model
        self.cache = cache
        self.device = cache.device
        self.vocab_size = model.vocab_size
        self.last_step: Optional[StepState] = None

    # requests ------------------------------------------------------------------
    def admit(self) -> int:
        return self.cache.admit()

    def release(self, slot: int) -> None:
        self.cache.release(slot)

    # one step -----------------------------------------------------------------------
    def check(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        for e in entries:
            if e.slot in seen:
                raise ValueError(f"request slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            if not self.cache.is_live(e.slot):
                raise ValueError(f"request slot {e.slot} is not in use")
            if len(e.tokens) == 0:
                raise ValueError("an entry needs at least one token")
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    raise ValueError(f"token id {t} outside [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"wanted place {w} outside the entry's {len(e.tokens)} tokens")

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run the entries as one batch.  Returns float32 logits [wanted, vocab] in
        the order of the entries and of their `want`.  Raises cache.OutOfPages,
        with nothing changed, when the pages for this step are not there."""
        self.check(entries)
        cache = self.cache
        wants = [(e.slot, cache.length(e.slot) + len(e.tokens)) for e in entries]
        cache.extend_many(wants)
        state = build_step(entries, cache, self.vocab_size, self.device)
        self.last_step = state
        logits = self.model.forward(state, cache)
        for slot, new_len in wants:
            cache.commit(slot, new_len)
        return logits
