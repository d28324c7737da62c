"""A decoder language model as data: an embedding, a set of blocks, the list
that says in which order they run (and with which cache), a final norm and an
output head.

The reference hard-wires embed -> layer 0..L-1 -> norm -> lm_head on all rows
(src/model/qwen3.cpp:1242-1278, :1501).  Here the order is a list of
`PlanEntry`: an entry may name a block that another entry names too (the
block's weights are then shared and it runs twice), and an entry may read the
cache that another entry writes instead of owning one.  The head runs on the
wanted rows only.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence

import torch

from ..parts.base import Block, BuildContext, Norm, Prenormed
from ..parts.embedding import Embedding
from ..parts.linear import Linear
from ..weights.spec import TensorSpec


@dataclasses.dataclass(frozen=True)
class PlanEntry:
    """One call of a block.  `cache` names the cache layer the mixer works on
    (default: one of its own, numbered like the entry); `writes=False` makes the
    entry a reader of a cache that an earlier entry fills."""

    block: int
    cache: Optional[int] = None
    writes: bool = True


class DecoderLM:
    def __init__(
        self,
        config,
        embedding: Embedding,
        blocks: Sequence[Block],
        plan: Sequence[PlanEntry],
        final_norm: Norm,
        head: Linear,
        tied_head: bool,
    ):
        self.config = config
        self.embedding = embedding
        self.blocks = list(blocks)
        self.plan = [
            PlanEntry(e.block, i if e.cache is None else e.cache, e.writes) for i, e in enumerate(plan)
        ]
        self.final_norm = final_norm
        self.head = head
        self.tied_head = tied_head
        writers = {e.cache for e in self.plan if e.writes}
        for e in self.plan:
            if not 0 <= e.block < len(self.blocks):
                raise ValueError(f"plan names block {e.block}, the model has {len(self.blocks)}")
            if not e.writes and e.cache not in writers:
                raise ValueError(f"plan entry reads cache {e.cache} that no entry writes")

    # -- structure ---------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.embedding.vocab_size

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = dict(self.embedding.tensor_specs())
        for b in self.blocks:
            specs.update(b.tensor_specs())
        specs.update(self.final_norm.tensor_specs())
        specs.update(self.head.tensor_specs())
        return specs

    def cache_layers(self):
        """cache id -> the mixer that defines its needs (the writer)."""
        out = {}
        for e in self.plan:
            if e.writes:
                mixer = self.blocks[e.block].mixer
                if e.cache in out and out[e.cache] is not mixer:
                    raise ValueError(f"two different mixers write cache {e.cache}")
                out[e.cache] = mixer
        return out

    # -- weights -------------------------------------------------------------
    def bind(self, weights: Dict[str, torch.Tensor], ctx: BuildContext) -> None:
        self.ctx = ctx
        self.embedding.bind(weights, ctx)
        for b in self.blocks:
            b.bind(weights, ctx)
        self.final_norm.bind(weights, ctx)
        head_name = self.head.names[0]
        if head_name in weights:
            self.head.bind(weights, ctx)
        elif self.tied_head:
            self.head.bind_tensor(self.embedding.weight, ctx)
        else:
            raise KeyError(head_name)

    # -- one step --------------------------------------------------------------
    def forward(self, step, caches) -> torch.Tensor:
        """Run the tokens of `step` (engine.batch.StepState) through the plan and
        return float32 logits [len(step.logit_rows), vocab]."""
        step.scratch.clear()  # per-step tables are made anew in every run (also when a graph is captured)
        first_norm = self.blocks[self.plan[0].block].input_norm() if self.plan else None
        if first_norm is not None:
            hidden, delta = self.embedding.forward(step.token_ids, step, norm=first_norm)
        else:
            hidden, delta = self.embedding.forward(step.token_ids, step), None
        last = len(self.plan) - 1
        for i, e in enumerate(self.plan):
            # the norm that the next block starts with, if the products around it may do its work
            if i < last:
                next_norm = self.blocks[self.plan[i + 1].block].entry_norm()
            else:  # the final norm, where the head's product can take its place (every row goes to the head)
                next_norm = self.final_norm if step.every_row_wanted and not self.head.has_bias else None
            delta = self.blocks[e.block].forward(hidden, delta, step, caches.layer(i), next_norm=next_norm)
        if step.logit_rows.shape[0] == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=hidden.device)
        x = delta if isinstance(delta, Prenormed) else self.final_norm.forward(hidden, delta, rows=step.logit_rows)
        return self.head.forward(x, out_dtype=torch.float32)
