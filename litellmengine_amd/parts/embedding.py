"""Token embedding: h[t, :] = E[ids[t], :] (src/layers/embedding.cu:75-87); the
rows leave as float32, the type of the residual stream."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.spec import INIT_NORMAL, TensorSpec
from .base import BuildContext, Normed, Part


class Embedding(Part):
    def __init__(self, name: str, vocab_size: int, hidden_size: int):
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.name: TensorSpec((self.vocab_size, self.hidden_size), INIT_NORMAL)}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.weight = weights[self.name].to(ctx.dtype).contiguous()

    def forward(self, ids: torch.Tensor, step=None, norm=None):
        """`step` (engine.batch.StepState): where it carries `token_feedback`, ids below zero are
        the tokens that the step before left on the device for their requests.  With `norm` (the
        parts.base.Norm that the first block begins with) the result is (rows, Normed or None):
        the norm's result comes along where one kernel makes both."""
        if norm is not None:
            both = norm.of_embedding(ids, self.weight, step)
            if both is not None:
                return both[0], Normed(both[1])
            return self.forward(ids, step), None
        if step is not None and step.token_feedback is not None:
            return self.ctx.ops.embedding(ids, self.weight, step.token_feedback, step.token_seq, step.seq_slots)
        return self.ctx.ops.embedding(ids, self.weight)
