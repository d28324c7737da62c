"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w; the weight multiplies directly,
no bias, no mean subtraction (src/layers/rms_norm.cu:81-93).  The residual add
that precedes a norm in the block is folded into the same kernel."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.spec import INIT_NORM, TensorSpec
from .base import BuildContext, Norm, NormFold


class RMSNorm(Norm):
    def __init__(self, name: str, size: int, eps: float):
        self.name = name
        self.size = size
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.name: TensorSpec((self.size,), INIT_NORM)}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.weight = weights[self.name].contiguous()  # bfloat16 or float32, as stored

    def forward(self, hidden, delta, rows=None) -> torch.Tensor:
        return self.ctx.ops.add_rmsnorm(hidden, delta, self.weight, self.eps, self.ctx.dtype, rows)

    def of_embedding(self, ids, table, step=None):
        if table.dtype != self.ctx.dtype or table.shape[1] != self.size:
            return None
        if step is not None and step.token_feedback is not None:
            return self.ctx.ops.embedding_rmsnorm(ids, table, self.weight, self.eps, step.token_feedback,
                                                  step.token_seq, step.seq_slots)
        return self.ctx.ops.embedding_rmsnorm(ids, table, self.weight, self.eps)

    def fold(self, hidden) -> Optional[NormFold]:
        if not self.ctx.ops.can_fold_norm(hidden.shape[0], self.size, self.ctx.dtype):
            return None
        return NormFold(hidden, self.weight, self.eps)
