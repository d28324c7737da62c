"""Linear projection y = x W^T, W [out, in] row-major, no bias
(src/layers/linear.cu:169-215; Qwen3 uses no bias, src/model/qwen3.cpp:181-205).
Several checkpoint tensors may be stacked along `out` into one product
(q, k, v  /  gate, up), which the reference runs as separate products."""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..weights.spec import INIT_NORMAL, TensorSpec
from .base import BuildContext, Part


class Linear(Part):
    def __init__(self, names: Sequence[str], in_features: int, out_features: Sequence[int], optional: bool = False,
                 to_residual: bool = False):
        """`to_residual`: the result is a delta of the residual stream and goes nowhere but into
        Norm.forward(hidden, delta); it may then come as parts.base.PartialSums (a product taken
        in slices of `in`), which that call adds up."""
        self.names = list(names)
        self.in_features = in_features
        self.out_features = list(out_features)
        self.optional = optional
        self.to_residual = to_residual
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            n: TensorSpec((o, self.in_features), INIT_NORMAL, optional=self.optional)
            for n, o in zip(self.names, self.out_features)
        }

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        parts = [weights[n].to(ctx.dtype) for n in self.names]
        self.weight = parts[0].contiguous() if len(parts) == 1 else torch.cat(parts, dim=0).contiguous()

    def bind_tensor(self, tensor: torch.Tensor, ctx: BuildContext) -> None:
        """Use an existing tensor (a tied output head shares the embedding table)."""
        self.ctx = ctx
        self.weight = tensor

    def forward(self, x, out_dtype=None, fold=None):
        """`x` may be a parts.base.Prenormed; with `fold` (a parts.base.NormFold) the result
        is added into the residual stream and comes back as the Prenormed of that norm."""
        if fold is None:
            if self.to_residual and out_dtype is None:
                return self.ctx.ops.linear(x, self.weight, out_dtype, sums_ok=True)
            return self.ctx.ops.linear(x, self.weight, out_dtype)
        return self.ctx.ops.linear(x, self.weight, out_dtype, fold=fold)
