"""Linear projection y = x W^T (+ b), W [out, in] row-major
(src/layers/linear.cu:169-215; Qwen3 uses no bias, src/model/qwen3.cpp:181-205).
Several checkpoint tensors may be stacked along `out` into one product
(q, k, v  /  gate, up), which the reference runs as separate products; a checkpoint
that holds them stacked already is one name with the whole width."""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..weights.spec import INIT_NORMAL, TensorSpec
from .base import BuildContext, Part


class Linear(Part):
    def __init__(self, names: Sequence[str], in_features: int, out_features: Sequence[int], optional: bool = False,
                 to_residual: bool = False, bias_names: Optional[Sequence[str]] = None):
        """`to_residual`: the result is a delta of the residual stream and goes nowhere but into
        Norm.forward(hidden, delta); it may then come as parts.base.PartialSums (a product taken
        in slices of `in`), which that call adds up.  `bias_names`: one bias tensor [out] for every
        weight tensor, added to the product (a projection with a bias takes no part in a folded norm)."""
        self.names = list(names)
        self.in_features = in_features
        self.out_features = list(out_features)
        self.optional = optional
        self.to_residual = to_residual
        self.bias_names = list(bias_names) if bias_names else []
        if self.bias_names and len(self.bias_names) != len(self.names):
            raise ValueError("a bias for every weight tensor, or none")
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    @property
    def has_bias(self) -> bool:
        return bool(self.bias_names)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {
            n: TensorSpec((o, self.in_features), INIT_NORMAL, optional=self.optional)
            for n, o in zip(self.names, self.out_features)
        }
        for n, o in zip(self.bias_names, self.out_features):
            specs[n] = TensorSpec((o,), INIT_NORMAL, optional=self.optional)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        parts = [weights[n].to(ctx.dtype) for n in self.names]
        self.weight = parts[0].contiguous() if len(parts) == 1 else torch.cat(parts, dim=0).contiguous()
        if self.bias_names:
            self.bias = torch.cat([weights[n].to(ctx.dtype).reshape(-1) for n in self.bias_names]).contiguous()

    def bind_tensor(self, tensor: torch.Tensor, ctx: BuildContext) -> None:
        """Use an existing tensor (a tied output head shares the embedding table)."""
        self.ctx = ctx
        self.weight = tensor

    def forward(self, x, out_dtype=None, fold=None):
        """`x` may be a parts.base.Prenormed; with `fold` (a parts.base.NormFold) the result
        is added into the residual stream and comes back as the Prenormed of that norm."""
        ops = self.ctx.ops
        if self.bias is not None:
            if fold is not None:
                raise ValueError("a projection with a bias cannot add into the residual stream for a folded norm")
            return ops.add_bias(ops.linear(x, self.weight, out_dtype), self.bias)
        if fold is None:
            if self.to_residual and out_dtype is None:
                return ops.linear(x, self.weight, out_dtype, sums_ok=True)
            return ops.linear(x, self.weight, out_dtype)
        return ops.linear(x, self.weight, out_dtype, fold=fold)
