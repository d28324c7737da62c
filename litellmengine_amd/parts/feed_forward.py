"""Dense gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(src/model/qwen3.cpp:88-105, :143-152; src/ops/silu_and_mul.cu:44-46).  gate and
up are one stacked product here; the activation is computed in 32-bit."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.spec import TensorSpec
from .base import BuildContext, FeedForward
from .linear import Linear


class GatedMLP(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int):
        # the products that do a folded norm's work read their inner dimension eight elements at a time
        self.folds_norm = intermediate_size % 8 == 0
        self.gate_up = Linear(
            [prefix + "gate_proj.weight", prefix + "up_proj.weight"], hidden_size, [intermediate_size] * 2
        )
        self.down = Linear([prefix + "down_proj.weight"], intermediate_size, [hidden_size], to_residual=True)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {**self.gate_up.tensor_specs(), **self.down.tensor_specs()}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.gate_up.bind(weights, ctx)
        self.down.bind(weights, ctx)

    def forward(self, x, fold=None):
        return self.down.forward(self.ctx.ops.gate_up_silu(x, self.gate_up.weight), fold=fold)
