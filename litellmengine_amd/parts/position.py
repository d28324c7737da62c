"""Position encodings applied to q and k inside a mixer."""
from __future__ import annotations

from typing import Optional

import torch

from .base import BuildContext, PositionEncoding


class RotaryHalfSplit(PositionEncoding):
    """Rotary encoding with half-split pairing: element i pairs with i + rot/2,
    inv_freq_i = theta^(-2i/rot), angle = pos * inv_freq_i
      y[i] = x[i] cos - x[i + rot/2] sin,  y[i + rot/2] = x[i + rot/2] cos + x[i] sin
    (src/layers/rotary.cu:81-83, :96-116; the reference rotates the whole head,
    rot = head_dim, and computes angles on the fly with no table).  The
    frequencies are computed once in double precision and rounded to float32;
    the angle, sine and cosine are float32 in the kernel, computed once per step for
    all heads and layers."""

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError("rotary_dim must be even and within the head")
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        inv = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -(2.0 * i) / self.rotary_dim)
        self.inv_freq = inv.to(torch.float32).to(ctx.device)

    def fused_rotary(self, step):
        # cosines and sines of this step's positions: made by the first layer that asks,
        # shared by every layer with the same rotation
        key = ("rope_table", self.theta, self.rotary_dim)
        table = step.scratch.get(key)
        if table is None:
            table = self.ctx.ops.rope_table(step.positions, self.inv_freq)
            step.scratch[key] = table
        return table, self.rotary_dim


class NoPositionEncoding(PositionEncoding):
    """q and k pass unchanged (a mixer whose order comes from elsewhere)."""

    def fused_rotary(self, step):
        return None, 0
