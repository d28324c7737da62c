"""Pre-norm residual block: r = x + mixer(norm_in(x)); y = r + ff(norm_post(r))
(src/model/qwen3.cpp:948-968).  The adds run inside the norm kernels on the
32-bit residual stream; the last add of a block is left to the next norm."""
from __future__ import annotations

from typing import Dict

from ..weights.spec import TensorSpec
from .base import Block, BuildContext, FeedForward, Mixer, Norm, Normed, Prenormed


class PreNormBlock(Block):
    def __init__(self, norm_in: Norm, mixer: Mixer, norm_post: Norm, feed_forward: FeedForward):
        self.norm_in = norm_in
        self.mixer = mixer
        self.norm_post = norm_post
        self.feed_forward = feed_forward

    def _parts(self):
        return (self.norm_in, self.mixer, self.norm_post, self.feed_forward)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in self._parts():
            p.bind(weights, ctx)

    def entry_norm(self):
        return self.norm_in if self.mixer.folds_norm else None

    def input_norm(self):
        return self.norm_in

    def forward(self, hidden, delta, step, cache, next_norm=None):
        if isinstance(delta, Prenormed):  # made for norm_in by the block before: the add and the norm are done
            x = delta
        elif isinstance(delta, Normed):  # norm_in's result, made together with the rows of `hidden`
            x = delta.x
        else:
            x = self.norm_in.forward(hidden, delta)
        fold = self.norm_post.fold(hidden) if self.mixer.folds_norm and self.feed_forward.folds_norm else None
        if fold is not None:
            x = self.mixer.forward(x, step, cache, fold=fold)
        else:
            x = self.norm_post.forward(hidden, self.mixer.forward(x, step, cache))
        fold = next_norm.fold(hidden) if next_norm is not None and self.feed_forward.folds_norm else None
        if fold is not None:
            return self.feed_forward.forward(x, fold=fold)
        return self.feed_forward.forward(x)
