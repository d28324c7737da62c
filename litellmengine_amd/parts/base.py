"""Interfaces of the parts a model is put together from.

A part knows its own sizes and constants (given as parameters when it is made)
and the names of its tensors; it never knows which model it sits in.  Parts are
made without touching memory; `bind` hands them their tensors, and `forward`
runs them on the flat token batch of one step.

To add a part of some kind, subclass the matching interface below and use it
from an architecture's builder; nothing else in the package refers to the
concrete classes.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple

import torch

from ..weights.spec import TensorSpec


@dataclasses.dataclass
class BuildContext:
    """Where and how a model is materialised."""

    dtype: torch.dtype  # activation/weight type: torch.bfloat16 or torch.float32
    device: torch.device
    ops: Any  # the kernel operations (csrc.ops.HipOps)


@dataclasses.dataclass(frozen=True)
class CacheField:
    """One named part of what a mixer keeps per token: `num_heads` vectors of `width`
    elements.  Inside a page the vectors of a head lie token after token
    ([head][token][width]) or, `transposed`, element after element ([head][width][token])."""

    name: str
    num_heads: int
    width: int
    transposed: bool = False

    @property
    def elems_per_token(self) -> int:
        return self.num_heads * self.width


@dataclasses.dataclass(frozen=True)
class CacheSpec:
    """Per-token cache need of a mixer: a record of named fields for every token.  A page
    holds the fields one after the other, each for all of the page's tokens.  With a
    `window` only the last `window` positions stay needed and pages behind it are given back.
    `page_size`: tokens per page, if the mixer's kernels want a size of their own (None: the
    engine's).  Mixers with equal specs share a group of pages and block tables; every group
    has a page size and a pool of its own."""

    fields: Tuple[CacheField, ...]
    window: Optional[int] = None
    page_size: Optional[int] = None

    def __post_init__(self):
        names = [f.name for f in self.fields]
        if not names or len(set(names)) != len(names):
            raise ValueError("a cache record needs at least one field, and every field a name of its own")
        for f in self.fields:
            if f.num_heads <= 0 or f.width <= 0:
                raise ValueError(f"cache field {f.name!r} needs positive sizes")
        if self.page_size is not None and self.page_size <= 0:
            raise ValueError("a cache record's page size must be positive")

    @property
    def elems_per_token(self) -> int:
        return sum(f.elems_per_token for f in self.fields)

    def keys_and_values(self) -> Optional[Tuple[int, int]]:
        """(kv heads, head size) if the record is the pair that the attention kernels read:
        keys token after token, then values transposed, of the same shape; else None."""
        if len(self.fields) != 2:
            return None
        k, v = self.fields
        if k.transposed or not v.transposed or (k.num_heads, k.width) != (v.num_heads, v.width):
            return None
        return k.num_heads, k.width


def KVCacheSpec(num_kv_heads: int, head_dim: int, window: Optional[int] = None,
                page_size: Optional[int] = None) -> CacheSpec:
    """Keys and values of `num_kv_heads` heads of `head_dim`, in the layout the attention
    kernels read: K as [head][token][d], V transposed as [head][d][token]."""
    return CacheSpec((CacheField("k", num_kv_heads, head_dim), CacheField("v", num_kv_heads, head_dim, True)), window,
                     page_size)


@dataclasses.dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state of a mixer (zeroed when a request is admitted).  The state
    tensor has one row per request slot and one more, which belongs to nobody: rows that pad a
    decode batch to a graph's size name it in `step.seq_slots`, and what they leave there is
    never read by a request."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Checkpoint tensors of this part, by full name."""
        return {}

    def bind(self, weights: Dict[str, torch.Tensor], ctx: BuildContext) -> None:
        """Take the tensors named by `tensor_specs` out of `weights`."""
        self.ctx = ctx


@dataclasses.dataclass
class NormFold:
    """A request to the product that precedes a norm: add your result into the 32-bit
    residual stream `hidden` in place and hand on the norm's input as a `Prenormed`,
    so that the norm needs no launch of its own."""

    hidden: torch.Tensor
    weight: torch.Tensor
    eps: float


@dataclasses.dataclass
class Prenormed:
    """Normed rows whose last factor is still outstanding: row m of the norm's result is
    `xw[m] * rsqrt(sum(sums[m]) / width + eps)`.  That factor commutes with a
    product, so the product that follows applies it to its own result.  Only
    `ops.linear` and `ops.gate_up_silu` take one, and each value is used once."""

    xw: torch.Tensor  # [N, width], hidden * norm weight, activation type
    sums: torch.Tensor  # float32 [16 or 32, parts]: row m's sums of squares of hidden over column ranges
    eps: float


@dataclasses.dataclass
class Normed:
    """Rows that a block's first norm has been applied to already (by the kernel that made the
    rows of the residual stream): the block takes `x` for its norm's result and adds nothing."""

    x: torch.Tensor  # [N, width], activation type


@dataclasses.dataclass
class PartialSums:
    """A product that was taken in slices of its inner dimension and not added up yet:
    `sums` is float32 [slices, N, width], and the product is their sum in slice order.  Only a
    Linear made with `to_residual` returns one, and only Norm.forward takes it (it is no tensor:
    a block that adds its delta by hand fails loudly instead of broadcasting over the slices)."""

    sums: torch.Tensor

    def total(self) -> torch.Tensor:
        """The product itself, float32 [N, width] (the plain way to take it)."""
        return self.sums.sum(0)


class Norm(Part):
    """forward(hidden, delta) adds `delta` (or nothing) into the 32-bit residual
    stream `hidden` in place and returns the normed rows in the activation type;
    with `rows` only those rows are read and `hidden` is left alone.  `delta` is
    [N, hidden] in the activation type, or the PartialSums that a Linear made with
    `to_residual` may leave (`delta.total()` is the plain way to take them).

    fold(hidden) may return a NormFold when the step is small enough that the
    products on both sides of the norm can do its work (None: call forward).

    of_embedding(ids, table, step) may return (hidden, normed rows) where a kernel makes the
    rows of the residual stream from the embedding table and norms them in one go (None: the
    embedding is taken on its own, then forward(hidden, None))."""

    def forward(self, hidden: torch.Tensor, delta: Optional[torch.Tensor], rows=None) -> torch.Tensor:
        raise NotImplementedError

    def of_embedding(self, ids: torch.Tensor, table: torch.Tensor, step=None):
        return None

    def fold(self, hidden: torch.Tensor) -> Optional[NormFold]:
        return None


class PositionEncoding(Part):
    """Encodes positions into q and k.  `fused_rotary(step)` may return
    (cos_sin float32 [N, rotary_dim / 2, 2], rotary_dim) when the encoding is a
    half-split rotation that the fused q/k kernel can apply itself (`step.scratch`
    is a dictionary that lives for one step: tables made once go there);
    otherwise `apply` is called on q [N, nq, d] and k [N, nkv, d]."""

    def fused_rotary(self, step):
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor):
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the tokens of a request.

    forward(x [N, hidden], step, cache) -> [N, hidden].  `step` is the
    engine.batch.StepState of this step; `cache` is the cache.manager.LayerCache
    of the plan entry being run (pages of its group, the state rows, and whether
    this entry writes)."""

    # True if forward() uses only device arrays of the step (no host-side view of
    # the batch, no sizes that depend on the step's values): decode steps of such
    # mixers may be captured into a graph and replayed.  A replay runs forward() once
    # per step, like a step without graphs: state may be kept and advanced.  What runs
    # before a capture to warm the kernels up runs on padding rows only.
    graph_safe = False
    # True if forward() takes a Prenormed for x (passing it to one product only) and
    # a keyword `fold` (a NormFold for its last product, whose Prenormed it then returns).
    folds_norm = False

    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """forward(x [N, hidden]) -> [N, hidden], token by token."""

    folds_norm = False  # as Mixer.folds_norm

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of norm, mixer and feed-forward around the residual stream.

    forward(hidden, delta, step, cache) -> delta': `hidden` is the 32-bit
    residual stream [N, hidden]; `delta` is what the previous block still has to
    add to it (None for the first); the return value is what this block leaves
    to be added by whoever comes next.

    A block whose first norm can be folded into the products around it says so
    with entry_norm(); the model then passes the next block's as `next_norm`, and
    the block may return a Prenormed made for that norm instead of a delta.

    A block that begins with a norm of the residual stream and takes a `Normed` for
    `delta` (the norm's result, made elsewhere) names that norm with input_norm()."""

    mixer: Mixer

    def entry_norm(self) -> Optional[Norm]:
        return None

    def input_norm(self) -> Optional[Norm]:
        return None

    def forward(self, hidden, delta, step, cache, next_norm=None):
        raise NotImplementedError
