"""Grouped-query attention over the paged cache.

q/k/v projections (no bias) -> RMSNorm of each q and k head over head_dim with
one weight [head_dim] for all heads, before the position encoding; v untouched
-> position encoding of q and k -> K (ready to dot) and V written to the pages
-> attention of every token of the step through the block table -> output
projection.  src/model/qwen3.cpp:375-377, :391-407, :443-449, :464-481,
:498-557, :565-567.  scale = 1/sqrt(head_dim) (src/ops/attention.cu:201); kv
head of q head h is h // (nq // nkv) (:196-199).  The q/k norm is optional and
the position encoding is a part of its own, so the same mixer serves models
without either; `window` limits a query to the last `window` keys (the
reference has full attention only).
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import torch

from ..csrc.limits import check_head_dim
from ..weights.spec import INIT_NORM, TensorSpec
from .base import BuildContext, CacheSpec, KVCacheSpec, Mixer, PositionEncoding
from .linear import Linear


class PagedAttention(Mixer):
    graph_safe = True
    folds_norm = True

    def __init__(
        self,
        prefix: str,
        hidden_size: int,
        num_q_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: PositionEncoding,
        qk_norm_eps: Optional[float] = None,
        window: Optional[int] = None,
        scale: Optional[float] = None,
        qkv_names: Optional[Sequence[str]] = None,
        o_name: Optional[str] = None,
        qkv_bias: bool = False,
        o_bias: bool = False,
        qk_norm_names: Optional[Sequence[str]] = None,
    ):
        """`qkv_names`: the checkpoint's names of the projections' weights after `prefix`, three
        (q, k, v; default q_proj.weight, k_proj.weight, v_proj.weight) or one that holds the three
        stacked in that order; `o_name` the output projection's (default o_proj.weight);
        `qk_norm_names` the two norm weights' (default q_norm.weight, k_norm.weight).  With
        `qkv_bias` / `o_bias` every weight `x.weight` has a bias `x.bias`."""
        if num_q_heads % num_kv_heads:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads")
        check_head_dim(head_dim, getattr(position, "rotary_dim", 0))  # what no kernel takes is refused now, not at the first step
        self.prefix = prefix
        self.nq, self.nkv, self.d = num_q_heads, num_kv_heads, head_dim
        self.position = position
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)
        widths = [num_q_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim]
        names = list(qkv_names) if qkv_names else ["q_proj.weight", "k_proj.weight", "v_proj.weight"]
        if len(names) == 1:
            widths = [sum(widths)]  # the three stacked in one checkpoint tensor
        elif len(names) != 3:
            raise ValueError("qkv_names holds three names (q, k, v) or one (the three stacked)")
        o_name = o_name or "o_proj.weight"
        bias_of = lambda name: prefix + (name[: -len("weight")] + "bias" if name.endswith("weight") else name + ".bias")
        self.qkv = Linear([prefix + n for n in names], hidden_size, widths,
                          bias_names=[bias_of(n) for n in names] if qkv_bias else None)
        self.o = Linear([prefix + o_name], num_q_heads * head_dim, [hidden_size], to_residual=True,
                        bias_names=[bias_of(o_name)] if o_bias else None)
        self.folds_norm = not o_bias  # (the product before a folded norm adds into the residual stream itself)
        self.qk_norm_names = list(qk_norm_names) if qk_norm_names else ["q_norm.weight", "k_norm.weight"]
        if len(self.qk_norm_names) != 2:
            raise ValueError("qk_norm_names holds two names (q, k)")
        self.q_norm_w = None
        self.k_norm_w = None

    def cache_spec(self) -> CacheSpec:
        return KVCacheSpec(self.nkv, self.d, self.window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {**self.qkv.tensor_specs(), **self.o.tensor_specs()}
        if self.qk_norm_eps is not None:
            for name in self.qk_norm_names:
                specs[self.prefix + name] = TensorSpec((self.d,), INIT_NORM)
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.qkv.bind(weights, ctx)
        self.o.bind(weights, ctx)
        self.position.bind(weights, ctx)
        if self.qk_norm_eps is not None:
            qw = weights[self.prefix + self.qk_norm_names[0]]
            kw = weights[self.prefix + self.qk_norm_names[1]]
            if qw.dtype != kw.dtype:
                qw, kw = qw.float(), kw.float()
            self.q_norm_w, self.k_norm_w = qw.contiguous(), kw.contiguous()

    def forward(self, x, step, cache, fold=None):
        ops = self.ctx.ops
        qkv = self.qkv.forward(x)
        fused = self.position.fused_rotary(step)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        group = cache.group
        if fused is not None:
            cos_sin, rot = fused
            if ops.can_fuse_rope_attention(qkv.dtype, self.d, rot, cache.kv.shape[3], self.nq // self.nkv,
                                           step.max_q_len, step.max_kv_len, step.seq_slots.shape[0]):
                # a decode step: norm, rotation, cache write and attention in one launch
                a = ops.qk_norm_rope_attention(
                    qkv, group.slot_mapping, self.q_norm_w, self.k_norm_w, cos_sin, eps, cache.kv, self.nq,
                    self.nkv, self.d, cache.writes, group.block_table, step.seq_slots, step.cu_tokens,
                    step.kv_lens, step.token_seq, self.window, self.scale, step.max_kv_len,
                )
                return self.o.forward(a, fold=fold)
            q = ops.qk_norm_rope_write(
                qkv, group.slot_mapping, self.q_norm_w, self.k_norm_w, cos_sin, rot, eps,
                cache.kv, self.nq, self.nkv, self.d, cache.writes,
            )
        else:
            # an encoding the fused kernel does not know: norm, encode, then write
            N = qkv.shape[0]
            qw, kw = self.nq * self.d, self.nkv * self.d
            q = qkv[:, :qw].reshape(N * self.nq, self.d).contiguous()
            k = qkv[:, qw : qw + kw].reshape(N * self.nkv, self.d).contiguous()
            if self.qk_norm_eps is not None:
                q = ops.rmsnorm(q, self.q_norm_w, eps)
                k = ops.rmsnorm(k, self.k_norm_w, eps)
            q, k = self.position.apply(q.view(N, self.nq, self.d), k.view(N, self.nkv, self.d), step.positions)
            packed = torch.cat([q.reshape(N, qw), k.reshape(N, kw), qkv[:, qw + kw :]], dim=1).contiguous()
            q = ops.qk_norm_rope_write(
                packed, group.slot_mapping, None, None, None, 0, 0.0,
                cache.kv, self.nq, self.nkv, self.d, cache.writes,
            )
        a = ops.paged_attention(
            q, cache.kv, group.block_table, step.seq_slots, step.cu_tokens, step.kv_lens, step.token_seq,
            self.window, self.scale, step.min_q_len, step.max_q_len, step.max_kv_len,
        )
        return self.o.forward(a, fold=fold)
