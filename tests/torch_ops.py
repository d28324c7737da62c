"""Plain torch forms of the kernel operations (tests only).

Two uses: (1) the GPU tests compare every HIP kernel with the function of the
same name here; (2) CPU tests hand an instance to the engine in place of the
HIP operations, so that the cache, the step function and the scheduler can be
exercised without a GPU.  Nothing in the package imports this file.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def v_pages(kv_layer):
    """The value half of the pages [pages, 2, nkv, P, d]: stored transposed, [pages, nkv, d, P]."""
    pages, _, nkv, P, d = kv_layer.shape
    return kv_layer[:, 1].reshape(pages, nkv, d, P)


class TorchOps:
    def __init__(self, compute_dtype=torch.float64):
        self.cd = compute_dtype

    def embedding(self, ids, table, feedback=None, token_seq=None, seq_slots=None):
        ids = ids.long()
        if feedback is not None:
            ids = torch.where(ids < 0, feedback.long()[seq_slots.long()[token_seq.long()]], ids)
        return table[ids].to(torch.float32)

    def embedding_rmsnorm(self, ids, table, weight, eps, feedback=None, token_seq=None, seq_slots=None):
        hidden = self.embedding(ids, table, feedback, token_seq, seq_slots)
        x = hidden.to(self.cd)
        x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight.to(self.cd)
        return hidden, x.to(table.dtype)

    # the fused and sliced forms are the HIP kernels' own: this stand-in offers none of them
    def can_fold_norm(self, rows, width, dtype):
        return False

    def can_fuse_rope_attention(self, *sizes):
        return False

    def slices_for(self, M, N, K):
        return 0

    def add_rmsnorm(self, hidden, delta, weight, eps, out_dtype, rows=None):
        if hasattr(delta, "sums"):  # parts.base.PartialSums
            delta = delta.sums
        if delta is not None and delta.dim() == 3:  # partial sums of a product taken in slices
            delta = delta.to(self.cd).sum(0)
        if rows is None:
            if delta is not None:
                hidden += delta.to(hidden.dtype)
            h = hidden
        else:
            h = hidden[rows.long()]
            if delta is not None:
                h = h + delta[rows.long()].to(hidden.dtype)
        x = h.to(self.cd)
        y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight.to(self.cd)
        return y.to(out_dtype)

    def rmsnorm(self, x, weight, eps):
        xx = x.to(self.cd)
        y = xx / torch.sqrt((xx * xx).mean(-1, keepdim=True) + eps) * weight.to(self.cd)
        return y.to(x.dtype)

    def linear(self, x, weight, out_dtype=None, fold=None, sums_ok=False):
        assert fold is None, "this stand-in folds no norm (can_fold_norm says so)"
        return (x.to(self.cd) @ weight.to(self.cd).t()).to(out_dtype or x.dtype)

    def add_bias(self, x, bias):
        x += bias.to(x.dtype)
        return x

    def rope_table(self, positions, inv_freq):
        ang = (positions.to(torch.float32)[:, None] * inv_freq[None, :]).double()  # float32 product
        return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(torch.float32)

    def qk_norm_rope_write(self, qkv, slots, q_weight, k_weight, cos_sin, rotary_dim, eps, kv_layer,
                           num_q_heads, num_kv_heads, head_dim, write_kv=True):
        nq, nkv, d = num_q_heads, num_kv_heads, head_dim
        N = qkv.shape[0]
        x = qkv.to(self.cd)
        q = x[:, : nq * d].reshape(N, nq, d)
        k = x[:, nq * d : (nq + nkv) * d].reshape(N, nkv, d)
        v = x[:, (nq + nkv) * d :].reshape(N, nkv, d)

        def norm(t, w):
            if w is None:
                return t
            return t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * w.to(self.cd)

        def rope(t):
            if rotary_dim == 0:
                return t
            half = rotary_dim // 2
            c, s = cos_sin[:, None, :, 0].to(self.cd), cos_sin[:, None, :, 1].to(self.cd)
            x1, x2 = t[..., :half], t[..., half:rotary_dim]
            return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, t[..., rotary_dim:]], dim=-1)

        q = rope(norm(q, q_weight))
        k = rope(norm(k, k_weight))
        if write_kv:
            P = kv_layer.shape[3]
            for n in range(N):
                slot = int(slots[n])
                if slot < 0:
                    continue
                page, off = slot // P, slot % P
                kv_layer[page, 0, :, off, :] = k[n].to(kv_layer.dtype)
                v_pages(kv_layer)[page, :, :, off] = v[n].to(kv_layer.dtype)
        return q.to(qkv.dtype).contiguous()

    def paged_attention(self, q, kv_layer, block_table, seq_slots, cu_tokens, kv_lens, token_seq, window, scale,
                        min_q_len=0, max_q_len=0, max_kv_len=0):
        N, nq, d = q.shape
        nkv, P = kv_layer.shape[2], kv_layer.shape[3]
        group = nq // nkv
        out = torch.zeros((N, nq, d), dtype=self.cd, device=q.device)
        for s in range(seq_slots.shape[0]):
            slot = int(seq_slots[s])
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            kv_len = int(kv_lens[s])
            for t in range(q0, q1):
                pos = kv_len - (q1 - q0) + (t - q0)
                lo = max(0, pos - window + 1) if window else 0
                idx = torch.arange(lo, pos + 1, device=q.device)
                pages = block_table[slot, (idx // P).long()].long()
                assert int(pages.min()) >= 0, "attention reads a page that was given back"
                offs = (idx % P).long()
                keys = kv_layer[pages, 0, :, offs, :].to(self.cd)  # [n, nkv, d]
                vals = v_pages(kv_layer)[pages, :, :, offs].to(self.cd)  # [n, nkv, d]
                keys = keys.repeat_interleave(group, dim=1)
                vals = vals.repeat_interleave(group, dim=1)
                sc = torch.einsum("hd,nhd->hn", q[t].to(self.cd), keys) * scale
                p = torch.softmax(sc, dim=-1)
                out[t] = torch.einsum("hn,nhd->hd", p, vals)
        return out.reshape(N, nq * d).to(q.dtype)

    def silu_mul(self, gate_up):
        I = gate_up.shape[1] // 2
        g, u = gate_up[:, :I].to(self.cd), gate_up[:, I:].to(self.cd)
        return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)

    def gate_up_silu(self, x, weight):
        return self.silu_mul(self.linear(x, weight))

    def argmax(self, logits, scatter=None):
        out = torch.argmax(logits, dim=-1).to(torch.int32)  # torch returns the first maximum
        if scatter is not None:
            scatter[0][scatter[1].long()] = out
        return out

    def sample(self, logits, temperature, uniform):
        out = []
        for r in range(logits.shape[0]):
            T = float(temperature[r])
            if T <= 0:
                out.append(int(torch.argmax(logits[r])))
                continue
            z = logits[r].double() / T
            p = torch.exp(z - z.max())
            cdf = torch.cumsum(p, 0)
            target = float(uniform[r]) * float(cdf[-1])
            i = int(torch.searchsorted(cdf, torch.tensor(target, dtype=cdf.dtype), right=True))
            out.append(min(i, logits.shape[1] - 1))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
