"""The attention kernels at the context lengths that the benchmark and the command line reach:
4096, 8192 and 32768 keys (decode rows at batch 1 and 8, with as many key splits as the host
then chooses), prompt portions of 64 and 2048 tokens after a past of 30000 keys, and single
keys made to stand out at the first key and at both ends of every key split.  Against a plain
form in float64 that is written here (whole requests, no splits, no tiles).  The reference
checks its paged kernel the same way at small sizes, tests/test_paged_attention_cuda.cpp:545-744."""
import math

import pytest
import torch

from litellmengine_amd.csrc.ops import default_ops
from tests.torch_ops import v_pages

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def long_case(dtype, nq, nkv, d, P, lens, seed):
    """Random pages (made on the GPU), a scrambled block table, random q.  lens: [(past, q_len)]."""
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(seed)
    need = [(p + l + P - 1) // P for p, l in lens]
    pages = sum(need) + 3
    kv = torch.randn((pages, 2, nkv, P, d), generator=g, device=dev, dtype=torch.float32).to(dtype)
    gc = torch.Generator().manual_seed(seed + 1)
    perm = torch.randperm(pages, generator=gc).tolist()
    S = len(lens)
    table = torch.full((S + 2, max(need) + 1), -1, dtype=torch.int32)
    slots = torch.randperm(S + 2, generator=gc)[:S].tolist()
    cu, kv_lens, token_seq = [0], [], []
    for s, (past, ql) in enumerate(lens):
        table[slots[s], : need[s]] = torch.tensor([perm.pop() for _ in range(need[s])], dtype=torch.int32)
        cu.append(cu[-1] + ql)
        kv_lens.append(past + ql)
        token_seq += [s] * ql
    q = torch.randn((cu[-1], nq, d), generator=g, device=dev, dtype=torch.float32).to(dtype)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    return dict(q=q, kv=kv, table=table.to(dev), slots=i32(slots), cu=i32(cu), kv_lens=i32(kv_lens),
                token_seq=i32(token_seq), scale=1.0 / math.sqrt(d), lens=lens, host_slots=slots, host_table=table)


def run(case, window=None):
    lens = case["lens"]
    return default_ops().paged_attention(
        case["q"], case["kv"], case["table"], case["slots"], case["cu"], case["kv_lens"], case["token_seq"], window,
        case["scale"], min(l for _, l in lens), max(l for _, l in lens), max(p + l for p, l in lens))


def keys_and_values(case, s):
    """All keys and values of request s in position order, float64: [kv_len, nkv, d] each."""
    kv, P = case["kv"], case["kv"].shape[3]
    past, ql = case["lens"][s]
    n = past + ql
    pages = case["host_table"][case["host_slots"][s], : (n + P - 1) // P].long().to(kv.device)
    k = kv[pages, 0].permute(0, 2, 1, 3).reshape(-1, kv.shape[2], kv.shape[4])[:n].double()
    v = v_pages(kv)[pages].permute(0, 3, 1, 2).reshape(-1, kv.shape[2], kv.shape[4])[:n].double()
    return k, v


def plain_rows(case, s, rows, window=None):
    """Attention of the rows `rows` (indices within request s's portion): [len(rows), nq * d] float64."""
    past, ql = case["lens"][s]
    k, v = keys_and_values(case, s)
    nkv, d = k.shape[1], k.shape[2]
    q0 = int(case["cu"][s])
    q = case["q"][q0 + torch.tensor(rows, device=k.device)].double()  # [R, nq, d]
    R, nq = q.shape[0], q.shape[1]
    q = q.reshape(R, nkv, nq // nkv, d)
    scores = torch.einsum("rngd,knd->rngk", q, k) * case["scale"]
    pos = past + torch.tensor(rows, device=k.device)
    j = torch.arange(past + ql, device=k.device)
    seen = j[None, :] <= pos[:, None]
    if window:
        seen &= j[None, :] > pos[:, None] - window
    scores = scores.masked_fill(~seen[:, None, None, :], float("-inf"))
    return torch.einsum("rngk,knd->rngd", torch.softmax(scores, dim=-1), v).reshape(R, nq * d)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bfloat16", "float32"])
@pytest.mark.parametrize("context", [4096, 8192, 32768])
@pytest.mark.parametrize("batch,nq,nkv,splits", [(1, 32, 8, None), (8, 32, 8, None), (1, 8, 2, 64)],
                         ids=["batch1", "batch8", "batch1-two-kv-heads"])
def test_decode_rows_at_long_contexts(dtype, context, batch, nq, nkv, splits):
    """Every decode row against float64.  The longest request has exactly `context` keys, the
    others a few less (other offsets within a page and a step), so the host picks the key
    splits that it picks for the benchmark at this context."""
    d, P = 128, 16
    lens = [(context - 1 - off, 1) for off in (0, 1, 17, 32, 250, 1023, 5, 2049)[:batch]]
    case = long_case(dtype, nq, nkv, d, P, lens, seed=context + batch)
    o = default_ops()
    if dtype == torch.bfloat16:
        ns = o.decode_splits(batch, nkv, context, 0)
        expect = {(1, 8): {4096: 16, 8192: 32, 32768: 32}, (8, 8): {4096: 4, 8192: 4, 32768: 4},
                  (1, 2): {4096: 16, 8192: 32, 32768: 64}}[(batch, nkv)][context]
        assert ns == expect, f"the test means to reach {expect} key splits, the host chose {ns}"
    got = run(case).double()
    for s in range(batch):
        want = plain_rows(case, s, [0])
        err = (got[s : s + 1] - want).abs().max().item()
        assert err < TOL[dtype], (s, lens[s], err)


@pytest.mark.parametrize("context", [4096, 32768])
def test_fused_decode_attention_at_long_contexts(context):
    """The decode launch that also norms, rotates and writes the new K and V, at batch 1 and 8:
    its output against float64 over the pages that the separate kernel wrote, and those pages."""
    nq, nkv, d, P = 32, 8, 128, 16
    o = default_ops()
    for batch in (1, 8):
        lens = [(context - 1 - off, 1) for off in (0, 1, 17, 32, 250, 1023, 5, 2049)[:batch]]
        case = long_case(torch.bfloat16, nq, nkv, d, P, lens, seed=context + 77 + batch)
        g = torch.Generator(device="cuda").manual_seed(5)
        qkv = (torch.randn((batch, (nq + 2 * nkv) * d), generator=g, device="cuda") * 1.5).bfloat16()
        positions = torch.tensor([p for p, _ in lens], dtype=torch.int32, device="cuda")
        table, hs = case["host_table"], case["host_slots"]
        slots = torch.tensor([int(table[hs[s], p // P]) * P + p % P for s, (p, _) in enumerate(lens)],
                             dtype=torch.int32, device="cuda")
        inv = (1e6 ** (-(2.0 * torch.arange(d // 2, dtype=torch.float64)) / d)).float().cuda()
        cs = o.rope_table(positions, inv)
        qw = (1 + 0.2 * torch.randn(d, generator=g, device="cuda")).bfloat16()
        kw = (1 + 0.2 * torch.randn(d, generator=g, device="cuda")).bfloat16()
        kv_a, kv_b = case["kv"].clone(), case["kv"].clone()
        q = o.qk_norm_rope_write(qkv, slots, qw, kw, cs, d, 1e-6, kv_a, nq, nkv, d, True)
        assert o.can_fuse_rope_attention(torch.bfloat16, d, d, P, nq // nkv, 1, context, batch)
        got = o.qk_norm_rope_attention(qkv, slots, qw, kw, cs, 1e-6, kv_b, nq, nkv, d, True, case["table"], case["slots"],
                                       case["cu"], case["kv_lens"], case["token_seq"], None, case["scale"], context)
        assert (kv_a.float() - kv_b.float()).abs().max() <= 2.0 ** -7 * kv_a.float().abs().max()
        case["kv"], case["q"] = kv_a, q
        for s in range(batch):
            want = plain_rows(case, s, [0])
            err = (got[s : s + 1].double() - want).abs().max().item()
            assert err < 2e-2, (batch, s, err)


def sample_rows(q_len, seed):
    """The first and the last row, the edges of the 16-, 64- and 128-row tiles, and a few others."""
    g = torch.Generator().manual_seed(seed)
    rows = {0, 1, q_len - 1, q_len - 2, q_len // 2}
    for edge in (16, 64, 128, 1024):
        rows |= {r for r in (edge - 1, edge, edge + 1, q_len - edge, q_len - edge - 1) if 0 <= r < q_len}
    rows |= set(torch.randint(0, q_len, (12,), generator=g).tolist())
    return sorted(rows)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bfloat16", "float32"])
@pytest.mark.parametrize("q_len", [64, 2048])
@pytest.mark.parametrize("window", [None, 5000], ids=["full", "window5000"])
def test_prompt_portions_after_a_long_past(dtype, q_len, window):
    """A portion of 64 and of 2048 tokens after 30000 keys (and a second, shorter request beside
    it): a sample of rows against float64.  The short portion has its keys split over workgroups."""
    nq, nkv, d, P = 32, 8, 128, 16
    lens = [(30000, q_len), (4100, 17)]
    case = long_case(dtype, nq, nkv, d, P, lens, seed=q_len + 3)
    o = default_ops()
    if dtype == torch.bfloat16 and q_len == 64 and window is None:
        assert o.prefill_splits(len(lens), nkv, nq // nkv, d, q_len, 30000 + q_len, 0) > 1
    got = run(case, window).double()
    for s, (past, ql) in enumerate(lens):
        rows = sample_rows(ql, s)
        want = plain_rows(case, s, rows, window)
        q0 = int(case["cu"][s])
        err = (got[[q0 + r for r in rows]] - want).abs().max(dim=1).values
        assert err.max().item() < TOL[dtype], (s, rows[int(err.argmax())], err.max().item())


def split_edges(first_step, last_step, splits, keys_per_step, kv_len):
    """First and last key of every key split, as the kernels cut them: the steps first .. last in
    `splits` runs of ceil(steps / splits)."""
    per = (last_step - first_step + 1 + splits - 1) // splits
    keys = {0, kv_len - 1}
    for i in range(splits):
        b = first_step + i * per
        e = min(last_step + 1, b + per)
        if b < e:
            keys |= {b * keys_per_step, min(kv_len, e * keys_per_step) - 1}
    return sorted(keys)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bfloat16", "float32"])
@pytest.mark.parametrize("context", [4096, 8192])
def test_far_keys_at_the_ends_of_every_key_split(dtype, context):
    """One decode row over `context` keys.  The first key and the first and last key of every key
    split are made, one at a time, to carry the whole softmax of one head: that key's value row
    must come back.  A split that drops its last key, reads into its neighbour's, or is merged
    with the wrong weight fails here."""
    nq, nkv, d, P = 32, 8, 128, 16
    case = long_case(dtype, nq, nkv, d, P, [(context - 1, 1)], seed=context + 9)
    o = default_ops()
    if dtype == torch.bfloat16:
        splits, step = o.decode_splits(1, nkv, context, 0), 32
        assert splits == {4096: 16, 8192: 32}[context]
    else:
        splits, step = o.f32_attention_splits(1, nkv, 1, 1, context, 0), 16
        assert splits >= 16
    keys = split_edges(0, (context - 1) // step, splits, step, context)
    assert len(keys) >= 2 * splits
    q, kv, table, slot = case["q"], case["kv"], case["host_table"], case["host_slots"][0]
    group = nq // nkv
    for at in range(0, len(keys), nkv):  # kv head h carries key keys[at + h] in this launch
        chunk = keys[at : at + nkv]
        saved = []
        for h, j in enumerate(chunk):
            page, off = int(table[slot, j // P]), j % P
            saved.append((page, h, off, kv[page, 0, h, off].clone()))
            kv[page, 0, h, off] = (q[0, h * group].float() * 4.0).to(dtype)
        got = run(case).reshape(1, nq, d)
        for h, j in enumerate(chunk):
            page, off = int(table[slot, j // P]), j % P
            want = v_pages(kv)[page, h, :, off]
            err = (got[0, h * group].float() - want.float()).abs().max().item()
            assert err < (2e-2 if dtype == torch.bfloat16 else 1e-3), (j, err)
        for page, h, off, old in saved:
            kv[page, 0, h, off] = old
