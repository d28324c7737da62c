"""Each HIP kernel alone against its plain torch form (tests/torch_ops.py), in
float32 and bfloat16, at sizes other than the tiny models': widths and
vocabularies that are no power of two, head sizes in steps of 16, odd page sizes."""
import math

import pytest
import torch

from tests.torch_ops import TorchOps, v_pages

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
REF = TorchOps(torch.float64)


def ops():
    from litellmengine_amd.csrc.ops import default_ops

    return default_ops()


def tol(dtype, scale=1.0):
    return (2e-5 if dtype == torch.float32 else 2e-2) * scale


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [48, 1000, 4096])
def test_embedding(dtype, H):
    table = rnd((333, H), dtype, 1)
    ids = torch.tensor([0, 332, 5, 5, 17], dtype=torch.int32).cuda()
    got = ops().embedding(ids, table)
    assert got.dtype == torch.float32
    assert torch.equal(got, table[ids.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,wdtype", [(48, None), (1000, torch.float32), (4096, None), (4098, None), (9000, torch.float32)])
def test_embedding_with_its_first_norm(dtype, H, wdtype):
    """The rows of the table and their RMSNorm from one launch: the rows are the embedding's own
    bit by bit, the normed rows what the norm kernel makes of them (and the float64 form); ids
    below zero are looked up in the feedback table.  Row 5 is made large in one place, so a sum
    over a part of the row shows."""
    o = ops()
    table = rnd((333, H), dtype, 1)
    table[5, H - 1] = 30.0
    w = (1 + 0.1 * rnd((H,), torch.float32, 4)).to(wdtype or dtype)
    ids = torch.tensor([0, 332, 5, 5, 17], dtype=torch.int32).cuda()
    hidden, x = o.embedding_rmsnorm(ids, table, w, 1e-3)
    assert hidden.dtype == torch.float32 and x.dtype == dtype and x.shape == (5, H)
    assert torch.equal(hidden, table[ids.long()].float())
    want = REF.add_rmsnorm(hidden.clone(), None, w, 1e-3, dtype)
    assert (x.double() - want.double()).abs().max() < tol(dtype, 4)
    feedback = torch.tensor([7, 332, 5, 0], dtype=torch.int32).cuda()
    seq_slots = torch.tensor([2, 0, 1], dtype=torch.int32).cuda()
    token_seq = torch.tensor([0, 0, 1, 2, 2], dtype=torch.int32).cuda()
    ids = torch.tensor([-1, 9, -1, 4, -1], dtype=torch.int32).cuda()
    hidden, x = o.embedding_rmsnorm(ids, table, w, 1e-3, feedback, token_seq, seq_slots)
    real = torch.tensor([5, 9, 7, 4, 332]).cuda()
    assert torch.equal(hidden, table[real].float())
    assert (x.double() - REF.add_rmsnorm(hidden.clone(), None, w, 1e-3, dtype).double()).abs().max() < tol(dtype, 4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,wdtype", [(80, None), (1000, torch.float32), (5120, None), (9000, None)])
def test_add_rmsnorm(dtype, H, wdtype):
    N = 7
    hidden = rnd((N, H), torch.float32, 2, 3.0)
    delta = rnd((N, H), dtype, 3)
    w = (1 + 0.1 * rnd((H,), torch.float32, 4)).to(wdtype or dtype)
    h_ref = hidden.clone()
    want = REF.add_rmsnorm(h_ref, delta, w, 1e-5, dtype)
    got = ops().add_rmsnorm(hidden, delta, w, 1e-5, dtype)
    assert torch.allclose(hidden, h_ref, atol=1e-6), "the residual sum is written back"
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
    # no delta: hidden unchanged
    before = hidden.clone()
    got = ops().add_rmsnorm(hidden, None, w, 1e-5, dtype)
    assert torch.equal(hidden, before)
    assert (got.double() - REF.add_rmsnorm(before.clone(), None, w, 1e-5, dtype).double()).abs().max() < tol(dtype, 4)
    # row list: only those rows, nothing written back
    rows = torch.tensor([6, 0, 3], dtype=torch.int32).cuda()
    got = ops().add_rmsnorm(hidden, delta, w, 1e-5, dtype, rows=rows)
    assert torch.equal(hidden, before)
    want = REF.add_rmsnorm(before.clone(), delta, w, 1e-5, dtype, rows=rows)
    assert got.shape == (3, H)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)


def test_rmsnorm_reference_vector():
    # input and weight of tests/test_rms_norm.cpp:57-64; expected by hand:
    # row 0: mean(x^2) = 7.5, row 1: mean(x^2) = 6
    x = torch.tensor([[1.0, 2, 3, 4], [2, 0, -2, 4]]).cuda()
    w = torch.tensor([1.0, 1.5, 2.0, 0.5]).cuda()
    got = ops().rmsnorm(x, w, 1e-6).cpu()
    r0, r1 = 1 / math.sqrt(7.5 + 1e-6), 1 / math.sqrt(6 + 1e-6)
    want = torch.tensor([[1 * r0, 3 * r0, 6 * r0, 2 * r0], [2 * r1, 0, -4 * r1, 2 * r1]])
    assert torch.allclose(got, want, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("I", [8, 200, 12288])
def test_silu_mul(dtype, I):
    gu = rnd((5, 2 * I), dtype, 5, 2.0)
    got = ops().silu_mul(gu)
    want = REF.silu_mul(gu)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(1, 128, 64), (5, 200, 96), (8, 12288, 4096), (8, 136, 80), (9, 100, 72), (40, 64, 48),
                                   (3, 12277, 4096), (1, 8189, 4096), (7, 4500, 200), (16, 5003, 72)])
def test_gate_up_silu(dtype, M, I, K):
    x = rnd((M, K), dtype, 21, 2.0)
    w = rnd((2 * I, K), dtype, 22, 0.1)
    got = ops().gate_up_silu(x, w)
    gu = x.double() @ w.double().t()
    want = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
    assert got.shape == (M, I)
    lim = 1e-5 if dtype == torch.float32 else 2e-2
    assert (got.double() - want).abs().max() < lim * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,H,K,N", [(1, 64, 40, 48), (3, 136, 72, 100), (8, 4096, 1024, 512), (5, 1000, 64, 30),
                                     (6, 4096, 256, 8189), (1, 4096, 128, 12288), (16, 4096, 256, 6151), (11, 5120, 128, 260),
                                     (7, 24, 8, 6), (16, 1024, 2048, 3072), (13, 520, 96, 70), (32, 1024, 2048, 3072),
                                     (17, 72, 40, 22), (29, 2048, 512, 128),
                                     # 17 to 32 rows against so many tiles of W that a workgroup takes several (an output head)
                                     (32, 1024, 128, 20000), (19, 520, 64, 16387),
                                     # more tiles than CUs, no whole rounds: tiles of fewer than 16 rows
                                     (9, 4600, 64, 4700), (16, 5120, 128, 5000), (3, 6152, 40, 4099)])
def test_norm_folded_into_products(wdtype, M, H, K, N):
    """RMSNorm between two products, done by them: the first adds its result into the
    residual stream and leaves hidden * w and sums of squares, the second (plain or
    gated) scales its rows.  Compared with add, norm, product in float64; the hidden row
    is made large in one place so that a missing or doubled part of the sum shows."""
    from litellmengine_amd.parts import NormFold

    o = ops()
    assert o.can_fold_norm(M, H, torch.bfloat16) and not o.can_fold_norm(33, H, torch.bfloat16)
    assert o.can_fold_norm(17, H, torch.bfloat16) == (H <= 2048), "more than 16 rows only for narrow models"
    assert not o.can_fold_norm(M, H, torch.float32) and not o.can_fold_norm(M, H + 4, torch.bfloat16)
    a = rnd((M, K), torch.bfloat16, 31)
    w1 = rnd((H, K), torch.bfloat16, 32, 0.2)
    hidden = rnd((M, H), torch.float32, 33, 1.5)
    hidden[:, H - 3] += 20.0  # a column of the last, partly filled, workgroup dominates the mean
    nw = (1 + 0.3 * rnd((H,), torch.float32, 34)).to(wdtype)
    eps = 1e-3
    for gated in (False, True):
        w2 = rnd((2 * N if gated else N, H), torch.bfloat16, 35, 0.1)
        h = hidden.clone()
        pre = o.linear(a, w1, fold=NormFold(h, nw, eps))
        want_h = hidden.double() + a.double() @ w1.double().t()
        assert (h.double() - want_h).abs().max() < 1e-4 * max(1.0, want_h.abs().max().item())
        assert pre.sums.shape == (16 if M <= 16 else 32, o.norm_sum_parts(H)) and o.norm_sum_parts(H) >= (H + 15) // 16
        ss = pre.sums.double().sum(1)[:M]
        assert torch.allclose(ss, (want_h ** 2).sum(1), rtol=1e-5)
        normed = want_h * torch.rsqrt((want_h ** 2).mean(1, keepdim=True) + eps) * nw.double()
        y = normed @ w2.double().t()
        if gated:
            got = o.gate_up_silu(pre, w2)
            want = torch.nn.functional.silu(y[:, :N]) * y[:, N:]
        else:
            got = o.linear(pre, w2)
            want = y
        assert got.dtype == torch.bfloat16 and got.shape == want.shape
        assert (got.double() - want).abs().max() < 2e-2 * max(1.0, want.abs().max().item())
        if not gated:
            # the same product left in float32 (an output head after the final norm): the bfloat16
            # result is this one rounded, and against float64 only the operands' rounding is left
            wide = o.linear(pre, w2, out_dtype=torch.float32)
            assert wide.dtype == torch.float32 and wide.shape == want.shape
            assert torch.equal(wide.to(torch.bfloat16), got)
            assert (wide.double() - want).abs().max() < 1e-2 * max(1.0, want.abs().max().item())
        # against the unfolded kernels on the same numbers: the two differ by rounding only
        h2 = hidden.clone()
        x2 = o.add_rmsnorm(h2, o.linear(a, w1), nw, eps, torch.bfloat16)
        ref = o.gate_up_silu(x2, w2) if gated else o.linear(x2, w2)
        assert (got.double() - ref.double()).abs().max() < 2e-2 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("M", [17, 31, 32, 33, 48, 64, 65, 81, 96, 97, 128])
@pytest.mark.parametrize("N,K,slices", [(4096, 4096, 4), (4096, 12288, 4), (320, 2048, 2), (64, 1024, 1), (128, 3072, 3), (640, 17408, 17)])
def test_product_in_slices_of_k(M, N, K, slices):
    """The product of 17 to 128 rows taken in slices of K: the float32 partial sums add up to the
    float64 product, each slice is the product over its own columns, and the residual add + norm
    that reads them gives what it gives for the summed delta.  W is made of rows that tell their
    own number and X of rows that tell theirs, so a tile written to the wrong place shows."""
    o = ops()
    x = rnd((M, K), torch.bfloat16, 61)
    w = rnd((N, K), torch.bfloat16, 62, 0.05)
    w[:, 0] = (torch.arange(N) % 64).to(torch.bfloat16) / 16
    x[:, 1] = (torch.arange(M) % 16).to(torch.bfloat16) / 8
    got = o.linear_slices(x, w, slices)
    assert got.shape == (slices, M, N) and got.dtype == torch.float32
    part = K // slices
    for s in range(slices):
        want = x[:, s * part:(s + 1) * part].double() @ w[:, s * part:(s + 1) * part].double().t()
        assert (got[s].double() - want).abs().max() < 2e-4 * max(1.0, want.abs().max().item()), s
    if N % 4 == 0 and N <= 8192:
        hidden = rnd((M, N), torch.float32, 63, 1.5)
        nw = (1 + 0.3 * rnd((N,), torch.float32, 64)).to(torch.bfloat16)
        h_ref = hidden.clone()
        want = REF.add_rmsnorm(h_ref, got, nw, 1e-6, torch.bfloat16)
        h_got = hidden.clone()
        out = o.add_rmsnorm(h_got, got, nw, 1e-6, torch.bfloat16)
        assert (h_got.double() - h_ref.double()).abs().max() < 1e-5 * max(1.0, h_ref.abs().max().item())
        assert (out.double() - want.double()).abs().max() < 2e-2
        rows = torch.tensor([M - 1, 0, 5], dtype=torch.int32, device="cuda")
        h_keep = hidden.clone()
        picked = o.add_rmsnorm(h_keep, got, nw, 1e-6, torch.bfloat16, rows=rows)
        assert torch.equal(h_keep, hidden)  # with rows nothing is written back
        assert (picked.double() - want[rows.long()].double()).abs().max() < 2e-2


def test_key_splits_of_prompt_portions():
    """The choice of key splits for prompt portions, from the sizes and the CU count: none from an
    empty cache, none where the row blocks fill the CUs by themselves (a 2048-token portion of a
    long prompt), several for a short portion after a long past."""
    o = ops()
    units = o.compute_units()
    full = units // 8 * 128 // 4  # tokens whose row blocks (8 kv heads, groups of 4, 128 rows) fill the CUs once
    assert o.prefill_splits(1, 8, 4, 128, 2048, 2048, 0) == 1
    assert o.prefill_splits(1, 8, 4, 128, 2 * full, 2 * full + 2048, 0) == 1
    assert o.prefill_splits(1, 8, 4, 128, full, full + 8192, 0) == 1
    assert o.prefill_splits(1, 8, 4, 128, full // 2, full // 2 + 4096, 0) == 4
    assert o.prefill_splits(1, 8, 4, 128, full // 2, full // 2 + 1024, 0) == 1
    assert o.prefill_splits(1, 8, 4, 128, full // 8, full // 8 + 1024, 0) == 4
    assert o.prefill_splits(1, 8, 4, 128, full // 8, full // 8 + 1024, 64) == 1  # a window of 64 keys
    # one row block a head (the keys come from memory once, one workgroup a CU is best) against sixteen
    assert o.prefill_splits(4, 8, 4, 128, 32, 32 + 16384, 0) == units // 32
    assert o.prefill_splits(1, 8, 4, 128, full // 2, full // 2 + 16384, 0) == 4
    # the low workgroup shape for a launch of at most one workgroup a CU, whatever its past
    assert o.prefill_form(2, 8, 4, 128, 128, 128 + 256, 0, 1, None) == 1
    assert o.prefill_form(1, 8, 4, 128, 2048, 4096, 0, 1, None) == 3


def test_which_products_are_taken_in_slices():
    """The choice is made from the sizes and the CU count: few rows per CU (o_proj, down_proj of the
    8B sizes) in whole rounds of workgroups; not below 17 or above 128 rows, not for wide weights,
    not where no slice count fills the CUs; and the engine's Linear asks only for deltas of the
    residual stream."""
    o = ops()
    units = o.compute_units()
    n = 16 * units  # 16 rows a CU
    assert o.slices_for(64, n, 4096) == 4 and o.slices_for(17, n, 12288) == 4
    assert o.slices_for(128, n, 4096) == 4 and o.slices_for(16, n, 4096) == 0 and o.slices_for(129, n, 4096) == 0
    assert o.slices_for(64, 64 * units, 4096) == 0      # wide: rows enough for every CU
    assert o.slices_for(64, n + 8, 4096) == 0           # no multiple of 64 rows
    assert o.slices_for(64, 8192 + 64, 32768) == 0      # wider than the norm that adds the slices up takes
    assert o.slices_for(64, n, 4096 + 256) == 0         # no whole slices
    if units == 256:
        # a long K beside few rows (down_proj of the 32B and 14B sizes): slices although the workgroups fill
        # no whole rounds; a square weight in a round and a quarter (o_proj of the 32B sizes) stays the library's
        assert o.slices_for(64, 5120, 25600) == 5 and o.slices_for(64, 5120, 17408) == 17
        assert o.slices_for(64, 5120, 8192) == 0 and o.slices_for(64, 1024, 3072) == 0
    if units == 256:
        # the library's products (more than 128 rows) of a weight with few rows and a long K: slices while the
        # CUs have room for the tiles; not for square weights, not when the tiles fill the CUs anyway
        assert [o.library_slices_for(m, 4096, 12288) for m in (128, 129, 512, 1024, 2048, 4096)] == [0, 4, 4, 4, 2, 0]
        assert o.library_slices_for(2048, 4096, 4096) == 0 and o.library_slices_for(1024, 5120, 25600) == 2
        assert o.library_slices_for(512, 8192 + 256, 32768) == 0  # wider than the norm that adds the slices up takes
    x = rnd((300, 12288), torch.bfloat16, 67, 0.5)
    w = rnd((1024, 12288), torch.bfloat16, 68, 0.05)
    got = o.linear(x, w, sums_ok=True)
    assert got.sums.shape == (4, 300, 1024) and got.sums.dtype == torch.float32
    want = x.double() @ w.double().t()
    assert (got.total().double() - want).abs().max() < 1e-3 * want.abs().max()  # float32 sums of bfloat16 products
    hidden = rnd((300, 1024), torch.float32, 69)
    nw = (1 + 0.1 * rnd((1024,), torch.float32, 70)).bfloat16()
    h_want = hidden.double() + want
    normed = o.add_rmsnorm(hidden, got, nw, 1e-6, torch.bfloat16)
    assert (hidden.double() - h_want).abs().max() < 1e-3 * want.abs().max()
    n_want = h_want / torch.sqrt((h_want * h_want).mean(-1, keepdim=True) + 1e-6) * nw.double()
    assert (normed.double() - n_want).abs().max() < 3e-2
    x = rnd((40, 4096), torch.bfloat16, 65)
    w = rnd((n, 4096), torch.bfloat16, 66, 0.05)
    assert o.linear(x, w).shape == (40, n)                       # a caller that said nothing gets the product
    assert o.linear(x, w, sums_ok=True).sums.shape == (4, 40, n)  # a delta of the residual stream may come in slices


@pytest.mark.parametrize("K", [1024, 2048, 3072, 4096, 5120, 6144, 8192])
@pytest.mark.parametrize("M", [1, 7, 16])
def test_streaming_products_at_every_width(M, K):
    """The weight-streaming forms (one workgroup per CU walking over its share of W, X held in
    registers) at every K they take, rows of W that leave the last tile of a share partly empty:
    plain (both result types), gated, and both after a folded norm, against float64.  W is made
    of rows that tell their own number, so a row written to the wrong place shows."""
    from litellmengine_amd.parts import NormFold

    o = ops()
    units = torch.cuda.get_device_properties(0).multi_processor_count
    N = 16 * units + 16 * 5 + 7  # more than one tile per CU, and no multiple of anything
    x = rnd((M, K), torch.bfloat16, 51)
    w = rnd((N, K), torch.bfloat16, 52, 0.05)
    w[:, 0] = (torch.arange(N) % 64).to(torch.bfloat16) / 16  # tells the row
    want = x.double() @ w.double().t()
    lim = 2e-2 * max(1.0, want.abs().max().item())
    for out_dtype in (torch.bfloat16, torch.float32):
        got = o.linear(x, w, out_dtype)
        assert (got.double() - want).abs().max() < (lim if out_dtype == torch.bfloat16 else lim / 100)
    if K <= 5120:  # the gated form holds two tiles of W: it streams up to this width
        half = N  # gate rows, then as many up rows
        wg = torch.cat([w, rnd((half, K), torch.bfloat16, 53, 0.05)]).contiguous()
        y = x.double() @ wg.double().t()
        wantg = torch.nn.functional.silu(y[:, :half]) * y[:, half:]
        got = o.gate_up_silu(x, wg)
        assert got.shape == (M, half)
        assert (got.double() - wantg).abs().max() < 2e-2 * max(1.0, wantg.abs().max().item())
    # after a folded norm: the product before it makes the sums, this one applies the row factors
    a = rnd((M, 64), torch.bfloat16, 54)
    w1 = rnd((K, 64), torch.bfloat16, 55, 0.2)
    hidden = rnd((M, K), torch.float32, 56, 1.5)
    nw = (1 + 0.3 * rnd((K,), torch.float32, 57)).to(torch.bfloat16)
    pre = o.linear(a, w1, fold=NormFold(hidden, nw, 1e-3))
    h = hidden.double()
    normed = h * torch.rsqrt((h ** 2).mean(1, keepdim=True) + 1e-3) * nw.double()
    got = o.linear(pre, w)
    wantn = normed @ w.double().t()
    assert (got.double() - wantn).abs().max() < 2e-2 * max(1.0, wantn.abs().max().item())


@pytest.mark.parametrize("K", [1024, 2048, 3072, 4096])
@pytest.mark.parametrize("M", [17, 25, 32])
def test_streaming_products_with_two_tiles_of_rows(M, K):
    """17 to 32 rows of X in the weight-streaming forms: plain (both result types) against a weight
    with many rows for every CU at every K they take, and, at the widths of narrow models, gated
    and after a folded norm; against float64.  Row 16 of X is made large, so a second tile of rows
    that is dropped or read twice shows, and W is made of rows that tell their own number."""
    from litellmengine_amd.parts import NormFold

    o = ops()
    units = torch.cuda.get_device_properties(0).multi_processor_count
    x = rnd((M, K), torch.bfloat16, 71)
    x[16] *= 4.0
    N = o.tuning.stream_32_rows_min_share * units + 16 * 5 + 7
    w = rnd((N, K), torch.bfloat16, 72, 0.05)
    w[:, 0] = (torch.arange(N) % 64).to(torch.bfloat16) / 16
    want = x.double() @ w.double().t()
    lim = 2e-2 * max(1.0, want.abs().max().item())
    for out_dtype in (torch.bfloat16, torch.float32):
        got = o.linear(x, w, out_dtype)
        assert (got.double() - want).abs().max() < (lim if out_dtype == torch.bfloat16 else lim / 100)
    if K > 2048:
        return
    assert o.can_fold_norm(M, K, torch.bfloat16)
    n = 17 * units + 16 * 5 + 7  # more than one tile per CU
    wg = rnd((2 * n, K), torch.bfloat16, 73, 0.05)
    y = x.double() @ wg.double().t()
    wantg = torch.nn.functional.silu(y[:, :n]) * y[:, n:]
    got = o.gate_up_silu(x, wg)
    assert (got.double() - wantg).abs().max() < 2e-2 * max(1.0, wantg.abs().max().item())
    a = rnd((M, 64), torch.bfloat16, 74)
    w1 = rnd((K, 64), torch.bfloat16, 75, 0.2)
    hidden = rnd((M, K), torch.float32, 76, 1.5)
    hidden[16] *= 3.0
    nw = (1 + 0.3 * rnd((K,), torch.float32, 77)).to(torch.bfloat16)
    pre = o.linear(a, w1, fold=NormFold(hidden, nw, 1e-3))
    h = hidden.double()
    normed = h * torch.rsqrt((h ** 2).mean(1, keepdim=True) + 1e-3) * nw.double()
    for weight, gated in ((w[: 17 * units + 87], False), (wg, True)):
        yn = normed @ weight.double().t()
        wantn = torch.nn.functional.silu(yn[:, :n]) * yn[:, n:] if gated else yn
        got = o.gate_up_silu(pre, weight) if gated else o.linear(pre, weight.contiguous())
        assert (got.double() - wantn).abs().max() < 2e-2 * max(1.0, wantn.abs().max().item())
        if not gated:
            wide = o.linear(pre, weight.contiguous(), out_dtype=torch.float32)
            assert (wide.double() - wantn).abs().max() < 1e-2 * max(1.0, wantn.abs().max().item())


@pytest.mark.parametrize("M", [3, 16, 24, 32, 40, 100, 300])
def test_the_numbers_that_choose_a_kernel_change_no_result(M):
    """ProductTuning decides which kernel takes a product, never what it gives: with every
    threshold pushed to one end and to the other (the library for everything it may take; the
    weight-streaming and sliced kernels for everything they take), plain and gated products and
    a product that leaves its result as a delta of the residual stream agree with float64."""
    import dataclasses

    from litellmengine_amd.csrc.ops import HipOps
    from litellmengine_amd.csrc.tuning import ProductTuning

    units = torch.cuda.get_device_properties(0).multi_processor_count
    K, N, I = 2048, 64 * units + 64, 1024
    x = rnd((M, K), torch.bfloat16, 81)
    w = rnd((N, K), torch.bfloat16, 82, 0.05)
    wg = rnd((2 * I, K), torch.bfloat16, 83, 0.05)
    wd = rnd((K, 4 * K), torch.bfloat16, 84, 0.05)  # K at least twice N: a candidate for slices
    xd = rnd((M, 4 * K), torch.bfloat16, 85)
    want = x.double() @ w.double().t()
    y = x.double() @ wg.double().t()
    want_g = torch.nn.functional.silu(y[:, :I]) * y[:, I:]
    want_d = xd.double() @ wd.double().t()
    base = ProductTuning()
    ends = [
        base,
        dataclasses.replace(base, skinny_max_rows=0, skinny_small_weight=0, skinny_small_width=0,
                            stream_32_rows_min_share=1 << 30, sliced_min_fill=2.0, sliced_long_k_min_weight=1 << 62,
                            library_max_slices=1),
        dataclasses.replace(base, skinny_small_weight=1 << 62, skinny_small_width=1 << 30, stream_32_rows_min_share=1,
                            sliced_min_fill=0.0, sliced_long_k_min_weight=0),
    ]
    for tuning in ends:
        o = HipOps(tuning=tuning)
        got = o.linear(x, w)
        assert (got.double() - want).abs().max() < 2e-2 * max(1.0, want.abs().max().item())
        got = o.linear(x, w, torch.float32)
        assert (got.double() - want).abs().max() < 2e-4 * max(1.0, want.abs().max().item())
        got = o.gate_up_silu(x, wg)
        assert (got.double() - want_g).abs().max() < 2e-2 * max(1.0, want_g.abs().max().item())
        delta = o.linear(xd, wd, sums_ok=True)
        total = delta.total() if hasattr(delta, "total") else delta
        assert (total.double() - want_d).abs().max() < 2e-2 * max(1.0, want_d.abs().max().item())


def test_silu_mul_reference_vector():
    # tests/test_silu_and_mul.cpp:48-56
    g = torch.tensor([[-3.0, -1, 0, 1], [2, 4, 0.5, -0.5]])
    u = torch.tensor([[1.0, 2, -1, 0.5], [3, -2, 4, -3]])
    got = ops().silu_mul(torch.cat([g, u], dim=1).cuda()).cpu()
    want = torch.nn.functional.silu(g) * u
    assert torch.allclose(got, want, atol=1e-6)


@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                                (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("M,N,K", [(1, 503, 96), (2, 4, 3), (5, 130, 70), (67, 257, 200), (33, 1000, 4096),
                                   (8, 6144, 4096), (16, 311, 136), (17, 48, 64), (64, 4096, 1536), (49, 72, 40),
                                   (3, 151936, 128), (5, 8189, 4096), (2, 6151, 4096), (16, 4112, 4096),
                                   (5, 5120, 1600), (16, 4200, 72), (9, 4603, 25600)])
def test_linear(in_dtype, out_dtype, M, N, K):
    x = rnd((M, K), in_dtype, 6)
    w = rnd((N, K), in_dtype, 7, 0.05)
    got = ops().linear(x, w, out_dtype)
    want = x.double() @ w.double().t()
    assert got.dtype == out_dtype
    lim = 1e-5 if out_dtype == torch.float32 and in_dtype == torch.float32 else (2e-5 if out_dtype == torch.float32 else 2e-2)
    assert (got.double() - want).abs().max() < lim * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("M,N,K", [(65, 64, 16), (130, 96, 72), (300, 513, 1024), (2048, 1000, 136), (77, 151, 4)])
def test_linear_float32_many_rows(M, N, K):
    """The tiled float32 kernel (float32 matrix instruction) and the plain-FMA kernel it stands beside."""
    x = rnd((M, K), torch.float32, 61)
    w = rnd((N, K), torch.float32, 62, 0.05)
    want = x.double() @ w.double().t()
    o = ops()
    got = o.linear(x, w)
    o.force_simt_gemm = True
    try:
        plain = o.linear(x, w)
    finally:
        o.force_simt_gemm = False
    lim = 1e-5 * max(1.0, want.abs().max().item())
    assert (got.double() - want).abs().max() < lim and (plain.double() - want).abs().max() < lim
    # a row's result does not depend on what else is in the batch
    part = o.linear(x[40:].contiguous(), w)
    assert torch.equal(part, got[40:])


def test_linear_reference_vector():
    # tests/test_linear.cpp:63-78: X 2x3, W 4x3
    x = torch.tensor([[1.0, 2, 3], [4, 5, 6]]).cuda()
    w = torch.tensor([[1.0, 2, 3], [4, 5, 6], [-1, 0, 1], [2, -3, 4]]).cuda()
    want = torch.tensor([[14.0, 32, 2, 8], [32, 77, 2, 17]])
    assert torch.equal(ops().linear(x, w).cpu(), want)


def make_cache(num_pages, nkv, P, d, dtype, seed):
    return rnd((num_pages, 2, nkv, P, d), dtype, seed)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P,rot,norm", [(4, 2, 16, 4, 16, True), (6, 3, 48, 3, 48, True),
                                                 (8, 1, 128, 16, 128, True), (2, 2, 80, 8, 32, False),
                                                 (3, 1, 256, 5, 0, True), (4, 2, 64, 16, 32, True),
                                                 (5, 5, 32, 8, 32, False), (32, 8, 128, 16, 128, True)])
def test_qk_norm_rope_write(dtype, nq, nkv, d, P, rot, norm):
    N, pages = 9, 6
    qkv = rnd((N, (nq + 2 * nkv) * d), dtype, 8)
    positions = torch.tensor([0, 1, 2, 50, 51, 7, 1000, 3, 4], dtype=torch.int32).cuda()
    slots = torch.tensor([0, 5, 9, -1, pages * P - 1, 2, 3, 11, 7], dtype=torch.int32).cuda()
    qw = (1 + 0.1 * rnd((d,), torch.float32, 9)).to(dtype) if norm else None
    kw = (1 + 0.1 * rnd((d,), torch.float32, 10)).to(dtype) if norm else None
    inv = None
    if rot:
        i = torch.arange(rot // 2, dtype=torch.float64)
        inv = (1e6 ** (-(2.0 * i) / rot)).float().cuda()
    kv_got = make_cache(pages, nkv, P, d, dtype, 11)
    kv_ref = kv_got.clone()
    cs = ops().rope_table(positions, inv) if rot else None
    if rot:
        assert (cs.double() - REF.rope_table(positions, inv).double()).abs().max() < 2e-6
    q_got = ops().qk_norm_rope_write(qkv, slots, qw, kw, cs, rot, 1e-6, kv_got, nq, nkv, d)
    q_ref = REF.qk_norm_rope_write(qkv, slots, qw, kw, REF.rope_table(positions, inv) if rot else None, rot, 1e-6,
                                   kv_ref, nq, nkv, d)
    t = tol(dtype, 8)
    assert (q_got.double() - q_ref.double()).abs().max() < t
    assert (kv_got.double() - kv_ref.double()).abs().max() < t
    # a reader entry leaves the pages alone
    kv2 = kv_ref.clone()
    ops().qk_norm_rope_write(qkv, slots, qw, kw, cs, rot, 1e-6, kv2, nq, nkv, d, write_kv=False)
    assert torch.equal(kv2, kv_ref)


@pytest.mark.parametrize("P", [8, 16, 64])
def test_qk_norm_rope_write_many_tokens(P):
    """Enough tokens for the transposing V writer: a prompt portion in consecutive slots that
    starts in the middle of a page, single tokens elsewhere, and tokens that are not written."""
    dtype, nq, nkv, d = torch.bfloat16, 8, 2, 128
    pages = 40
    end = 3 * P + 5 + 83
    slots = list(range(3 * P + 5, end)) + [-1, 1, end + 3, -1, end + 2 * P - 1, 0, 2]
    N = len(slots)
    qkv = rnd((N, (nq + 2 * nkv) * d), dtype, 31)
    positions = torch.arange(N, dtype=torch.int32).cuda() + 11
    slots = torch.tensor(slots, dtype=torch.int32).cuda()
    qw = (1 + 0.1 * rnd((d,), torch.float32, 32)).to(dtype)
    kw = (1 + 0.1 * rnd((d,), torch.float32, 33)).to(dtype)
    i = torch.arange(d // 2, dtype=torch.float64)
    inv = (1e6 ** (-(2.0 * i) / d)).float().cuda()
    kv_got = make_cache(pages, nkv, P, d, dtype, 34)
    kv_ref = kv_got.clone()
    cs = ops().rope_table(positions, inv)
    q_got = ops().qk_norm_rope_write(qkv, slots, qw, kw, cs, d, 1e-6, kv_got, nq, nkv, d)
    q_ref = REF.qk_norm_rope_write(qkv, slots, qw, kw, REF.rope_table(positions, inv), d, 1e-6, kv_ref, nq, nkv, d)
    assert (q_got.double() - q_ref.double()).abs().max() < 0.1
    assert (kv_got.double() - kv_ref.double()).abs().max() < 0.1
    assert torch.equal(v_pages(kv_got), v_pages(kv_ref))  # values are copied, not computed


def test_rotary_reference_vector():
    # q of tests/test_rotary.cpp:98-122: positions {0, 2}, d = 4, theta 1e4.
    # position 0 is the identity; at position 2 pair (x[i], x[i+2]) turns by 2 * theta^(-2i/4)
    q = torch.tensor([[1.0, 2, 3, 4, -1, 0.5, 2, -0.5], [0, 1, -2, 3, 4, -1, 0.25, -0.75]])
    qkv = torch.cat([q, torch.zeros(2, 8)], dim=1).cuda()  # nq = 2, nkv = 1, d = 4
    positions = torch.tensor([0, 2], dtype=torch.int32).cuda()
    slots = torch.tensor([-1, -1], dtype=torch.int32).cuda()
    inv = torch.tensor([1.0, 1e4 ** -0.5]).cuda()
    kv = torch.zeros(1, 2, 1, 4, 4).cuda()
    got = ops().qk_norm_rope_write(qkv, slots, None, None, ops().rope_table(positions, inv), 4, 0.0, kv, 2, 1, 4).cpu()
    assert torch.allclose(got[0].reshape(-1), q[0], atol=1e-7)
    x = q[1].reshape(2, 4)
    want = torch.empty(2, 4)
    for i, f in enumerate([1.0, 0.01]):
        c, s = math.cos(2 * f), math.sin(2 * f)
        want[:, i] = x[:, i] * c - x[:, i + 2] * s
        want[:, i + 2] = x[:, i + 2] * c + x[:, i] * s
    assert torch.allclose(got[1], want, atol=1e-6)


def attention_case(dtype, nq, nkv, d, P, window, lens, seed=12, pages=40, max_pages=12):
    """lens: list of (past, q_len).  Builds a cache with random pages in a
    scrambled block table and random q."""
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    kv = make_cache(pages, nkv, P, d, dtype, seed + 1)
    perm = torch.randperm(pages, generator=g).tolist()
    table = torch.full((5, max_pages), -1, dtype=torch.int32)
    slots = torch.randperm(5, generator=g)[:S].tolist()
    cu, kv_lens, token_seq = [0], [], []
    for s, (past, ql) in enumerate(lens):
        n_pages = (past + ql + P - 1) // P
        assert n_pages <= max_pages
        for i in range(n_pages):
            table[slots[s], i] = perm.pop()
        cu.append(cu[-1] + ql)
        kv_lens.append(past + ql)
        token_seq += [s] * ql
    N = cu[-1]
    q = rnd((N, nq, d), dtype, seed + 2)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32).cuda()
    args = (q, kv, table.cuda(), i32(slots), i32(cu), i32(kv_lens), i32(token_seq), window, 1.0 / math.sqrt(d))
    return args, (min(l for _, l in lens), max(l for _, l in lens)), max(kv_lens)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,P,window", [(4, 2, 16, 4, None), (6, 3, 48, 3, None), (8, 2, 128, 16, None),
                                               (8, 8, 64, 16, 7), (5, 1, 80, 8, 20), (2, 1, 256, 16, None)])
def test_paged_attention(dtype, nq, nkv, d, P, window):
    lens = [(0, 9), (17, 1), (30, 2), (5, 11)]
    args, mq, mk = attention_case(dtype, nq, nkv, d, P, window, lens)
    got = ops().paged_attention(*args, *mq, mk)
    want = REF.paged_attention(*args)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 2)


@pytest.mark.parametrize("nq,nkv,d,P,window", [(8, 2, 128, 16, None), (4, 4, 16, 16, None), (16, 2, 64, 32, None),
                                               (6, 1, 48, 16, 40), (2, 1, 256, 16, None), (32, 8, 128, 16, 700),
                                               (3, 1, 160, 48, None), (5, 5, 80, 16, 9),
                                               # groups of 16 and 32: a decoded token fills a tile, or is more than one
                                               (32, 2, 128, 16, None), (32, 1, 64, 16, None), (32, 1, 128, 32, 300),
                                               (32, 2, 64, 16, None)])
@pytest.mark.parametrize("lens", [
    [(0, 9), (17, 1), (30, 2), (5, 11)],          # portions beside decoded tokens
    [(1999, 1), (640, 1), (31, 1), (0, 1)],       # decoding only, long contexts: key splits
    [(0, 150), (100, 70)],                        # prompt portions only, one after a past
    [(2000, 49)],                                 # a short tail after a long past: keys split over workgroups
    [(1500, 40), (1900, 1), (3, 30)],
])
def test_float32_matrix_core_attention(nq, nkv, d, P, window, lens):
    """The float32 matrix-core kernel (float32 operands, products and sums) against the plain
    form in float64 and against the generic kernel it stands beside."""
    need = max((p + l + P - 1) // P for p, l in lens)
    args, mq, mk = attention_case(torch.float32, nq, nkv, d, P, window, lens,
                                  pages=sum((p + l + P - 1) // P for p, l in lens) + 3, max_pages=need + 1)
    o = ops()
    want = REF.paged_attention(*args).double()
    got = o.paged_attention(*args, *mq, mk)
    o.force_generic_attention = True
    try:
        generic = o.paged_attention(*args, *mq, mk)
    finally:
        o.force_generic_attention = False
    assert (got.double() - want).abs().max() < tol(torch.float32, 2)
    assert (generic.double() - want).abs().max() < tol(torch.float32, 2)
    # one key made to stand out among all that a row sees: its value row comes back
    q, kv, table, slots = args[0], args[1], args[2], args[3]
    past, ql = lens[-1]
    far = max(0, past + ql - 1 - (window - 1 if window else past + ql - 1))  # the first key the last row sees
    page, off = int(table[int(slots[len(lens) - 1]), far // P]), far % P
    kv[page, 0, 0, off, :] = q[-1, 0] * (60.0 / max(1.0, float((q[-1, 0] ** 2).sum()) ** 0.5))
    got = o.paged_attention(*args, *mq, mk).reshape(-1, nq, d)
    assert torch.allclose(got[-1, 0], v_pages(kv)[page, 0, :, off], atol=1e-3)


@pytest.mark.parametrize("nq,nkv,d,P,window", [(8, 2, 128, 16, None), (4, 4, 32, 16, None), (16, 2, 64, 32, None),
                                               (6, 1, 96, 16, 40), (8, 2, 256, 16, None), (32, 8, 128, 16, 700),
                                               (3, 1, 160, 48, None), (8, 2, 128, 48, None), (4, 1, 128, 32, 100),
                                               # groups of 16 and 32: a decoded token fills a tile, or is more than one
                                               (32, 2, 128, 16, None), (32, 1, 64, 16, None), (32, 1, 128, 32, 300),
                                               (32, 2, 64, 16, None), (48, 1, 32, 16, None)])
@pytest.mark.parametrize("lens", [
    [(0, 9), (17, 1), (30, 2), (5, 11)],          # portions beside decoded tokens
    [(1999, 1), (640, 1), (31, 1), (0, 1)],       # decoding only, long contexts: key splits
    [(0, 150), (100, 70)],                        # prompt portions only, one after a past
    [(1200, 3), (64, 64), (15, 1)],
    [(2000, 49)],                                 # a short tail after a long past: keys split over workgroups
    [(1500, 40), (1900, 1), (3, 30)],
])
def test_matrix_core_attention(nq, nkv, d, P, window, lens):
    """The bfloat16 matrix-core kernels against the plain form and the generic kernel; prompt
    portions with every shape of workgroup (four wavefronts of one or of two row tiles, eight of one)."""
    need = max((p + l + P - 1) // P for p, l in lens)
    args, mq, mk = attention_case(torch.bfloat16, nq, nkv, d, P, window, lens, pages=sum((p + l + P - 1) // P for p, l in lens) + 3,
                                  max_pages=need + 1)
    o = ops()
    want = REF.paged_attention(*args)
    for row_tiles in (1, 2, 3):
        o.force_prefill_form = row_tiles
        try:
            got = o.paged_attention(*args, *mq, mk)
        finally:
            o.force_prefill_form = 0
        err = (got.double() - want.double()).abs().max().item()
        assert err < 2e-2, (row_tiles, err)
    o.force_generic_attention = True
    try:
        generic = o.paged_attention(*args, *mq, mk)
    finally:
        o.force_generic_attention = False
    assert (got.double() - generic.double()).abs().max() < 2e-2


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32, None])
@pytest.mark.parametrize("nq,nkv,d,P,window", [(32, 8, 128, 16, None), (4, 4, 64, 32, None), (16, 2, 64, 16, 50),
                                               (6, 1, 192, 48, None), (8, 2, 256, 16, 900),
                                               (32, 2, 128, 16, None), (16, 1, 64, 16, 1100)])  # a group of 16: one token a tile
@pytest.mark.parametrize("lens", [
    [(1999, 1), (640, 1), (31, 1), (0, 1)],   # long contexts: the new key lies in the last of several key splits
    [(15, 1), (16, 1), (47, 1)],              # the new key is the last of a page / the first of a new one
    [(100, 2), (31, 2), (0, 1), (2047, 2)],   # two tokens of a request in one step, across a page's and a step's edge
])
def test_fused_decode_attention_equals_its_two_halves(wdtype, nq, nkv, d, P, window, lens):
    """Norm, rotation, cache write and attention of a decode step in one launch against the
    two kernels it replaces, on the same inputs: the same pages afterwards, the same output."""
    group = nq // nkv
    lens = [(p, min(l, 16 // group)) for p, l in lens if 16 // group >= 1]
    need = max((p + l + P - 1) // P for p, l in lens)
    args, mq, mk = attention_case(torch.bfloat16, nq, nkv, d, P, window, lens,
                                  pages=sum((p + l + P - 1) // P for p, l in lens) + 3, max_pages=need + 1)
    _, kv, table, seq_slots, cu, kv_lens, token_seq, _, scale = args
    N = int(cu[-1])
    qkv = rnd((N, (nq + 2 * nkv) * d), torch.bfloat16, 70, 1.5)
    positions, slots = [], []
    for s, (past, ql) in enumerate(lens):
        for t in range(ql):
            pos = past + t
            positions.append(pos)
            slots.append(int(table[int(seq_slots[s]), pos // P]) * P + pos % P)
    positions = torch.tensor(positions, dtype=torch.int32).cuda()
    slots = torch.tensor(slots, dtype=torch.int32).cuda()
    i = torch.arange(d // 2, dtype=torch.float64)
    inv = (1e6 ** (-(2.0 * i) / d)).float().cuda()
    o = ops()
    cs = o.rope_table(positions, inv)
    qw = kw = None
    if wdtype is not None:
        qw = (1 + 0.2 * rnd((d,), torch.float32, 71)).to(wdtype)
        kw = (1 + 0.2 * rnd((d,), torch.float32, 72)).to(wdtype)
    assert o.can_fuse_rope_attention(torch.bfloat16, d, d, P, group, mq[1], mk, len(lens))
    kv_a, kv_b = kv.clone(), kv.clone()
    q = o.qk_norm_rope_write(qkv, slots, qw, kw, cs, d, 1e-5, kv_a, nq, nkv, d, True)
    want = o.paged_attention(q, kv_a, table, seq_slots, cu, kv_lens, token_seq, window, scale, *mq, mk)
    got = o.qk_norm_rope_attention(qkv, slots, qw, kw, cs, 1e-5, kv_b, nq, nkv, d, True, table, seq_slots, cu,
                                   kv_lens, token_seq, window, scale, mk)
    assert not torch.equal(kv_b, kv), "the new keys and values are written"
    # both round the same 32-bit results to bfloat16; one unit in the last place where a product was fused differently
    assert (kv_a.float() - kv_b.float()).abs().max() <= 2.0 ** -7 * kv_a.float().abs().max()
    assert (got.double() - want.double()).abs().max() < 2e-2
    # without writing (a layer that reads another layer's pages): the pages stay, q is still made
    kv_c = kv_a.clone()
    again = o.qk_norm_rope_attention(qkv, slots, qw, kw, cs, 1e-5, kv_c, nq, nkv, d, False, table, seq_slots, cu,
                                     kv_lens, token_seq, window, scale, mk)
    assert torch.equal(kv_c, kv_a) and (again.double() - want.double()).abs().max() < 2e-2


def test_matrix_core_attention_far_key_and_window_edge():
    """A key hundreds of positions back is made to dominate, with the window
    ending exactly on it (seen) or one short of it (not seen)."""
    nq, nkv, d, P = 8, 2, 128, 16
    for window, seen in ((None, True), (1000 - 37, True), (1000 - 38, False)):
        args, mq, mk = attention_case(torch.bfloat16, nq, nkv, d, P, window, [(999, 1)], pages=70, max_pages=64)
        q, kv, table, slots = args[0], args[1], args[2], args[3]
        far = 37
        page, off = int(table[int(slots[0]), far // P]), far % P
        kv[page, 0, 0, off, :] = q[0, 2] * 4.0  # q head 2 belongs to kv head 0
        got = ops().paged_attention(*args, *mq, mk).reshape(1, nq, d)
        hit = torch.allclose(got[0, 2].float(), v_pages(kv)[page, 0, :, off].float(), atol=2e-2)
        assert hit == seen, (window, hit)


def test_attention_single_token_returns_value():
    # tests/test_attention.cpp:220-281: one token sees only itself, out == V
    args, mq, mk = attention_case(torch.float32, 4, 2, 16, 4, None, [(0, 1)])
    got = ops().paged_attention(*args, *mq, mk).reshape(1, 4, 16)
    q, kv, table, slots = args[0], args[1], args[2], args[3]
    page = int(table[int(slots[0]), 0])
    v = v_pages(kv)[page, :, :, 0]  # [nkv, d]
    assert torch.allclose(got[0], v.repeat_interleave(2, dim=0), atol=1e-6)


def test_attention_far_key_stands_out():
    """One key far back is made to dominate: the output must be its value row."""
    dtype, nq, nkv, d, P = torch.float32, 2, 1, 32, 16
    args, mq, mk = attention_case(dtype, nq, nkv, d, P, None, [(299, 1)], pages=40, max_pages=20)
    q, kv, table, slots = args[0], args[1], args[2], args[3]
    far = 37
    page, off = int(table[int(slots[0]), far // P]), far % P
    kv[page, 0, 0, off, :] = q[0, 0] * 50.0
    got = ops().paged_attention(*args, *mq, mk).reshape(1, nq, d)
    assert torch.allclose(got[0, 0], v_pages(kv)[page, 0, :, off], atol=1e-4)


@pytest.mark.parametrize("V", [7, 503, 151936])
def test_argmax_and_sample(V):
    g = torch.Generator().manual_seed(3)
    logits = torch.randn((6, V), generator=g).cuda()
    logits[1, V // 2] = 50.0
    logits[2, 0] = 60.0
    logits[3, V - 1] = 60.0
    logits[4, :] = 1.0  # all equal: the first wins
    logits[5, V - 1] = 9.0
    logits[5, V // 3] = 9.0  # tie: the lower index wins
    got = ops().argmax(logits).cpu().tolist()
    want = torch.argmax(logits.cpu(), dim=-1).tolist()
    assert got == want
    assert got[4] == 0 and got[5] == V // 3
    temperature = torch.tensor([0.7, 1.0, 0.0, 2.5, 1.0, 0.3]).cuda()
    for seed in range(4):
        u = torch.rand((6,), generator=torch.Generator().manual_seed(seed)).cuda()
        got = ops().sample(logits, temperature, u).cpu().tolist()
        want = REF.sample(logits.cpu(), temperature.cpu(), u.cpu()).tolist()
        for r in range(6):
            if got[r] != want[r]:
                # rounding may move a pick across a boundary of the running sum by one id
                p = torch.softmax(logits[r].double().cpu() / max(float(temperature[r]), 1e-9), 0)
                cdf = torch.cumsum(p, 0)
                lo, hi = sorted((got[r], want[r]))
                assert abs(float(cdf[hi - 1]) - float(u[r])) < 1e-4 and hi - lo <= 2, (r, got[r], want[r])
    assert ops().sample(logits, temperature, u).cpu().tolist()[2] == 0
    # a uniform number that rounds to 1.0 in float32 still picks an id that has weight: row 1 is
    # peaked (all but 1e-17 of the weight on one id), so the running sum passes the target there
    ones = torch.ones((6,), dtype=torch.float32).cuda()
    assert ops().sample(logits, temperature, ones).cpu().tolist()[1] == V // 2
    below = torch.full((6,), 1.0 - 2.0 ** -24, dtype=torch.float32).cuda()
    assert ops().sample(logits, temperature, below).cpu().tolist()[1] == V // 2


@pytest.mark.parametrize("V", [1024, 1025, 70000, 151936])
def test_sample_every_region_of_the_row(V):
    """Uniform numbers spread over [0, 1) against a flat-ish row: picks land in every segment
    of the row and must agree with the exact running sum up to a boundary's rounding."""
    g = torch.Generator().manual_seed(11)
    R = 64
    logits = (0.5 * torch.randn((R, V), generator=g)).cuda()
    temperature = torch.full((R,), 0.9).cuda()
    u = ((torch.arange(R, dtype=torch.float64) + 0.37) / R).float().cuda()
    got = ops().sample(logits, temperature, u).cpu().tolist()
    p = torch.softmax(logits.double().cpu() / 0.9, dim=1)
    cdf = torch.cumsum(p, dim=1)
    want = torch.searchsorted(cdf, u.double().cpu().unsqueeze(1) * cdf[:, -1:], right=True).squeeze(1).tolist()
    assert len(set(w * 8 // V for w in want)) == 8  # every eighth of the row is hit
    for r in range(R):
        if got[r] != want[r]:
            lo, hi = sorted((got[r], want[r]))
            assert hi - lo <= 2 and abs(float(cdf[r, hi - 1]) - float(u[r])) < 1e-5, (r, got[r], want[r])


@pytest.mark.parametrize("V", [1500, 151936])
def test_sample_skips_logits_that_are_no_numbers(V):
    """NaN logits in the middle of a row (and a row with an infinite logit) get no weight: the
    picks are those of the same row with the NaNs set to -inf, wherever the NaNs stand; a row
    whose maximum is +inf is that id."""
    g = torch.Generator().manual_seed(13)
    R = 32
    logits = (0.5 * torch.randn((R, V), generator=g))
    bad = torch.randint(0, V, (R, 5), generator=g)
    bad[:, 0] = V // 2  # one of them in the middle of every row
    clean = logits.clone()
    for r in range(R):
        logits[r, bad[r]] = float("nan")
        clean[r, bad[r]] = float("-inf")
    temperature = torch.full((R,), 0.8)
    u = ((torch.arange(R, dtype=torch.float64) + 0.41) / R).float()
    o = ops()
    got = o.sample(logits.cuda(), temperature.cuda(), u.cuda()).cpu().tolist()
    same = o.sample(clean.cuda(), temperature.cuda(), u.cuda()).cpu().tolist()
    assert got == same
    p = torch.softmax(clean.double() / 0.8, dim=1)
    cdf = torch.cumsum(p, dim=1)
    want = torch.searchsorted(cdf, u.double().unsqueeze(1) * cdf[:, -1:], right=True).squeeze(1).tolist()
    for r in range(R):
        assert got[r] not in bad[r].tolist()
        assert abs(got[r] - want[r]) <= 2 + 5, (r, got[r], want[r])  # a boundary's rounding, and the ids skipped
    logits[3, 77] = float("inf")
    assert o.sample(logits.cuda(), temperature.cuda(), u.cuda()).cpu().tolist()[3] == 77
