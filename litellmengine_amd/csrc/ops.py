"""Python face of the HIP kernels: checks operands on the host, then launches
on the current stream.  Tensors are torch tensors on the GPU (torch is the
allocator and the stream owner; the arithmetic is in `*.hip`).  There is no
CPU path: without a GPU or without the compiled libraries these raise.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..parts.base import PartialSums, Prenormed
from . import build
from .tuning import ProductTuning
from .limits import MAX_HEAD_DIM, MAX_SUMMED_NORM_WIDTH

F32, BF16 = 0, 1
_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64
_F = ctypes.c_float


class KernelError(RuntimeError):
    pass


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, not {dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(t: torch.Tensor, name: str, dtype=None) -> None:
    # (on every operand of every launch: the messages are made only when they are needed)
    if not t.is_cuda:
        raise KernelError(f"{name} must live on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, is {t.dtype}")


# the current stream's handle without the Stream object around it (a launch is a few microseconds
# of Python as it is; torch.cuda.current_stream() alone costs as much again)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream_handle() -> int:
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


class HipOps:
    """The operations a model part may call.  One instance per process is enough."""

    MAX_HEAD_DIM = MAX_HEAD_DIM

    def __init__(self, tuning: Optional[ProductTuning] = None):
        if not torch.cuda.is_available():
            raise KernelError("litellmengine_amd needs a GPU: its kernels have no CPU form")
        self._fn = {}
        self.tuning = tuning or ProductTuning()  # which kernel takes a product (never what it gives)

    # -- plumbing ---------------------------------------------------------
    def _get(self, lib: str, name: str, argtypes):
        key = (lib, name)
        fn = self._fn.get(key)
        if fn is None:
            fn = getattr(build.load_library(lib), name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
            self._fn[key] = fn
        return fn

    def _run(self, lib: str, name: str, argtypes, *args):
        fn = self._get(lib, name, argtypes)
        code = fn(*args, _stream_handle())
        if code != 0:
            msg = build.load_library(lib).lle_error_string(code).decode()
            raise KernelError(f"{name} failed to launch: {msg} (hip error {code})")

    # -- embedding -----------------------------------------------------------
    def embedding(self, ids: torch.Tensor, table: torch.Tensor, feedback=None, token_seq=None,
                  seq_slots=None) -> torch.Tensor:
        """ids int32 [N], table [V, H] -> float32 [N, H] (the residual stream).  With `feedback`
        (int32, indexed by request slot), `token_seq` [N] and `seq_slots`: an id below zero is
        replaced by feedback[seq_slots[token_seq[n]]], the token that argmax(..., scatter=...) left there."""
        _dev(ids, "ids", torch.int32)
        _dev(table, "embedding table")
        _need(ids.dim() == 1 and table.dim() == 2, "embedding wants ids [N] and a table [V, H]")
        N, H = ids.shape[0], table.shape[1]
        if feedback is not None:
            for t, name in ((feedback, "feedback"), (token_seq, "token_seq"), (seq_slots, "seq_slots")):
                _need(t is not None, "feedback, token_seq and seq_slots come together")
                _dev(t, name, torch.int32)
            _need(token_seq.shape == (N,), "token_seq must be [N]")
        out = torch.empty((N, H), dtype=torch.float32, device=table.device)
        self._run("elementwise", "lle_embedding_feedback", [_P, _P, _P, _I, _I, _I, _P, _P, _P, _P],
                  _ptr(ids), _ptr(table), _ptr(out), N, H, dtype_code(table.dtype), _ptr(feedback),
                  _ptr(token_seq) if feedback is not None else None, _ptr(seq_slots) if feedback is not None else None)
        return out

    def embedding_rmsnorm(self, ids, table, weight, eps: float, feedback=None, token_seq=None, seq_slots=None):
        """embedding() and the RMSNorm of its rows in one launch: (float32 [N, H] residual stream,
        [N, H] normed rows in the table's type)."""
        _dev(ids, "ids", torch.int32)
        _dev(table, "embedding table")
        _dev(weight, "norm weight")
        _need(ids.dim() == 1 and table.dim() == 2, "embedding wants ids [N] and a table [V, H]")
        N, H = ids.shape[0], table.shape[1]
        _need(weight.shape == (H,), f"norm weight must be [{H}], is {list(weight.shape)}")
        if feedback is not None:
            for t, name in ((feedback, "feedback"), (token_seq, "token_seq"), (seq_slots, "seq_slots")):
                _need(t is not None, "feedback, token_seq and seq_slots come together")
                _dev(t, name, torch.int32)
            _need(token_seq.shape == (N,), "token_seq must be [N]")
        hidden = torch.empty((N, H), dtype=torch.float32, device=table.device)
        out = torch.empty((N, H), dtype=table.dtype, device=table.device)
        self._run("norm", "lle_embedding_rmsnorm", [_P, _P, _P, _P, _I, _P, _I, _I, _F, _I, _P, _P, _P, _P],
                  _ptr(ids), _ptr(table), _ptr(hidden), _ptr(weight), dtype_code(weight.dtype), _ptr(out), N, H,
                  float(eps), dtype_code(table.dtype), _ptr(feedback),
                  _ptr(token_seq) if feedback is not None else None, _ptr(seq_slots) if feedback is not None else None)
        return hidden, out

    # -- norms ---------------------------------------------------------------
    def add_rmsnorm(self, hidden, delta, weight, eps: float, out_dtype, rows=None) -> torch.Tensor:
        """hidden float32 [N, H] (+ delta [N, H] of out_dtype, or float32 partial sums
        [slices, N, H], bare or as PartialSums, that are added in slice order) -> norm * weight, out_dtype.
        Without `rows` the sum is written back to `hidden` and every row is normed;
        with `rows` (int32 [R]) only those rows are read and nothing is written back."""
        _dev(hidden, "hidden", torch.float32)
        _dev(weight, "norm weight")
        N, H = hidden.shape
        _need(weight.shape == (H,), f"norm weight must be [{H}], is {list(weight.shape)}")
        if isinstance(delta, PartialSums):
            delta = delta.sums
        sums = delta is not None and delta.dim() == 3  # partial sums of a product taken in slices of K
        if sums:
            _dev(delta, "partial sums", torch.float32)
            _need(delta.shape[1:] == hidden.shape and H % 4 == 0 and H <= MAX_SUMMED_NORM_WIDTH,
                  f"partial sums {list(delta.shape)} do not fit the residual stream {list(hidden.shape)}")
        elif delta is not None:
            _dev(delta, "delta", out_dtype)
            _need(delta.shape == hidden.shape, "delta must have the shape of hidden")
        if rows is not None:
            _dev(rows, "rows", torch.int32)
            R = rows.shape[0]
        else:
            R = N
        out = torch.empty((R, H), dtype=out_dtype, device=hidden.device)
        if sums:
            self._run("norm", "lle_add_rmsnorm_sums", [_P, _P, _I, _L, _P, _P, _I, _P, _I, _I, _F, _I, _P],
                      _ptr(hidden), _ptr(delta), delta.shape[0], delta.stride(0), _ptr(rows), _ptr(weight),
                      dtype_code(weight.dtype), _ptr(out), R, H, float(eps), dtype_code(out_dtype))
            return out
        self._run("norm", "lle_add_rmsnorm", [_P, _P, _P, _P, _I, _P, _I, _I, _F, _I, _P],
                  _ptr(hidden), _ptr(delta), _ptr(rows), _ptr(weight), dtype_code(weight.dtype), _ptr(out),
                  R, H, float(eps), dtype_code(out_dtype))
        return out

    def rmsnorm(self, x, weight, eps: float) -> torch.Tensor:
        """x [R, H] -> x * rsqrt(mean(x^2) + eps) * weight, same type."""
        _dev(x, "x")
        _dev(weight, "norm weight")
        R, H = x.shape
        _need(weight.shape == (H,), f"norm weight must be [{H}], is {list(weight.shape)}")
        out = torch.empty_like(x)
        self._run("norm", "lle_rmsnorm", [_P, _P, _I, _P, _I, _I, _F, _I, _P],
                  _ptr(x), _ptr(weight), dtype_code(weight.dtype), _ptr(out), R, H, float(eps), dtype_code(x.dtype))
        return out

    # -- matrix products -------------------------------------------------------
    def can_fold_norm(self, rows: int, width: int, dtype) -> bool:
        """Whether an RMSNorm over `width` of a step of `rows` tokens can be done by the
        products before and after it (the weight-streaming kernel's few-rows forms)."""
        most = 32 if width <= self.tuning.skinny_small_width else self.tuning.skinny_max_rows
        return dtype == torch.bfloat16 and 0 < rows <= most and width % 8 == 0 and not self.force_library_gemm

    def norm_sum_parts(self, width: int) -> int:
        """Into how many column ranges the product before a folded norm over `width` splits the
        sums of squares (one per tile of its launch; the kernel library decides the tiles)."""
        fn = getattr(build.load_library("gemm"), "lle_gemm_skinny_resid_parts")
        fn.argtypes, fn.restype = [_I], _I
        return int(fn(int(width)))

    def _linear_folded(self, x, weight, fold, gated: bool, out_dtype=torch.bfloat16):
        """The forms of the weight-streaming product around a folded norm: `x` a Prenormed
        (its row factors are applied to the result), `fold` a NormFold (the result goes
        into the residual stream and comes back as the next Prenormed)."""
        pre = x if isinstance(x, Prenormed) else None
        xin = pre.xw if pre is not None else x
        _dev(xin, "x", torch.bfloat16)
        _dev(weight, "weight", torch.bfloat16)
        M, K = xin.shape
        N = weight.shape[0]
        _need(weight.shape[1] == K, f"weight [{N}, {weight.shape[1]}] does not fit x [{M}, {K}]")
        _need(K % 8 == 0, f"the weight-streaming product needs a multiple of 8 columns, not {K}")
        _need(pre is None or fold is None, "a product takes a Prenormed or makes one, not both")
        if pre is not None:
            _need(self.can_fold_norm(M, K, xin.dtype), f"a norm over {K} cannot be folded for {M} rows")
            _dev(pre.sums, "sums", torch.float32)
            parts = pre.sums.shape[1]
            _need(pre.sums.shape == (16 if M <= 16 else 32, parts) and pre.xw.shape[1] == K,
                  "sums of squares do not fit")
            _need(not gated or N % 2 == 0, "a gated weight has an even number of rows")
            _need(out_dtype == torch.bfloat16 or (out_dtype == torch.float32 and not gated),
                  "the product after a folded norm writes bfloat16, or float32 where it is not gated")
            out = torch.empty((M, N // 2 if gated else N), dtype=out_dtype, device=xin.device)
            self._run("gemm", "lle_gemm_skinny_scaled_bf16", [_P, _P, _P, _P, _I, _F, _I, _I, _I, _I, _I, _P],
                      _ptr(xin), _ptr(weight), _ptr(out), _ptr(pre.sums), parts, float(pre.eps), M, N, K, int(gated),
                      dtype_code(out_dtype))
            return out
        _dev(fold.hidden, "hidden", torch.float32)
        _dev(fold.weight, "norm weight")
        _need(not gated and fold.hidden.shape == (M, N) and fold.weight.shape == (N,),
              f"residual stream {list(fold.hidden.shape)} does not fit a product [{M}, {N}]")
        _need(self.can_fold_norm(M, N, xin.dtype), f"a norm over {N} cannot be folded for {M} rows")
        xw = torch.empty((M, N), dtype=torch.bfloat16, device=xin.device)
        sums = torch.empty((16 if M <= 16 else 32, self.norm_sum_parts(N)), dtype=torch.float32, device=xin.device)
        self._run("gemm", "lle_gemm_skinny_resid_bf16", [_P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _P],
                  _ptr(xin), _ptr(weight), _ptr(fold.hidden), _ptr(fold.weight), dtype_code(fold.weight.dtype),
                  _ptr(xw), _ptr(sums), M, N, K)
        return Prenormed(xw, sums, fold.eps)

    def linear(self, x, weight, out_dtype=None, fold=None, sums_ok=False):
        """x [M, K] . weight [N, K]^T -> [M, N].  With `sums_ok` the caller takes the result also as
        PartialSums (float32 [slices, M, N], what add_rmsnorm adds into the residual stream).  float32 operands take a true 32-bit
        product: few rows the weight-streaming kernel, more rows a tiled kernel, both
        with the float32 matrix instruction; the plain-FMA kernel where K is no multiple of 4.  bfloat16 operands: few rows take the
        weight-streaming matrix-core kernel, more rows the library product; both
        accumulate in 32-bit and write either result type.  `x` a Prenormed or `fold`
        a NormFold: see _linear_folded."""
        if fold is not None or isinstance(x, Prenormed):
            _need(out_dtype in (None, torch.bfloat16) or (fold is None and out_dtype == torch.float32),
                  "a product that makes a folded norm's input writes bfloat16")
            return self._linear_folded(x, weight, fold, gated=False, out_dtype=out_dtype or torch.bfloat16)
        _dev(x, "x")
        _dev(weight, "weight", x.dtype)
        M, K = x.shape
        N = weight.shape[0]
        _need(weight.shape[1] == K, f"weight [{N}, {weight.shape[1]}] does not fit x [{M}, {K}]")
        out_dtype = out_dtype or x.dtype
        if x.dtype == torch.bfloat16:
            if sums_ok and out_dtype == torch.bfloat16:
                slices = self.slices_for(M, N, K)
                if slices:
                    return PartialSums(self.linear_slices(x, weight, slices))
                slices = self.library_slices_for(M, N, K)
                if slices:
                    # one batched library product over the slices of K, partial sums left in 32-bit
                    xs = x.view(M, slices, K // slices).permute(1, 0, 2)
                    ws = weight.view(N, slices, K // slices).permute(1, 2, 0)
                    return PartialSums(torch.bmm(xs, ws, out_dtype=torch.float32))
            t = self.tuning
            skinny = K % 8 == 0 and not self.force_library_gemm and (
                M <= t.skinny_max_rows
                or (M <= 32 and K <= t.skinny_small_width and N * K <= t.skinny_small_weight)
                # 17 to 32 rows against a weight with many rows for every CU: the streaming kernel with two
                # tiles of X rows in its registers (K a multiple of 1024 up to 4096)
                or (M <= 32 and K % 1024 == 0 and K <= 4096 and N >= t.stream_32_rows_min_share * self.compute_units()))
            if skinny:
                out = torch.empty((M, N), dtype=out_dtype, device=x.device)
                self._run("gemm", "lle_gemm_skinny_bf16", [_P, _P, _P, _I, _I, _I, _I, _P],
                          _ptr(x), _ptr(weight), _ptr(out), M, N, K, dtype_code(out_dtype))
                return out
            # the library product accumulates in 32-bit and can leave the result so
            return torch.mm(x, weight.t()) if out_dtype == torch.bfloat16 else torch.mm(x, weight.t(), out_dtype=out_dtype)
        _need(out_dtype == torch.float32, "a float32 product has a float32 result")
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        if M <= self.tuning.skinny_f32_max_rows and K % 4 == 0 and not self.force_library_gemm:
            # few rows: W streamed once, float32 matrix instruction
            self._run("gemm", "lle_gemm_skinny_f32", [_P, _P, _P, _I, _I, _I, _P], _ptr(x), _ptr(weight), _ptr(out),
                      M, N, K)
            return out
        if K % 4 == 0 and not self.force_simt_gemm:
            # many rows: 64 x 64 tiles through the float32 matrix instruction
            self._run("gemm", "lle_gemm_nt_mfma_f32", [_P, _P, _P, _I, _I, _I, _L, _L, _L, _P],
                      _ptr(x), _ptr(weight), _ptr(out), M, N, K, K, K, N)
            return out
        self._run("gemm", "lle_gemm_nt_simt", [_P, _P, _P, _I, _I, _I, _L, _L, _L, _I, _I, _P],
                  _ptr(x), _ptr(weight), _ptr(out), M, N, K, K, K, N, dtype_code(x.dtype), dtype_code(out_dtype))
        return out

    SLICED_MIN_ROWS, SLICED_MAX_ROWS = 17, 128  # (lle_gemm_mid_slices_max_rows)
    SLICED_UNIT = 1024  # columns of K that a slice is a multiple of (lle_gemm_mid_slices_unit)

    def slices_for(self, M: int, N: int, K: int) -> int:
        """In how many slices of K the product of 17 to 128 rows with a weight [N, K] is taken
        (see linear_slices), or 0 where the library product stays.  Weights with rows enough for
        every CU need no slices.  For the others the slice count is the one that a small model of
        the kernel's time likes best (rounds of N / 64 x slices workgroups over the CUs, each
        taking in its W and X at what a CU takes in, plus the way of the partial sums to the norm
        and back), and it is used where the workgroups fill the CUs in whole rounds (at least
        0.85 of them: o_proj, down_proj of the 8B sizes), or where K is at least twice N and the
        weight is not small: there the library's tiles are too few for the CUs and it does not
        split K (measured at 64 rows: down_proj of the 32B sizes, 5120 x 25600, in 5 slices 76 us
        against the library's 158; of the 14B sizes, 5120 x 17408, in 17 slices 70 against 132)."""
        if not (self.SLICED_MIN_ROWS <= M <= self.SLICED_MAX_ROWS) or N % 64 != 0 or self.force_library_gemm:
            return 0
        if N > MAX_SUMMED_NORM_WIDTH:  # the only reader of the partial sums (add_rmsnorm) takes no wider rows
            return 0
        units, t = self.compute_units(), self.tuning
        groups = N // 64
        if groups > units // 2 or K % self.SLICED_UNIT != 0:  # (rows enough for the library's own tiles)
            return 0
        parts = K // self.SLICED_UNIT
        rows = 32 if M <= 32 else 64 if M <= 64 else 96 if M <= 96 else 128  # the kernel's tiles of X
        best, best_time, best_fill = 0, 0.0, 0.0
        for slices in range(1, min(parts, 32) + 1):
            if parts % slices != 0:
                continue
            rounds = -(-groups * slices // units)
            taken_in = (64 + rows) * (K // slices) * 2  # bytes of W and X through a CU
            seconds = (rounds * (t.sliced_round_seconds + taken_in / t.cu_intake_bytes_per_s)
                       + slices * M * N * 8 / t.partial_sums_bytes_per_s)
            if best == 0 or seconds < best_time:
                best, best_time, best_fill = slices, seconds, groups * slices / (rounds * units)
        if best_fill >= t.sliced_min_fill or (K >= 2 * N and N * K >= t.sliced_long_k_min_weight):
            return best
        return 0

    def library_slices_for(self, M: int, N: int, K: int) -> int:
        """In how many slices of K the LIBRARY takes a product of more than 128 rows whose result is a
        delta of the residual stream, or 0 for the whole product.  The library cuts the result into
        tiles of up to 256 x 256 and does not split K: a weight with few rows and a long K
        (down_proj) leaves CUs without a tile or gets small tiles.  Slices are tiles as well (one
        batched product), up to 4 while the CUs have room for them; the residual add + norm then
        reads float32 partial sums, which costs part of the gain.  Measured at 4096 x 12288 against
        the whole product, both with the norm: 512 rows 90 -> 65 us (4 slices), 1024 rows 126 -> 106
        (4), 2048 rows 214 -> 205 (2), 4096 rows slower (not taken); square weights (o_proj) gain nothing."""
        if M <= self.SLICED_MAX_ROWS or self.force_library_gemm or K < 2 * N:
            return 0
        if N > MAX_SUMMED_NORM_WIDTH or N % 4 != 0:
            return 0
        tiles = -(-M // 256) * -(-N // 256)
        slices = min(self.tuning.library_max_slices, self.compute_units() // tiles)
        while slices > 1 and K % (8 * slices) != 0:
            slices -= 1
        return slices if slices > 1 else 0

    def linear_slices(self, x, weight, slices: int) -> torch.Tensor:
        """x [M, K] . weight [N, K]^T as float32 partial sums over `slices` equal parts of K:
        [slices, M, N], to be added up by the reader in slice order (M <= 128)."""
        _dev(x, "x", torch.bfloat16)
        _dev(weight, "weight", torch.bfloat16)
        M, K = x.shape
        N = weight.shape[0]
        _need(weight.shape[1] == K, f"weight [{N}, {weight.shape[1]}] does not fit x [{M}, {K}]")
        _need(0 < M <= self.SLICED_MAX_ROWS and N % 64 == 0 and slices > 0 and K % (self.SLICED_UNIT * slices) == 0,
              f"no product in {slices} slices for [{M}, {K}] x [{N}, {K}]")
        out = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
        self._run("gemm", "lle_gemm_mid_slices_bf16", [_P, _P, _P, _I, _I, _I, _I, _P], _ptr(x), _ptr(weight), _ptr(out),
                  M, N, K, slices)
        return out

    # (which of these kernels takes a product is decided by the numbers in self.tuning)
    force_library_gemm = False
    force_simt_gemm = False  # tests flip this to reach the plain-FMA kernel at sizes the matrix instruction takes

    # -- attention ---------------------------------------------------------------
    def rope_table(self, positions, inv_freq) -> torch.Tensor:
        """cos and sin of float(position) * inv_freq for every token: float32 [N, len(inv_freq), 2].
        Made once per step; every head of every layer with this rotation reads it."""
        _dev(positions, "positions", torch.int32)
        _dev(inv_freq, "inv_freq", torch.float32)
        N, half = positions.shape[0], inv_freq.shape[0]
        out = torch.empty((N, half, 2), dtype=torch.float32, device=positions.device)
        self._run("rope_kv", "lle_rope_table", [_P, _P, _P, _I, _I, _P], _ptr(positions), _ptr(inv_freq), _ptr(out),
                  N, half)
        return out

    def qk_norm_rope_write(self, qkv, slots, q_weight, k_weight, cos_sin, rotary_dim: int, eps: float, kv_layer,
                           num_q_heads: int, num_kv_heads: int, head_dim: int, write_kv: bool = True) -> torch.Tensor:
        """qkv [N, (nq + 2 nkv) d] -> q [N, nq, d] normed and rotated; K (normed, rotated)
        and V go to the pages `kv_layer` [pages, 2, nkv, page_size, d] at `slots` [N].
        `cos_sin` is rope_table()'s [N, rotary_dim / 2, 2] (None when rotary_dim is 0)."""
        _dev(qkv, "qkv")
        _dev(slots, "slots", torch.int32)
        _dev(kv_layer, "kv_layer", qkv.dtype)
        nq, nkv, d = num_q_heads, num_kv_heads, head_dim
        N = qkv.shape[0]
        _need(qkv.shape == (N, (nq + 2 * nkv) * d), "qkv has the wrong width")
        _need(slots.shape == (N,), "slots must be [N]")
        _need(kv_layer.dim() == 5 and kv_layer.shape[1] == 2 and kv_layer.shape[2] == nkv
              and kv_layer.shape[4] == d, "kv_layer must be [pages, 2, nkv, page_size, d]")
        _need(0 <= rotary_dim <= d and rotary_dim % 2 == 0, "rotary_dim must be even and <= head_dim")
        wd = F32
        for w, name in ((q_weight, "q_norm weight"), (k_weight, "k_norm weight")):
            if w is not None:
                _dev(w, name)
                _need(w.shape == (d,), f"{name} must be [{d}]")
                wd = dtype_code(w.dtype)
        if q_weight is not None and k_weight is not None:
            _need(q_weight.dtype == k_weight.dtype, "q_norm and k_norm weights must share a type")
        if rotary_dim > 0:
            _dev(cos_sin, "cos_sin", torch.float32)
            _need(cos_sin.shape == (N, rotary_dim // 2, 2), "cos_sin must be [N, rotary_dim / 2, 2]")
        page_size = kv_layer.shape[3]
        q_out = torch.empty((N, nq, d), dtype=qkv.dtype, device=qkv.device)
        self._run("rope_kv", "lle_qk_norm_rope_write",
                  [_P, _P, _P, _P, _I, _P, _I, _F, _P, _P, _I, _I, _I, _I, _I, _L, _I, _I, _P],
                  _ptr(qkv), _ptr(slots), _ptr(q_weight), _ptr(k_weight), wd,
                  _ptr(cos_sin) if rotary_dim > 0 else None, rotary_dim, float(eps), _ptr(q_out), _ptr(kv_layer),
                  N, nq, nkv, d, page_size, kv_layer.stride(0), 1 if write_kv else 0, dtype_code(qkv.dtype))
        return q_out

    def paged_attention(self, q, kv_layer, block_table, seq_slots, cu_tokens, kv_lens, token_seq,
                        window: Optional[int], scale: float, min_q_len: int = 0, max_q_len: int = 0,
                        max_kv_len: int = 0) -> torch.Tensor:
        """q [N, nq, d] against the pages -> [N, nq * d].  `min_q_len`, `max_q_len`
        and `max_kv_len` are host-side bounds of this batch; they choose the kernels
        and the number of key splits, never the result.  bfloat16 with head_dim a
        multiple of 32 and a page size a multiple of 16 runs on the matrix cores;
        everything else takes the generic kernel."""
        _dev(q, "q")
        _dev(kv_layer, "kv_layer", q.dtype)
        for t, name in ((block_table, "block_table"), (seq_slots, "seq_slots"), (cu_tokens, "cu_tokens"),
                        (kv_lens, "kv_lens"), (token_seq, "token_seq")):
            _dev(t, name, torch.int32)
        N, nq, d = q.shape
        nkv, page_size = kv_layer.shape[2], kv_layer.shape[3]
        _need(kv_layer.shape[4] == d and kv_layer.shape[1] == 2, "kv_layer must be [pages, 2, nkv, page_size, d]")
        _need(nq % nkv == 0, "q heads must be a multiple of kv heads")
        _need(d <= self.MAX_HEAD_DIM, f"head_dim {d} is larger than the attention kernels take ({self.MAX_HEAD_DIM})")
        _need(token_seq.shape == (N,), "token_seq must be [N]")
        S = seq_slots.shape[0]
        _need(cu_tokens.shape == (S + 1,) and kv_lens.shape == (S,), "cu_tokens [S + 1], kv_lens [S]")
        _need(block_table.dim() == 2, "block_table must be [slots, pages]")
        out = torch.empty((N, nq * d), dtype=q.dtype, device=q.device)
        win = int(window) if window else 0
        mfma = (q.dtype == torch.bfloat16 and d % 32 == 0 and page_size % 16 == 0 and max_q_len > 0
                and max_kv_len > 0 and S <= 65535 and not self.force_generic_attention)
        group = nq // nkv
        if (q.dtype == torch.float32 and d % 16 == 0 and page_size % 16 == 0 and max_q_len > 0 and max_kv_len > 0
                and S <= 65535 and not self.force_generic_attention):
            # float32 on the matrix cores (float32 operands, products and sums)
            rows = max_q_len * group
            row_blocks = 1 if rows <= 16 else -(-rows // 64)
            ns = self.f32_attention_splits(S, nkv, row_blocks, max_q_len, max_kv_len, win)
            ws_o = ws_ml = None
            if ns > 1:
                ws_o = torch.empty((N * nq * ns * d,), dtype=torch.float32, device=q.device)
                ws_ml = torch.empty((N * nq * ns * 2,), dtype=torch.float32, device=q.device)
            self._run("attention", "lle_paged_attention_mfma_f32",
                      [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _I, _I, _F, _I, _I, _P],
                      _ptr(q), _ptr(kv_layer), _ptr(block_table), _ptr(seq_slots), _ptr(cu_tokens), _ptr(kv_lens),
                      _ptr(out), _ptr(ws_o), _ptr(ws_ml), N, S, nq, nkv, d, page_size, kv_layer.stride(0),
                      block_table.shape[1], win, float(scale), row_blocks, ns)
            return out
        if not mfma:
            self._run("attention", "lle_paged_attention_generic",
                      [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _L, _I, _I, _F, _I, _P],
                      _ptr(q), _ptr(kv_layer), _ptr(block_table), _ptr(seq_slots), _ptr(cu_tokens), _ptr(kv_lens),
                      _ptr(token_seq), _ptr(out), N, nq, nkv, d, page_size, kv_layer.stride(0), block_table.shape[1],
                      win, float(scale), dtype_code(q.dtype))
            return out
        min_q_len = min_q_len or 1
        run_decode = min_q_len * group <= 16
        run_prefill = max_q_len * group > 16
        ns_decode = self.decode_splits(S, nkv, max_kv_len, win) if run_decode else 1
        ns_prefill = self.prefill_splits(S, nkv, group, d, max_q_len, max_kv_len, win) if run_prefill else 1
        row_tiles = (self.prefill_form(S, nkv, group, d, max_q_len, max_kv_len, win, ns_prefill, q.device)
                     if run_prefill else 0)
        ns = max(ns_decode, ns_prefill)
        ws_o = ws_ml = None
        if ns > 1:
            ws_o = torch.empty((N * nq * ns * d,), dtype=torch.float32, device=q.device)
            ws_ml = torch.empty((N * nq * ns * 2,), dtype=torch.float32, device=q.device)
        self._run("attention", "lle_paged_attention_mfma",
                  [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _I, _I, _F, _I, _I, _I, _I, _I, _I,
                   _P],
                  _ptr(q), _ptr(kv_layer), _ptr(block_table), _ptr(seq_slots), _ptr(cu_tokens), _ptr(kv_lens),
                  _ptr(token_seq), _ptr(out), _ptr(ws_o), _ptr(ws_ml), N, S, nq, nkv, d, page_size,
                  kv_layer.stride(0), block_table.shape[1], win, float(scale), int(run_decode), ns_decode,
                  int(run_prefill), ns_prefill, max_q_len, row_tiles)
        return out

    def can_fuse_rope_attention(self, dtype, head_dim: int, rotary_dim: int, page_size: int, group: int,
                                max_q_len: int, max_kv_len: int, num_seqs: int) -> bool:
        """Whether qk_norm_rope_attention takes this step: bfloat16, a rotation over the whole head
        of a multiple of 64 elements, and only requests of at most 16 / group tokens (decode steps)."""
        return (dtype == torch.bfloat16 and head_dim % 64 == 0 and head_dim <= self.MAX_HEAD_DIM
                and rotary_dim == head_dim and page_size % 16 == 0 and 0 < max_q_len and max_q_len * group <= 16
                and max_kv_len > 0 and num_seqs <= 65535 and not self.force_generic_attention
                and not self.force_separate_rope)

    def qk_norm_rope_attention(self, qkv, slots, q_weight, k_weight, cos_sin, eps: float, kv_layer, nq: int,
                               nkv: int, d: int, write_kv: bool, block_table, seq_slots, cu_tokens, kv_lens,
                               token_seq, window: Optional[int], scale: float, max_kv_len: int) -> torch.Tensor:
        """qk_norm_rope_write and paged_attention of a decode step in one launch (see
        can_fuse_rope_attention): the workgroup whose keys include a new token's position writes
        its K and V, every workgroup norms and rotates the q rows it multiplies."""
        _dev(qkv, "qkv", torch.bfloat16)
        _dev(kv_layer, "kv_layer", torch.bfloat16)
        _dev(cos_sin, "cos_sin", torch.float32)
        for t, name in ((slots, "slots"), (block_table, "block_table"), (seq_slots, "seq_slots"),
                        (cu_tokens, "cu_tokens"), (kv_lens, "kv_lens"), (token_seq, "token_seq")):
            _dev(t, name, torch.int32)
        N = qkv.shape[0]
        page_size = kv_layer.shape[3]
        _need(qkv.shape[1] == (nq + 2 * nkv) * d, "qkv must be [N, (nq + 2 nkv) * d]")
        _need(tuple(kv_layer.shape[1:]) == (2, nkv, page_size, d), "kv_layer must be [pages, 2, nkv, page_size, d]")
        _need(slots.shape == (N,) and token_seq.shape == (N,), "slots and token_seq must be [N]")
        _need(cos_sin.shape == (N, d // 2, 2), f"cos_sin must be [{N}, {d // 2}, 2]")
        _need((q_weight is None) == (k_weight is None), "q and k norm weights come together")
        wcode = 0
        if q_weight is not None:
            _dev(q_weight, "q_weight")
            _dev(k_weight, "k_weight", q_weight.dtype)
            _need(q_weight.shape == (d,) and k_weight.shape == (d,), f"q/k norm weights must be [{d}]")
            wcode = dtype_code(q_weight.dtype)
        S = seq_slots.shape[0]
        _need(cu_tokens.shape == (S + 1,) and kv_lens.shape == (S,), "cu_tokens [S + 1], kv_lens [S]")
        _need(nq % nkv == 0 and d % 64 == 0 and page_size % 16 == 0 and S <= 65535,
              "the fused decode attention does not take these sizes")
        win = int(window) if window else 0
        ns = self.decode_splits(S, nkv, max_kv_len, win)
        out = torch.empty((N, nq * d), dtype=torch.bfloat16, device=qkv.device)
        ws_o = ws_ml = None
        if ns > 1:
            ws_o = torch.empty((N * nq * ns * d,), dtype=torch.float32, device=qkv.device)
            ws_ml = torch.empty((N * nq * ns * 2,), dtype=torch.float32, device=qkv.device)
        self._run("attention", "lle_qk_norm_rope_attention_decode",
                  [_P, _P, _P, _P, _I, _P, _F, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _I, _I,
                   _F, _I, _P],
                  _ptr(qkv), _ptr(slots), _ptr(q_weight), _ptr(k_weight), wcode, _ptr(cos_sin), float(eps),
                  int(bool(write_kv)), _ptr(kv_layer), _ptr(block_table), _ptr(seq_slots), _ptr(cu_tokens),
                  _ptr(kv_lens), _ptr(token_seq), _ptr(out), _ptr(ws_o), _ptr(ws_ml), N, S, nq, nkv, d, page_size,
                  kv_layer.stride(0), block_table.shape[1], win, float(scale), ns)
        return out

    force_generic_attention = False  # tests flip this to compare the two families of kernels
    force_prefill_form = 0           # tests set 1, 2 or 3 to reach every shape of the prompt-portion workgroups
    force_separate_rope = False      # tests flip this to compare the fused decode step with its two halves
    # measured on MI355X: about one workgroup per CU and at least 8 32-key steps (two per
    # wavefront) per split are best; more splits cost more in partial results than they gain
    DECODE_MIN_STEPS_PER_SPLIT = 8
    DECODE_MIN_STEPS_TO_SPLIT = 32

    PREFILL_MIN_STEPS_PER_SPLIT = 8

    def prefill_splits(self, num_seqs: int, num_kv_heads: int, group: int, head_dim: int, max_q_len: int,
                       max_kv_len: int, window: int) -> int:
        """Key splits of the prompt-portion kernel: 1 unless the portions are short and come after a
        long past, when their row blocks alone leave most of the chip idle.  Only the keys that
        every row sees count (the past; a prompt from an empty cache is never split: measured
        twice as slow at 512 tokens).  A split keeps at least 8 steps of 32 keys while the row
        blocks fill less than half the CUs and 32 otherwise, the splits fill the CUs once, and
        twice where every split still keeps 32 steps, at least two row blocks share the keys of a
        head and the row blocks alone fill at most half the CUs (measured: 128 tokens after 1 k keys 26 -> 20 us with 4 splits, 512 tokens after 16 k
        keys 289 -> 149 us with 4, 512 tokens after 1 k keys best unsplit; row blocks that fill the
        CUs by themselves are never split: 2048 tokens after 2048 keys 115 us unsplit, 151 in two;
        four requests of 32 tokens after 16 k keys 57 us in 8 splits, one workgroup a CU, 70 in 16)."""
        units = self.compute_units()
        rows_per_block = 128 if head_dim <= 128 else 64
        blocks = ((max_q_len * group + rows_per_block - 1) // rows_per_block) * num_kv_heads * max(1, num_seqs)
        past = max_kv_len - max_q_len
        if window:
            past = min(past, window)
        steps = max(0, past) // 32
        by_work = max(1, steps // (self.PREFILL_MIN_STEPS_PER_SPLIT if 2 * blocks < units else 32))
        by_fill = max(1, units // blocks)
        splits = min(by_work, by_fill)
        shared_keys = max_q_len * group >= 2 * rows_per_block  # else the keys' way from memory bounds the launch
        if splits == by_fill and 2 * blocks <= units and shared_keys and steps // (2 * splits) >= 32:
            splits *= 2
        return int(min(splits, 64))

    _compute_units: dict = {}

    def compute_units(self, device=None) -> int:
        """CUs of `device` (the current one if not given), asked once per device."""
        key = device.index if device is not None and device.index is not None else torch.cuda.current_device()
        if key not in self._compute_units:
            self._compute_units[key] = torch.cuda.get_device_properties(key).multi_processor_count
        return self._compute_units[key]

    def prefill_form(self, num_seqs: int, num_kv_heads: int, group: int, head_dim: int, max_q_len: int,
                     max_kv_len: int, window: int, nsplit: int, device) -> int:
        """The shape of the prompt-portion kernel's workgroups:
          1: four wavefronts of one 16-row tile each (64 rows a workgroup),
          2: four wavefronts of two tiles each (128 rows; every operand read from LDS serves both tiles),
          3: eight wavefronts of one tile each (128 rows; four wavefronts a SIMD; heads of 128 only).
        The low form when its workgroups all fit the chip at once (a short portion; at heads of 128
        at most one workgroup a CU, or one prompt from an empty cache); else the tall ones, which share a pass over the keys between more
        rows: form 3 at heads of 128, form 2 below.  Measured on MI355X at heads of 128 (forms 1 / 2 / 3): 2048 tokens from an empty cache
        60 / 65 / 57 us, 2048 tokens after 2048 keys 148 / 128 / 118 us, 49 tokens after 2048 keys
        17 / 21 / 19 us."""
        if head_dim > 128:
            return 1
        if self.force_prefill_form:
            return self.force_prefill_form if head_dim == 128 or self.force_prefill_form < 3 else 2
        resident = 2 * self.compute_units(device)
        rows = max_q_len * group
        low = -(-rows // 64) * num_kv_heads * max(1, num_seqs) * max(1, nsplit)
        if head_dim == 128:
            # (measured: a launch of at most one low workgroup a CU is about 1 us, up to 10 %, faster in
            # the low form, whatever its past and however many requests; so is one prompt from an empty
            # cache while the low form fits the chip at once; else form 3 wins by 5-15 %)
            units = resident // 2
            return 1 if low <= units or (low <= resident and max_kv_len <= max_q_len and num_seqs <= 1) else 3
        return 1 if low <= resident else 2

    def f32_attention_splits(self, num_seqs: int, num_kv_heads: int, row_blocks: int, max_q_len: int,
                             max_kv_len: int, window: int) -> int:
        """Key splits of the float32 matrix-core kernel: enough workgroups for one round of the CUs
        (measured: more cost 10 % at batch 8 and at 512-token portions), at least 4 of its 16-key
        steps each (measured at 512 keys: batch 1 in 2 / 8 splits 20 / 12 us, batch 8 in 2 / 4 splits
        22 / 18 us)."""
        span = min(max_kv_len, window + max_q_len) if window else max_kv_len
        steps = (span + 15) // 16
        by_work = max(1, steps // 4)
        by_fill = max(1, self.compute_units() // max(1, num_seqs * num_kv_heads * row_blocks))
        return int(min(by_work, by_fill, 64))

    def decode_splits(self, num_seqs: int, num_kv_heads: int, max_kv_len: int, window: int) -> int:
        """Key splits of the decode kernel: enough workgroups to fill the chip, but
        at least DECODE_MIN_STEPS_PER_SPLIT 32-key steps each, and none below DECODE_MIN_STEPS_TO_SPLIT steps: the merge
        that splits need is a launch of its own and costs what those steps take (measured at 512 keys:
        batch 16 unsplit 12.1 us, in two 14.2; batch 1 the same either way)."""
        span = min(max_kv_len, window + 32) if window else max_kv_len
        steps = (span + 31) // 32 + (1 if window else 0)
        by_work = max(1, steps // self.DECODE_MIN_STEPS_PER_SPLIT) if steps >= self.DECODE_MIN_STEPS_TO_SPLIT else 1
        by_fill = max(1, self.compute_units() // max(1, num_seqs * num_kv_heads))
        return int(min(by_work, by_fill, 64))

    def add_bias(self, x, bias) -> torch.Tensor:
        """x [M, N] += bias [N], in place (the sum in 32-bit); returns x."""
        _dev(x, "x")
        _dev(bias, "bias")
        _need(x.dim() == 2 and bias.shape == (x.shape[1],), f"bias {list(bias.shape)} does not fit x {list(x.shape)}")
        self._run("elementwise", "lle_add_bias", [_P, _P, _I, _I, _I, _I, _P], _ptr(x), _ptr(bias), x.shape[0],
                  x.shape[1], dtype_code(x.dtype), dtype_code(bias.dtype))
        return x

    # -- feed-forward --------------------------------------------------------------
    def silu_mul(self, gate_up) -> torch.Tensor:
        """gate_up [N, 2 I] (gate columns first) -> silu(gate) * up, [N, I]."""
        _dev(gate_up, "gate_up")
        N, two_i = gate_up.shape
        _need(two_i % 2 == 0, "gate_up must have an even width")
        out = torch.empty((N, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
        self._run("elementwise", "lle_silu_mul", [_P, _P, _I, _I, _I, _P],
                  _ptr(gate_up), _ptr(out), N, two_i // 2, dtype_code(gate_up.dtype))
        return out

    def gate_up_silu(self, x, weight) -> torch.Tensor:
        """x [M, K], weight [2 I, K] (gate rows, then up rows) -> silu(x gate^T) * (x up^T), [M, I].
        Few bfloat16 rows run as ONE weight-streaming launch with the activation in its
        epilogue; otherwise the product and silu_mul."""
        if isinstance(x, Prenormed):
            return self._linear_folded(x, weight, None, gated=True)
        _dev(x, "x")
        _dev(weight, "weight", x.dtype)
        M, K = x.shape
        N2 = weight.shape[0]
        _need(weight.shape[1] == K and N2 % 2 == 0, f"weight {list(weight.shape)} does not fit x [{M}, {K}]")
        few = M <= self.tuning.skinny_max_rows or (M <= 32 and N2 * K <= self.tuning.skinny_small_weight)
        if x.dtype == torch.bfloat16 and few and K % 8 == 0 and not self.force_library_gemm:
            out = torch.empty((M, N2 // 2), dtype=x.dtype, device=x.device)
            self._run("gemm", "lle_gemm_skinny_gated_bf16", [_P, _P, _P, _I, _I, _I, _P],
                      _ptr(x), _ptr(weight), _ptr(out), M, N2, K)
            return out
        return self.silu_mul(self.linear(x, weight))

    # -- picking tokens --------------------------------------------------------------
    def argmax(self, logits, scatter=None) -> torch.Tensor:
        """float32 [R, V] -> int32 [R], first maximum wins.  `scatter` = (dst int32, index int32 [R]):
        the pick of row r is also written to dst[index[r]] (the host has made sure that index is in range)."""
        _dev(logits, "logits", torch.float32)
        R, V = logits.shape
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
        chunks = max(1, min(64, V // 2048))  # enough workgroups to stream a long row from all CUs
        part_val = torch.empty((R * chunks,), dtype=torch.float32, device=logits.device)
        part_idx = torch.empty((R * chunks,), dtype=torch.int32, device=logits.device)
        dst = index = None
        if scatter is not None:
            dst, index = scatter
            _dev(dst, "scatter destination", torch.int32)
            _dev(index, "scatter index", torch.int32)
            _need(index.shape == (R,), "one scatter index for every row")
        self._run("sampling", "lle_argmax_rows_scatter", [_P, _P, _P, _P, _I, _I, _I, _P, _P, _P],
                  _ptr(logits), _ptr(out), _ptr(part_val), _ptr(part_idx), R, V, chunks, _ptr(dst), _ptr(index))
        return out

    def sample(self, logits, temperature, uniform) -> torch.Tensor:
        """float32 logits [R, V], temperature [R] (<= 0: greedy), uniform [R] in [0, 1) -> int32 [R]."""
        _dev(logits, "logits", torch.float32)
        _dev(temperature, "temperature", torch.float32)
        _dev(uniform, "uniform", torch.float32)
        R, V = logits.shape
        _need(temperature.shape == (R,) and uniform.shape == (R,), "temperature and uniform must be [R]")
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
        self._run("sampling", "lle_sample_rows", [_P, _P, _P, _P, _I, _I, _P],
                  _ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(out), R, V)
        return out


    # -- measured peaks (the benchmark's rooflines) ---------------------------------------------
    def probe_read_stream(self, data: torch.Tensor, blocks: int) -> None:
        """Launch a kernel that only reads `data` (any type, a multiple of 16 bytes), `blocks` workgroups."""
        _dev(data, "data")
        nbytes = data.numel() * data.element_size()
        _need(nbytes % 16 == 0 and nbytes > 0, "the read probe takes a multiple of 16 bytes")
        self._run("probe", "lle_probe_read_stream", [_P, _L, _I, _P, _P], _ptr(data), nbytes, int(blocks), None)

    def probe_mfma(self, dtype, blocks: int, iters: int) -> float:
        """Launch a kernel of nothing but matrix instructions on registers; returns its flops."""
        self._run("probe", "lle_probe_mfma", [_I, _I, _I, _P, _P], dtype_code(dtype), int(blocks), int(iters), None)
        per_instruction = 2.0 * 16 * 16 * (32 if dtype == torch.bfloat16 else 4)
        return per_instruction * 16 * iters * 4 * blocks


_default: Optional[HipOps] = None


def default_ops() -> HipOps:
    global _default
    if _default is None:
        _default = HipOps()
    return _default
