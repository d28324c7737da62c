"""What was measured on one chip and decides WHICH kernel takes a product: never a result.

Every number here was found on an MI355X (256 CUs, HBM3E) with the weights of the Qwen3 sizes
from 0.6B to 32B.  They sit in one object, `HipOps.tuning`, so that another chip or another family
of widths replaces the numbers and not the code that reads them; `HipOps(tuning=...)` takes
another set."""
from __future__ import annotations

import dataclasses


@dataclasses.dataclass(frozen=True)
class ProductTuning:
    # bfloat16 products of up to this many rows (one tile of matrix-core columns) take the
    # weight-streaming kernels, with the norm folded into them: at batch 12 / 16 of the 8B sizes 14 % /
    # 10 % faster than the library products beside separate norms; more rows take the sliced kernel
    # or the library (the 32-row forms at batch 17 / 32 of the 8B sizes: 7.3 / 9.2 against 6.3 / 7.5 ms a step)
    skinny_max_rows: int = 16
    # ... up to 32 rows where the weight is this small (elements) or the model this narrow: a launch
    # is then as short as a launch can be, and one launch with the norm in it beats two
    skinny_small_weight: int = 1 << 25
    skinny_small_width: int = 2048
    # 17 to 32 rows: the weight-streaming kernel (two tiles of X rows in its registers, K up to 4096)
    # takes a plain product whose weight has at least this many rows for every CU (gate_up and the
    # head of the 8B sizes: 41-43 against the library's 49 us, 239-250 against 270; qkv, 24 rows a CU,
    # is the library's: 15-17 against 15 us)
    stream_32_rows_min_share: int = 64
    # the float32 twin takes up to this many rows (the tiled float32 kernel wastes its 64-row tiles on fewer)
    skinny_f32_max_rows: int = 64
    # the sliced product (17 to 128 rows) is taken where its workgroups fill at least this share
    # of whole rounds of the CUs ...
    sliced_min_fill: float = 0.85
    # ... or where K is at least twice N and the weight has at least this many elements
    sliced_long_k_min_weight: int = 1 << 23
    # the small model of the sliced kernel's time: a round of workgroups costs `sliced_round_seconds`
    # plus the bytes of W and X that a CU takes in, at `cu_intake_bytes_per_s`; the partial sums
    # travel to the norm that adds them at `partial_sums_bytes_per_s`
    sliced_round_seconds: float = 3e-6
    cu_intake_bytes_per_s: float = 29e9
    partial_sums_bytes_per_s: float = 5e12
    # most slices of K that a library product of more than 128 rows is cut into
    library_max_slices: int = 4
