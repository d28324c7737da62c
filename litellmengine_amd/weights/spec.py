"""What a model expects of a checkpoint: tensor names with shapes."""
from __future__ import annotations

import dataclasses
from typing import Tuple

# how the random-weights mode fills a tensor
INIT_NORMAL = "normal"  # N(0, 0.02): projections, embedding tables
INIT_NORM = "norm"  # 1 + U(-0.1, 0.1): norm weights


@dataclasses.dataclass(frozen=True)
class TensorSpec:
    shape: Tuple[int, ...]
    init: str = INIT_NORMAL
    optional: bool = False  # may be absent from the checkpoint (a tied output head)
    integer: bool = False  # an integer table: kept as int32 in every mode
