"""Seeded random weights: in memory (benchmarks) or written as a model folder.

The reference has no such mode in product code; its tests write literals or
patterns by hand (tests/test_paged_generate_engine.cpp:64-91).  Distributions:
projections and embedding tables N(0, 0.02), norm weights 1 + U(-0.1, 0.1).
Every tensor has a generator of its own, seeded by (seed, name), so the values
of a tensor do not depend on which other tensors exist or in which order they
are made.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Dict, Mapping

import torch

from .loader import WEIGHTS_FILE
from .spec import INIT_NORM, INIT_NORMAL, TensorSpec


def _seed_of(seed: int, name: str) -> int:
    return (int(seed) * 1000003 + zlib.crc32(name.encode())) % (2**63 - 1)


def random_tensor(name: str, spec: TensorSpec, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(_seed_of(seed, name))
    if spec.integer:
        raise ValueError(f"{name}: no random rule for integer tables")
    if spec.init == INIT_NORMAL:
        t = torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, 0.02, generator=gen)
    elif spec.init == INIT_NORM:
        t = torch.empty(spec.shape, dtype=torch.float32, device=device).uniform_(-0.1, 0.1, generator=gen) + 1.0
    else:
        raise ValueError(f"{name}: unknown init rule {spec.init!r}")
    return t.to(dtype)


def random_weights(
    expected: Mapping[str, TensorSpec],
    seed: int,
    dtype: torch.dtype,
    device="cpu",
    include_optional: bool = False,
) -> Dict[str, torch.Tensor]:
    out = {}
    for name, spec in expected.items():
        if spec.optional and not include_optional:
            continue
        out[name] = random_tensor(name, spec, seed, dtype, device)
    return out


def write_model_dir(config, path: str, seed: int, dtype: torch.dtype = torch.bfloat16) -> None:
    """Write `config.json` and `model.safetensors` for `config` (a typed
    configuration of a registered architecture) with seeded random weights."""
    from safetensors.torch import save_file

    from ..config import get_architecture
    from ..models.build import expected_tensors

    arch = get_architecture(config.architecture)
    tensors = random_weights(expected_tensors(arch, config), seed, dtype)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, WEIGHTS_FILE))
