"""Weights from safetensors, bound by tensor name.

The reference reads a private per-tensor `.bin` format made offline from
safetensors (src/weights/weight_loader.cpp:122-178, scripts/convert_weights.py)
and binds by the checkpoint's names with `WeightMap::take`
(include/weights/weight_map.hpp:12-57); a missing name throws, a wrong shape
throws, and tensors left over after binding are an error (src/main.cpp:161-165).
This loader reads `model.safetensors` (or the shards named by
`model.safetensors.index.json`) directly and reports all three kinds of fault
in ONE error before any tensor is copied.

Storage policy: the engine's 16-bit mode keeps float tensors in bfloat16 (F16
is converted), a tensor stored in 32-bit stays 32-bit, integer tables become
int32.  The 32-bit mode converts every float tensor to float32.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Iterable, List, Mapping, Tuple

import torch

from .spec import TensorSpec

_FLOAT_DTYPES = {"F64", "F32", "F16", "BF16"}
_INT_DTYPES = {"I64", "I32", "I16", "I8", "U8"}
WEIGHTS_FILE = "model.safetensors"
INDEX_FILE = "model.safetensors.index.json"


class WeightError(ValueError):
    """A checkpoint that does not fit the model; the message lists every fault."""


def _shard_files(model_dir: str) -> List[str]:
    index = os.path.join(model_dir, INDEX_FILE)
    single = os.path.join(model_dir, WEIGHTS_FILE)
    if os.path.isfile(index):
        with open(index) as f:
            weight_map = json.load(f).get("weight_map", {})
        files = sorted(set(weight_map.values()))
        missing = [n for n in files if not os.path.isfile(os.path.join(model_dir, n))]
        if missing:
            raise WeightError(f"{index} names shard files that do not exist: {', '.join(missing)}")
        return [os.path.join(model_dir, n) for n in files]
    if os.path.isfile(single):
        return [single]
    raise WeightError(f"no {WEIGHTS_FILE} (or {INDEX_FILE}) in {model_dir}")


def checkpoint_header(model_dir: str) -> Dict[str, Tuple[str, Tuple[int, ...], str]]:
    """name -> (file, shape, safetensors dtype string), from the headers only."""
    from safetensors import safe_open

    header: Dict[str, Tuple[str, Tuple[int, ...], str]] = {}
    duplicates = []
    for path in _shard_files(model_dir):
        with safe_open(path, framework="pt") as f:
            for name in f.keys():
                if name in header:
                    duplicates.append(name)  # scripts/convert_weights.py:103-119
                sl = f.get_slice(name)
                header[name] = (path, tuple(int(s) for s in sl.get_shape()), str(sl.get_dtype()))
    if duplicates:
        raise WeightError(f"tensors stored in more than one shard: {', '.join(sorted(duplicates))}")
    return header


def check_against(header: Mapping[str, Tuple[str, Tuple[int, ...], str]], expected: Mapping[str, TensorSpec]) -> None:
    missing = sorted(n for n, s in expected.items() if n not in header and not s.optional)
    unexpected = sorted(n for n in header if n not in expected)
    wrong_shape = []
    wrong_dtype = []
    for name, spec in expected.items():
        if name not in header:
            continue
        _, shape, dtype = header[name]
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append(f"{name}: stored {list(shape)}, model wants {list(spec.shape)}")
        ok = _INT_DTYPES if spec.integer else _FLOAT_DTYPES
        if dtype not in ok:
            wrong_dtype.append(f"{name}: stored as {dtype}")
    if missing or unexpected or wrong_shape or wrong_dtype:
        parts = []
        if missing:
            parts.append(f"missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            parts.append(f"unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            parts.append(f"wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        if wrong_dtype:
            parts.append(f"unsupported dtypes ({len(wrong_dtype)}): " + "; ".join(wrong_dtype))
        raise WeightError("checkpoint does not fit the model:\n  " + "\n  ".join(parts))


def storage_dtype(stored: str, integer: bool, compute_dtype: torch.dtype) -> torch.dtype:
    if integer:
        return torch.int32
    if compute_dtype == torch.float32:
        return torch.float32
    if stored in ("F32", "F64"):
        return torch.float32  # stored in 32-bit: stays so
    return torch.bfloat16


def load_checkpoint(
    model_dir: str,
    expected: Mapping[str, TensorSpec],
    compute_dtype: torch.dtype,
    device,
) -> Dict[str, torch.Tensor]:
    """Check the whole checkpoint against `expected`, then read every tensor to `device`."""
    from safetensors import safe_open

    header = checkpoint_header(model_dir)
    check_against(header, expected)
    by_file: Dict[str, List[str]] = {}
    for name in expected:
        if name in header:
            by_file.setdefault(header[name][0], []).append(name)
    out: Dict[str, torch.Tensor] = {}
    for path, names in by_file.items():
        with safe_open(path, framework="pt") as f:
            for name in names:
                t = f.get_tensor(name)
                dt = storage_dtype(header[name][2], expected[name].integer, compute_dtype)
                out[name] = t.to(device=device, dtype=dt).contiguous()
    return out
