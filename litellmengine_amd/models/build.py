"""From a configuration or a model folder to a model with its weights bound."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import Architecture, architecture_of, get_architecture
from ..config.model_config import read_config_json
from ..parts.base import BuildContext
from ..weights.loader import load_checkpoint
from ..weights.random_init import random_weights
from ..weights.spec import TensorSpec


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float32):
            return name
        raise ValueError(f"the engine computes in bfloat16 or float32, not {name}")
    table = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}
    try:
        return table[str(name)]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}; use bfloat16 or float32") from None


def expected_tensors(arch: Architecture, config) -> Dict[str, TensorSpec]:
    return arch.build(config).tensor_specs()


def make_context(dtype, device=None, ops=None) -> BuildContext:
    dtype = parse_dtype(dtype)
    if ops is None:
        from ..csrc.ops import default_ops

        ops = default_ops()
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    return BuildContext(dtype=dtype, device=torch.device(device), ops=ops)


def load_model(model_dir: str, dtype, device=None, ops=None):
    """config.json picks the architecture; the checkpoint is checked against the
    model's tensor list and bound by name."""
    d = read_config_json(model_dir)
    arch = architecture_of(d)
    config = arch.config_class.from_dict(d)
    model = arch.build(config)
    ctx = make_context(dtype, device, ops)
    weights = load_checkpoint(model_dir, model.tensor_specs(), ctx.dtype, ctx.device)
    model.bind(weights, ctx)
    return model


def random_model(config, seed: int, dtype, device=None, ops=None):
    """A model of `config` with seeded random weights made on the device (no files)."""
    arch = get_architecture(config.architecture)
    model = arch.build(config)
    ctx = make_context(dtype, device, ops)
    weights = random_weights(model.tensor_specs(), seed, ctx.dtype, ctx.device)
    model.bind(weights, ctx)
    return model
