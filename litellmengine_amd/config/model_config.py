"""Typed model configurations, read from an architecture's own config.json keys.

The reference keeps one flat `ModelConfig` filled by `load_model_config`
(include/model/model_config.hpp:7-24, src/model/model_config.cpp:33-90) and
validates it in `check_qwen3_config` (src/model/qwen3.cpp:19-75).  Here every
architecture owns a frozen dataclass with a `from_dict`, and the registry
(`registry.py`) picks the class by `architectures[0]`.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a model this engine can build."""


def _required(d: Dict[str, Any], key: str, kind):
    if key not in d or d[key] is None:
        raise ConfigError(f"Missing required config field: {key}")
    return _typed(d[key], key, kind)


def _optional(d: Dict[str, Any], key: str, kind, default):
    if key not in d or d[key] is None:
        return default
    return _typed(d[key], key, kind)


def _typed(value, key, kind):
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"config field {key} must be an integer, got {value!r}")
        return value
    if kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"config field {key} must be a number, got {value!r}")
        return float(value)
    if kind is bool:
        if not isinstance(value, bool):
            raise ConfigError(f"config field {key} must be true or false, got {value!r}")
        return value
    raise TypeError(kind)


FULL_ATTENTION = "full_attention"
SLIDING_ATTENTION = "sliding_attention"


@dataclasses.dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense.  Field names are the config.json keys.

    Keys and defaults follow src/model/model_config.cpp:45-87:
    `num_key_value_heads` defaults to `num_attention_heads`, `head_dim` to
    `hidden_size // num_attention_heads` (real Qwen3 files carry it
    explicitly: q width may differ from hidden), `rms_norm_eps` to 1e-6,
    `rope_theta` to 1e4, `tie_word_embeddings` to false,
    `max_position_embeddings` to 32768 (parsed, never used by the reference).
    `sliding_window` + `layer_types` are read in addition: the reference
    ignores them (all layers attend to all keys), here a layer typed
    "sliding_attention" sees the last `sliding_window` keys only.
    eps and theta stay double here and are cast where a kernel takes them.
    """

    architecture: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    sliding_window: Optional[int]
    layer_types: Tuple[str, ...]

    ARCHITECTURE = "Qwen3ForCausalLM"
    MODEL_TYPE = "qwen3"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Qwen3Config":
        archs = d.get("architectures") or [cls.ARCHITECTURE]
        heads = _required(d, "num_attention_heads", int)
        hidden = _required(d, "hidden_size", int)
        layers = _required(d, "num_hidden_layers", int)
        if heads <= 0:
            raise ConfigError("num_attention_heads must be positive")
        if d.get("attention_bias", False):
            raise ConfigError("attention_bias=true is not supported (Qwen3 projections carry no bias)")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act={act!r} is not supported (Qwen3 uses silu)")
        if d.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported")
        window = _optional(d, "sliding_window", int, None)
        types = d.get("layer_types")
        if types is None:
            if d.get("use_sliding_window", False) and window is not None:
                first = _optional(d, "max_window_layers", int, layers)
                types = [SLIDING_ATTENTION if i >= first else FULL_ATTENTION for i in range(layers)]
            else:
                types = [FULL_ATTENTION] * layers
        cfg = cls(
            architecture=str(archs[0]),
            vocab_size=_required(d, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=_required(d, "intermediate_size", int),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=_optional(d, "num_key_value_heads", int, heads),
            head_dim=_optional(d, "head_dim", int, hidden // heads),
            rms_norm_eps=_optional(d, "rms_norm_eps", float, 1e-6),
            rope_theta=_optional(d, "rope_theta", float, 10000.0),
            tie_word_embeddings=_optional(d, "tie_word_embeddings", bool, False),
            max_position_embeddings=_optional(d, "max_position_embeddings", int, 32768),
            sliding_window=window,
            layer_types=tuple(str(t) for t in types),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        """src/model/qwen3.cpp:19-75, plus the keys the reference does not read."""
        for key in (
            "vocab_size",
            "hidden_size",
            "intermediate_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
            "max_position_embeddings",
        ):
            if getattr(self, key) <= 0:
                raise ConfigError(f"Qwen3 config {key} must be positive")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("Qwen3 config num_attention_heads must be divisible by num_key_value_heads")
        if self.head_dim % 2 != 0:
            raise ConfigError("Qwen3 config head_dim must be even (rotary pairs)")
        if not self.rms_norm_eps > 0.0:
            raise ConfigError("Qwen3 config rms_norm_eps must be positive")
        if not self.rope_theta > 0.0:
            raise ConfigError("Qwen3 config rope_theta must be positive")
        if len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError("Qwen3 config layer_types must name every layer")
        for t in self.layer_types:
            if t not in (FULL_ATTENTION, SLIDING_ATTENTION):
                raise ConfigError(f"Qwen3 config layer_types entry {t!r} is unknown")
        if SLIDING_ATTENTION in self.layer_types and (self.sliding_window is None or self.sliding_window <= 0):
            raise ConfigError("Qwen3 config sliding_window must be positive when a layer uses it")

    def window_of_layer(self, i: int) -> Optional[int]:
        return self.sliding_window if self.layer_types[i] == SLIDING_ATTENTION else None

    def to_dict(self) -> Dict[str, Any]:
        d = {
            "architectures": [self.architecture],
            "model_type": self.MODEL_TYPE,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
        }
        if SLIDING_ATTENTION in self.layer_types:
            d["sliding_window"] = self.sliding_window
            d["layer_types"] = list(self.layer_types)
        return d


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except OSError as e:
        raise ConfigError(f"Failed to open config file: {path}") from e  # src/model/model_config.cpp:36-38
    if not isinstance(d, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return d
