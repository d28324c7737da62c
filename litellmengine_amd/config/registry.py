"""One registry from an architecture's name (config.json `architectures[0]`) to
its configuration class and its model builder.

The reference never dispatches: `main` builds `Qwen3ForCausalLM` whatever
`model_type` says (src/main.cpp:158).  Here an unknown name is an error that
lists what is registered, and a new architecture is one `register_architecture`
call (the tests register a toy one without touching this package).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, Dict, Optional

from .model_config import ConfigError, read_config_json


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any  # has from_dict(dict) and to_dict()
    build: Callable[..., Any]  # build(config) -> models.decoder.DecoderLM
    # chat_template(user_prompt, enable_thinking) -> the text that is tokenised for a text prompt;
    # None: the prompt is tokenised as it is
    chat_template: Optional[Callable[[str, bool], str]] = None


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class, build, chat_template=None) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, build, chat_template)


def registered_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(sorted(_ARCHITECTURES)) or '(none)'}"
        ) from None


def architecture_of(config_dict: Dict[str, Any]) -> Architecture:
    archs = config_dict.get("architectures")
    if not archs or not isinstance(archs, list):
        raise ConfigError("config.json has no `architectures` list to choose a model by")
    return get_architecture(str(archs[0]))


def architecture_of_model_dir(model_dir: str) -> Architecture:
    return architecture_of(read_config_json(model_dir))


def load_config(model_dir: str):
    """config.json of a model folder -> the typed configuration of its architecture."""
    d = read_config_json(model_dir)
    return architecture_of(d).config_class.from_dict(d)


def _ensure_builtin() -> None:
    # the built-in architectures register themselves when their module is imported
    from .. import models  # noqa: F401
