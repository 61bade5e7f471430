"""One registry from an architecture's name (config.json "architectures"[0]) to the
functions that turn its config.json into a typed configuration and that configuration
into a model description (a ModelSpec of parts).

The reference has no registry: nanovllm/engine/model_runner.py:9,31 names
Qwen3ForCausalLM directly.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping

from .model_config import ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[Mapping[str, Any]], Any]   # config.json dict -> typed config
    build_spec: Callable[[Any], Any]                   # typed config -> parts.spec.ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, parse_config, build_spec, *, replace: bool = False) -> Architecture:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    arch = Architecture(name, parse_config, build_spec)
    _ARCHITECTURES[name] = arch
    return arch


def known_architectures():
    _load_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f"unknown architecture {name!r}; known: {known_architectures()}") from None


def architecture_of(config_json: Mapping[str, Any]) -> Architecture:
    names = config_json.get("architectures")
    if not names or not isinstance(names, (list, tuple)):
        raise ConfigError("config.json: key 'architectures' is missing or empty; "
                          f"known architectures: {known_architectures()}")
    return get_architecture(names[0])


def _load_builtin() -> None:
    # The built-in architectures register themselves on import.
    from .. import models  # noqa: F401
