"""One registry from an architecture's name (config.json ``architectures[0]``) to its typed
configuration and to the function that builds its model. The reference has a single hard-wired
model; every place in this framework that needs a model asks here."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .base import ConfigError, ModelConfig, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build: Callable  # (config, precision) -> mini_llm_amd.models.base.Model, weights not loaded


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, build: Callable) -> None:
    """Adds (or replaces) an architecture. ``build(config, precision)`` returns the model made
    of parts, without weights."""
    _ARCHITECTURES[name] = Architecture(name, config_class, build)


def registered_architectures() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(sorted(_ARCHITECTURES))}"
        )
    return _ARCHITECTURES[name]


def architecture_name(raw: dict) -> str:
    names = raw.get("architectures")
    if not isinstance(names, list) or not names or not isinstance(names[0], str):
        raise ConfigError("config.json has no 'architectures' list naming the model class")
    return names[0]


def config_from_dict(raw: dict) -> ModelConfig:
    return get_architecture(architecture_name(raw)).config_class.from_dict(raw)


def load_config(model_dir) -> ModelConfig:
    """config.json of a model folder as the typed configuration of its architecture."""
    return config_from_dict(read_config_json(model_dir))


def _load_builtin() -> None:
    # The built-in architectures register themselves when their module is imported.
    from .. import models  # noqa: F401
