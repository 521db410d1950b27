"""What every architecture's typed configuration has in common."""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path


class ConfigError(ValueError):
    """config.json is missing, names an unknown architecture or holds a value that cannot be run."""


@dataclass(frozen=True)
class ModelConfig:
    """Base of the typed configurations. A subclass reads its own config.json keys in
    ``from_dict`` and checks them there; nothing downstream reads the raw dictionary."""

    architecture: str

    @classmethod
    def from_dict(cls, raw: dict) -> "ModelConfig":  # pragma: no cover - interface
        raise NotImplementedError

    def to_dict(self) -> dict:  # pragma: no cover - interface
        """The config.json content that ``from_dict`` reads back to an equal configuration."""
        raise NotImplementedError


def read_config_json(model_dir) -> dict:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"no config.json in {model_dir}")
    try:
        raw = json.loads(path.read_text())
    except json.JSONDecodeError as error:
        raise ConfigError(f"{path} is not valid JSON: {error}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return raw


def take_int(raw: dict, key: str, default=None, minimum: int = 1) -> int:
    value = raw.get(key, default)
    if value is None:
        raise ConfigError(f"config.json has no '{key}'")
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"'{key}' must be an integer, not {value!r}")
    if value < minimum:
        raise ConfigError(f"'{key}' must be at least {minimum}, not {value}")
    return value


def take_float(raw: dict, key: str, default=None) -> float:
    value = raw.get(key, default)
    if value is None:
        raise ConfigError(f"config.json has no '{key}'")
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"'{key}' must be a number, not {value!r}")
    return float(value)
