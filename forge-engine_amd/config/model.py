"""Base of the typed model configurations and the reader of config.json.

A model configuration holds exactly what the architecture's config.json gives;
no size or constant of a model is written anywhere else in the package.
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass
from pathlib import Path
from typing import Any, ClassVar


class ConfigError(ValueError):
    """config.json is missing a key, has a value out of range, or names an
    architecture or option that is not supported."""


@dataclass(frozen=True)
class ModelConfig:
    """Common base: each architecture subclasses this with its own keys."""

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict[str, Any]:
        """config.json form (round-trips through ``from_dict``)."""
        data = asdict(self)
        data["architectures"] = [self.architecture]
        return data

    @classmethod
    def from_file(cls, path: str | Path) -> "ModelConfig":
        return cls.from_dict(read_config_json(path))

    def save(self, folder: str | Path) -> Path:
        path = Path(folder) / "config.json"
        path.write_text(json.dumps(self.to_dict(), indent=2) + "\n")
        return path


def read_config_json(path: str | Path) -> dict[str, Any]:
    path = Path(path)
    if path.is_dir():
        path = path / "config.json"
    try:
        raw = json.loads(path.read_text())
    except FileNotFoundError:
        raise ConfigError(f"no config.json at {path}") from None
    except json.JSONDecodeError as error:
        raise ConfigError(f"{path} is not valid JSON: {error}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return raw


def architecture_name(raw: dict[str, Any]) -> str:
    names = raw.get("architectures")
    if not isinstance(names, list) or not names or not isinstance(names[0], str):
        raise ConfigError("config.json must name the model under 'architectures'")
    return names[0]


def load_model_config(source: str | Path | dict[str, Any]) -> ModelConfig:
    """Read config.json (a path, a folder, or the parsed dict) into the typed
    configuration of the architecture it names."""
    from ..registry import architecture  # late: the registry imports the configs

    raw = source if isinstance(source, dict) else read_config_json(source)
    return architecture(architecture_name(raw)).config_class.from_dict(raw)


class KeyReader:
    """Reads typed values out of a config.json dict with clear errors."""

    def __init__(self, raw: dict[str, Any]) -> None:
        self.raw = raw

    def _get(self, key: str, default: Any, required: bool) -> Any:
        if key in self.raw and self.raw[key] is not None:
            return self.raw[key]
        if required:
            raise ConfigError(f"config.json is missing '{key}'")
        return default

    def integer(self, key: str, default: int | None = None, *, required: bool = True, minimum: int = 1) -> int | None:
        value = self._get(key, default, required and default is None)
        if value is None:
            return None
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value.is_integer():
                value = int(value)
            else:
                raise ConfigError(f"'{key}' must be an integer, got {value!r}")
        if value < minimum:
            raise ConfigError(f"'{key}' must be at least {minimum}, got {value}")
        return value

    def number(self, key: str, default: float | None = None) -> float:
        value = self._get(key, default, default is None)
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"'{key}' must be a number, got {value!r}")
        value = float(value)
        if not value > 0.0 or value != value or value == float("inf"):
            raise ConfigError(f"'{key}' must be finite and positive, got {value}")
        return value

    def boolean(self, key: str, default: bool) -> bool:
        value = self._get(key, default, False)
        if not isinstance(value, bool):
            raise ConfigError(f"'{key}' must be true or false, got {value!r}")
        return value
