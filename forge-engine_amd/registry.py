"""Two registries: architectures (config.json name -> configuration class and
layer plan) and parts (role and kind -> class).

Adding an architecture is one ``register_architecture`` call with a function
from its configuration to a ``ModelPlan``; adding a mixer, feed-forward, norm,
position encoding or block arrangement is one ``register_part`` call.  Nothing
else in the package names a model or a part kind.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .config.model import ConfigError

ROLES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    plan: Callable  # (config) -> parts.plan.ModelPlan


_ARCHITECTURES: dict[str, Architecture] = {}
_PARTS: dict[str, dict[str, type]] = {role: {} for role in ROLES}


def register_architecture(name: str, config_class: type, plan: Callable, *, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, plan)


def architecture(name: str) -> Architecture:
    _load_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        known = ", ".join(sorted(_ARCHITECTURES)) or "none"
        raise ConfigError(f"unknown architecture '{name}' (registered: {known})") from None


def architectures() -> tuple[str, ...]:
    _load_builtin()
    return tuple(sorted(_ARCHITECTURES))


def register_part(role: str, kind: str, cls: type, *, replace: bool = False) -> None:
    if role not in _PARTS:
        raise ValueError(f"unknown part role '{role}' (roles: {', '.join(ROLES)})")
    if kind in _PARTS[role] and not replace:
        raise ValueError(f"{role} '{kind}' is already registered")
    _PARTS[role][kind] = cls


def part_class(role: str, kind: str) -> type:
    _load_builtin()
    try:
        return _PARTS[role][kind]
    except KeyError:
        known = ", ".join(sorted(_PARTS.get(role, {}))) or "none"
        raise ConfigError(f"unknown {role} kind '{kind}' (registered: {known})") from None


_BUILTIN_LOADED = False


def _load_builtin() -> None:
    global _BUILTIN_LOADED
    if _BUILTIN_LOADED:
        return
    _BUILTIN_LOADED = True
    from . import parts  # noqa: F401  registers the built-in parts
    from .models import qwen3  # noqa: F401  registers Qwen3ForCausalLM
