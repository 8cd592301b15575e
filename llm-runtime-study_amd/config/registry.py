"""One registry from an architecture's name (config.json `architectures[0]`) to its model.

An entry holds the typed configuration class and the function that turns a configuration
into a ModelSpec.  Reference: mini_llm/model/loader.py:13-33 and mini_llm/config.py:501-512
dispatch on `model_type`; here the key is the architecture name and `model_type` is checked
by the configuration class itself.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from ..errors import ConfigError
from .fields import read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build_spec: Callable


_ARCHITECTURES: dict[str, Architecture] = {}
_builtin_loaded = False


def _load_builtin() -> None:
    """Register the architectures that ship with the package (on first use, to keep imports acyclic)."""
    global _builtin_loaded
    if _builtin_loaded:
        return
    _builtin_loaded = True
    from ..models.qwen3 import build_spec
    from .qwen3 import Qwen3Config

    _ARCHITECTURES.setdefault(Qwen3Config.ARCHITECTURE, Architecture(Qwen3Config.ARCHITECTURE, Qwen3Config, build_spec))


def register_architecture(name: str, config_class: type, build_spec: Callable) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec)


def registered_architectures() -> tuple[str, ...]:
    _load_builtin()
    return tuple(sorted(_ARCHITECTURES))


def architecture_for(raw: dict) -> Architecture:
    names = raw.get("architectures")
    if not isinstance(names, list) or len(names) != 1 or not isinstance(names[0], str):
        raise ConfigError(f"config.json must name exactly one architecture in `architectures`, got {names!r}")
    _load_builtin()
    try:
        return _ARCHITECTURES[names[0]]
    except KeyError:
        known = ", ".join(registered_architectures()) or "none"
        raise ConfigError(f"no model is registered for architecture {names[0]!r} (registered: {known})") from None


def load_config(model_dir):
    """Typed configuration of the model folder, chosen by its architecture name."""
    raw = read_config_json(model_dir)
    return architecture_for(raw).config_class.from_dict(raw)


def config_from_dict(raw: dict):
    return architecture_for(raw).config_class.from_dict(raw)


def spec_for(config):
    """ModelSpec of a typed configuration."""
    _load_builtin()
    for arch in _ARCHITECTURES.values():
        if isinstance(config, arch.config_class):
            return arch.build_spec(config)
    raise ConfigError(f"no architecture is registered for configuration type {type(config).__name__}")
