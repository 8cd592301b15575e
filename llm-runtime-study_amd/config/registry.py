"""One registry from an architecture's name (config.json `architectures[0]`) to its model.

An entry holds the typed configuration class, the function that turns a configuration
into a ModelSpec, and the architecture's chat template.  Reference: mini_llm/model/loader.py:13-33
and mini_llm/config.py:501-512 dispatch on `model_type` (and mini_llm/tokenizer.py picks the chat
template by it); here the key is the architecture name and `model_type` is checked by the
configuration class itself.

What the engine, the loader and the scheduler read of a configuration object is stated once, as
ModelConfig below; `register_architecture` refuses a class that lacks any of it.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Protocol, Sequence, runtime_checkable

from ..errors import ConfigError
from .fields import read_config_json


@runtime_checkable
class ModelConfig(Protocol):
    """What everything outside an architecture's own files reads of its typed configuration."""

    model_type: str                      # named in checkpoint errors
    vocab_size: int                      # token ids are checked against it
    eos_token_ids: Sequence[int]         # generation ends at any of them

    @classmethod
    def from_dict(cls, raw: dict) -> "ModelConfig": ...

    def validate_context_length(self, max_seq_len: int) -> None: ...

    def to_json_dict(self) -> dict: ...  # the config.json content that reads back as this configuration (random-weights folders)


CONFIG_ATTRIBUTES = ("model_type", "vocab_size", "eos_token_ids")
CONFIG_METHODS = ("from_dict", "validate_context_length", "to_json_dict")
# Modules named here (comma-separated import paths) are imported when the registry is first used: each registers its
# parts and architectures as it is imported, so that a program started as a process of its own (the command line,
# bin/trace_run) knows an architecture that lives outside this package.
PLUGINS_VARIABLE = "LLM_RUNTIME_STUDY_PLUGINS"


def _config_fields(config_class: type) -> set:
    """Names a configuration class declares: annotations (dataclass fields), attributes and properties."""
    names = set()
    for klass in getattr(config_class, "__mro__", (config_class,)):
        names.update(getattr(klass, "__annotations__", {}))
        names.update(vars(klass))
    return names


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build_spec: Callable
    chat_template: Callable | None = None    # (messages, *, enable_thinking) -> prompt text; None: token ids only


_ARCHITECTURES: dict[str, Architecture] = {}
_builtin_loaded = False


def _load_builtin() -> None:
    """Register the architectures that ship with the package (on first use, to keep imports acyclic)."""
    global _builtin_loaded
    if _builtin_loaded:
        return
    _builtin_loaded = True
    from ..models.qwen3 import build_spec
    from ..text.chat import format_qwen3_chat
    from .qwen3 import Qwen3Config

    if Qwen3Config.ARCHITECTURE not in _ARCHITECTURES:
        register_architecture(Qwen3Config.ARCHITECTURE, Qwen3Config, build_spec, chat_template=format_qwen3_chat)
    import importlib
    import os

    for name in filter(None, (piece.strip() for piece in os.environ.get(PLUGINS_VARIABLE, "").split(","))):
        try:
            importlib.import_module(name)
        except ImportError as exc:
            raise ConfigError(f"{PLUGINS_VARIABLE} names the module {name!r}, which cannot be imported: {exc}") from exc


def register_architecture(name: str, config_class: type, build_spec: Callable, chat_template: Callable | None = None) -> None:
    """Make `name` (config.json `architectures[0]`) load as `config_class` and build through `build_spec`.

    `config_class` must provide what ModelConfig lists; `chat_template(messages, *, enable_thinking)`
    turns chat messages into the prompt text of this architecture (None: it takes token ids only)."""
    fields = _config_fields(config_class)
    lacking = [n for n in CONFIG_ATTRIBUTES if n not in fields] + [n for n in CONFIG_METHODS if not callable(getattr(config_class, n, None))]
    if lacking:
        raise ConfigError(f"configuration class {config_class.__name__} of architecture {name!r} lacks: {', '.join(lacking)}")
    if not callable(build_spec) or (chat_template is not None and not callable(chat_template)):
        raise ConfigError(f"architecture {name!r}: build_spec (and chat_template, if given) must be callable")
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec, chat_template)


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


def architecture_of(config) -> Architecture:
    """The registry entry whose configuration class is `config`'s own class (else one it inherits from)."""
    _load_builtin()
    for exact in (True, False):
        for arch in _ARCHITECTURES.values():
            if type(config) is arch.config_class if exact else isinstance(config, arch.config_class):
                return arch
    raise ConfigError(f"no architecture is registered for configuration type {type(config).__name__}")


def spec_for(config):
    """ModelSpec of a typed configuration."""
    return architecture_of(config).build_spec(config)


def chat_template_for(config) -> Callable | None:
    """The chat template of the configuration's architecture (None if it has none)."""
    return architecture_of(config).chat_template
