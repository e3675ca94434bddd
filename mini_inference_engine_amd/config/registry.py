"""One registry from an architecture's name to its configuration type and builder.

The reference constructs its Llama model unconditionally
(inference_engine/engine.py:44) and never reads ``architectures``; here the name
in config.json chooses the model everywhere (engine, replay, command line).

A builder is ``build(config) -> DecoderSpec``: it only assembles parts with
their sizes and constants as parameters; it computes nothing itself.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping

from .model_config import ConfigError, ModelConfig, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_type: type
    build: Callable[[Any], Any]
    shapes: Mapping[str, Mapping[str, Any]] = None     # named sizes: shape name -> config.json keys


_ARCHITECTURES: dict[str, Architecture] = {}
_MODEL_TYPES: dict[str, str] = {}


def register_architecture(name: str, config_type: type, build: Callable, *, model_type: str | None = None,
                          shapes: Mapping[str, Mapping[str, Any]] | None = None, replace: bool = False) -> None:
    """``shapes``: sizes of this architecture that have a name (``--shape`` of the command line and of the
    benchmark): shape name -> the config.json keys of that size, without ``architectures``."""
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    for shape in shapes or {}:
        owner = next((a.name for a in _ARCHITECTURES.values() if a.name != name and shape in (a.shapes or {})), None)
        if owner:
            raise ValueError(f"shape '{shape}' is already a named size of architecture '{owner}'")
    _ARCHITECTURES[name] = Architecture(name, config_type, build, dict(shapes or {}))
    if model_type is not None:
        _MODEL_TYPES[model_type] = name


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)
    for k in [k for k, v in _MODEL_TYPES.items() if v == name]:
        del _MODEL_TYPES[k]


def known_shapes() -> list[str]:
    """Every named size of every registered architecture."""
    _ensure_builtin()
    return sorted(shape for a in _ARCHITECTURES.values() for shape in (a.shapes or {}))


def shape_config(shape: str, **overrides) -> ModelConfig:
    """The typed configuration of a named size; ``overrides`` replace config.json keys of it (fewer layers,
    say) before it is read."""
    _ensure_builtin()
    for a in _ARCHITECTURES.values():
        if shape in (a.shapes or {}):
            return a.config_type.from_dict({**a.shapes[shape], **overrides, "architectures": [a.name]})
    raise ConfigError(f"no registered architecture has a size named '{shape}'; known: {known_shapes()}")


def known_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def _ensure_builtin() -> None:
    # Importing the models package registers what ships with the engine.
    from .. import models  # noqa: F401


def architecture_for(config: Mapping[str, Any]) -> Architecture:
    """Choose by ``architectures[0]``; fall back on ``model_type``."""
    _ensure_builtin()
    names = config.get("architectures") or []
    if isinstance(names, str):
        names = [names]
    for n in names:
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n]
    mt = config.get("model_type")
    if not names and mt in _MODEL_TYPES:
        return _ARCHITECTURES[_MODEL_TYPES[mt]]
    asked = names if names else (f"model_type={mt!r}" if mt else "nothing (no 'architectures' key)")
    raise ConfigError(f"config.json names {asked}; registered architectures: {sorted(_ARCHITECTURES)}")


def architecture_of(config: ModelConfig) -> Architecture:
    _ensure_builtin()
    name = type(config).architecture
    if name not in _ARCHITECTURES:
        raise ConfigError(f"architecture '{name}' is not registered; known: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def load_model_config(path_or_dict) -> tuple[ModelConfig, Architecture]:
    d = path_or_dict if isinstance(path_or_dict, Mapping) else read_config_json(path_or_dict)
    arch = architecture_for(d)
    return arch.config_type.from_dict(d), arch
