"""One registry from an architecture's name to its typed configuration.

``config.json`` names its architecture twice: ``model_type`` (e.g. ``qwen3``)
and ``architectures`` (e.g. ``["Qwen3ForCausalLM"]``).  Either name finds the
configuration class; the class turns the file into a ``ModelSpec`` and the
generic builder in ``lockstep_amd.engine.model`` turns that into a model, so
registering a configuration class is all that adding an architecture takes.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping

from .base import ConfigError, ModelConfig

_ARCHITECTURES: dict[str, type[ModelConfig]] = {}


def register_architecture(config_cls: type[ModelConfig]) -> type[ModelConfig]:
    """Class decorator: make ``config_cls`` answer to its ``architecture_names``."""
    if not config_cls.architecture_names:
        raise ConfigError(f"{config_cls.__name__} declares no architecture_names")
    for name in config_cls.architecture_names:
        known = _ARCHITECTURES.get(name)
        if known is not None and known is not config_cls:
            raise ConfigError(f"architecture name {name!r} is already taken by {known.__name__}")
        _ARCHITECTURES[name] = config_cls
    return config_cls


def unregister_architecture(config_cls: type[ModelConfig]) -> None:
    for name in config_cls.architecture_names:
        if _ARCHITECTURES.get(name) is config_cls:
            del _ARCHITECTURES[name]


def known_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def config_class_for(raw: Mapping[str, Any]) -> type[ModelConfig]:
    """The class registered for ``raw["model_type"]`` or ``raw["architectures"]``."""
    names = []
    if raw.get("model_type") is not None:
        names.append(raw["model_type"])
    names.extend(raw.get("architectures") or [])
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
    raise ConfigError(
        f"no architecture is registered for model_type={raw.get('model_type')!r}, "
        f"architectures={raw.get('architectures')!r}; known: {', '.join(known_architectures()) or 'none'}"
    )


def config_from_dict(raw: Mapping[str, Any]) -> ModelConfig:
    return config_class_for(raw).from_dict(raw)


def config_from_dir(model_dir) -> ModelConfig:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"{path} does not exist")
    return config_from_dict(json.loads(path.read_text()))
