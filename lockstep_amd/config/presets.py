"""Named configurations for the random-weights mode, kept as data
(``presets.json``): the two tiny test sizes and the sizes the engine is
measured at."""

from __future__ import annotations

import json
from pathlib import Path

from .base import ConfigError, ModelConfig
from .registry import config_from_dict

_PATH = Path(__file__).with_name("presets.json")


def preset_names() -> list[str]:
    return sorted(json.loads(_PATH.read_text()))


def preset(name: str, **overrides) -> ModelConfig:
    table = json.loads(_PATH.read_text())
    if name not in table:
        raise ConfigError(f"no preset {name!r}; known: {', '.join(sorted(table))}")
    raw = dict(table[name])
    raw.update(overrides)
    return config_from_dict(raw)
