"""Typed description of a model: what config.json says, turned into parts.

Two levels live here.

``ModelConfig`` is the architecture's own view of ``config.json``: a frozen
dataclass whose fields are that architecture's keys.  ``ModelSpec`` is what
the rest of the framework consumes: per-layer ``LayerSpec`` records naming a
mixer, a feed-forward, norms and an arrangement (each a ``PartSpec`` with its
constants as parameters), and a ``schedule`` that says in which order the
layers run and whose cache each run uses.  An architecture is the function
from the first to the second; nothing below this level knows which model it
is in.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field, fields
from pathlib import Path
from typing import Any, Mapping


class ConfigError(ValueError):
    """config.json is missing a key, names an unknown architecture, or holds
    values that no kernel can take."""


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: its registered kind and its constants."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]


@dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement and the parts it wires.

    ``prefix`` is the layer's tensor-name prefix in the checkpoint, e.g.
    ``model.layers.3``; each part appends its own names to it.

    The four named fields are the common case (one mixer, one feed-forward, a
    norm in front of each) and are all optional: an arrangement reads the parts
    it knows by name with ``part(name)`` and need not use these names at all.
    Whatever else a layer is made of (a norm behind each part as well, a second
    feed-forward, a gate) goes into ``parts``, an open mapping from names of the
    arrangement's choosing to ``PartSpec``s.
    """

    prefix: str
    arrangement: PartSpec
    mixer: PartSpec | None = None
    feed_forward: PartSpec | None = None
    mixer_norm: PartSpec | None = None
    feed_forward_norm: PartSpec | None = None
    parts: Mapping[str, PartSpec] = field(default_factory=dict)

    COMMON = ("mixer", "feed_forward", "mixer_norm", "feed_forward_norm")

    def __post_init__(self):
        clash = [name for name in self.parts if name in self.COMMON or name in ("prefix", "arrangement", "parts")]
        if clash:
            raise ConfigError(f"layer {self.prefix!r}: the names {clash} in 'parts' are fields of the layer itself")
        wrong = [name for name, spec in self.named_parts().items() if not isinstance(spec, PartSpec)]
        if wrong:
            raise ConfigError(f"layer {self.prefix!r}: the parts {wrong} are not PartSpecs")

    def named_parts(self) -> dict:
        """Every part of the layer by name: the common fields that are set, then ``parts``."""
        out = {name: getattr(self, name) for name in self.COMMON if getattr(self, name) is not None}
        out.update(self.parts)
        return out

    def part(self, name: str) -> PartSpec:
        found = self.named_parts().get(name)
        if found is None:
            raise ConfigError(f"layer {self.prefix!r} has no part named {name!r}; it has: "
                              f"{', '.join(self.named_parts()) or 'none'}")
        return found

    def has(self, name: str) -> bool:
        return name in self.named_parts()


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may be named by several
    entries).  ``cache`` is the cache unit the mixer uses in this run; units
    are numbered by the model spec.  ``writes_cache`` is False when the run
    only reads a unit that another entry fills (sharing another layer's keys
    and values).
    """

    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    """Everything the engine needs to build a model from parts."""

    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    #: positions a request may use (its tokens are at positions 0 .. max_positions - 1); None: no bound
    max_positions: int | None = None

    def cache_units(self) -> int:
        return 1 + max((e.cache for e in self.schedule), default=-1)


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's typed configuration."""

    #: value(s) of ``model_type`` / ``architectures`` this class answers to
    architecture_names = ()

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ModelConfig":
        missing = [f.name for f in fields(cls) if f.name not in raw]
        if missing:
            raise ConfigError(
                f"config.json for {cls.__name__} lacks the key(s) {', '.join(missing)}"
            )
        config = cls(**{f.name: raw[f.name] for f in fields(cls)})
        config.validate()
        return config

    @classmethod
    def from_file(cls, path) -> "ModelConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def to_dict(self) -> dict[str, Any]:
        """What a config.json of this architecture holds."""
        out: dict[str, Any] = {
            "model_type": self.architecture_names[0],
            "architectures": [n for n in self.architecture_names[1:2]] or [self.architecture_names[0]],
        }
        out.update({f.name: getattr(self, f.name) for f in fields(self)})
        return out

    def validate(self) -> None:  # pragma: no cover - overridden
        pass

    def model_spec(self) -> ModelSpec:
        raise NotImplementedError

    def init_scheme(self) -> Mapping[str, Any]:
        """Defaults of the random-weights mode (may be overridden by the caller)."""
        return {"std": 0.02, "norm_std": 0.0}
