"""Weights by tensor name, checked against what the model's parts expect.

``load_weights`` opens a model folder, compares the names and shapes it holds
with the ``WeightSpec`` list of the model and raises one ``WeightError`` that
lists every missing, unexpected and mis-shaped tensor.  Tensors stay on the
CPU here (memory-mapped); parts move what they use to the device.

Dtypes are normalised, not chosen: bfloat16 and float16 tensors are kept as
stored, integer tables become int32, and a tensor stored in 32-bit (or
64-bit) floating point stays float32.  The cast to the compute dtype happens
where a part puts a tensor on the device (``Runtime.matrix`` / ``vector``),
which also keeps the record of what a lossy cast cost.

A tied head follows the reference (engine/model/qwen3.py:159-174,201-202):
when the configuration ties the head to the embedding and the checkpoint
holds both tensors they must be equal, else the load is refused; the head
then aliases the embedding.
"""

from __future__ import annotations

from typing import Mapping, Sequence

import torch

from ..parts.base import WeightSpec
from .safetensors_io import open_model_tensors


class WeightError(ValueError):
    """The checkpoint does not hold what the model needs."""

    def __init__(self, message: str, missing=(), unexpected=(), mismatched=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.mismatched = list(mismatched)


def normalise_dtype(tensor: torch.Tensor) -> torch.Tensor:
    if tensor.dtype in (torch.bfloat16, torch.float32, torch.float16):
        return tensor
    if tensor.dtype is torch.float64:
        return tensor.to(torch.float32)
    if tensor.dtype in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool):
        return tensor.to(torch.int32)
    raise WeightError(f"cannot hold a tensor of dtype {tensor.dtype}")


def check_names_and_shapes(
    specs: Sequence[WeightSpec],
    available: Mapping[str, tuple[int, ...]],
    aliases: Mapping[str, str] | None = None,
) -> None:
    """Raise one error listing all missing, unexpected and mis-shaped tensors.

    ``aliases`` maps a tensor name to the name it may be taken from when the
    checkpoint does not hold it (a tied head).
    """
    aliases = dict(aliases or {})
    expected = {s.name: s for s in specs}
    missing, mismatched = [], []
    for name, spec in expected.items():
        source = name if name in available else aliases.get(name)
        if source is None or source not in available:
            if not spec.optional:
                missing.append(name)
            continue
        if tuple(available[source]) != tuple(spec.shape):
            mismatched.append((name, tuple(spec.shape), tuple(available[source])))
    unexpected = sorted(n for n in available if n not in expected)
    if missing or unexpected or mismatched:
        lines = ["the checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(sorted(missing)))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if mismatched:
            lines.append(f"  wrong shape ({len(mismatched)}): " + "; ".join(
                f"{n} expected {list(e)} found {list(f)}" for n, e, f in sorted(mismatched)))
        raise WeightError("\n".join(lines), missing=sorted(missing), unexpected=unexpected,
                          mismatched=sorted(mismatched))


class WeightStore:
    """Name -> CPU tensor, read on demand and dtype-normalised."""

    def __init__(self, where, aliases: Mapping[str, str] | None = None):
        self._where = where
        self._aliases = dict(aliases or {})

    def names(self) -> list[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where or self._aliases.get(name) in self._where

    def source_name(self, name: str) -> str:
        """The name the tensor is read from (differs for an aliased tensor)."""
        if name in self._where:
            return name
        return self._aliases[name]

    def get(self, name: str) -> torch.Tensor:
        handle, key = self._where[self.source_name(name)]
        return normalise_dtype(handle.get(key))


class DictWeightStore(WeightStore):
    """The same interface over tensors already in memory."""

    def __init__(self, tensors: Mapping[str, torch.Tensor], aliases: Mapping[str, str] | None = None):
        self._tensors = dict(tensors)
        self._where = self._tensors
        self._aliases = dict(aliases or {})

    def get(self, name: str) -> torch.Tensor:
        return normalise_dtype(self._tensors[self.source_name(name)])


def resolve_ties(shapes: dict, ties: Mapping[str, str], same) -> dict[str, str]:
    """Handle tied tensors.  ``ties`` maps a name to the name it is tied to;
    ``same(a, b)`` compares two stored tensors.  Returns the aliases to use
    and removes a redundant duplicate from ``shapes``."""
    aliases: dict[str, str] = {}
    for name, target in ties.items():
        if name in shapes and target in shapes:
            if not same(name, target):
                raise WeightError(
                    f"the configuration ties {name} to {target} but the two tensors differ "
                    "in this checkpoint; refusing to alias them")
            del shapes[name]
        aliases[name] = target
    return aliases


def load_weights(model_dir, specs: Sequence[WeightSpec], ties: Mapping[str, str] | None = None) -> WeightStore:
    where = open_model_tensors(model_dir)
    shapes = {name: handle.shape(key) for name, (handle, key) in where.items()}

    def same(a: str, b: str) -> bool:
        ta, tb = where[a][0].get(where[a][1]), where[b][0].get(where[b][1])
        return ta.shape == tb.shape and ta.dtype == tb.dtype and torch.equal(ta, tb)

    aliases = resolve_ties(shapes, ties or {}, same)
    check_names_and_shapes(specs, shapes, aliases)
    return WeightStore({n: where[n] for n in shapes}, aliases)


def weights_from_dict(tensors: Mapping[str, torch.Tensor], specs: Sequence[WeightSpec],
                      ties: Mapping[str, str] | None = None) -> WeightStore:
    shapes = {name: tuple(t.shape) for name, t in tensors.items()}
    aliases = resolve_ties(shapes, ties or {}, lambda a, b: torch.equal(tensors[a], tensors[b]))
    check_names_and_shapes(specs, shapes, aliases)
    return DictWeightStore({n: tensors[n] for n in shapes}, aliases)
