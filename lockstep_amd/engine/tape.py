"""Repeating one layer's launches for the layers that are like it.

A step that is not replayed from a captured graph launches some eight kernels a layer, and the
Python that leads up to each launch (the part's ``forward``, the checks of the kernel wrapper,
building the arguments) costs twice what the launch itself costs.  Layers of one model mostly
differ in nothing but the addresses of their weights and of their unit of the cache.  So within a
step the engine runs a layer's ``forward`` in Python only for the first two layers of a kind: the
second run is noted launch by launch (``Kernels.tape``), and for every further layer of that kind
the noted launches are made again with this layer's addresses in the place of that layer's.

What makes two schedule entries *alike* (``RunKinds``): parts that all say ``repeatable``, equal
layer specifications apart from the tensor-name prefix, the same answer to ``writes_cache``, and
cache units in the same group of the cache.  The first run of a kind is never noted, because parts
may do once a step what later layers find done.  A noted run stands for later ones only while they
arrive in the same situation: the same pending addition (or none) and an unchanged workspace.

A tape is refused (``TapeRefused``; the layers of that kind then run their ``forward`` every time)
when a launch of the noted layer passes an address that lies inside a tensor of *another* layer and
is not among the noted layer's own: the part holds a per-layer tensor where ``device_constants``
does not find it, and repeating the launch would run every later layer on that one tensor.

The first layer that a tape of its kind could stand for (once per model and cache) runs in Python all
the same and its launches are compared, argument by argument, with what the tape would have launched;
only when they agree do later layers repeat the tape, and a disagreement (a per-layer tensor that
neither walk finds, a per-layer number passed to a kernel) switches the repetition off for the kind.
``LOCKSTEP_VERIFY_TAPE=1`` does the same for every layer of every step, and raises.
"""

from __future__ import annotations

import bisect
import dataclasses
from ctypes import c_float, c_int, c_long, c_void_p

import torch

from ..ops.kernels import KernelError
from ..parts.base import Part


def device_constants(part: Part) -> dict:
    """Device tensors that ``part`` and the parts below it hold, by a name that is the same for
    every layer of the same build: attribute names along the path through ``parts()``."""
    found: dict = {}

    def collect(value, name):
        if isinstance(value, torch.Tensor):
            if value.is_cuda and value.numel():
                found[name] = value
        elif isinstance(value, (list, tuple)):
            for i, v in enumerate(value):
                if isinstance(v, torch.Tensor):
                    collect(v, f"{name}[{i}]")
        elif isinstance(value, dict):
            for k, v in value.items():
                if isinstance(v, torch.Tensor):
                    collect(v, f"{name}[{k!r}]")

    def walk(p, path):
        for name, value in vars(p).items():
            if not isinstance(value, Part):
                collect(value, f"{path}{name}")
        for i, child in enumerate(p.parts()):
            walk(child, f"{path}{i}/")

    walk(part, "")
    return found


def repeatable_tree(part: Part) -> bool:
    return bool(getattr(part, "repeatable", False)) and all(repeatable_tree(p) for p in part.parts())


def _spec_without_prefix(layer_spec):
    if dataclasses.is_dataclass(layer_spec):
        fields = {f.name: getattr(layer_spec, f.name) for f in dataclasses.fields(layer_spec)}
        fields.pop("prefix", None)
        return fields
    return layer_spec


class RunKinds:
    """For one model and one cache: which schedule entries are alike, and every entry's addresses."""

    def __init__(self, model, cache):
        self.kind: list = []            # per schedule entry: a small int, or None (always run in Python)
        self.verified: set = set()      # kinds whose tape was once compared with a layer run in Python, and agreed
        self.addresses: list = []       # per schedule entry: name -> (address, bytes)
        seen: list = []
        for run in model.schedule:
            layer = model.layers[run.layer]
            tensors = dict(device_constants(layer))
            for i, t in enumerate(cache.unit_tensors(run.cache)):
                tensors[f"cache[{i}]"] = t
            group = cache.unit_place.get(run.cache, (None,))[0]
            self.addresses.append({name: (t.data_ptr(), t.numel() * t.element_size()) for name, t in tensors.items()})
            if not repeatable_tree(layer):
                self.kind.append(None)
                continue
            key = (_spec_without_prefix(model.spec.layers[run.layer]), bool(run.writes_cache), group,
                   tuple((name, tuple(t.shape), t.dtype) for name, t in tensors.items()))
            for i, known in enumerate(seen):
                if known == key:
                    self.kind.append(i)
                    break
            else:
                seen.append(key)
                self.kind.append(len(seen) - 1)
        # per schedule entry: the address ranges of tensors that belong to other entries and not to this one
        owners: dict = {}
        for index, names in enumerate(self.addresses):
            for base, size in names.values():
                owners.setdefault((base, base + size), set()).add(index)
        self.foreign: list = [sorted(r for r, who in owners.items() if index not in who)
                              for index in range(len(self.addresses))]

    def refuse(self, kind) -> None:
        """Layers of this kind run their ``forward`` every time from now on."""
        self.kind = [None if k == kind else k for k in self.kind]


def _value(arg):
    return getattr(arg, "value", arg)


class TapeMismatch(RuntimeError):
    """A layer run in Python launched something else than the tape of its kind would have."""


class TapeRefused(RuntimeError):
    """A noted launch names a tensor of another layer that the noted layer is not known to hold."""


class LayerTape:
    """The launches of one layer run, with the places marked where an address of that layer stands."""

    def __init__(self, launches, addresses: dict, foreign=()):
        """``foreign``: sorted (first, end) address ranges of the other layers' own tensors."""
        ranges = sorted((base, base + size, name) for name, (base, size) in addresses.items())
        starts = [lo for lo, _ in foreign]
        self.calls = []
        for lib, entry, args in launches:
            marks = []
            for i, a in enumerate(args):
                if isinstance(a, c_void_p) and a.value:
                    for lo, hi, name in ranges:
                        if lo <= a.value < hi:
                            marks.append((i, name, a.value - lo))
                            break
                    else:
                        at = bisect.bisect_right(starts, a.value) - 1
                        if at >= 0 and a.value < foreign[at][1]:
                            raise TapeRefused(
                                f"argument {i} of {getattr(entry, '__name__', entry)} points into a tensor of "
                                "another layer that this layer's parts do not list among their own")
            self.calls.append((lib, entry, args, tuple(marks)))
        self.names = sorted({name for _, _, _, marks in self.calls for _, name, _ in marks})
        self._bases: dict = {}       # id of an addresses mapping -> its base addresses in the order of names
        self.words = None            # the launches as one list for Kernels.run_list, if every entry point is listed

    def as_words(self, kernels) -> bool:
        """Lay the launches out as the list of words that the core library runs in one call
        (``Kernels.run_list``); False if a launch names an entry point that cannot be listed."""
        import struct

        import numpy as np

        words, at_word, name_at, offset, libs = [], [], [], [], []
        for lib, entry, args, marks in self.calls:
            listed = kernels.listed(lib, entry)
            if listed is None:
                return False
            libs.append((len(words), listed[2]))
            words += [listed[0], listed[1], len(args)]
            first = len(words)
            for a in args:
                if isinstance(a, c_float):
                    words.append(struct.unpack("<I", struct.pack("<f", a.value))[0])
                elif isinstance(a, (c_void_p, c_int, c_long)):
                    words.append(a.value or 0)
                else:
                    return False
            for i, name, off in marks:
                at_word.append(first + i)
                name_at.append(self.names.index(name))
                offset.append(off)
        self.words = np.asarray(words, dtype=np.int64)
        self._at_word = np.asarray(at_word, dtype=np.int64)
        self._name_at = np.asarray(name_at, dtype=np.int64)
        self._offset = np.asarray(offset, dtype=np.int64)
        self._libs = libs
        return True

    def _bases_of(self, addresses: dict):
        import numpy as np

        held = self._bases.get(id(addresses))
        if held is None:
            held = np.asarray([addresses[name][0] for name in self.names], dtype=np.int64)
            self._bases[id(addresses)] = held
        return held

    def repeat_many(self, kernels, layers) -> None:
        """The launches for every mapping of addresses in ``layers``, one layer after the other, in one call."""
        import numpy as np

        n, size = len(layers), self.words.size
        words = np.tile(self.words, n)
        if self._at_word.size:
            bases = np.stack([self._bases_of(a) for a in layers])                       # [layers, names]
            values = bases[:, self._name_at] + self._offset[None, :]                    # [layers, marks]
            places = self._at_word[None, :] + (np.arange(n, dtype=np.int64) * size)[:, None]
            words[places.reshape(-1)] = values.reshape(-1)
        kernels.run_list(words, self._libs, size)

    def arguments(self, addresses: dict):
        """(library, entry point, arguments) of every launch, for the layer with these addresses."""
        for lib, entry, args, marks in self.calls:
            if marks:
                args = list(args)
                for i, name, offset in marks:
                    args[i] = c_void_p(addresses[name][0] + offset)
            yield lib, entry, args

    def repeat(self, addresses: dict) -> None:
        for lib, entry, args in self.arguments(addresses):
            if entry(*args) != 0:
                raise KernelError(lib.ls_last_error().decode())

    def compare(self, launches, addresses: dict, what: str) -> None:
        """Raise unless ``launches`` (of a layer run in Python) are what ``repeat`` would launch."""
        mine = list(self.arguments(addresses))
        if len(mine) != len(launches):
            raise TapeMismatch(f"{what}: the layer launched {len(launches)} kernels, the tape holds {len(mine)}")
        for n, ((_, entry, args), (_, entry2, args2)) in enumerate(zip(mine, launches)):
            same = entry == entry2 and len(args) == len(args2) and all(
                _value(a) == _value(b) for a, b in zip(args, args2))
            if not same:
                raise TapeMismatch(f"{what}: launch {n} ({getattr(entry2, '__name__', entry2)}) differs from the "
                                   f"tape's: {[_value(a) for a in args2]} against {[_value(a) for a in args]}")
