"""Reader and writer for the safetensors container, by tensor name.

File layout: an unsigned 64-bit little-endian header length ``n``; ``n`` bytes
of JSON mapping each tensor name to ``{"dtype", "shape", "data_offsets":
[begin, end]}`` (offsets relative to the end of the header; the key
``__metadata__`` is free text); then the raw little-endian data.  Tensors are
returned as views of a copy-on-write memory map, so opening a large file
costs nothing until a tensor is touched.
"""

from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path
from typing import Mapping

import numpy as np
import torch

_DTYPES = {
    "F64": (np.float64, torch.float64),
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.uint16, torch.bfloat16),
    "I64": (np.int64, torch.int64),
    "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16),
    "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8),
    "BOOL": (np.bool_, torch.bool),
}
_NAMES = {t: name for name, (_, t) in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One ``.safetensors`` file opened for reading."""

    def __init__(self, path):
        self.path = Path(path)
        with open(self.path, "rb") as handle:
            head = handle.read(8)
            if len(head) != 8:
                raise SafetensorsError(f"{self.path}: shorter than a safetensors header")
            (length,) = struct.unpack("<Q", head)
            size = self.path.stat().st_size
            if length > size - 8:
                raise SafetensorsError(f"{self.path}: header length {length} exceeds the file")
            try:
                header = json.loads(handle.read(length).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as exc:
                raise SafetensorsError(f"{self.path}: header is not JSON: {exc}") from None
            self._data_start = 8 + length
            self._map = mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_COPY) if size else None
        self.metadata = header.pop("__metadata__", None) or {}
        self.entries: dict[str, dict] = header
        for name, entry in self.entries.items():
            if entry.get("dtype") not in _DTYPES:
                raise SafetensorsError(f"{self.path}: tensor {name!r} has unknown dtype {entry.get('dtype')!r}")
            begin, end = entry["data_offsets"]
            count = int(np.prod(entry["shape"], dtype=np.int64)) if entry["shape"] else 1
            width = np.dtype(_DTYPES[entry["dtype"]][0]).itemsize
            if end - begin != count * width or self._data_start + end > size:
                raise SafetensorsError(f"{self.path}: tensor {name!r} has inconsistent offsets")

    def keys(self) -> list[str]:
        return list(self.entries)

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self.entries[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name]["dtype"]][1]

    def get(self, name: str) -> torch.Tensor:
        entry = self.entries[name]
        np_dtype, torch_dtype = _DTYPES[entry["dtype"]]
        begin, end = entry["data_offsets"]
        count = (end - begin) // np.dtype(np_dtype).itemsize
        if count == 0:
            return torch.empty(tuple(entry["shape"]), dtype=torch_dtype)
        array = np.frombuffer(self._map, dtype=np_dtype, count=count, offset=self._data_start + begin)
        tensor = torch.from_numpy(array)
        if torch_dtype is torch.bfloat16:
            tensor = tensor.view(torch.bfloat16)
        return tensor.reshape(tuple(entry["shape"]))


def open_model_tensors(model_dir) -> dict[str, tuple[SafetensorsFile, str]]:
    """Map each tensor name in a model folder to the file that holds it.

    A folder holds either ``model.safetensors`` or shards listed by
    ``model.safetensors.index.json`` (``weight_map``: name -> file).
    """
    model_dir = Path(model_dir)
    single = model_dir / "model.safetensors"
    index = model_dir / "model.safetensors.index.json"
    where: dict[str, tuple[SafetensorsFile, str]] = {}
    if single.is_file():
        handle = SafetensorsFile(single)
        for name in handle.keys():
            where[name] = (handle, name)
    elif index.is_file():
        weight_map = json.loads(index.read_text())["weight_map"]
        files: dict[str, SafetensorsFile] = {}
        for name, file_name in weight_map.items():
            if file_name not in files:
                files[file_name] = SafetensorsFile(model_dir / file_name)
            where[name] = (files[file_name], name)
    else:
        raise FileNotFoundError(f"{model_dir} holds neither model.safetensors nor model.safetensors.index.json")
    return where


def save_file(tensors: Mapping[str, torch.Tensor], path, metadata: Mapping[str, str] | None = None) -> None:
    """Write ``tensors`` (CPU) to one safetensors file, names in sorted order."""
    header: dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r} has dtype {t.dtype}, which safetensors cannot hold")
        size = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + size]}
        offset += size
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)))
        handle.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            if t.dtype is torch.bfloat16:
                t = t.view(torch.int16)
            elif t.dtype is torch.bool:
                t = t.view(torch.uint8)
            handle.write(t.numpy().tobytes())
