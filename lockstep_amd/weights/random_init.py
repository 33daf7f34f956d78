"""Random-weights mode: write a model folder from a configuration and a seed.

Each tensor gets its own generator seeded from ``(seed, tensor name)``, so a
tensor's values do not depend on which other tensors the model has.  Matrices
are N(0, std), norm weights are 1 + N(0, norm_std) (exactly 1 when norm_std is
0); values are drawn in float32 and stored in ``dtype``.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from ..config import ModelConfig
from .safetensors_io import save_file


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return torch.Generator().manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))


def random_tensors(config: ModelConfig, seed: int, std: float | None = None, norm_std: float | None = None,
                   dtype: torch.dtype = torch.bfloat16) -> dict[str, torch.Tensor]:
    from ..engine.model import collect_ties, collect_weight_specs

    scheme = dict(config.init_scheme())
    std = scheme["std"] if std is None else std
    norm_std = scheme["norm_std"] if norm_std is None else norm_std
    spec = config.model_spec()
    tied = collect_ties(spec)
    tensors: dict[str, torch.Tensor] = {}
    for w in collect_weight_specs(spec):
        if w.name in tied:
            continue  # the tied tensor is not stored; it aliases its target
        gen = _generator(seed, w.name)
        if w.kind == "int":
            value = torch.zeros(w.shape, dtype=torch.int32)
        elif w.init == "norm":
            value = torch.ones(w.shape, dtype=torch.float32)
            if norm_std:
                value = value + torch.randn(w.shape, generator=gen, dtype=torch.float32) * norm_std
        elif w.init == "zeros":
            value = torch.zeros(w.shape, dtype=torch.float32)
        else:
            value = torch.randn(w.shape, generator=gen, dtype=torch.float32) * std
        tensors[w.name] = value if w.kind == "int" else value.to(dtype)
    return tensors


def write_random_model(config: ModelConfig, out_dir, seed: int, std: float | None = None,
                       norm_std: float | None = None, dtype: torch.dtype = torch.bfloat16) -> Path:
    """Create ``out_dir`` with ``config.json`` and ``model.safetensors``."""
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    (out_dir / "config.json").write_text(json.dumps(config.to_dict(), indent=2) + "\n")
    save_file(random_tensors(config, seed, std, norm_std, dtype), out_dir / "model.safetensors",
              metadata={"format": "pt", "seed": str(seed)})
    return out_dir
