"""Shared fixtures: the two tiny configurations, model folders in temporary
directories, and the ``gpu`` marker."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations that differ in every size and option.
TINY_A = dict(
    hidden_size=64, intermediate_size=192, num_hidden_layers=2, num_attention_heads=4,
    num_key_value_heads=2, head_dim=16, vocab_size=512, rms_norm_eps=1e-6, rope_theta=10000.0,
    max_position_embeddings=256, tie_word_embeddings=True,
)
TINY_A_INIT = dict(seed=0, std=0.02, norm_std=0.0, page_size=16)
TINY_B = dict(
    hidden_size=96, intermediate_size=256, num_hidden_layers=3, num_attention_heads=6,
    num_key_value_heads=3, head_dim=32, vocab_size=1000, rms_norm_eps=1e-5, rope_theta=1000000.0,
    max_position_embeddings=512, tie_word_embeddings=False,
)
TINY_B_INIT = dict(seed=2, std=0.05, norm_std=0.1, page_size=8)
TINY = {"A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT)}


# The configurations' own position bounds (256 and 512) hold the workloads they are defined with; the
# tests of tile, split and page edges run longer sequences, so their folders carry wider bounds
# (still different from each other).  ``max_position=None`` keeps the configuration's own.
LONG_POSITIONS = {"A": 1024, "B": 2048}


def make_model_dir(tmp_path_factory, name: str, sharpen: float = 1.0, std: float | None = None,
                   max_position: int | None = -1, overrides: dict | None = None) -> Path:
    """Write tiny configuration ``name`` with random weights.  ``sharpen``
    multiplies the per-head q/k norm weights so that attention is peaked and a
    wrong key or a wrong position changes the logits visibly (the float32 path
    is compared on such weights; in bfloat16 the rounding of queries and keys
    is amplified by the same factor squared, so the bfloat16 comparison with
    the plain implementation uses the unsharpened weights and the sharpened
    ones serve its bit-for-bit comparisons).  ``std`` overrides the spread of
    the matrices (larger values separate the logits, for token comparisons).
    ``overrides`` replaces keys of the configuration (more layers, for instance)."""
    from lockstep_amd.config import Qwen3Config
    from lockstep_amd.weights import random_tensors, save_file
    import json

    raw, init = TINY[name]
    if max_position == -1:
        max_position = LONG_POSITIONS[name]
    if max_position is not None:
        raw = dict(raw, max_position_embeddings=max_position)
    if overrides:
        raw = dict(raw, **overrides)
    config = Qwen3Config.from_dict(raw)
    out = tmp_path_factory.mktemp(f"tiny{name}")
    tensors = random_tensors(config, init["seed"], std or init["std"], init["norm_std"], torch.bfloat16)
    if sharpen != 1.0:
        for key in tensors:
            if key.endswith("q_norm.weight") or key.endswith("k_norm.weight"):
                tensors[key] = (tensors[key].float() * sharpen).to(torch.bfloat16)
    (out / "config.json").write_text(json.dumps(config.to_dict()))
    save_file(tensors, out / "model.safetensors")
    return out


@pytest.fixture(scope="session")
def tiny_a_dir(tmp_path_factory):
    return make_model_dir(tmp_path_factory, "A", sharpen=2.0)


@pytest.fixture(scope="session")
def tiny_b_dir(tmp_path_factory):
    return make_model_dir(tmp_path_factory, "B", sharpen=2.0)


@pytest.fixture(scope="session")
def tiny_dirs(tmp_path_factory, tiny_a_dir, tiny_b_dir):
    """(configuration, variant) -> model folder; variants: ``sharp`` (peaked
    attention), ``soft`` (weights as drawn), ``gen`` (well separated logits)."""
    return {
        ("A", "sharp"): tiny_a_dir, ("B", "sharp"): tiny_b_dir,
        ("A", "soft"): make_model_dir(tmp_path_factory, "A"), ("B", "soft"): make_model_dir(tmp_path_factory, "B"),
        ("A", "gen"): make_model_dir(tmp_path_factory, "A", std=0.3),
        ("B", "gen"): make_model_dir(tmp_path_factory, "B", std=0.3),
    }
