"""Static gates on the sources (in the spirit of the reference's
scripts/static_checks.py:14-49): nothing on the product path may make a
result depend on scheduling order or on a library's choice of algorithm."""

from __future__ import annotations

import re
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "lockstep_amd" / "csrc"
PACKAGE = ROOT / "lockstep_amd"


def strip_comments(text: str) -> str:
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def test_kernels_use_no_atomics_and_no_library_math():
    for path in sorted(CSRC.glob("*.hip")) + sorted(CSRC.glob("*.h")):
        code = strip_comments(path.read_text())
        for banned in ("atomicAdd", "atomicMax", "atomicMin", "atomicExch", "atomicCAS", "__hip_atomic",
                       "rocblas", "hipblas", "miopen", "hipcub", "rocprim", "__shfl_down", "__reduce_"):
            assert banned not in code, f"{path.name} uses {banned}"
        assert "-ffast-math" not in code


def test_kernels_are_built_without_contraction_and_for_gfx950_only():
    from lockstep_amd.ops import build

    assert "-ffp-contract=off" in build.FLAGS and "--offload-arch=gfx950" in build.FLAGS
    assert "-packed-fp32-ops" in build.FLAGS
    assert not any("fast-math" in f for f in build.FLAGS)


def test_product_path_calls_no_library_model_code():
    """No torch matrix products, attention, softmax or norms in the package:
    those are the hand-written kernels' job (the sampler's float64 top-p on the
    host is the named exception, as in the reference)."""
    banned = [r"torch\.matmul", r"torch\.bmm", r"torch\.einsum", r"F\.linear", r"scaled_dot_product_attention",
              r"torch\.nn\.functional", r"torch\.softmax", r"\.softmax\(", r"F\.rms_norm", r"torch\.rms_norm", r"layer_norm\(",
              r"import transformers", r"from transformers", r"import vllm", r"@ self\.", r"\.mm\("]
    for path in sorted(PACKAGE.rglob("*.py")):
        code = path.read_text()
        for pattern in banned:
            assert not re.search(pattern, code), f"{path.relative_to(ROOT)} matches {pattern}"


def test_engine_does_not_import_tests_or_working_files():
    for path in sorted(PACKAGE.rglob("*.py")) + [ROOT / "bench.py", ROOT / "bin" / "trace_run"]:
        code = path.read_text()
        assert "_work" not in code, path
        assert not re.search(r"^\s*(from|import)\s+(tests|plain)\b", code, flags=re.M), path
