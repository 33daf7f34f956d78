"""bin/trace_run as a user drives it: a subprocess fed steps on standard
input, logits read from the files it writes, compared with the plain
implementation under four ways of cutting the same requests."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

from helpers import make_mixed_trace, max_live_tokens, random_tokens, rel_err, tol_for

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


def run_trace(model_dir, dtype, steps, out_dir, vocab, max_tokens):
    """Feed the steps one by one, waiting for ``done <step>`` each time."""
    proc = subprocess.Popen(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {step['step']}", f"expected 'done {step['step']}', got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    logits: dict[str, list] = {}
    for step in steps:
        wanted = sum(len(e["want"]) for e in step["entries"])
        path = Path(out_dir) / f"{step['step']}.f32"
        if not wanted:
            assert not path.exists()
            continue
        data = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        row = 0
        for e in step["entries"]:
            for w in e["want"]:
                logits.setdefault(e["id"], []).append(data[row])
                row += 1
    return {rid: np.stack(rows) for rid, rows in logits.items()}


def read_digests(out_dir) -> dict:
    """(request, position) -> sha256 of the logit row, from the ``<step>.sha256`` files."""
    digests = {}
    for path in Path(out_dir).glob("*.sha256"):
        for line in path.read_text().splitlines():
            rid, position, digest = line.split()
            assert (rid, int(position)) not in digests, f"position {position} of {rid} was written twice"
            digests[(rid, int(position))] = digest
    return digests


def whole(requests):
    return [{"step": i, "entries": [{"id": rid, "tokens": t, "want": list(range(len(t)))}], "end": [rid]}
            for i, (rid, t) in enumerate(requests.items())]


def tail_one_by_one(requests, tail=32):
    steps = []
    for rid, t in requests.items():
        head = max(len(t) - tail, 1)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": t[:head], "want": list(range(head))}],
                      "end": []})
        for i in range(head, len(t)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": t[i:i + 1], "want": [0]}],
                          "end": [rid] if i == len(t) - 1 else []})
        if head == len(t):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=(7, 2, 17, 3, 37, 2, 16, 15, 64)):
    steps = []
    for rid, t in requests.items():
        pos, k = 0, 0
        while pos < len(t):
            take = min(sizes[k % len(sizes)], len(t) - pos)
            if len(t) - pos - take == 1:
                take += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": t[pos:pos + take],
                                                           "want": list(range(take))}],
                          "end": [rid] if pos + take == len(t) else []})
            pos += take
            k += 1
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_under_four_cuttings(tiny_dirs, tmp_path, dtype, name):
    from plain.qwen3_plain import PlainModel, bf16

    # the sharpened weights; float32 against exact arithmetic, bfloat16 against the plain forward
    # that stores in bfloat16 where the engine does
    folder = tiny_dirs[(name, "sharp")]
    plain = PlainModel(folder)
    vocab = plain.cfg["vocab_size"]
    requests = {f"t{i}": random_tokens(n, vocab, seed=40 + i) for i, n in enumerate((150, 40, 3, 97, 300, 66))}
    store = None if dtype == "float32" else bf16
    want = {rid: plain.logits(t, store=store).numpy() for rid, t in requests.items()}
    runs = {
        "whole": whole(requests),
        "tail": tail_one_by_one(requests),
        "portions": portions(requests),
        "mixed": make_mixed_trace(requests, seed=9, decode_tail=32),
    }
    results = {}
    for label, steps in runs.items():
        out = tmp_path / label
        results[label] = run_trace(folder, dtype, steps, out, vocab, max_live_tokens(steps))
        for rid in requests:
            err = rel_err(results[label][rid], want[rid])
            assert err < tol_for(dtype, name), f"{label} {rid}: rel err {err:.3e}"
    for label in ("tail", "portions", "mixed"):
        for rid in requests:
            assert np.array_equal(results[label][rid], results["whole"][rid]), f"{label} {rid} differs from whole"
    # the digests written beside the logits name every (request, position) once and agree between the cuttings
    import hashlib

    reference = read_digests(tmp_path / "whole")
    assert set(reference) == {(rid, i) for rid, t in requests.items() for i in range(len(t))}
    assert reference[("t2", 1)] == hashlib.sha256(results["whole"]["t2"][1].astype("<f4").tobytes()).hexdigest()
    for label in ("tail", "portions", "mixed"):
        assert read_digests(tmp_path / label) == reference, label


def test_steps_without_wanted_logits_write_no_file(tiny_a_dir, tmp_path):
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": [1, 2, 3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": [4, 5], "want": [1]}], "end": ["x"]}]
    got = run_trace(tiny_a_dir, "float32", steps, tmp_path / "o", 512, 64)
    assert got["x"].shape == (1, 512) and not (tmp_path / "o" / "0.f32").exists()
