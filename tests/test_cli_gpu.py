"""``lockstep init`` + ``run --model`` + ``run --random`` as a user starts them, against the
plain implementation (float32) and against the Python entry point (bfloat16)."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest

from helpers import random_tokens

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent
LOCKSTEP = [sys.executable, str(ROOT / "bin" / "lockstep")]


def run(*args):
    done = subprocess.run([*LOCKSTEP, *args], capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    return {rec["uid"]: rec["tokens"] for rec in map(json.loads, done.stdout.strip().splitlines())}


def test_init_then_run_a_model_folder(tmp_path):
    from plain.qwen3_plain import PlainModel

    folder = tmp_path / "m"
    subprocess.run([*LOCKSTEP, "init", "--preset", "tiny-a", "--out", str(folder), "--seed", "1", "--std", "0.3"],
                   check=True, capture_output=True, timeout=300)
    prompts = [random_tokens(n, 512, seed=70 + n) for n in (7, 13, 32)]
    plain = PlainModel(folder)
    want = {f"r{i:02d}": plain.generate_greedy(p, 6) for i, p in enumerate(prompts)}
    args = [x for p in prompts for x in ("--prompt-ids", ",".join(map(str, p)))]
    got = run("run", "--model", str(folder), "--dtype", "float32", "--max-new-tokens", "6", *args)
    assert got == want
    cut = run("run", "--model", str(folder), "--dtype", "float32", "--max-new-tokens", "6", "--prefill-chunk", "5",
              "--max-batched-tokens", "12", "--block-size", "8", "--num-blocks", "24", "--decode-burst", "1", *args)
    assert cut == want
    eos = want["r00"][2]
    stopped = run("run", "--model", str(folder), "--dtype", "float32", "--max-new-tokens", "6", "--eos", str(eos),
                  *args[:2])
    assert stopped == {"r00": want["r00"][: want["r00"].index(eos) + 1]}


def test_run_random_weights_with_a_prompt_file(tmp_path):
    """``--random tiny-b --prefill-chunk 12`` with sampled and greedy requests from a file: the
    tokens equal those of the Python entry point on the same random weights."""
    from lockstep_amd import LLM, Request
    from lockstep_amd.config.presets import preset
    from lockstep_amd.weights import write_random_model

    prompts = [random_tokens(n, 1000, seed=80 + n) for n in (1, 9, 17, 40)]
    lines = [{"uid": f"q{i}", "prompt": p, "max_new_tokens": 5 + i, "temperature": 0.8 if i % 2 else 0.0,
              "top_p": 0.9, "seed": 3 + i} for i, p in enumerate(prompts)]
    (tmp_path / "prompts.jsonl").write_text("\n".join(json.dumps(d) for d in lines) + "\n")
    got = run("run", "--random", "tiny-b", "--seed", "6", "--prefill-chunk", "12", "--block-size", "8",
              "--prompt-file", str(tmp_path / "prompts.jsonl"))
    folder = write_random_model(preset("tiny-b"), tmp_path / "b", 6)
    llm = LLM(folder, num_pages=512, page_size=8)
    want = llm.generate([Request(uid=d["uid"], prompt=d["prompt"], seed=d["seed"], max_new_tokens=d["max_new_tokens"],
                                 temperature=d["temperature"], top_p=d["top_p"]) for d in lines])
    assert got == want and [len(got[f"q{i}"]) for i in range(4)] == [5, 6, 7, 8]
