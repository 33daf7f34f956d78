"""The command line: one dispatcher, one function per command (reference lockstep:32-95).
The commands that need no GPU are run here as subprocesses; the others in test_cli_gpu.py."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
LOCKSTEP = [sys.executable, str(ROOT / "bin" / "lockstep")]


def run(*args, **kw):
    return subprocess.run([*LOCKSTEP, *args], capture_output=True, text=True, timeout=300, **kw)


def test_help_lists_every_command_and_says_what_is_not_built():
    done = run("--help")
    assert done.returncode == 0
    for name in ("run", "replay", "bench", "init", "verify", "certify"):
        assert name in done.stdout
    assert "not built" in done.stdout
    assert run().returncode == 0


def test_unknown_and_unbuilt_commands_exit_with_2():
    assert run("frobnicate").returncode == 2
    done = run("certify")
    assert done.returncode == 2 and "not built" in done.stdout


def test_init_writes_a_model_folder_from_a_preset_and_from_a_config(tmp_path):
    from lockstep_amd.config import config_from_dir
    from lockstep_amd.weights import SafetensorsFile

    done = run("init", "--preset", "tiny-b", "--out", str(tmp_path / "b"), "--seed", "4", "--norm-std", "0.1")
    assert done.returncode == 0, done.stderr
    assert done.stdout.strip() == str(tmp_path / "b")
    config = config_from_dir(tmp_path / "b")
    assert config.hidden_size == 96 and not config.tie_word_embeddings
    names = SafetensorsFile(tmp_path / "b" / "model.safetensors").keys()
    assert "lm_head.weight" in names and "model.layers.2.self_attn.q_norm.weight" in names
    raw = json.loads((tmp_path / "b" / "config.json").read_text())
    raw["num_hidden_layers"] = 1
    (tmp_path / "one.json").write_text(json.dumps(raw))
    done = run("init", "--config", str(tmp_path / "one.json"), "--out", str(tmp_path / "c"))
    assert done.returncode == 0, done.stderr
    assert config_from_dir(tmp_path / "c").num_hidden_layers == 1
    assert run("init", "--preset", "no-such", "--out", str(tmp_path / "d")).returncode != 0


def test_run_needs_prompts_and_a_model():
    assert run("run", "--random", "tiny-a").returncode == 2          # no prompts
    assert run("run", "--prompt-ids", "1 2 3").returncode == 2       # neither --model nor --random
