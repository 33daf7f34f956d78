"""``lockstep <command> [args]``: one dispatcher, one module per command, in
the manner of the reference's root script (lockstep:32-95).

Built here: ``run`` (a workload through the scheduler -- the reference names
this command and leaves it unbuilt), ``replay`` (feed a trace of given tokens
step by step and write logits), ``bench`` (the throughput measurement) and
``init`` (write a random-weights model folder).  The reference's other
commands drive its verification harness, certifier and report generator,
which are not part of this engine; they are listed as not built.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

NOT_BUILT = {
    "verify": "the metamorphic-relation harness is covered by this repository's tests (pytest -m gpu)",
    "fuzz": "no fuzzing campaign in this engine",
    "mutate": "no seeded-fault campaign in this engine",
    "minimize": "no delta-debugging of cases in this engine",
    "certify": "the HTTP certifier for external servers is out of scope",
    "report": "no HTML report generator",
    "publish": "no report publisher",
    "witness": "no witness artifacts; use `replay` with a trace",
}


def _ids(text: str) -> list[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def cmd_run(argv) -> int:
    p = argparse.ArgumentParser(prog="lockstep run", description="Run a workload through the scheduler.")
    src = p.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="folder with config.json and model.safetensors")
    src.add_argument("--random", metavar="PRESET", help="random weights of a named configuration")
    p.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"])
    p.add_argument("--prompt-ids", action="append", default=[], metavar="IDS",
                   help="token ids of one prompt, comma or space separated (repeatable)")
    p.add_argument("--prompt-file", help="JSON lines: {uid, prompt, seed, max_new_tokens, temperature, top_p}")
    p.add_argument("--max-new-tokens", type=int, default=8)
    p.add_argument("--temperature", type=float, default=0.0, help="<= 0 is greedy")
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--req-seed", type=int, default=0, help="per-request sampling seed")
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    p.add_argument("--num-blocks", type=int, default=512, help="pages in the cache pool")
    p.add_argument("--prefill-chunk", type=int, default=None, help="cut prompts into portions of this many tokens")
    p.add_argument("--max-batched-tokens", type=int, default=None, help="token budget of one step")
    p.add_argument("--max-running", type=int, default=64)
    p.add_argument("--eos", type=int, action="append", default=[], help="end-of-sequence token id (repeatable)")
    p.add_argument("--enable-prefix-cache", action="store_true")
    p.add_argument("--reserve", default="full", choices=["full", "lazy"],
                   help="take a request's pages at admission (full) or step by step (lazy)")
    p.add_argument("--decode-burst", type=int, default=32,
                   help="up to this many greedy decode steps run on the GPU without the host in between (1: none)")
    args = p.parse_args(argv)

    import tempfile

    from .engine.config import EngineConfig
    from .engine.llm import LLM
    from .engine.scheduler import Request

    requests = []
    for i, text in enumerate(args.prompt_ids):
        requests.append(Request(uid=f"r{i:02d}", prompt=_ids(text), seed=args.req_seed,
                                max_new_tokens=args.max_new_tokens, temperature=args.temperature,
                                top_p=args.top_p))
    if args.prompt_file:
        for line in Path(args.prompt_file).read_text().splitlines():
            if line.strip():
                d = json.loads(line)
                requests.append(Request(uid=d.get("uid", f"f{len(requests):02d}"), prompt=list(d["prompt"]),
                                        seed=d.get("seed", args.req_seed),
                                        max_new_tokens=d.get("max_new_tokens", args.max_new_tokens),
                                        temperature=d.get("temperature", args.temperature),
                                        top_p=d.get("top_p", args.top_p)))
    if not requests:
        p.error("no prompts: give --prompt-ids or --prompt-file")

    with tempfile.TemporaryDirectory() as scratch:
        folder = args.model
        if args.random:
            from .config.presets import preset
            from .weights import write_random_model

            folder = write_random_model(preset(args.random), scratch, args.seed)
        engine = EngineConfig(dtype=args.dtype, num_pages=args.num_blocks, page_size=args.block_size,
                              max_batched_tokens=args.max_batched_tokens, prefill_chunk=args.prefill_chunk,
                              max_running=args.max_running, enable_prefix_cache=args.enable_prefix_cache,
                              eos_token_ids=tuple(args.eos), reserve=args.reserve, decode_burst=args.decode_burst)
        outputs = LLM(folder, engine).generate(requests)
    for uid in sorted(outputs):
        print(json.dumps({"uid": uid, "tokens": outputs[uid]}))
    return 0


def cmd_init(argv) -> int:
    p = argparse.ArgumentParser(prog="lockstep init", description="Write a model folder with random weights.")
    src = p.add_mutually_exclusive_group(required=True)
    src.add_argument("--preset", help="a named configuration")
    src.add_argument("--config", help="a config.json to take the sizes from")
    p.add_argument("--out", required=True)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--std", type=float, default=None, help="standard deviation of the matrices (default 0.02)")
    p.add_argument("--norm-std", type=float, default=None, help="norm weights are 1 + N(0, this) (default 0)")
    args = p.parse_args(argv)
    from .config import config_from_dict
    from .config.presets import preset
    from .weights import write_random_model

    config = preset(args.preset) if args.preset else config_from_dict(json.loads(Path(args.config).read_text()))
    out = write_random_model(config, args.out, args.seed, args.std, args.norm_std)
    print(out)
    return 0


def cmd_replay(argv) -> int:
    import runpy

    script = Path(__file__).resolve().parent.parent / "bin" / "trace_run"
    sys.argv = [str(script), *argv]
    try:
        runpy.run_path(str(script), run_name="__main__")
    except SystemExit as done:
        return int(done.code or 0)
    return 0


def cmd_bench(argv) -> int:
    import runpy

    script = Path(__file__).resolve().parent.parent / "bench.py"
    sys.argv = [str(script), *argv]
    try:
        runpy.run_path(str(script), run_name="__main__")
    except SystemExit as done:
        return int(done.code or 0)
    return 0


COMMANDS = {"run": cmd_run, "replay": cmd_replay, "bench": cmd_bench, "init": cmd_init}


def usage() -> int:
    print("lockstep <command> [args]\n")
    width = max(len(n) for n in list(COMMANDS) + list(NOT_BUILT))
    docs = {"run": "run prompts through the scheduler and print the generated token ids",
            "replay": "feed a trace of given tokens step by step and write logits (bin/trace_run)",
            "bench": "measure decode and prefill throughput (bench.py)",
            "init": "write a model folder with random weights"}
    for name in COMMANDS:
        print(f"  {name:<{width}}  {docs[name]}")
    for name, why in NOT_BUILT.items():
        print(f"  {name:<{width}}  not built: {why}")
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] in ("-h", "--help", "help"):
        return usage()
    command, rest = argv[0], argv[1:]
    if command in NOT_BUILT:
        print(f"lockstep {command} is not built: {NOT_BUILT[command]}")
        return 2
    if command not in COMMANDS:
        print(f"unknown command {command!r}. Try --help.")
        return 2
    return COMMANDS[command](rest)


if __name__ == "__main__":
    raise SystemExit(main())
