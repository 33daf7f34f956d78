"""Throughput of the engine on one MI355X: decoded tokens a second at batch 8
(the headline value), at batch 1 and 64, and prefill of one 2,048-token
prompt, with random weights at the Qwen3-0.6B layer sizes.

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the whole batch: the engine's step function
followed by greedy sampling of every request's next token, which is fed back
in the next step.  By default the pick is fed back on the device
(``Model.decode_greedy``: the captured step is launched K times and the host
reads the tokens once at the end); ``--host-sampling`` brings every step's
logits to the ``Sampler`` on the host instead.  Requests start from 512-token random prompts (prefilled
outside the timed region); K timed steps follow W untimed ones, bracketed by
device synchronisation.  One JSON line is printed.  The reference publishes no
tokens-a-second figure (it states ratios only), so ``vs_baseline`` is null.
"""

from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}   # dense MFMA peaks of MI355X
PEAK_HBM = 8.0e12                                  # bytes a second


def build_model(args):
    import torch

    from lockstep_amd.config.presets import preset
    from lockstep_amd.engine.model import model_from_tensors
    from lockstep_amd.weights import random_tensors

    overrides = {}
    if args.layers:
        overrides["num_hidden_layers"] = args.layers
    config = preset(args.model, **overrides)
    full_layers = preset(args.model).num_hidden_layers
    tensors = random_tensors(config, seed=0, std=0.02, norm_std=0.0, dtype=torch.bfloat16)
    model = model_from_tensors(config, tensors, dtype="bfloat16" if args.dtype == "bf16" else "float32")
    del tensors
    return model, config, full_layers


def matrix_params_per_layer(cfg) -> int:
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim * cfg.hidden_size
    out = cfg.hidden_size * cfg.num_attention_heads * cfg.head_dim
    mlp = 3 * cfg.intermediate_size * cfg.hidden_size
    return qkv + out + mlp


def step_flops(cfg, tokens: int, start: int, wanted: int) -> float:
    """Multiply-adds times two of a step of ``tokens`` new tokens at positions
    ``start``.. of one request with ``wanted`` logit rows."""
    dense = 2.0 * tokens * matrix_params_per_layer(cfg)
    pairs = sum(start + i + 1 for i in range(tokens))               # visible (query, key) pairs
    attention = 4.0 * cfg.head_dim * cfg.num_attention_heads * pairs
    return cfg.num_hidden_layers * (dense + attention) + 2.0 * wanted * cfg.vocab_size * cfg.hidden_size


def decode_bytes(cfg, batch: int, context: float, element: int) -> float:
    """Bytes a decode step has to read: every weight it uses once, and the
    cache of the live requests."""
    weights = cfg.num_hidden_layers * (matrix_params_per_layer(cfg) * element + 2 * cfg.hidden_size * 4
                                       + 2 * cfg.head_dim * 4)
    weights += cfg.vocab_size * cfg.hidden_size * element + cfg.hidden_size * 4     # head and final norm
    weights += batch * cfg.hidden_size * element                                     # embedding rows
    kv = batch * context * cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * cfg.head_dim * element
    return weights + kv


def random_prompts(n: int, length: int, vocab: int, seed: int):
    import torch

    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(n)]


def measure_decode(model, cfg, batch: int, prompt_len: int, steps: int, warmup: int, page_size: int,
                   device_loop: bool = True):
    """(seconds of the timed steps, mean context length during them)."""
    import torch

    from lockstep_amd.engine.batch import StepEntry
    from lockstep_amd.engine.scheduler import Request
    from lockstep_amd.sampling import Sampler

    total = prompt_len + max(steps, warmup) + 1
    pages = batch * (-(-total // page_size)) + 8
    cache = model.make_cache(num_pages=pages, page_size=page_size, max_requests=batch,
                             max_tokens_per_request=total)
    sampler = Sampler(model.rt.kernels)
    requests = [Request(uid=f"b{i}", prompt=p, max_new_tokens=steps + warmup)
                for i, p in enumerate(random_prompts(batch, prompt_len, cfg.vocab_size, seed=batch))]

    def prefill():
        tokens = []
        for lo in range(0, batch, 4):
            group = requests[lo:lo + 4]
            for r in group:
                cache.open(r.uid)
            logits = model.step(cache, [StepEntry(r.uid, r.prompt, [len(r.prompt) - 1]) for r in group])
            tokens += sampler.sample(logits, group)
        return tokens

    def decode(tokens, n):
        if n <= 0:
            return tokens
        if device_loop:
            # the greedy pick of every step is fed back on the device; the host reads the tokens at the end
            picked = model.decode_greedy(cache, [r.uid for r in requests], tokens, n)
            return picked[-1].tolist()
        for _ in range(n):
            logits = model.step(cache, [StepEntry(r.uid, [t], [0]) for r, t in zip(requests, tokens)])
            tokens = sampler.sample(logits, requests)
        return tokens

    tokens = prefill()
    decode(tokens, warmup)
    for r in requests:
        cache.close(r.uid)
    tokens = prefill()
    decode(tokens, 1)          # the first step of a shape records its graph; keep that out of the timing
    torch.cuda.synchronize()
    started = time.perf_counter()
    decode(tokens, steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    for r in requests:
        cache.close(r.uid)
    del cache
    return elapsed, prompt_len + 1 + steps / 2.0


def measure_prefill(model, cfg, length: int, page_size: int, repeats: int = 5):
    import torch

    from lockstep_amd.engine.batch import StepEntry

    cache = model.make_cache(num_pages=-(-length // page_size) + 1, page_size=page_size, max_requests=1,
                             max_tokens_per_request=length)
    prompt = random_prompts(1, length, cfg.vocab_size, seed=2048)[0]
    times = []
    for i in range(repeats + 1):
        cache.open("p")
        torch.cuda.synchronize()
        started = time.perf_counter()
        model.step(cache, [StepEntry("p", prompt, [length - 1])])
        torch.cuda.synchronize()
        if i:
            times.append(time.perf_counter() - started)
        cache.close("p")
    return statistics.median(times)


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=256, help="timed decode steps (default: the workload's 256 new tokens)")
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--model", default="qwen3-0.6b", help="named configuration (layer sizes)")
    p.add_argument("--layers", type=int, default=0, help="run fewer layers than the configuration has (reported)")
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--prompt-len", type=int, default=512)
    p.add_argument("--prefill-len", type=int, default=2048)
    p.add_argument("--page-size", type=int, default=16)
    p.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    p.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points and the prefill")
    p.add_argument("--host-sampling", action="store_true",
                   help="pick every step's tokens on the host (Model.step + Sampler) instead of the device-side loop")
    p.add_argument("--only-prefill", action="store_true",
                   help="run the prefill measurement alone and print its record (for profiling)")
    args = p.parse_args(argv)

    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {args.gpus})")
        return 2

    import torch

    model, cfg, full_layers = build_model(args)
    element = 2 if args.dtype == "bf16" else 4

    if args.only_prefill:
        seconds = measure_prefill(model, cfg, args.prefill_len, args.page_size)
        print(json.dumps({"prefill": {"value": round(args.prefill_len / seconds, 1), "tokens": args.prefill_len,
                                      "ms": round(1e3 * seconds, 3)}}))
        return 0

    elapsed, context = measure_decode(model, cfg, args.batch, args.prompt_len, args.steps, args.warmup,
                                      args.page_size, not args.host_sampling)
    ms_per_step = 1e3 * elapsed / args.steps
    value = args.batch * args.steps / elapsed
    bytes_step = decode_bytes(cfg, args.batch, context, element)
    achieved = bytes_step / (elapsed / args.steps)

    record = {
        "metric": f"decode tok/s at batch {args.batch} ({args.model} layer sizes, {args.prompt_len}-token prompts, greedy)",
        "value": round(value, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
        "config": {
            "model": args.model, "layers": cfg.num_hidden_layers, "layers_of_model": full_layers,
            "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "tie_word_embeddings": cfg.tie_word_embeddings,
            "global_batch": args.batch, "prompt_len": args.prompt_len, "new_tokens": args.steps,
            "seq_len": args.prompt_len + args.steps, "max_context": 4096, "page_size": args.page_size,
            "prefill_len": args.prefill_len, "parallelism": "single GPU", "hip_graphs": bool(model.use_graphs),
            "token_feedback": "host" if args.host_sampling else "device",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM, 4)},
    }

    if not args.no_points:
        seconds = measure_prefill(model, cfg, args.prefill_len, args.page_size)
        flops = step_flops(cfg, args.prefill_len, 0, 1)
        record["prefill"] = {"value": round(args.prefill_len / seconds, 1), "tokens": args.prefill_len,
                             "ms": round(1e3 * seconds, 3),
                             "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
        points = {}
        for batch, steps in ((1, args.steps), (64, args.steps)):
            t, _ = measure_decode(model, cfg, batch, args.prompt_len, steps, min(args.warmup, 4), args.page_size,
                                  not args.host_sampling)
            points[f"decode_b{batch}"] = round(batch * steps / t, 1)
        record["points"] = points
    torch.cuda.synchronize()
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
