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
device synchronisation; the run is repeated (``--repeats``, default 5) from freshly
prefilled requests and the median run is reported with the fastest and slowest beside it
(reference bench/lockstep_runner.py:30-42 and README.md:184-222: an untimed warm-up pass, then
the median of at least five runs with their spread).  One JSON line is printed.  The reference
publishes no tokens-a-second figure (it states ratios only), so ``vs_baseline`` is null.

    python bench.py --workload serve --model qwen3-8b

runs a whole workload through the scheduler instead, as the reference's own benchmark does
(bench/lockstep_runner.py:35-51: every request submitted at once, ``Scheduler.run()``, one
untimed pass first): 64 requests with prompt lengths uniform in [128, 4096] and 256 new tokens
each in prompt portions of 2,048 tokens (``qwen3-0.6b``, ``qwen3-8b``), or 16 requests of 8,192
tokens with 128 new tokens each (``qwen3-32b``).  ``--workload reference-trace`` runs the shape
of the reference's committed trace (eight prompts of 64 to 700 tokens, 32 new tokens each,
bench/throughput.py:35-45).  The value is all tokens (prompt and new) a second.

    python bench.py --workload contexts --model qwen3-8b --steps 32

measures a prompt in portions of 2,048 tokens and decode steps at batch 1, 8 and 64 at the
context lengths of ``--contexts`` (default 4,096, 8,192 and 16,384 tokens).
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
    print(f"[bench] drawing random weights for {args.model}", file=sys.stderr, flush=True)
    tensors = random_tensors(config, seed=0, std=0.02, norm_std=0.0, dtype=torch.bfloat16)
    print("[bench] weights drawn; loading them onto the GPU", file=sys.stderr, flush=True)
    model = model_from_tensors(config, tensors, dtype="bfloat16" if args.dtype == "bf16" else "float32")
    del tensors
    return model, config, full_layers


class Workload:
    """What a step costs, read from the model's own description rather than from one
    architecture's formulas: per run of a layer the elements of its matrices and vectors; what
    its mixer keeps between steps (``cache_spec()``: keys and values a token, or a state a
    request) and what mixing costs beyond the matrices (``mixing_flops``); the head's matrix."""

    def __init__(self, model):
        from lockstep_amd.parts import part_class

        spec = model.spec
        per_layer = []
        for layer_spec, layer in zip(spec.layers, model.layers):
            tensors = part_class(layer_spec.arrangement.kind).weight_specs(layer_spec)
            matrices = sum(_numel(w.shape) for w in tensors if w.kind == "matrix")
            vectors = sum(_numel(w.shape) for w in tensors if w.kind != "matrix")
            per_layer.append((matrices, vectors, layer.mixer))
        self.runs = [per_layer[run.layer] for run in spec.schedule]
        self.writers = [per_layer[run.layer][2] for run in spec.schedule if run.writes_cache]
        self.head = spec.vocab_size * spec.hidden_size
        self.hidden = spec.hidden_size

    def step_flops(self, tokens: int, start: int, wanted: int) -> float:
        """Multiply-adds times two of a step of ``tokens`` new tokens at positions ``start``.. of
        one request with ``wanted`` logit rows."""
        total = 2.0 * wanted * self.head
        for matrices, _, mixer in self.runs:
            total += 2.0 * tokens * matrices + (mixer.mixing_flops(tokens, start) if mixer is not None else 0.0)
        return total

    def decode_bytes(self, batch: int, context: float, element: int) -> float:
        """Bytes a decode step has to read: every weight it uses once, and what the mixers hold
        of the live requests."""
        weights = sum(matrices * element + vectors * 4 for matrices, vectors, _ in self.runs)
        weights += self.head * element + self.hidden * 4                     # head and final norm
        weights += batch * self.hidden * element                             # embedding rows
        held = sum(batch * cache_bytes(mixer.cache_spec(), context, element) for mixer in self.writers
                   if mixer is not None)
        return weights + held


def cache_bytes(spec, context: float, element: int) -> float:
    """Bytes one request of ``context`` tokens holds in a cache unit of this description."""
    from lockstep_amd.parts import PagedKVSpec, StateSpec

    if spec is None:
        return 0.0
    if isinstance(spec, PagedKVSpec):
        return min(context, spec.window or context) * 2 * spec.num_kv_heads * spec.head_dim * element
    if isinstance(spec, StateSpec):
        return _numel(spec.shape) * {"float32": 4, "int32": 4, "bfloat16": 2}[spec.dtype]
    raise TypeError(f"a cache unit described by {type(spec).__name__}: bench.py does not know its size")


def _numel(shape) -> int:
    n = 1
    for size in shape:
        n *= int(size)
    return n


def gpu_state() -> dict:
    """Clocks and temperatures of the GPU at this moment, as ``rocm-smi`` reports them (the
    reference records the same beside its measurements, bench/throughput.py:88-104); empty if
    the tool is missing or says nothing."""
    import re
    import subprocess

    try:
        out = subprocess.run(["rocm-smi", "--showclocks", "--showtemp", "--showpower", "--json"],
                             capture_output=True, text=True, timeout=20).stdout
        cards = json.loads(out[out.index("{"):])
    except (OSError, ValueError, subprocess.SubprocessError):
        return {}
    card = cards.get("card0") or next(iter(cards.values()), {})
    state = {}
    for key, value in card.items():
        number = re.search(r"-?\d+(\.\d+)?", str(value))
        if number is None:
            continue
        low = key.lower()
        for name, wanted in (("sclk_mhz", "sclk clock speed"), ("mclk_mhz", "mclk clock speed"),
                             ("fclk_mhz", "fclk clock speed"), ("temp_junction_c", "sensor junction"),
                             ("temp_memory_c", "sensor memory"), ("power_w", "power (w)")):
            if wanted in low:
                state[name] = float(number.group())
    return state


def states_record(before: dict, after: dict) -> dict:
    """Two readings of ``gpu_state`` as one flat record."""
    return {**{f"{k}_before": v for k, v in before.items()}, **{f"{k}_after": v for k, v in after.items()}}


def random_prompts(n: int, length: int, vocab: int, seed: int):
    import torch

    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(n)]


def measure_decode(model, cfg, batch: int, prompt_len: int, steps: int, warmup: int, page_size: int,
                   device_loop: bool = True, repeats: int = 1, progress: bool = False):
    """(seconds of the timed steps of every repeat, mean context length during them).  Every
    repeat starts from freshly prefilled requests and times exactly ``steps`` decode steps."""
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
            if progress:
                print(f"[bench] prompts of {lo + len(group)} of {batch} requests are in", file=sys.stderr, flush=True)
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

    def close_all():
        for r in requests:
            cache.close(r.uid)

    tokens = prefill()
    decode(tokens, warmup)
    close_all()
    times = []
    for _ in range(max(1, repeats)):
        tokens = prefill()
        decode(tokens, 1)          # the first step of a shape records its graph; keep that out of the timing
        torch.cuda.synchronize()
        started = time.perf_counter()
        decode(tokens, steps)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - started)
        close_all()
    del cache
    return times, prompt_len + 1 + steps / 2.0


def spread(times, steps: int) -> dict:
    return {"runs": len(times), "min_ms_per_step": round(1e3 * min(times) / steps, 4),
            "max_ms_per_step": round(1e3 * max(times) / steps, 4)}


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


def measure_prefill_portions(model, cfg, length: int, portion: int, page_size: int, repeats: int = 3):
    """Median seconds of a ``length``-token prompt run in portions of ``portion`` tokens (one request)."""
    import torch

    from lockstep_amd.engine.batch import StepEntry

    cache = model.make_cache(num_pages=-(-length // page_size) + 1, page_size=page_size, max_requests=1,
                             max_tokens_per_request=length)
    prompt = random_prompts(1, length, cfg.vocab_size, seed=length)[0]
    times = []
    for i in range(repeats + 1):
        cache.open("p")
        torch.cuda.synchronize()
        started = time.perf_counter()
        for lo in range(0, length, portion):
            part = prompt[lo:lo + portion]
            model.step(cache, [StepEntry("p", part, [len(part) - 1] if lo + portion >= length else [])])
        torch.cuda.synchronize()
        if i:
            times.append(time.perf_counter() - started)
        cache.close("p")
    del cache
    return statistics.median(times)


def contexts_record(args, model, cfg, full_layers: int) -> dict:
    """Prefill and decode at longer contexts: for every context length a prompt of that length in
    portions of ``--prefill-chunk`` tokens, and ``--steps`` decode steps of batches of 1, 8 and 64
    requests that hold that many tokens each (batches whose cache would not fit are left out)."""
    import torch

    element = 2 if args.dtype == "bf16" else 4
    portion = args.prefill_chunk or 2048
    rows = {}
    for context in [int(c) for c in args.contexts.split(",")]:
        print(f"[bench] context {context}: prefill in portions of {portion}", file=sys.stderr, flush=True)
        seconds = measure_prefill_portions(model, cfg, context, portion, args.page_size)
        flops = sum(Workload(model).step_flops(min(portion, context - lo), lo, 0) for lo in range(0, context, portion))
        row = {"prefill_tok_s": round(context / seconds, 1), "prefill_ms": round(1e3 * seconds, 2),
               "prefill_frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
        for batch in (1, 8, 64):
            cache_bytes = (batch * (context + args.steps + 64) * cfg.num_hidden_layers * 2
                           * cfg.num_key_value_heads * cfg.head_dim * element)
            free, _ = torch.cuda.mem_get_info()
            if cache_bytes > free - (12 << 30):
                continue
            print(f"[bench] context {context}: decode at batch {batch}", file=sys.stderr, flush=True)
            t, mean_context = measure_decode(model, cfg, batch, context, args.steps, 2, args.page_size,
                                             not args.host_sampling, 1, progress=True)
            step_s = t[0] / args.steps
            row[f"decode_b{batch}_tok_s"] = round(batch / step_s, 1)
            row[f"decode_b{batch}_ms"] = round(1e3 * step_s, 3)
            row[f"decode_b{batch}_hbm_frac"] = round(Workload(model).decode_bytes(batch, mean_context, element) / step_s
                                                     / PEAK_HBM, 4)
            torch.cuda.empty_cache()
        rows[str(context)] = row
    return {
        "metric": f"prefill and decode tok/s by context length ({args.model} layer sizes)",
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "dtype": args.dtype,
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
        "config": {"model": args.model, "layers": cfg.num_hidden_layers, "layers_of_model": full_layers,
                   "prefill_portion": portion, "page_size": args.page_size, "kernels": kernel_digest(model)},
        "contexts": rows,
    }


def kernel_digest(model) -> str:
    """Names of the loaded kernel libraries; each carries a hash of its sources and flags, which
    fixes every tile and split constant (reference engine/kernels/registry.py:163-166)."""
    kernels = model.rt.kernels
    names = [Path(kernels.core_path).stem] + [Path(p).stem for _, p in sorted(kernels.attention_paths.items())]
    return ",".join(n.replace("liblockstep_", "") for n in names)


def serve_trace(kind: str, model_name: str, vocab: int, n_requests: int = 0):
    """(prompts, new tokens each, prompt portion) of a serving workload, seeded."""
    import random

    import torch

    g = torch.Generator().manual_seed(20260805)
    rng = random.Random(64)
    if kind == "reference-trace":
        lengths, new, chunk = [64, 544, 96, 600, 80, 520, 112, 700], 32, None
    elif model_name == "qwen3-32b":
        lengths, new, chunk = [8192] * 16, 128, 2048
    else:
        lengths, new, chunk = [rng.randint(128, 4096) for _ in range(64)], 256, 2048
    if n_requests:
        lengths = lengths[:n_requests]
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths], new, chunk


def measure_serve(model, prompts, new_tokens: int, chunk, page_size: int, max_batched_tokens, repeats: int,
                  temperature: float = 0.0, top_p: float = 1.0):
    """Run the workload ``repeats`` + 1 times through the scheduler (the first pass untimed).
    Returns per timed pass (seconds, seconds until no prompt token was left, scheduler steps,
    steps of the decode-only phase)."""
    import torch

    from lockstep_amd.engine.policy import DefaultPolicy, FixedChunkPolicy
    from lockstep_amd.engine.scheduler import Request, Scheduler

    n = len(prompts)
    longest = max(len(p) for p in prompts) + new_tokens
    pages = sum(-(-(len(p) + new_tokens) // page_size) for p in prompts) + 8
    cache = model.make_cache(num_pages=pages, page_size=page_size, max_requests=n, max_tokens_per_request=longest)
    passes = []
    for i in range(repeats + 1):
        policy = FixedChunkPolicy(chunk, max_running=n) if chunk else DefaultPolicy(max_running=n)
        scheduler = Scheduler(model, num_blocks=pages, policy=policy, audit=False, block_size=page_size,
                              max_batched_tokens=max_batched_tokens, cache=cache, decode_burst=32)
        for j, prompt in enumerate(prompts):
            scheduler.submit(Request(uid=f"r{j:02d}", prompt=prompt, seed=j, max_new_tokens=new_tokens,
                                     temperature=temperature, top_p=top_p))
        torch.cuda.synchronize()
        started = time.perf_counter()
        prompts_done_at, steps_at = None, 0
        while scheduler.advance():
            if prompts_done_at is None and not scheduler.waiting and all(
                    r.cached >= r.n_prompt for r in scheduler.running):
                torch.cuda.synchronize()
                prompts_done_at, steps_at = time.perf_counter() - started, scheduler.step_index
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        done = {r.uid: r.n_generated for r in scheduler.done}
        if len(done) != n or any(v != new_tokens for v in done.values()):
            raise RuntimeError(f"the workload did not finish: {len(done)} of {n} requests done")
        if i:
            passes.append((elapsed, prompts_done_at if prompts_done_at is not None else elapsed,
                           scheduler.step_index, scheduler.step_index - steps_at))
    del cache
    return passes


def serve_record(args, model, cfg, full_layers) -> dict:
    prompts, new_tokens, chunk = serve_trace(args.workload, args.model, cfg.vocab_size, args.requests)
    if args.prefill_chunk is not None:
        chunk = args.prefill_chunk or None
    if args.new_tokens:
        new_tokens = args.new_tokens
    state_before = gpu_state()
    passes = measure_serve(model, prompts, new_tokens, chunk, args.page_size, args.max_batched_tokens,
                           args.repeats, args.temperature, args.top_p)
    state_after = gpu_state()
    order = sorted(passes, key=lambda t: t[0])
    elapsed, prompts_done, steps, decode_steps = order[len(order) // 2]
    prompt_tokens = sum(len(p) for p in prompts)
    total_new = new_tokens * len(prompts)
    decode_seconds = elapsed - prompts_done
    return {
        "metric": (f"serve tok/s, prompt and new tokens ({args.model} layer sizes, {len(prompts)} requests through the "
                   f"scheduler, {args.workload})"),
        "value": round((prompt_tokens + total_new) / elapsed, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": 1,
        "ms_per_step": round(1e3 * elapsed / steps, 4),
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
            "requests": len(prompts), "prompt_tokens": prompt_tokens, "longest_prompt": max(len(p) for p in prompts),
            "new_tokens": new_tokens, "prefill_chunk": chunk or 0, "max_batched_tokens": args.max_batched_tokens or 0,
            "page_size": args.page_size, "parallelism": "single GPU", "decode_loop": "hip graphs, device token feedback",
            "kernels": kernel_digest(model),
        },
        "serve": {
            "seconds": round(elapsed, 4), "runs": len(passes), "min_s": round(order[0][0], 4),
            "max_s": round(order[-1][0], 4), "new_tokens_per_s": round(total_new / elapsed, 1),
            "until_prompts_done_s": round(prompts_done, 4), "decode_only_s": round(decode_seconds, 4),
            "decode_only_steps": decode_steps,
            "decode_only_step_ms": round(1e3 * decode_seconds / decode_steps, 4) if decode_steps else None,
            "sampling": "greedy" if args.temperature <= 0 else f"temperature {args.temperature}, top_p {args.top_p}",
        },
        "gpu_state": states_record(state_before, state_after),
    }


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
    p.add_argument("--workload", default="decode", choices=["decode", "serve", "reference-trace", "contexts"],
                   help="decode: fixed batches (the headline); serve / reference-trace: a workload through the "
                        "scheduler; contexts: prefill and decode at the context lengths of --contexts")
    p.add_argument("--contexts", default="4096,8192,16384", help="contexts: the context lengths, comma separated")
    p.add_argument("--repeats", type=int, default=5, help="timed runs; the median is reported with the spread")
    p.add_argument("--requests", type=int, default=0, help="serve: only the first N requests of the workload")
    p.add_argument("--prefill-chunk", type=int, default=None, help="serve: prompt portion (0: whole prompts)")
    p.add_argument("--max-batched-tokens", type=int, default=8192, help="serve: token budget of a step (0: none)")
    p.add_argument("--temperature", type=float, default=0.0,
                   help="serve: requests draw their tokens at this temperature (0: greedy), a seed a request")
    p.add_argument("--top-p", type=float, default=1.0, help="serve: nucleus of the requests that draw their tokens")
    p.add_argument("--new-tokens", type=int, default=0, help="serve: new tokens a request (0: the workload's own)")
    p.add_argument("--only-prefill", action="store_true",
                   help="run the prefill measurement alone and print its record (for profiling)")
    args = p.parse_args(argv)

    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {args.gpus})")
        return 2

    import torch

    model, cfg, full_layers = build_model(args)
    element = 2 if args.dtype == "bf16" else 4

    if args.workload == "contexts":
        print(json.dumps(contexts_record(args, model, cfg, full_layers)))
        return 0
    if args.workload != "decode":
        print(json.dumps(serve_record(args, model, cfg, full_layers)))
        return 0

    if args.only_prefill:
        seconds = measure_prefill(model, cfg, args.prefill_len, args.page_size)
        print(json.dumps({"prefill": {"value": round(args.prefill_len / seconds, 1), "tokens": args.prefill_len,
                                      "ms": round(1e3 * seconds, 3)}}))
        return 0

    state_before = gpu_state()
    times, context = measure_decode(model, cfg, args.batch, args.prompt_len, args.steps, args.warmup,
                                    args.page_size, not args.host_sampling, args.repeats)
    state_after = gpu_state()
    elapsed = statistics.median(times)
    ms_per_step = 1e3 * elapsed / args.steps
    value = args.batch * args.steps / elapsed
    bytes_step = Workload(model).decode_bytes(args.batch, context, element)
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
            "prefill_len": args.prefill_len, "parallelism": "single GPU",
            "decode_loop": ("hip graphs" if model.use_graphs else "eager") +
                           (", host sampling" if args.host_sampling else ", device token feedback"),
            "kernels": kernel_digest(model),
        },
        "spread": spread(times, args.steps),
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM, 4)},
        # clocks and temperatures right before and right after the headline's timed runs
        "gpu_state": states_record(state_before, state_after),
    }

    if not args.no_points:
        seconds = measure_prefill(model, cfg, args.prefill_len, args.page_size)
        flops = Workload(model).step_flops(args.prefill_len, 0, 1)
        record["prefill"] = {"value": round(args.prefill_len / seconds, 1), "tokens": args.prefill_len,
                             "ms": round(1e3 * seconds, 3),
                             "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4)}
        points, point_spread = {}, {}
        for batch, steps in ((1, args.steps), (64, args.steps)):
            t, _ = measure_decode(model, cfg, batch, args.prompt_len, steps, min(args.warmup, 4), args.page_size,
                                  not args.host_sampling, args.repeats)
            points[f"decode_b{batch}"] = round(batch * steps / statistics.median(t), 1)
            point_spread[f"decode_b{batch}"] = spread(t, steps)
        record["points"] = points
        record["points_spread"] = point_spread
    torch.cuda.synchronize()
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
