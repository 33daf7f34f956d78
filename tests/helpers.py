"""Helpers shared by the GPU tests: drive the engine's step function over a
request in portions and compare logits with the plain implementation."""

from __future__ import annotations

import math

import numpy as np
import torch

# Bounds on max |engine - plain| / max |plain| over a request.  Each is about three times the
# largest error measured on the MI355X for the weights it is used with, so a fault that moves
# the logits by a few times the rounding noise fails.
FP32_TOL = 2e-5        # 32-bit path on the sharpened weights (measured up to 7e-6: peaked attention
                       # multiplies the rounding of the scores; 1e-6 on weights as drawn)
FP32_TOL_SOFT = 5e-6   # 32-bit path on weights as drawn and on the generation weights (measured up to 2e-6)
BF16_TOL = 2e-2        # bfloat16 path against exact arithmetic, weights as drawn (measured up to 6e-3)
# bfloat16 path against the plain forward that stores in bfloat16 where the engine does
# (``store=bf16``): until the first value lands on the other side of a rounding boundary the two agree
# to 1e-7; afterwards the difference is that of a few flipped roundings.  One bound for each test
# configuration, some three times the largest error measured on its sharpened weights (A: 4e-3, B: 2.4e-2
# over 340 and 700 tokens).  B's is five times A's because B's attention is far more peaked: its matrices are drawn
# 2.5 times wider (std 0.05 against 0.02), its norm weights vary, and it has three
# layers to A's two.  Where one key holds most of a row's weight, a score that moves by one bfloat16 step moves
# the output by a visible fraction; the same sensitivity shows in what a single lost key does (A: 4.3e-2 of the
# largest logit, B: 0.78 -- eighteen times as much), so the ratio of fault to bound is no worse for B.  (The
# bfloat16 softmax also uses the fast exponential, good to about 2 ulp of float32: far below a bfloat16 step,
# but one more source of flipped roundings.)  A single lost key exceeds three times these bounds.
BF16_STORED_TOL = {"A": 1.2e-2, "B": 6e-2}
BF16_STORED_TOL_WINDOW_TOY = 4e-2   # the windowed toy of test_window_gpu.py (measured 1.3e-2; a window one key too wide: 0.57)
BF16_EXACT_PREFIX_TOL = 1e-6   # ... and the bound while no rounding has flipped yet (the first positions)


def tol_for(dtype: str, name: str) -> float:
    """The bound for the engine against the plain forward on the sharpened weights of configuration ``name``."""
    return FP32_TOL if dtype == "float32" else BF16_STORED_TOL[name]


def rel_err(got, want) -> float:
    got = torch.as_tensor(np.asarray(got)).double()
    want = torch.as_tensor(np.asarray(want)).double()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def feed(model, cache, rid, tokens, cuts, want_all=True):
    """Feed ``tokens`` of request ``rid`` in portions of the sizes ``cuts``
    (the last portion takes the rest); return logits ``[len(tokens), V]``."""
    from lockstep_amd.engine.batch import StepEntry

    if rid not in cache.requests:
        cache.open(rid)
    out = []
    pos = 0
    sizes = list(cuts)
    while pos < len(tokens):
        take = sizes.pop(0) if sizes else len(tokens) - pos
        take = min(take, len(tokens) - pos)
        chunk = tokens[pos:pos + take]
        logits = model.step(cache, [StepEntry(rid, chunk, list(range(take)) if want_all else [])])
        if logits is not None:
            out.append(logits.cpu())
        pos += take
    return torch.cat(out) if out else None


def make_mixed_trace(requests: dict, seed: int, max_live: int = 4, decode_tail: int = 8, max_portion: int = 19):
    """Steps in the trace-replay format that run ``requests`` (id -> tokens)
    with up to ``max_live`` live at a time: portions of changing size (down to
    two tokens) for prompts, the last ``decode_tail`` tokens of each request one
    by one, some requests sitting out a step, all logits wanted.  A finished
    request ends and the next one starts, so pages are used again."""
    import random

    rng = random.Random(seed)
    waiting = list(requests)
    live: dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                    # sits this step out
            tokens, pos = requests[rid], live[rid]
            left = len(tokens) - pos
            if left <= decode_tail:
                take = 1
            else:
                take = min(left - decode_tail, rng.choice([2, 2, 3, 5, 8, 13, max_portion]))
                if left - decode_tail - take == 1:          # never leave a portion of one token
                    take += 1
            entries.append({"id": rid, "tokens": tokens[pos:pos + take], "want": list(range(take))})
            live[rid] = pos + take
            if live[rid] == len(tokens):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def replay_in_process(model, cache, steps):
    """Run trace steps through ``model.step``; per-request logits in order."""
    from lockstep_amd.engine.batch import StepEntry

    out: dict[str, list] = {}
    for step in steps:
        entries = []
        for e in step["entries"]:
            if e["id"] not in cache.requests:
                cache.open(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = model.step(cache, entries)
        row = 0
        for e in step["entries"]:
            n = len(e["want"])
            if n:
                out.setdefault(e["id"], []).append(logits[row:row + n].cpu())
                row += n
        for rid in step["end"]:
            cache.close(rid)
        cache.audit()
    return {rid: torch.cat(parts) for rid, parts in out.items()}


def max_live_tokens(steps, round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up."""
    held: dict[str, int] = {}
    worst = 0
    for step in steps:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return worst


def sampling_rows_on_boundaries(vocab: int, rows: int = 24, seed: int = 0):
    """Logits rows and sampling requests on which a change in the order of any of the sampler's sums
    shows as another token.  A row takes four values a quarter apart, so its weights are a few long
    runs of equal, irrational addends; the nucleus is put exactly on the boundary between two tokens
    (top_p = the cumulative weight up to a token / the total, both summed here without rounding
    error, so that the quotient is off by its own rounding only), so whether that token is still
    inside is decided in the last bit of the kernel's own sums, and the head it leaves scales the draw.  Returns (float32 logits [rows, vocab], requests as ``sample_top_p`` takes them)."""
    from lockstep_amd.sampling import philox

    g = torch.Generator().manual_seed(seed + vocab)
    logits = torch.randint(0, 4, (rows, vocab), generator=g).float() * -0.25
    key = philox.uid_key("boundaries")
    requests = []
    for i in range(rows):
        temperature = [0.7, 1.0, 1.9, 0.45][i % 4]
        values = (logits[i] / torch.tensor(temperature, dtype=torch.float32)).double()
        weights = (values - values.max()).exp()
        ordered = torch.sort(weights, descending=True, stable=True)[0].tolist()
        at = int(vocab * (0.15 + 0.7 * (i + 1) / (rows + 1)))
        top_p = math.fsum(ordered[: at + 1]) / math.fsum(ordered)
        requests.append((i, temperature, top_p, (31 + i) ^ key, 2000 + 13 * i))
    return logits, requests
