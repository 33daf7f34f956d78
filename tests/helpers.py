"""Helpers shared by the GPU tests: drive the engine's step function over a
request in portions and compare logits with the plain implementation."""

from __future__ import annotations

import numpy as np
import torch

FP32_TOL = 5e-5    # max |engine - plain| / max |plain| over a request, 32-bit path
BF16_TOL = 4e-2    # same, bfloat16 path


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
