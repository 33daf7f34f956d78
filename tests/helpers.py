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
