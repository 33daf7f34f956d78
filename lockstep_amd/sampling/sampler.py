"""Greedy and temperature / nucleus sampling.

``greedy`` takes the lowest token id among the maxima of the row in float32
(reference engine/sampler/philox.py:64-68); on the GPU it is one arg-max
kernel over all rows of the step.  ``top_p`` follows the reference's
procedure in float64 (engine/sampler/philox.py:71-98), here on the host and,
for logits on the GPU, in a kernel that finds the same token without sorting
(``Kernels.sample_top_p``; the two can part only where a draw lands within
rounding of a token's boundary):
temperature <= 0 is greedy; else softmax of float32(row)/T, tokens ordered by
(-probability, id), the shortest head whose cumulative sum reaches ``p`` is
kept, and the draw ``u * sum(head)`` picks the first token whose cumulative
sum reaches it.  ``u`` comes from the counter-based generator keyed on
(seed, uid, position).
"""

from __future__ import annotations

import torch

from . import philox


def greedy(row: torch.Tensor) -> int:
    values = row.detach().to(torch.float32).cpu()
    best = values.max()
    return int(torch.nonzero(values == best)[0].item())


def top_p(row: torch.Tensor, seed: int, uid: str, position: int, p: float = 1.0, temperature: float = 1.0) -> int:
    if temperature <= 0:
        return greedy(row)
    values = (row.detach().to(torch.float32) / temperature).to(torch.float64).cpu()
    shifted = values - values.max()
    weights = shifted.exp()
    probs = weights / weights.sum()
    # descending and stable: equal probabilities stay in ascending id order
    ordered, order = torch.sort(probs, descending=True, stable=True)
    cumulative = torch.cumsum(ordered, dim=0)
    keep = int(torch.searchsorted(cumulative, torch.tensor(float(p), dtype=torch.float64)).item()) + 1
    keep = min(keep, ordered.numel())
    head = ordered[:keep]
    draw = philox.uniform(seed, uid, position) * float(head.sum())
    chosen = int(torch.searchsorted(torch.cumsum(head, dim=0), torch.tensor(draw, dtype=torch.float64)).item())
    return int(order[min(chosen, keep - 1)].item())


class Sampler:
    """Samples one token for each finished row of a step."""

    def __init__(self, kernels=None):
        self.kernels = kernels

    def sample(self, logits: torch.Tensor, requests) -> list[int]:
        """``logits [n, V]`` float32; ``requests[i]`` has ``uid, seed,
        temperature, top_p`` and ``total_tokens()``; row i is the row of the
        request's last token, whose position is ``total_tokens() - 1``
        (reference engine/sched/scheduler.py:293-310)."""
        n = len(requests)
        out: list[int | None] = [None] * n
        greedy_rows = [i for i, r in enumerate(requests) if r.temperature <= 0]
        if greedy_rows:
            if logits.is_cuda and self.kernels is not None:
                picked = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
                self.kernels.argmax(logits, picked)
                host = picked.cpu().tolist()
                for i in greedy_rows:
                    out[i] = int(host[i])
            else:
                for i in greedy_rows:
                    out[i] = greedy(logits[i])
        drawn = [i for i in range(n) if out[i] is None]
        if drawn and logits.is_cuda and self.kernels is not None:
            # the same procedure on the device, the draw included (csrc/sample.hip)
            picked = torch.empty(len(drawn), dtype=torch.int32, device=logits.device)
            self.kernels.sample_top_p(
                logits, [(i, float(requests[i].temperature), float(requests[i].top_p),
                          int(requests[i].seed) ^ philox.uid_key(requests[i].uid), requests[i].total_tokens() - 1)
                         for i in drawn], picked)
            for i, token in zip(drawn, picked.cpu().tolist()):
                out[i] = int(token)
            return out  # type: ignore[return-value]
        for i in drawn:
            r = requests[i]
            out[i] = top_p(logits[i], r.seed, r.uid, r.total_tokens() - 1, r.top_p, r.temperature)
        return out  # type: ignore[return-value]
