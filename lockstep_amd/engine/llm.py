"""Python entry points in the reference's manner.

The reference is driven as ``model = Qwen3(weights_dir, device, max_len)``;
``s = Scheduler(model, num_blocks, ...)``; ``s.submit(Request(...))``;
``outputs = s.run()`` and, for one prompt, ``model.generate_greedy(prompt,
max_new_tokens, eos_token_ids)`` (engine/model/qwen3.py:135,381-402;
engine/sched/scheduler.py:51-60,356-361).  Here ``load_model`` takes the
place of the hard-wired class (config.json picks the architecture), the
scheduler and the request keep their names and arguments, and ``LLM`` wraps
the three for the common case.
"""

from __future__ import annotations

from typing import Iterable, Sequence

from .batch import StepEntry
from .model import Model, load_model
from .policy import DefaultPolicy, FixedChunkPolicy, Policy
from .scheduler import Request, Scheduler


def generate_greedy(model: Model, prompt_ids: Sequence[int], max_new_tokens: int, eos_token_ids=None,
                    page_size: int = 16):
    """Greedy decoding of one prompt through the step function; returns the
    generated ids and the float32 logits each was picked from."""
    from ..sampling import Sampler

    total = len(prompt_ids) + max_new_tokens
    cache = model.make_cache(num_pages=-(-total // page_size), page_size=page_size, max_requests=1,
                             max_tokens_per_request=total)
    cache.open("seq")
    sampler = Sampler(model.rt.kernels)
    eos = set(eos_token_ids or ())
    request = Request(uid="seq", prompt=list(prompt_ids), max_new_tokens=max_new_tokens)
    tokens = list(prompt_ids)
    generated, step_logits = [], []
    for _ in range(max_new_tokens):
        logits = model.step(cache, [StepEntry("seq", tokens, [len(tokens) - 1])])
        step_logits.append(logits[0].clone())
        token = sampler.sample(logits, [request])[0]
        generated.append(token)
        request.generated.append(token)
        if token in eos:
            break
        tokens = [token]
    cache.close("seq")
    return generated, step_logits


class LLM:
    """A loaded model plus what a workload needs to run on it."""

    def __init__(self, model_dir, dtype: str = "bfloat16", device: str = "cuda:0", num_pages: int = 512,
                 page_size: int = 16, max_batched_tokens: int | None = None, prefill_chunk: int | None = None,
                 max_running: int = 64, enable_prefix_cache: bool = False, eos_token_ids=None,
                 reserve: str = "full", audit: bool = False, max_tokens_per_request: int | None = None,
                 decode_burst: int = 32):
        self.model = load_model(model_dir, dtype=dtype, device=device)
        self.options = dict(num_blocks=num_pages, block_size=page_size, max_batched_tokens=max_batched_tokens,
                            enable_prefix_cache=enable_prefix_cache, eos_token_ids=eos_token_ids, reserve=reserve,
                            audit=audit, max_tokens_per_request=max_tokens_per_request, decode_burst=decode_burst)
        self.prefill_chunk = prefill_chunk
        self.max_running = max_running

    def policy(self) -> Policy:
        if self.prefill_chunk:
            return FixedChunkPolicy(self.prefill_chunk, max_running=self.max_running)
        return DefaultPolicy(max_running=self.max_running)

    def scheduler(self, policy: Policy | None = None) -> Scheduler:
        return Scheduler(self.model, policy=policy or self.policy(), **self.options)

    def generate(self, requests: Iterable[Request], policy: Policy | None = None) -> dict:
        """Run the requests to completion; ``{uid: generated token ids}``."""
        scheduler = self.scheduler(policy)
        for request in requests:
            scheduler.submit(request)
        return scheduler.run()

    def generate_greedy(self, prompt_ids, max_new_tokens: int, eos_token_ids=None):
        return generate_greedy(self.model, prompt_ids, max_new_tokens, eos_token_ids)
