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
from .config import EngineConfig
from .model import Model, load_model
from .policy import Policy
from .scheduler import Request, Scheduler
from .scheduler import Sequence as SchedulerSequence


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
    seq = SchedulerSequence(Request(uid="seq", prompt=list(prompt_ids), max_new_tokens=max_new_tokens))
    feed = list(seq.tokens)
    step_logits = []
    for _ in range(max_new_tokens):
        logits = model.step(cache, [StepEntry("seq", feed, [len(feed) - 1])])
        step_logits.append(logits[0].clone())
        token = sampler.sample(logits, [seq])[0]
        seq.tokens.append(token)
        if token in eos:
            break
        feed = [token]
    cache.close("seq")
    return seq.generated, step_logits


class LLM:
    """A loaded model plus what a workload needs to run on it.  Options are an ``EngineConfig``
    or its fields as keywords."""

    def __init__(self, model_dir, config: EngineConfig | None = None, device: str = "cuda:0", **options):
        self.config = (config or EngineConfig()).with_(**options) if options else (config or EngineConfig())
        self.model = load_model(model_dir, dtype=self.config.dtype, device=device)

    def policy(self) -> Policy:
        return self.config.policy()

    def scheduler(self, policy: Policy | None = None) -> Scheduler:
        return Scheduler.from_config(self.model, self.config, policy)

    def generate(self, requests: Iterable[Request], policy: Policy | None = None) -> dict:
        """Run the requests to completion; ``{uid: generated token ids}``."""
        scheduler = self.scheduler(policy)
        for request in requests:
            scheduler.submit(request)
        return scheduler.run()

    def generate_greedy(self, prompt_ids, max_new_tokens: int, eos_token_ids=None):
        return generate_greedy(self.model, prompt_ids, max_new_tokens, eos_token_ids)
