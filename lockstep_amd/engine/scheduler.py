"""Continuous batching above the step function.

Each step: admit waiting requests while the policy and the pages allow; give
every running request its next tokens under a token budget (decoded tokens
first, then prompt portions in admission order, each cut by the policy); run
them as one batch; sample for the requests whose whole context is now cached;
finish and free.  The loop follows the reference scheduler
(engine/sched/scheduler.py:205-361); the token budget, the choice of when
pages are taken and the automatic preemption are additions.

When pages run out:

* ``submit`` refuses a request that could not fit an empty pool
  (``OversizedRequest``; reference engine/sched/scheduler.py:90-104).
* With ``reserve="full"`` (default, the reference's behaviour) a request's
  pages for prompt + max_new_tokens are taken at admission, so a request that
  does not fit simply waits and a running request never lacks a page.  Pages
  held only by the prefix index are evicted first (lowest id by default).
* With ``reserve="lazy"`` pages are taken step by step.  If a running request
  cannot grow, the most recently admitted other request is preempted: its
  pages are freed, it returns to the front of the queue and its context is
  recomputed later, which gives the same tokens because results do not depend
  on how the work is cut (reference engine/sched/scheduler.py:195-203).
* If nothing runs and nothing can be admitted the step raises ``OutOfPages``
  (reference engine/sched/scheduler.py:226-232).
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..cache import OutOfPages, PrefixIndex
from .audit import Counters, TrajectoryHash
from .batch import StepEntry
from .policy import DefaultPolicy, Event, Policy, SchedulerState


@dataclass
class Request:
    """Token ids in, token ids out (reference engine/sched/scheduler.py:19-43)."""

    uid: str
    prompt: list
    seed: int = 0
    max_new_tokens: int = 8
    temperature: float = 0.0
    top_p: float = 1.0

    generated: list = field(default_factory=list)
    finished: bool = False
    kv_len: int = 0
    preempt_count: int = 0
    cache_hit_tokens: int = 0

    def context(self) -> list:
        return list(self.prompt) + list(self.generated)

    def total_tokens(self) -> int:
        return len(self.prompt) + len(self.generated)


class OversizedRequest(ValueError):
    """The request cannot fit the pool even when the pool is empty."""


class Scheduler:
    def __init__(self, model, num_blocks: int, policy: Policy | None = None, eos_token_ids=None,
                 audit: bool = True, block_size: int = 16, enable_prefix_cache: bool = False, *,
                 max_batched_tokens: int | None = None, reserve: str = "full", max_requests: int | None = None,
                 max_tokens_per_request: int | None = None, sampler=None, cache=None, keep_logits: bool = False,
                 decode_burst: int = 1):
        """``num_blocks`` pages of ``block_size`` tokens (the reference's names).
        ``max_batched_tokens`` bounds the tokens of one step (None: no bound).
        ``decode_burst`` > 1: while nothing waits, every running request is decoding greedily and no
        decision could differ from step to step (default policy, pages reserved in full, no
        end-of-sequence ids, no audit), up to that many decode steps run as one call of the model's
        device-side loop (``decode_greedy``); the tokens are those of single steps."""
        if reserve not in ("full", "lazy"):
            raise ValueError("reserve must be 'full' or 'lazy'")
        self.model = model
        self.policy = policy or DefaultPolicy()
        self.eos = set(eos_token_ids or ())
        self.audit_enabled = audit
        self.reserve_mode = reserve
        self.max_batched_tokens = max_batched_tokens
        self.keep_logits = keep_logits
        self.decode_burst = max(1, int(decode_burst))
        self.counters = Counters()
        self.lifecycle: dict[str, list] = {}
        max_running = getattr(self.policy, "max_running", 64)
        if cache is None:
            cache = model.make_cache(num_pages=num_blocks, page_size=block_size,
                                     max_requests=max_requests or max(max_running, 1),
                                     max_tokens_per_request=max_tokens_per_request)
        self.cache = cache
        self.page_size = cache.page_size
        self.num_pages = min(g.pool.num_pages for g in cache.groups) if cache.groups else num_blocks
        self.prefix = PrefixIndex(self.page_size) if enable_prefix_cache and cache.shareable() else None
        if sampler is None:
            from ..sampling import Sampler

            sampler = Sampler(getattr(getattr(model, "rt", None), "kernels", None))
        self.sampler = sampler
        self.waiting: list[Request] = []
        self.running: list[Request] = []
        self.done: list[Request] = []
        self.step_index = 0
        self.evictions = 0
        self.trajectory = TrajectoryHash()
        self.emitted_logits: dict[str, list] = {}

    # -- bookkeeping -------------------------------------------------------------
    def _event(self, uid: str, event: Event) -> None:
        self.lifecycle.setdefault(uid, []).append(event)

    def _pages_for(self, tokens: int) -> int:
        return -(-tokens // self.page_size)

    def _pages_needed(self, request: Request) -> int:
        return self._pages_for(len(request.prompt) + request.max_new_tokens)

    def _free_pages(self) -> int:
        return min(self.cache.free_pages) if self.cache.groups else self.num_pages

    def _state(self) -> SchedulerState:
        return SchedulerState(
            step=self.step_index,
            waiting=tuple(r.uid for r in self.waiting),
            running=tuple(r.uid for r in self.running),
            free_pages=self._free_pages(),
            total_pages=self.num_pages,
            reclaimable_pages=len(self.prefix.evictable(self.cache)) if self.prefix else 0,
        )

    def submit(self, request: Request) -> None:
        if not len(request.prompt):
            raise ValueError(f"{request.uid} has an empty prompt")
        needed = self._pages_needed(request)
        if needed > self.num_pages or needed > self.cache.max_pages_per_request:
            raise OversizedRequest(
                f"{request.uid} needs {needed} pages ({len(request.prompt)} prompt + {request.max_new_tokens} "
                f"new tokens at {self.page_size} tokens a page) but the pool holds {self.num_pages} and a "
                f"request may map {self.cache.max_pages_per_request}; no eviction or preemption can satisfy it")
        self.waiting.append(request)

    # -- pages -----------------------------------------------------------------------
    def _reserve_with_eviction(self, uid: str, end: int, start: int | None = None) -> bool:
        """Reserve pages for positions < ``end``, evicting index-only pages if needed."""
        while True:
            try:
                self.cache.reserve(uid, end, start)
                return True
            except OutOfPages:
                candidates = self.prefix.evictable(self.cache) if self.prefix else []
                if not candidates:
                    return False
                victim = self.policy.evict_victim(self._state(), tuple(candidates))
                if victim not in candidates:
                    raise ValueError(f"policy {self.policy.name} chose page {victim}, which is not evictable")
                self.prefix.evict(victim, self.cache)
                self.evictions += 1
                self.counters.hit("eviction_taken")
                self._event(uid, Event.EVICT)

    def _admit(self, request: Request, state: SchedulerState) -> bool:
        self.cache.open(request.uid)
        request.kv_len = 0
        request.cache_hit_tokens = 0
        if self.prefix is not None:
            hit_tokens, pages = self.prefix.lookup(request.prompt)
            if hit_tokens >= len(request.prompt) and pages:
                # keep at least one token to compute logits from
                hit_tokens -= self.page_size
                pages = pages[:-1]
                self.counters.hit("cache_full_prompt_trimmed")
            if hit_tokens and not self.policy.honor_cache_hit(state, request.uid, hit_tokens):
                self.counters.hit("cache_hit_refused")
            elif hit_tokens:
                self.counters.hit("cache_hit")
                self._event(request.uid, Event.CACHE_HIT)
                self.cache.adopt(request.uid, pages)
                self.cache.commit(request.uid, hit_tokens)
                request.kv_len = hit_tokens
                request.cache_hit_tokens = hit_tokens
            else:
                self.counters.hit("cache_miss")
        if self.reserve_mode == "full":
            if not self._reserve_with_eviction(request.uid, len(request.prompt) + request.max_new_tokens,
                                               request.kv_len):
                self.cache.close(request.uid)
                request.kv_len = 0
                return False
        return True

    def _preempt(self, request: Request) -> None:
        """Recompute preemption: drop the cache, keep the tokens."""
        self.cache.close(request.uid)
        request.kv_len = 0
        request.preempt_count += 1
        self.running.remove(request)
        self.waiting.insert(0, request)
        self._event(request.uid, Event.PREEMPT)

    # -- one step --------------------------------------------------------------------
    def step(self) -> bool:
        if not self.waiting and not self.running:
            return False

        state = self._state()
        for request in list(self.waiting):
            if not self.policy.admit(state, request.uid, self._pages_needed(request)):
                self.counters.hit("admit_refused")
                continue
            if self.cache.free_slots == 0:
                self.counters.hit("admit_refused")
                continue
            if not self._admit(request, state):
                self.counters.hit("admit_no_pages")
                continue
            self.counters.hit("admit")
            if request.preempt_count:
                self.counters.hit("resume")
                self._event(request.uid, Event.RESUME)
            else:
                self._event(request.uid, Event.ADMIT)
            self.waiting.remove(request)
            self.running.append(request)
            state = self._state()

        if not self.running:
            smallest = min(self._pages_needed(r) for r in self.waiting)
            self.counters.hit("out_of_pages")
            raise OutOfPages(
                f"{len(self.waiting)} requests waiting, the smallest needs {smallest} pages, "
                f"{self._free_pages()} free and {state.reclaimable_pages} reclaimable, nothing running to free more")

        for request in list(self.running):
            if request.kv_len == 0 or not request.generated:
                continue
            if self.policy.should_preempt(state, request.uid):
                self._preempt(request)
                self.counters.hit("preempt_fired")
                state = self._state()
        if not self.running:
            self.step_index += 1
            return True

        # -- build the batch under the token budget: decoded tokens first ----------
        budget = self.max_batched_tokens if self.max_batched_tokens is not None else float("inf")
        plan: dict[str, int] = {}
        order = sorted(self.running, key=lambda r: 0 if (r.generated and r.total_tokens() - r.kv_len == 1) else 1)
        for request in order:
            remaining = request.total_tokens() - request.kv_len
            if budget < 1:
                self.counters.hit("budget_deferred")
                continue
            take = self.policy.chunk_boundary(state, request.uid, remaining)
            if not 1 <= take <= remaining:
                raise ValueError(f"policy {self.policy.name} returned chunk {take} for {request.uid} "
                                 f"with {remaining} remaining; must be in [1, remaining]")
            take = int(min(take, budget))
            plan[request.uid] = take
            budget -= take

        if self.reserve_mode == "lazy":
            for request in list(self.running):
                if request.uid not in plan or request not in self.running:
                    continue
                end = request.kv_len + plan[request.uid]
                while not self._reserve_with_eviction(request.uid, end, request.kv_len):
                    victims = [r for r in self.running if r is not request]
                    if not victims:
                        self.counters.hit("out_of_pages")
                        raise OutOfPages(f"{request.uid} cannot grow to {end} tokens and nothing is left to preempt")
                    victim = victims[-1]
                    plan.pop(victim.uid, None)
                    self._preempt(victim)
                    self.counters.hit("preempt_for_pages")

        work, entries, samplers, ran = [], [], [], []
        for request in self.running:
            take = plan.get(request.uid)
            if not take:
                continue
            context = request.context()
            start, end = request.kv_len, request.kv_len + take
            completes = end == len(context)
            work.append((request.uid, context[start:end], start))
            ran.append(request)
            entries.append(StepEntry(request.uid, context[start:end], [take - 1] if completes else []))
            if take == 1 and start == len(context) - 1 and request.generated:
                self.counters.hit("decode_step")
                self._event(request.uid, Event.DECODE)
            else:
                self.counters.hit("prefill_chunk")
                self._event(request.uid, Event.DECODE if completes else Event.CHUNK)
            if completes:
                samplers.append(request)

        logits = self.model.step(self.cache, entries) if entries else None

        emitted = []
        for request, (_, tokens, start) in zip(ran, work):
            request.kv_len = start + len(tokens)
            if request.kv_len == len(request.prompt) and not request.generated:
                self.counters.hit("prefill_complete")
        if samplers:
            tokens = self.sampler.sample(logits, samplers)
            for row, (request, token) in enumerate(zip(samplers, tokens)):
                if self.keep_logits:
                    self.emitted_logits.setdefault(request.uid, []).append(logits[row].detach().cpu().clone())
                request.generated.append(int(token))
                emitted.append((request.uid, int(token)))

        if self.audit_enabled:
            logits_bytes = logits.detach().cpu().numpy().tobytes() if logits is not None else b""
            self.trajectory.observe_step(
                self.step_index, work, emitted, logits_bytes,
                (self.cache.state_digest(), self.prefix.state_digest() if self.prefix else ()))
            self.cache.audit()

        self._retire_finished()

        self.step_index += 1
        return True

    def _retire_finished(self) -> None:
        for request in list(self.running):
            if not request.generated:
                continue
            if len(request.generated) >= request.max_new_tokens or request.generated[-1] in self.eos:
                request.finished = True
                self.counters.hit("finish")
                self.counters.hit("finish_eos" if request.generated[-1] in self.eos else "finish_limit")
                self._event(request.uid, Event.FINISH)
                self.running.remove(request)
                self.done.append(request)
                if self.prefix is not None:
                    created = self.prefix.insert(request.context()[: request.kv_len],
                                                 self.cache.request_pages(request.uid), self.cache)
                    if created:
                        self.counters.hit("cache_insert", created)
                self.cache.close(request.uid)

    def _burst(self, max_steps: int) -> bool:
        """Several decode steps in one call of the model's device-side loop, when every decision of
        those steps is known in advance (see ``decode_burst``).  Returns whether it ran."""
        if self.decode_burst <= 1 or self.waiting or not self.running or self.eos or self.audit_enabled:
            return False
        if self.keep_logits or self.reserve_mode != "full" or type(self.policy) is not DefaultPolicy:
            return False
        if not hasattr(self.model, "decode_greedy"):
            return False
        if self.max_batched_tokens is not None and self.max_batched_tokens < len(self.running):
            return False
        for r in self.running:
            if r.temperature > 0 or not r.generated or r.total_tokens() - r.kv_len != 1:
                return False
        steps = min(self.decode_burst, max_steps - self.step_index,
                    min(r.max_new_tokens - len(r.generated) for r in self.running))
        if steps <= 1:
            return False
        uids = [r.uid for r in self.running]
        picked = self.model.decode_greedy(self.cache, uids, [r.generated[-1] for r in self.running], steps)
        for row in picked:
            for request, token in zip(self.running, row):
                request.generated.append(int(token))
                request.kv_len += 1
                self.counters.hit("decode_step")
                self._event(request.uid, Event.DECODE)
            self.step_index += 1
        self._retire_finished()
        return True

    def advance(self, max_steps: int = 1 << 20) -> bool:
        """One iteration of the serving loop (a run of decode steps on the device, or one step);
        False when nothing waits and nothing runs, or ``max_steps`` steps have been taken."""
        return bool(self._burst(max_steps) or self.step()) and self.step_index < max_steps

    def run(self, max_steps: int = 1 << 20) -> dict:
        while self.advance(max_steps):
            pass
        if self.audit_enabled:
            self.cache.audit()
        return {r.uid: list(r.generated) for r in self.done}
