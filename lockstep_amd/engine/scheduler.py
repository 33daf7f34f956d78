"""Continuous batching above the step function.

A step has six phases, each a method: start waiting requests the policy and
the pages allow; preempt those the policy names; share the step's token
budget out (requests that decode first, then prompt portions in admission
order, each cut by the policy); under lazy reservation, grow the requests or
preempt for pages; run the batch and sample for every request whose whole
context is now cached; retire what finished.  What the loop does is the
reference scheduler's behaviour (engine/sched/scheduler.py:205-361); the token
budget, the choice of when pages are taken, the automatic preemption for
pages and the device-side decode bursts are additions.

When pages run out:

* ``submit`` refuses a request that an empty pool could not hold, or that
  would pass the model's last position (``OversizedRequest``; the reference
  refuses the former, engine/sched/scheduler.py:90-104).
* ``reserve="full"`` (default, the reference's behaviour): the pages for
  prompt + max_new_tokens are taken when a request starts, so one that does
  not fit waits and a running request never lacks a page.  Pages that only
  the prefix index holds are dropped first (lowest leaf by default).
* ``reserve="lazy"``: pages are taken step by step.  When a running request
  cannot grow, the request that started last among the others is preempted:
  its pages go back, it returns to the head of the queue, and its context is
  computed again later -- with the same tokens, because results do not depend
  on how the work is cut (reference engine/sched/scheduler.py:195-203).
* When nothing runs and nothing can start, the step raises ``OutOfPages``
  (reference engine/sched/scheduler.py:226-232).
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..cache import OutOfPages, PrefixIndex
from .audit import Counters, StepLedger
from .batch import StepEntry
from .policy import DefaultPolicy, Event, Policy, View


@dataclass
class Request:
    """What a caller submits: token ids in, sampling options (the reference's request fields,
    engine/sched/scheduler.py:19-29).  Token ids come back through ``Scheduler.run``."""

    uid: str
    prompt: list
    seed: int = 0
    max_new_tokens: int = 8
    temperature: float = 0.0
    top_p: float = 1.0


class Sequence:
    """The scheduler's record of one submitted request: its tokens (prompt, then what was
    generated, in one list) and how far the cache has got."""

    __slots__ = ("request", "tokens", "n_prompt", "cached", "preemptions", "reused", "finished")

    def __init__(self, request: Request):
        self.request = request
        self.tokens = [int(t) for t in request.prompt]
        self.n_prompt = len(self.tokens)
        self.cached = 0          # tokens whose keys and values the cache holds
        self.preemptions = 0
        self.reused = 0          # prompt tokens taken from the prefix index when it last started
        self.finished = False

    # what the sampler reads
    uid = property(lambda self: self.request.uid)
    seed = property(lambda self: self.request.seed)
    temperature = property(lambda self: self.request.temperature)
    top_p = property(lambda self: self.request.top_p)

    def total_tokens(self) -> int:
        return len(self.tokens)

    @property
    def generated(self) -> list:
        return self.tokens[self.n_prompt:]

    @property
    def n_generated(self) -> int:
        return len(self.tokens) - self.n_prompt

    @property
    def remaining(self) -> int:
        """Tokens that still have to go through the model before the next one can be sampled."""
        return len(self.tokens) - self.cached

    @property
    def decoding(self) -> bool:
        return self.n_generated > 0 and self.remaining == 1

    @property
    def budget_left(self) -> int:
        return self.request.max_new_tokens - self.n_generated


class OversizedRequest(ValueError):
    """No state of the engine could ever run this request."""


@dataclass
class _Portion:
    seq: Sequence
    start: int
    count: int
    samples: bool            # the portion ends the context: a token is sampled from its last row


@dataclass
class _Batch:
    portions: list = field(default_factory=list)

    def work(self) -> list:
        return [(p.seq.uid, p.seq.tokens[p.start:p.start + p.count], p.start) for p in self.portions]


class Scheduler:
    def __init__(self, model, num_blocks: int, policy: Policy | None = None, eos_token_ids=None,
                 audit: bool = True, block_size: int = 16, enable_prefix_cache: bool = False, *,
                 max_batched_tokens: int | None = None, reserve: str = "full", max_requests: int | None = None,
                 max_tokens_per_request: int | None = None, sampler=None, cache=None, keep_logits: bool = False,
                 decode_burst: int = 1):
        """``num_blocks`` pages of ``block_size`` tokens, ``eos_token_ids``, ``audit`` and
        ``enable_prefix_cache`` carry the reference's names (engine/sched/scheduler.py:51-60).
        ``max_batched_tokens`` bounds the tokens of one step (None: no bound).  ``decode_burst`` > 1:
        while nothing waits, every running request decodes and no answer of the policy can change
        from step to step, up to that many decode steps run as one call of the model's device-side
        loop (``decode_greedy``, or ``decode_sampled`` where requests draw their tokens); tokens,
        counters and marks are those of single steps."""
        if reserve not in ("full", "lazy"):
            raise ValueError("reserve must be 'full' or 'lazy'")
        self.model = model
        self.policy = policy or DefaultPolicy()
        self.eos = frozenset(int(t) for t in (eos_token_ids or ()))
        self.audit_enabled = bool(audit)
        self.lazy = reserve == "lazy"
        self.max_batched_tokens = max_batched_tokens
        self.keep_logits = keep_logits
        self.decode_burst = max(1, int(decode_burst))
        if cache is None:
            slots = max_requests or max(getattr(self.policy, "max_running", 64), 1)
            cache = model.make_cache(num_pages=num_blocks, page_size=block_size, max_requests=slots,
                                     max_tokens_per_request=max_tokens_per_request)
        self.cache = cache
        self.page_size = cache.page_size
        self.num_pages = min((g.pool.num_pages for g in cache.groups), default=num_blocks)
        self.max_positions = getattr(getattr(model, "spec", None), "max_positions", None)
        self.prefix = PrefixIndex(self.page_size) if enable_prefix_cache and cache.shareable() else None
        if sampler is None:
            from ..sampling import Sampler

            sampler = Sampler(getattr(getattr(model, "rt", None), "kernels", None))
        self.sampler = sampler
        self.waiting: list[Sequence] = []
        self.running: list[Sequence] = []
        self.done: list[Sequence] = []
        self.step_index = 0
        self.evictions = 0
        self.counters = Counters()
        self.lifecycle: dict[str, list] = {}
        self.trajectory = StepLedger()
        self.emitted_logits: dict[str, list] = {}

    @classmethod
    def from_config(cls, model, config, policy: Policy | None = None, **overrides) -> "Scheduler":
        """A scheduler as an ``EngineConfig`` describes it."""
        options = dict(num_blocks=config.num_pages, block_size=config.page_size, policy=policy or config.policy(),
                       eos_token_ids=config.eos_token_ids, audit=config.audit,
                       enable_prefix_cache=config.enable_prefix_cache, max_batched_tokens=config.max_batched_tokens,
                       reserve=config.reserve, max_requests=config.max_running,
                       max_tokens_per_request=config.max_tokens_per_request, decode_burst=config.decode_burst)
        options.update(overrides)
        return cls(model, **options)

    # -- small helpers -----------------------------------------------------------------
    def _mark(self, uid: str, event: Event) -> None:
        self.lifecycle.setdefault(uid, []).append(event)

    def _pages_for(self, total_tokens: int) -> int:
        """Pages the neediest cache group takes for a request of that many tokens."""
        if not self.cache.groups:
            return 0
        return max(self.cache.pages_to_reserve(None, 0, total_tokens))

    def _need(self, seq: Sequence) -> int:
        return self._pages_for(seq.n_prompt + seq.request.max_new_tokens)

    def _free(self) -> int:
        return min(self.cache.free_pages) if self.cache.groups else self.num_pages

    def _view(self) -> View:
        return View(step=self.step_index, waiting=tuple(s.uid for s in self.waiting),
                    running=tuple(s.uid for s in self.running), free_pages=self._free(),
                    total_pages=self.num_pages,
                    reclaimable_pages=self.prefix.reclaimable(self.cache) if self.prefix else 0)

    # -- in ---------------------------------------------------------------------------------
    def submit(self, request: Request) -> None:
        if not len(request.prompt):
            raise ValueError(f"request {request.uid!r} has no prompt tokens")
        total = len(request.prompt) + request.max_new_tokens
        if self.max_positions is not None and total > self.max_positions:
            self.counters.hit("position_limit")
            raise OversizedRequest(
                f"request {request.uid!r} would reach {total} tokens ({len(request.prompt)} of prompt and "
                f"{request.max_new_tokens} new); the model's positions end at {self.max_positions}")
        need = self._pages_for(total)
        if need > self.num_pages or need > self.cache.max_pages_per_request:
            raise OversizedRequest(
                f"request {request.uid!r} would hold {need} pages of {self.page_size} tokens for its {total} tokens; "
                f"the pool has {self.num_pages} and a block table {self.cache.max_pages_per_request} columns, so it "
                "could not run even alone")
        self.waiting.append(Sequence(request))

    # -- pages --------------------------------------------------------------------------
    def _reserve(self, seq: Sequence, end: int, start: int) -> bool:
        """Take the pages for positions below ``end``; while the pool is short, give up leaves of
        the prefix index that nobody maps, one at a time, the policy choosing which."""
        while True:
            try:
                self.cache.reserve(seq.uid, end, start)
                return True
            except OutOfPages:
                leaves = self.prefix.droppable(self.cache) if self.prefix else []
                if not leaves:
                    return False
                choice = self.policy.evict_victim(self._view(), tuple(leaves))
                if choice not in leaves:
                    raise ValueError(f"policy {self.policy.name} wants page {choice} dropped; the index can only "
                                     f"give up one of {leaves}")
                self.prefix.drop(choice, self.cache)
                self.evictions += 1
                self.counters.hit("eviction_taken")
                self._mark(seq.uid, Event.EVICT)

    def _start(self, seq: Sequence, view: View) -> bool:
        """Give the request a slot, map what the prefix index has of its prompt, and (unless pages
        are taken lazily) reserve all it will need.  False: the pages could not be had."""
        self.cache.open(seq.uid)
        seq.cached = seq.reused = 0
        if self.prefix is not None:
            pages = self.prefix.match(seq.tokens[: seq.n_prompt])
            if pages and len(pages) * self.page_size >= seq.n_prompt:
                pages = pages[:-1]            # the last prompt token must run: its row gives the first logits
                self.counters.hit("cache_full_prompt_trimmed")
            reuse = len(pages) * self.page_size
            if not reuse:
                self.counters.hit("cache_miss")
            elif not self.policy.honor_cache_hit(view, seq.uid, reuse):
                self.counters.hit("cache_hit_refused")
            else:
                self.cache.adopt(seq.uid, pages)
                self.cache.commit(seq.uid, reuse)
                seq.cached = seq.reused = reuse
                self.counters.hit("cache_hit")
                self._mark(seq.uid, Event.CACHE_HIT)
        if not self.lazy and not self._reserve(seq, seq.n_prompt + seq.request.max_new_tokens, seq.cached):
            self.cache.close(seq.uid)
            seq.cached = seq.reused = 0
            return False
        return True

    def _preempt(self, seq: Sequence) -> None:
        """Drop the request's cache and put it at the head of the queue; its tokens stay."""
        self.cache.close(seq.uid)
        seq.cached = 0
        seq.preemptions += 1
        self.running.remove(seq)
        self.waiting.insert(0, seq)
        self._mark(seq.uid, Event.PREEMPT)

    # -- the phases of a step -------------------------------------------------------------
    def _start_waiting(self) -> None:
        view = self._view()
        for seq in list(self.waiting):           # a request that has to wait does not hold up those behind it
            if self.cache.free_slots == 0 or not self.policy.admit(view, seq.uid, self._need(seq)):
                self.counters.hit("admit_refused")
                continue
            if not self._start(seq, view):
                self.counters.hit("admit_no_pages")
                continue
            self.waiting.remove(seq)
            self.running.append(seq)
            self.counters.hit("admit")
            if seq.preemptions:
                self.counters.hit("resume")
                self._mark(seq.uid, Event.RESUME)
            else:
                self._mark(seq.uid, Event.ADMIT)
            view = self._view()

    def _preempt_on_request(self) -> None:
        view = self._view()
        for seq in list(self.running):
            # only a request that has cached something and produced a token has anything to lose
            if seq.cached and seq.n_generated and self.policy.should_preempt(view, seq.uid):
                self._preempt(seq)
                self.counters.hit("preempt_fired")
                view = self._view()

    def _share_out_tokens(self) -> dict:
        """How many tokens each running request gets this step: decoding requests first, then the
        others in admission order, while the budget lasts."""
        view = self._view()
        left = float("inf") if self.max_batched_tokens is None else self.max_batched_tokens
        shares: dict[str, int] = {}
        for seq in [s for s in self.running if s.decoding] + [s for s in self.running if not s.decoding]:
            if left < 1:
                self.counters.hit("budget_deferred")
                continue
            asked = self.policy.chunk_boundary(view, seq.uid, seq.remaining)
            if not 1 <= asked <= seq.remaining:
                raise ValueError(f"policy {self.policy.name} gave request {seq.uid!r} a portion of {asked} tokens; "
                                 f"{seq.remaining} remain, so it has to lie between 1 and {seq.remaining}")
            shares[seq.uid] = int(min(asked, left))
            left -= shares[seq.uid]
        return shares

    def _grow_or_preempt(self, shares: dict) -> None:
        """Lazy reservation: take each request's pages for this step; a request that cannot grow
        has the most recently started other request preempted, until it can."""
        for seq in list(self.running):
            if seq.uid not in shares or seq not in self.running:
                continue
            end = seq.cached + shares[seq.uid]
            while not self._reserve(seq, end, seq.cached):
                others = [s for s in self.running if s is not seq]
                if not others:
                    self.counters.hit("out_of_pages")
                    raise OutOfPages(f"request {seq.uid!r} needs pages up to token {end} and runs alone: "
                                     "there is no one left to preempt for it")
                shares.pop(others[-1].uid, None)
                self._preempt(others[-1])
                self.counters.hit("preempt_for_pages")

    def _build_batch(self, shares: dict) -> _Batch:
        batch = _Batch()
        for seq in self.running:
            count = shares.get(seq.uid)
            if not count:
                continue
            portion = _Portion(seq, seq.cached, count, samples=seq.cached + count == len(seq.tokens))
            batch.portions.append(portion)
            if seq.decoding:
                self.counters.hit("decode_step")
                self._mark(seq.uid, Event.DECODE)
            else:
                self.counters.hit("prefill_chunk")
                self._mark(seq.uid, Event.DECODE if portion.samples else Event.CHUNK)
        return batch

    def _run_and_sample(self, batch: _Batch) -> None:
        entries = [StepEntry(p.seq.uid, p.seq.tokens[p.start:p.start + p.count], [p.count - 1] if p.samples else [])
                   for p in batch.portions]
        work = batch.work() if self.audit_enabled else None
        logits = self.model.step(self.cache, entries) if entries else None
        for p in batch.portions:
            before = p.seq.cached
            p.seq.cached = p.start + p.count
            if before < p.seq.n_prompt <= p.seq.cached and not p.seq.n_generated:
                self.counters.hit("prefill_complete")
        sampled = [p.seq for p in batch.portions if p.samples]
        emitted = []
        if sampled:
            picks = self.sampler.sample(logits, sampled)
            for row, (seq, token) in enumerate(zip(sampled, picks)):
                if self.keep_logits:
                    self.emitted_logits.setdefault(seq.uid, []).append(logits[row].detach().cpu().clone())
                seq.tokens.append(int(token))
                emitted.append((seq.uid, int(token)))
        if self.audit_enabled:
            raw = logits.detach().cpu().numpy().tobytes() if logits is not None else b""
            self.trajectory.observe_step(self.step_index, work, emitted, raw,
                                         (self.cache.state_digest(content=bool(self.cache.state_units)),
                                          self.prefix.digest() if self.prefix else ()))
            self.cache.audit()

    def _retire(self) -> None:
        for seq in list(self.running):
            if not seq.n_generated:
                continue
            stopped = seq.tokens[-1] in self.eos
            if not stopped and seq.budget_left > 0:
                continue
            seq.finished = True
            self.counters.hit("finish")
            self.counters.hit("finish_eos" if stopped else "finish_limit")
            self._mark(seq.uid, Event.FINISH)
            self.running.remove(seq)
            self.done.append(seq)
            if self.prefix is not None:
                fresh = self.prefix.remember(seq.tokens[: seq.cached], self.cache.request_pages(seq.uid), self.cache)
                if fresh:
                    self.counters.hit("cache_insert", fresh)
            self.cache.close(seq.uid)

    # -- one step ---------------------------------------------------------------------------
    def step(self) -> bool:
        """Run one step; False when there is nothing to do."""
        if not self.waiting and not self.running:
            return False
        self._start_waiting()
        if not self.running:
            self.counters.hit("out_of_pages")
            least = min(self._need(s) for s in self.waiting)
            reclaimable = self.prefix.reclaimable(self.cache) if self.prefix else 0
            raise OutOfPages(
                f"nothing running and none of the {len(self.waiting)} waiting requests can start: the smallest "
                f"asks for {least} pages; {self._free()} are free and {reclaimable} more are held by the prefix "
                "index alone")
        self._preempt_on_request()
        if self.running:                      # preemption may have emptied the step: it still counts
            shares = self._share_out_tokens()
            if self.lazy:
                self._grow_or_preempt(shares)
            self._run_and_sample(self._build_batch(shares))
            self._retire()
        self.step_index += 1
        return True

    # -- several decode steps without the host ---------------------------------------------------
    def _burst(self, max_steps: int) -> bool:
        """Run decode steps through the model's device-side loop while every decision of those
        steps is known beforehand (see ``decode_burst``).  Returns whether any ran."""
        if self.decode_burst <= 1 or self.waiting or not self.running or self.audit_enabled:
            return False
        if self.keep_logits or self.lazy or not hasattr(self.model, "decode_greedy"):
            return False
        if not getattr(self.policy, "same_answers_every_step", lambda: False)():
            return False
        if self.max_batched_tokens is not None and self.max_batched_tokens < len(self.running):
            return False
        if any(not s.decoding for s in self.running):
            return False
        steps = min(self.decode_burst, max_steps - self.step_index, min(s.budget_left for s in self.running))
        if steps <= 1:
            return False
        uids, last = [s.uid for s in self.running], [s.tokens[-1] for s in self.running]
        if any(s.temperature > 0 for s in self.running):
            if not hasattr(self.model, "decode_sampled"):
                return False
            from ..sampling import philox

            picked = self.model.decode_sampled(self.cache, uids, last, steps, [
                None if s.temperature <= 0 else (s.temperature, s.top_p, int(s.request.seed) ^ philox.uid_key(s.uid))
                for s in self.running])
            if picked is None:
                return False
        else:
            picked = self.model.decode_greedy(self.cache, uids, last, steps)
        # A request that draws an end-of-sequence id stops there: the steps the loop ran for it beyond that
        # are dropped (its pages go back when it retires below; the others' tokens do not depend on it).
        stopped = set()
        for row in picked:
            for seq, token in zip(self.running, row):
                if seq.uid in stopped:
                    continue
                seq.tokens.append(int(token))
                seq.cached += 1
                self.counters.hit("decode_step")
                self._mark(seq.uid, Event.DECODE)
                if int(token) in self.eos:
                    stopped.add(seq.uid)
            self.step_index += 1
            if len(stopped) == len(self.running):
                break                              # single steps would have stopped here as well
        self._retire()
        return True

    def advance(self, max_steps: int = 1 << 20) -> bool:
        """One iteration of the serving loop (a burst of decode steps, or one step); False when
        nothing waits and nothing runs, or ``max_steps`` steps have been taken."""
        return bool(self._burst(max_steps) or self.step()) and self.step_index < max_steps

    def run(self, max_steps: int = 1 << 20) -> dict:
        """Serve until everything submitted has finished: ``{uid: generated token ids}``."""
        while self.advance(max_steps):
            pass
        if self.audit_enabled:
            self.cache.audit()
        return {seq.uid: seq.generated for seq in self.done}
