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

import math

from ..cache import OutOfPages, PrefixIndex
from . import lifecycle
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


class InvalidRequest(ValueError):
    """A field of the request is out of range, or its uid is already in use."""


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
        #: why the prefix cache that was asked for is off (None: it is on, or was not asked for)
        self.prefix_cache_refused = None
        if enable_prefix_cache and self.prefix is None:
            import warnings

            self.prefix_cache_refused = cache.why_not_shareable()
            warnings.warn(f"enable_prefix_cache was asked for, but this model's cache cannot share pages between "
                          f"requests ({self.prefix_cache_refused}); requests are served without prefix reuse",
                          RuntimeWarning, stacklevel=2)
        #: keys of an attention split (None if the model does not say): the split counters are about these
        self.split_keys = getattr(model, "split_keys", None)
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
        self._known: set = set()                 # every uid this scheduler has accepted
        self._states: dict = {}                  # uid -> lifecycle.State (kept while auditing)
        self._steps_table = lifecycle.steps(self.lazy)

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
        if self.audit_enabled:
            state = self._states.get(uid, lifecycle.FIRST)
            target = self._steps_table.get((state, event))
            if target is None:
                raise lifecycle.IllegalMark(f"step {self.step_index}: request {uid!r} is {state.value} and was "
                                            f"marked {event.value}")
            self._states[uid] = target

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
    def _refuse(self, message: str):
        self.counters.hit("request_refused")
        raise InvalidRequest(message)

    def submit(self, request: Request) -> None:
        """Queue a request.  Everything that can be wrong with it is found here, before anything of
        the scheduler has changed: a uid that this scheduler has seen before (waiting, running or
        finished: records are kept by uid), an empty prompt, ``max_new_tokens`` below one, a negative
        or non-finite ``temperature``, a ``top_p`` outside [0, 1], a size that no state of the engine
        could hold."""
        uid = request.uid
        if uid in self._known:
            where = ("waiting" if any(s.uid == uid for s in self.waiting) else
                     "running" if any(s.uid == uid for s in self.running) else "finished")
            self._refuse(f"a request with uid {uid!r} was submitted before (it is {where}); uids name the "
                         "records of a run and the draws of its sampler, so each is used once")
        if not len(request.prompt):
            self._refuse(f"request {uid!r} has no prompt tokens")
        new = request.max_new_tokens
        if isinstance(new, bool) or not isinstance(new, int) or new < 1:
            self._refuse(f"request {uid!r}: max_new_tokens must be an integer of at least 1, got {new!r}")
        for name, low, high in (("temperature", 0.0, math.inf), ("top_p", 0.0, 1.0)):
            value = getattr(request, name)
            if isinstance(value, bool) or not isinstance(value, (int, float)) or not low <= value <= high \
                    or value == math.inf:
                self._refuse(f"request {uid!r}: {name} must be a number in [{low}, {high}"
                             f"{')' if high == math.inf else ']'}, got {value!r}")
        if not isinstance(request.seed, int) or isinstance(request.seed, bool) or not 0 <= request.seed < 1 << 64:
            self._refuse(f"request {uid!r}: seed must be an integer in [0, 2^64), got {request.seed!r}")
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
        self._known.add(uid)
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
        if seq.preemptions == 2:
            self.counters.hit("preempt_depth_2")
        elif seq.preemptions > 2:
            self.counters.hit("preempt_depth_3_plus")

    # -- the phases of a step -------------------------------------------------------------
    def _start_waiting(self) -> None:
        view = self._view()
        for seq in list(self.waiting):           # a request that has to wait does not hold up those behind it
            if self.cache.free_slots == 0 or not self.policy.admit(view, seq.uid, self._need(seq)):
                self.counters.hit("admit_refused")
                continue
            # (the mark comes first: what starting does to the request -- a prefix hit, evictions -- follows it)
            marks_before = len(self.lifecycle.get(seq.uid, ()))
            state_before = self._states.get(seq.uid)
            self._mark(seq.uid, Event.RESUME if seq.preemptions else Event.ADMIT)
            if not self._start(seq, view):
                del self.lifecycle[seq.uid][marks_before:]          # it did not start after all
                if state_before is None:
                    self._states.pop(seq.uid, None)
                else:
                    self._states[seq.uid] = state_before
                self.counters.hit("admit_no_pages")
                continue
            self.waiting.remove(seq)
            self.running.append(seq)
            self.counters.hit("admit")
            if seq.preemptions:
                self.counters.hit("resume")
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
            self._count_edges(seq.cached + count, portion.samples)
        return batch

    def _count_edges(self, end: int, whole_context: bool) -> None:
        """Where the tokens a request ran in this step end, relative to pages and attention splits
        (the reference counts the same, engine/sched/scheduler.py:270-279)."""
        hit = self.counters.hit
        if not whole_context:
            hit("chunk_boundary_mid_block" if end % self.page_size else "chunk_boundary_on_block")
            if self.split_keys and end % self.split_keys:
                hit("chunk_boundary_mid_split")
        if self.split_keys:
            hit("attention_multi_split" if end > self.split_keys else "attention_single_split")

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
        self.counters.hit("decode_burst")
        if any(s.reused for s in self.running):
            self.counters.hit("burst_on_shared_prefix")
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
                self._count_edges(seq.cached, True)
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
