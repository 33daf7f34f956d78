"""The decisions of the scheduler, as objects a caller can replace.

The scheduler never decides by itself whether to admit, how much of a prompt
to run, whom to preempt, which indexed page to give up or whether to use a
prefix hit: it asks its policy, so a test can script an exact interleaving
and serving keeps a short default.  The five questions are those of the
reference's policy seam (engine/sched/policy.py:51-73); how they are answered
here is this engine's own: a policy is put together from small *rules*, one
per question, and the named policies are presets of rules.

    Policy(portion=EveryTokens(2048), preemption=AtSteps({("r0", 2)}))

Every rule sees a ``View``: a read-only snapshot of the scheduler taken just
before the question is asked.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum
from typing import Iterable


class Event(str, Enum):
    """Marks in a request's life, in the vocabulary of the reference
    (engine/sched/policy.py:13-23)."""

    ADMIT = "admit"
    CHUNK = "chunk"
    DECODE = "decode"
    PREEMPT = "preempt_rc"
    RESUME = "resume"
    EVICT = "evict"
    CACHE_HIT = "cache_hit"
    FINISH = "finish"


@dataclass(frozen=True)
class View:
    """What a rule may look at."""

    step: int
    waiting: tuple           # uids in queue order
    running: tuple           # uids in admission order
    free_pages: int          # of the scarcest cache group
    total_pages: int
    reclaimable_pages: int = 0   # pages only the prefix index holds

    @property
    def obtainable_pages(self) -> int:
        return self.free_pages + self.reclaimable_pages


# ---------------------------------------------------------------------------
# rules: one small object per question
# ---------------------------------------------------------------------------

class WhileRoom:
    """Admit while fewer than ``max_running`` requests run and the pages the
    request asks for can be had (free, or held by the prefix index alone)."""

    def __init__(self, max_running: int):
        self.max_running = max_running

    def __call__(self, view: View, uid: str, pages: int) -> bool:
        return len(view.running) < self.max_running and pages <= view.obtainable_pages


class Everything:
    """Run all of a request's remaining tokens in one step."""

    def __call__(self, view: View, uid: str, remaining: int) -> int:
        return remaining


class EveryTokens:
    """Cut into portions of at most ``size`` tokens."""

    def __init__(self, size: int):
        if size < 1:
            raise ValueError(f"a portion has at least one token, got {size}")
        self.size = size

    def __call__(self, view: View, uid: str, remaining: int) -> int:
        return min(self.size, remaining)


class Listed:
    """Portion sizes read off a list, one per question in the order asked;
    once the list is used up, everything that remains."""

    def __init__(self, sizes: Iterable[int]):
        self.sizes = list(sizes)
        self.used = 0

    def __call__(self, view: View, uid: str, remaining: int) -> int:
        if self.used >= len(self.sizes):
            return remaining
        size = self.sizes[self.used]
        self.used += 1
        return max(1, min(int(size), remaining))


class Never:
    def __call__(self, *_args) -> bool:
        return False


class Always:
    def __call__(self, *_args) -> bool:
        return True


class AtSteps:
    """True once for each listed (uid, step)."""

    def __init__(self, moments: Iterable[tuple]):
        self.pending = {(uid, int(step)) for uid, step in moments}
        self.fired: list[tuple] = []

    def __call__(self, view: View, uid: str) -> bool:
        moment = (uid, view.step)
        if moment not in self.pending:
            return False
        self.pending.discard(moment)
        self.fired.append(moment)
        return True


class ExceptAtSteps:
    """True except at the listed steps (for prefix hits to be refused there)."""

    def __init__(self, steps: Iterable[int]):
        self.steps = {int(s) for s in steps}

    def __call__(self, view: View, uid: str, tokens: int) -> bool:
        return view.step not in self.steps


class LowestPage:
    def __call__(self, view: View, candidates: tuple) -> int:
        return min(candidates)


# ---------------------------------------------------------------------------
# the policy: five questions, each answered by a rule
# ---------------------------------------------------------------------------

class Policy:
    """Answers the scheduler's questions by its rules.  Subclasses may override a method
    instead of passing a rule."""

    def __init__(self, max_running: int = 64, *, admission=None, portion=None, preemption=None, eviction=None,
                 prefix_hits=None, name: str | None = None):
        self.max_running = max_running
        self._admission = admission or WhileRoom(max_running)
        self._portion = portion or Everything()
        self._preemption = preemption or Never()
        self._eviction = eviction or LowestPage()
        self._prefix_hits = prefix_hits or Always()
        self.name = name or type(self).__name__

    def same_answers_every_step(self) -> bool:
        """Whether a run of decode steps may be decided once for all of them: portions and
        preemption are answered by rules that neither count the questions nor look at the step,
        and no subclass answers them itself."""
        cls = type(self)
        return (isinstance(self._portion, (Everything, EveryTokens)) and isinstance(self._preemption, Never)
                and cls.chunk_boundary is Policy.chunk_boundary and cls.should_preempt is Policy.should_preempt)

    def admit(self, view: View, uid: str, pages_needed: int) -> bool:
        """May the waiting request start now?"""
        return bool(self._admission(view, uid, pages_needed))

    def chunk_boundary(self, view: View, uid: str, remaining: int) -> int:
        """How many of the request's ``remaining`` tokens run in this step (1..remaining)."""
        return int(self._portion(view, uid, remaining))

    def should_preempt(self, view: View, uid: str) -> bool:
        """Give up the request's cache now and recompute it later?"""
        return bool(self._preemption(view, uid))

    def evict_victim(self, view: View, candidates: tuple) -> int:
        """Which of the pages that only the prefix index holds goes back to the pool."""
        return int(self._eviction(view, candidates))

    def honor_cache_hit(self, view: View, uid: str, hit_tokens: int) -> bool:
        """Use the indexed pages that match the request's prompt?"""
        return bool(self._prefix_hits(view, uid, hit_tokens))


class DefaultPolicy(Policy):
    """Serving default: admit while there is room, whole remainders, no preemption on request,
    lowest indexed page evicted first, every prefix hit used.  The reference's default admits 32
    requests at most (engine/sched/policy.py:75-103); 64 here, the largest workload measured."""

    def __init__(self, max_running: int = 64):
        super().__init__(max_running, name="default")


class FixedChunkPolicy(Policy):
    """Prompts in portions of ``chunk`` tokens (the reference's chunked prefill,
    engine/sched/policy.py:125-134)."""

    def __init__(self, chunk: int, max_running: int = 64):
        super().__init__(max_running, portion=EveryTokens(chunk), name=f"fixed-chunk({chunk})")
        self.chunk = chunk


class PreemptAtStepsPolicy(Policy):
    """Preempt request ``uid`` at each of ``at_steps``, once (the reference's scripted
    preemption, engine/sched/policy.py:137-171)."""

    def __init__(self, uid: str, at_steps, chunk: int | None = None, max_running: int = 64):
        rule = AtSteps((uid, step) for step in at_steps)
        super().__init__(max_running, portion=EveryTokens(chunk) if chunk else Everything(), preemption=rule,
                         name=f"preempt({uid}@{sorted(at_steps)})")
        self.uid = uid
        self._rule = rule

    @property
    def fired_at(self) -> list[int]:
        return [step for _, step in self._rule.fired]


class NoCacheHitPolicy(Policy):
    """Every prefix hit is declined (engine/sched/policy.py:174-179 of the reference)."""

    def __init__(self, max_running: int = 64):
        super().__init__(max_running, prefix_hits=Never(), name="no-cache-hit")


class ScriptedPolicy(Policy):
    """A whole interleaving from data: portion sizes in the order they are asked for,
    preemptions at (uid, step) pairs, steps at which prefix hits are declined (the reference's
    trace-driven policy, harness/sim/driver.py:100-129)."""

    def __init__(self, chunk_plan=(), preempt_at=(), refuse_cache_at=(), max_running: int = 64):
        super().__init__(max_running, portion=Listed(chunk_plan), preemption=AtSteps(preempt_at),
                         prefix_hits=ExceptAtSteps(refuse_cache_at), name="scripted")
