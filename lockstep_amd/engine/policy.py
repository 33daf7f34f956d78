"""The seam of the scheduler: every decision is a call into a policy object
(reference engine/sched/policy.py:51-180), so a test can script an exact
interleaving and the production heuristic stays a few lines."""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum


class Event(str, Enum):
    """What can happen to a request (reference engine/sched/policy.py:13-23)."""

    ADMIT = "admit"
    CHUNK = "chunk"
    DECODE = "decode"
    PREEMPT = "preempt_rc"
    RESUME = "resume"
    EVICT = "evict"
    CACHE_HIT = "cache_hit"
    FINISH = "finish"


@dataclass(frozen=True)
class SchedulerState:
    """What a policy may look at when it decides."""

    step: int
    waiting: tuple
    running: tuple
    free_pages: int
    total_pages: int
    reclaimable_pages: int = 0


class Policy:
    name = "base"

    def admit(self, state: SchedulerState, uid: str, pages_needed: int) -> bool:
        raise NotImplementedError

    def chunk_boundary(self, state: SchedulerState, uid: str, remaining: int) -> int:
        """How many of the request's ``remaining`` tokens to run in this step."""
        raise NotImplementedError

    def should_preempt(self, state: SchedulerState, uid: str) -> bool:
        return False

    def evict_victim(self, state: SchedulerState, candidates: tuple) -> int:
        return min(candidates)

    def honor_cache_hit(self, state: SchedulerState, uid: str, hit_length: int) -> bool:
        return True


class DefaultPolicy(Policy):
    """Admit while there is room, run whole remainders, never preempt, evict
    the lowest page id, honour every prefix hit (reference
    engine/sched/policy.py:75-103; ``max_running`` defaults to 32 there, 64
    here to hold the largest workload this engine is measured with)."""

    name = "default"

    def __init__(self, max_running: int = 64):
        self.max_running = max_running

    def admit(self, state, uid, pages_needed):
        if len(state.running) >= self.max_running:
            return False
        return pages_needed <= state.free_pages + state.reclaimable_pages

    def chunk_boundary(self, state, uid, remaining):
        return remaining


class FixedChunkPolicy(DefaultPolicy):
    """Cut prompts into portions of ``chunk`` tokens (reference
    engine/sched/policy.py:125-134)."""

    def __init__(self, chunk: int, max_running: int = 64):
        super().__init__(max_running)
        if chunk < 1:
            raise ValueError("chunk must be at least 1")
        self.chunk = chunk
        self.name = f"fixed-chunk({chunk})"

    def chunk_boundary(self, state, uid, remaining):
        return min(self.chunk, remaining)


class PreemptAtStepsPolicy(DefaultPolicy):
    """Preempt one named request at named steps, once each (reference
    engine/sched/policy.py:137-171)."""

    def __init__(self, uid: str, at_steps, chunk: int | None = None, max_running: int = 64):
        super().__init__(max_running)
        self.uid = uid
        self.at_steps = set(at_steps)
        self.fired_at: list[int] = []
        self.chunk = chunk
        self.name = f"preempt({uid}@{sorted(self.at_steps)})"

    def chunk_boundary(self, state, uid, remaining):
        return remaining if self.chunk is None else min(self.chunk, remaining)

    def should_preempt(self, state, uid):
        if uid != self.uid or state.step not in self.at_steps or state.step in self.fired_at:
            return False
        self.fired_at.append(state.step)
        return True


class NoCacheHitPolicy(DefaultPolicy):
    """Refuse every prefix hit (reference engine/sched/policy.py:174-179)."""

    name = "no-cache-hit"

    def honor_cache_hit(self, state, uid, hit_length):
        return False


class ScriptedPolicy(DefaultPolicy):
    """Chunk sizes taken from a plan, one per call, then whole remainders;
    preemptions at given (uid, step) pairs (reference
    harness/sim/driver.py:100-129)."""

    def __init__(self, chunk_plan=(), preempt_at=(), refuse_cache_at=(), max_running: int = 64):
        super().__init__(max_running)
        self.chunk_plan = list(chunk_plan)
        self.preempt_at = {(u, s) for u, s in preempt_at}
        self.refuse_cache_at = set(refuse_cache_at)
        self.fired: set = set()
        self.name = "scripted"

    def chunk_boundary(self, state, uid, remaining):
        if self.chunk_plan:
            return max(1, min(self.chunk_plan.pop(0), remaining))
        return remaining

    def should_preempt(self, state, uid):
        key = (uid, state.step)
        if key in self.preempt_at and key not in self.fired:
            self.fired.add(key)
            return True
        return False

    def honor_cache_hit(self, state, uid, hit_length):
        return state.step not in self.refuse_cache_at
