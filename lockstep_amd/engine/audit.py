"""Counters of the paths a run took, and a running digest of what it did.

A test that claims "preemption leaves tokens unchanged" must be able to show
that a preemption happened; the counters are that evidence (reference
engine/audit/counters.py:8-99).  The trajectory hash absorbs every step's
work list, emitted tokens, sampled logit rows and the cache manager's state,
so two runs can be compared step by step (reference
engine/audit/trajectory.py:15-59).
"""

from __future__ import annotations

import hashlib
from collections import Counter

PATHS = {
    "admit": "a waiting request was admitted",
    "admit_refused": "the policy declined to admit a waiting request",
    "admit_no_pages": "a request was admitted by the policy but its pages could not be reserved",
    "resume": "a preempted request was admitted again",
    "prefill_chunk": "a portion of a prompt (or of a recomputed context) ran",
    "prefill_complete": "a prompt's last portion ran",
    "decode_step": "a single decoded token ran",
    "budget_deferred": "a request got no tokens this step because the token budget was spent",
    "preempt_fired": "a running request was preempted for recompute",
    "preempt_for_pages": "a running request was preempted because another could not grow",
    "cache_hit": "a prefix hit was found and honoured",
    "cache_hit_refused": "a prefix hit was found and the policy declined it",
    "cache_miss": "a lookup found no usable prefix",
    "cache_insert": "whole pages were indexed after a request finished",
    "cache_full_prompt_trimmed": "a whole-prompt hit gave its last page back",
    "eviction_taken": "an indexed page was reclaimed under pressure",
    "finish": "a request finished and gave its pages back",
    "finish_eos": "a request finished on an end-of-sequence token",
    "finish_limit": "a request finished at max_new_tokens",
    "out_of_pages": "nothing could run and nothing could be admitted",
}


class VacuousRun(AssertionError):
    """A run that was meant to exercise a path never took it."""


class Counters:
    def __init__(self):
        self.counts: Counter = Counter()

    def hit(self, path: str, amount: int = 1) -> None:
        if path not in PATHS:
            raise KeyError(f"{path!r} is not a declared path; add it to PATHS with what firing it means")
        self.counts[path] += amount

    def __getitem__(self, path: str) -> int:
        return self.counts.get(path, 0)

    def require_fired(self, *paths: str) -> None:
        missing = [p for p in paths if not self.counts.get(p)]
        if missing:
            raise VacuousRun(f"the run never took: {', '.join(missing)}")


class TrajectoryHash:
    def __init__(self):
        self._digest = hashlib.sha256()
        self.per_step: list[str] = []

    def _absorb(self, label: str, payload: bytes) -> None:
        self._digest.update(label.encode())
        self._digest.update(len(payload).to_bytes(8, "big"))
        self._digest.update(payload)

    def observe_step(self, step: int, work, emitted, logits_bytes: bytes, cache_state) -> None:
        self._absorb("step", str(step).encode())
        self._absorb("work", repr(work).encode())
        self._absorb("emitted", repr(emitted).encode())
        self._absorb("logits", logits_bytes)
        self._absorb("cache", repr(cache_state).encode())
        self.per_step.append(self._digest.hexdigest())

    def hexdigest(self) -> str:
        return self._digest.hexdigest()

    def first_divergence(self, other: "TrajectoryHash"):
        for i, (a, b) in enumerate(zip(self.per_step, other.per_step)):
            if a != b:
                return i
        if len(self.per_step) != len(other.per_step):
            return min(len(self.per_step), len(other.per_step))
        return None
