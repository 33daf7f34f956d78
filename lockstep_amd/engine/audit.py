"""Evidence of what a run did: counters of the paths it took, and a ledger of
its steps that two runs can be compared by.

A test that claims "preemption leaves the tokens unchanged" has to show that
a preemption happened; ``Counters.require_fired`` is that check (the idea of
the reference's engine/audit/counters.py:86-99).  The ledger answers the other
question, "where did two runs part and in what": every step leaves one record
of four digests (the batch that ran, the tokens it emitted, the logit rows
they were sampled from, the state of cache manager and prefix index), and the
records are chained, so equal chains mean equal runs (the reference keeps one
rolling hash, engine/audit/trajectory.py:15-59; here the parts stay apart so
that a difference names what differs).
"""

from __future__ import annotations

import hashlib
from collections import Counter
from dataclasses import dataclass

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
    "position_limit": "a request was refused because it would pass the model's last position",
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


def _digest(*chunks: bytes) -> bytes:
    h = hashlib.sha256()
    for chunk in chunks:
        h.update(len(chunk).to_bytes(8, "little"))
        h.update(chunk)
    return h.digest()


@dataclass(frozen=True)
class StepRecord:
    """One step of a run, as digests of its four aspects, and the chain value after it."""

    step: int
    batch: bytes
    tokens: bytes
    logits: bytes
    state: bytes
    chain: bytes

    ASPECTS = ("batch", "tokens", "logits", "state")


class StepLedger:
    """The chained records of a run's steps."""

    def __init__(self):
        self.records: list[StepRecord] = []

    def observe_step(self, step: int, batch, emitted, logits_bytes: bytes, state) -> StepRecord:
        """``batch``: what ran (uid, tokens, start) per request; ``emitted``: (uid, token) pairs;
        ``logits_bytes``: the raw float32 rows the tokens were picked from; ``state``: any value
        with a stable ``repr`` that describes the cache manager and the prefix index."""
        previous = self.records[-1].chain if self.records else b"\0" * 32
        parts = (_digest(repr(batch).encode()), _digest(repr(emitted).encode()), _digest(logits_bytes),
                 _digest(repr(state).encode()))
        record = StepRecord(step, *parts, chain=_digest(previous, str(step).encode(), *parts))
        self.records.append(record)
        return record

    @property
    def per_step(self) -> list[str]:
        return [r.chain.hex() for r in self.records]

    def hexdigest(self) -> str:
        return self.records[-1].chain.hex() if self.records else _digest().hex()

    def first_divergence(self, other: "StepLedger"):
        """Index of the first step at which the two runs differ, or None."""
        found = self.first_difference(other)
        return None if found is None else found[0]

    def first_difference(self, other: "StepLedger"):
        """(index, aspects) of the first step that differs: the names of the digests that are not
        equal there ("length" when one run simply has more steps), or None for equal runs."""
        for i, (mine, theirs) in enumerate(zip(self.records, other.records)):
            if mine.chain != theirs.chain:
                aspects = tuple(a for a in StepRecord.ASPECTS if getattr(mine, a) != getattr(theirs, a))
                return i, aspects or ("step",)
        if len(self.records) != len(other.records):
            return min(len(self.records), len(other.records)), ("length",)
        return None
