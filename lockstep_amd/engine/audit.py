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

#: every path a run can be asked to prove it took: name -> what one count of it stands for.
#: The names follow the reference's counters (engine/audit/counters.py:8-37) where it has the
#: path, so that its relations can be stated against either engine.
PATHS = {
    # admission
    "admit": "one request left the queue and got a slot and its pages",
    "admit_refused": "the policy said no to a queued request (asked once per request and step)",
    "admit_no_pages": "the policy said yes, but the pool could not cover the request even after evictions",
    "resume": "the request admitted had been preempted before",
    "position_limit": "submit turned a request down: prompt plus new tokens pass the model's last position",
    "request_refused": "submit turned a request down for its fields (a uid in use, a value out of range)",
    # what a step ran
    "prefill_chunk": "a request ran more than its one newest token in a step (part of a prompt, or of a "
                     "context that is computed again)",
    "prefill_complete": "the step that cached the last prompt token of a request that has emitted nothing yet",
    "decode_step": "a request ran exactly its newest token",
    "budget_deferred": "the step's token budget was used up before this request's turn",
    "decode_burst": "a run of decode steps went through the device-side loop in one call",
    "burst_on_shared_prefix": "... while a request in it read pages adopted from the prefix index",
    "chunk_boundary_mid_block": "a portion stopped short of its context's end at a position inside a page",
    "chunk_boundary_on_block": "a portion stopped short of its context's end exactly where a page ends",
    "chunk_boundary_mid_split": "a portion stopped short of its context's end inside an attention split",
    "attention_multi_split": "a request's keys reached into a second attention split in this step",
    "attention_single_split": "all keys of a request lay in the first attention split in this step",
    # giving the cache up
    "preempt_fired": "the policy asked for a running request's cache to be dropped",
    "preempt_for_pages": "a request lost its cache so that another could take its next pages (lazy reservation)",
    "preempt_depth_2": "the request preempted had been preempted once before",
    "preempt_depth_3_plus": "the request preempted had been preempted at least twice before",
    # prefix index
    "cache_hit": "indexed pages matched a prompt's beginning and were mapped into the request",
    "cache_hit_refused": "indexed pages matched, and the policy chose to compute them anyway",
    "cache_miss": "no indexed page matched the prompt's beginning",
    "cache_insert": "counts the pages a finished request added to the index",
    "cache_full_prompt_trimmed": "the index held the whole prompt; its last page was left out so that the last "
                                 "prompt token runs",
    "eviction_taken": "a page that only the index held went back to the pool to make room",
    # endings
    "finish": "a request retired and its pages went back",
    "finish_eos": "... because its newest token is an end-of-sequence id",
    "finish_limit": "... because it has emitted max_new_tokens",
    "out_of_pages": "a step found nothing running and nothing it could start",
}


class VacuousRun(AssertionError):
    """A run that was meant to exercise a path never took it."""


class Counters:
    """How often a run took each declared path."""

    def __init__(self):
        self.counts: Counter = Counter()

    def hit(self, path: str, amount: int = 1) -> None:
        if path in PATHS:
            self.counts[path] += amount
            return
        raise KeyError(f"{path!r} is not a declared path; add it to PATHS with what one count of it stands for")

    def __getitem__(self, path: str) -> int:
        return self.counts[path]          # (a Counter answers 0 for what it never saw, without keeping it)

    def never_taken(self, *paths: str) -> list:
        """Those of ``paths`` (all declared ones if none are given) that the run did not take."""
        return [p for p in (paths or PATHS) if self.counts[p] == 0]

    def require_fired(self, *paths: str) -> None:
        missing = self.never_taken(*paths) if paths else []
        if missing:
            raise VacuousRun(f"the run never took: {', '.join(missing)}")

    def report(self) -> str:
        """One line per path taken: count, name, what it stands for."""
        return "\n".join(f"{n:8d}  {path}: {PATHS[path]}" for path, n in sorted(self.counts.items()) if n)


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
