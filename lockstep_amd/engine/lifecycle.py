"""A request's life as a table: which mark may follow in which state.

The scheduler leaves a mark (``policy.Event``) in a request's record whenever
something happens to it.  ``STEPS`` says, for every state, which marks are
legal there and where they lead; everything else about a life follows from
that table by search: the states that can be reached, and every run of ``n``
marks that some life can contain (the yardstick a set of tests is measured
against: which of the possible runs of marks did they produce?).  The idea,
the six states and the thirteen transitions under full reservation are those
of the reference (engine/sched/lifecycle.py:11-106); lazy reservation, which
the reference does not have, adds three more, listed apart.

With ``audit`` on, the scheduler walks every request through the table as it
marks, so a mark that the table does not allow stops the run where it happens.
"""

from __future__ import annotations

from enum import Enum

from .policy import Event


class State(str, Enum):
    WAITING = "waiting"          # submitted, or preempted and waiting for its turn again
    ADMITTED = "admitted"        # has a slot (and pages), nothing of it has run since
    PREFILLING = "prefilling"    # part of its context is cached
    DECODING = "decoding"        # its whole context is cached and it emits tokens
    PREEMPTED = "preempted"      # lost its cache, keeps its tokens
    DONE = "done"


def _table(text: str) -> dict:
    """``state: mark > state, mark > state`` a line."""
    out = {}
    for line in text.strip().splitlines():
        source, _, moves = line.partition(":")
        for move in moves.split(","):
            mark, _, target = move.partition(">")
            out[(State(source.strip()), Event(mark.strip()))] = State(target.strip())
    return out


#: transitions of a scheduler that takes a request's pages when it starts
STEPS = _table("""
    waiting:    admit > admitted
    admitted:   evict > admitted, cache_hit > prefilling, chunk > prefilling, decode > decoding
    prefilling: chunk > prefilling, decode > decoding, preempt_rc > preempted, evict > prefilling
    decoding:   decode > decoding, preempt_rc > preempted, finish > done
    preempted:  resume > admitted
""")

#: what taking pages step by step adds: a request that decodes may still have an indexed page
#: dropped for it, and the request that started last is the first to be preempted for pages,
#: also when nothing of it has run yet
STEPS_LAZY = _table("""
    decoding:   evict > decoding
    admitted:   preempt_rc > preempted
""")

#: pairs that can never occur although both halves exist, and why
NEVER = {
    (State.WAITING, Event.PREEMPT): "a request that holds no cache has nothing to give up",
    (State.ADMITTED, Event.FINISH): "a request retires only after a step sampled a token for it, which marks "
                                    "decode first",
    (State.PREFILLING, Event.FINISH): "as above: the step that completes the context marks decode",
}

FIRST = State.WAITING
LAST = frozenset({State.DONE})


def steps(lazy: bool = False) -> dict:
    return {**STEPS, **STEPS_LAZY} if lazy else dict(STEPS)


class IllegalMark(AssertionError):
    """The scheduler marked a request with something its state does not allow."""


def follow(marks, lazy: bool = False, start: State = FIRST) -> State:
    """The state a request is in after ``marks``; raises ``IllegalMark`` at the first one the table forbids."""
    table, state = steps(lazy), start
    for i, mark in enumerate(marks):
        target = table.get((state, Event(mark)))
        if target is None:
            raise IllegalMark(f"mark {i} ({Event(mark).value}) is not allowed in state {state.value}"
                              + (f": {NEVER[(state, Event(mark))]}" if (state, Event(mark)) in NEVER else ""))
        state = target
    return state


def reachable(lazy: bool = False) -> set:
    table, seen, todo = steps(lazy), {FIRST}, [FIRST]
    while todo:
        here = todo.pop()
        for (source, _), target in table.items():
            if source is here and target not in seen:
                seen.add(target)
                todo.append(target)
    return seen


def feasible_runs(n: int, lazy: bool = False) -> set:
    """Every run of ``n`` consecutive marks that some life contains."""
    if n < 1:
        raise ValueError("a run has at least one mark")
    table = steps(lazy)
    found, todo = set(), [(state, ()) for state in reachable(lazy)]
    while todo:
        state, so_far = todo.pop()
        if len(so_far) == n:
            found.add(so_far)
            continue
        for (source, mark), target in table.items():
            if source is state:
                todo.append((target, so_far + (mark,)))
    return found


def observed_runs(lives, n: int) -> set:
    """The runs of ``n`` consecutive marks in the given lives (``{uid: [marks]}`` or a list of them)."""
    if isinstance(lives, dict):
        lives = lives.values()
    out = set()
    for marks in lives:
        marks = [Event(m) for m in marks]
        out.update(tuple(marks[i:i + n]) for i in range(len(marks) - n + 1))
    return out
