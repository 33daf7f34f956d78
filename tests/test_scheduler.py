"""The scheduler's decisions, on the host with a stand-in model whose logits
are a pure function of a request's context."""

from __future__ import annotations

import hashlib

import pytest
import torch

from lockstep_amd.cache import CacheManager, OutOfPages
from lockstep_amd.engine.policy import (DefaultPolicy, Event, FixedChunkPolicy, NoCacheHitPolicy,
                                        PreemptAtStepsPolicy, ScriptedPolicy)
from lockstep_amd.engine.scheduler import OversizedRequest, Request, Scheduler
from lockstep_amd.parts import PagedKVSpec
from lockstep_amd.sampling import greedy, top_p

VOCAB = 40


def context_logits(context) -> torch.Tensor:
    seed = int.from_bytes(hashlib.sha256(repr(list(context)).encode()).digest()[:7], "big")
    return torch.randn(VOCAB, generator=torch.Generator().manual_seed(seed))


class StandInModel:
    """Keeps each request's tokens; logits at a place depend on the context up to it."""

    def __init__(self):
        self.history: dict[str, list[int]] = {}
        self.prompts: dict[str, list[int]] = {}
        self.batches: list[list[tuple]] = []

    def make_cache(self, num_pages, page_size=16, max_requests=64, max_tokens_per_request=None, **_):
        return CacheManager([PagedKVSpec(1, 16, None)], page_size, num_pages, max_requests,
                            max_tokens_per_request or num_pages * page_size)

    def step(self, cache, entries):
        rows, batch = [], []
        for e in entries:
            start = cache.length(e.request)
            if start == 0:
                self.history[e.request] = []
            hist = self.history.setdefault(e.request, [])
            if len(hist) < start:                       # a prefix hit: those tokens were never fed
                hist.extend(self.prompts[e.request][len(hist):start])
            assert len(hist) == start, "the step must continue where the cache ends"
            cache.reserve(e.request, start + len(e.tokens))
            hist.extend(e.tokens)
            batch.append((e.request, start, len(e.tokens)))
            for w in e.want:
                rows.append(context_logits(hist[: start + w + 1]))
        for e in entries:
            cache.commit(e.request, len(self.history[e.request]))
        self.batches.append(batch)
        return torch.stack(rows) if rows else None

    def decode_greedy(self, cache, requests, tokens, n_steps):
        """What the engine's device-side loop does, step by step."""
        import numpy as np
        from lockstep_amd.engine.batch import StepEntry

        self.bursts = getattr(self, "bursts", []) + [n_steps]
        out = []
        for _ in range(n_steps):
            logits = self.step(cache, [StepEntry(r, [t], [0]) for r, t in zip(requests, tokens)])
            tokens = [greedy(row) for row in logits]
            out.append(tokens)
        return np.asarray(out)


def expected_greedy(prompt, n, eos=()):
    context, out = list(prompt), []
    for _ in range(n):
        token = greedy(context_logits(context))
        out.append(token); context.append(token)
        if token in eos:
            break
    return out


def prompts(*lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, VOCAB, (n,), generator=g).tolist() for n in lengths]


def run(requests, **kw):
    model = StandInModel()
    for r in requests:
        model.prompts[r.uid] = list(r.prompt)
    kw.setdefault("num_blocks", 64)
    s = Scheduler(model, **kw)
    for r in requests:
        s.submit(r)
    return s.run(), s, model


def reqs(ps, n=6, **kw):
    return [Request(uid=f"r{i}", prompt=p, max_new_tokens=n, **kw) for i, p in enumerate(ps)]


def test_outputs_do_not_depend_on_chunking_budget_or_company():
    ps = prompts(1, 9, 17, 40, 64)
    want = {f"r{i}": expected_greedy(p, 6) for i, p in enumerate(ps)}
    assert run(reqs(ps))[0] == want
    assert run(reqs(ps), policy=FixedChunkPolicy(12))[0] == want
    assert run(reqs(ps), policy=FixedChunkPolicy(5), max_batched_tokens=16)[0] == want
    assert run(reqs(ps), policy=ScriptedPolicy(chunk_plan=[7, 2, 17, 3, 2]))[0] == want
    assert run(reqs(ps[2:3]))[0] == {"r0": want["r2"]}
    assert run(list(reversed(reqs(ps))))[0] == want


def test_token_budget_holds_and_decoded_tokens_go_first():
    ps = prompts(30, 30, 30)
    out, s, model = run(reqs(ps, n=4), policy=FixedChunkPolicy(8), max_batched_tokens=10)
    assert all(sum(n for _, _, n in b) <= 10 for b in model.batches)
    assert s.counters["budget_deferred"] > 0 and s.counters["prefill_chunk"] > 3
    # once r0 decodes, its token is in every batch although the budget is short for the others
    first_decode = next(i for i, b in enumerate(model.batches) if any(u == "r0" and n == 1 and st >= 30 for u, st, n in b))
    later = model.batches[first_decode: first_decode + 3]
    assert all(any(u == "r0" for u, _, _ in b) for b in later)
    assert out == {f"r{i}": expected_greedy(p, 4) for i, p in enumerate(ps)}


def test_admission_waits_for_pages_and_respects_max_running():
    ps = prompts(20, 20, 20)
    out, s, model = run(reqs(ps, n=4), num_blocks=4, block_size=8)        # each needs 3 of 4 pages
    assert [len(b) for b in model.batches].count(1) == len(model.batches)  # never two at once
    assert s.counters["admit_refused"] > 0 and s.counters["admit"] == 3
    assert out == {f"r{i}": expected_greedy(p, 4) for i, p in enumerate(ps)}
    out2, s2, model2 = run(reqs(ps, n=4), policy=DefaultPolicy(max_running=2))
    assert max(len(b) for b in model2.batches) == 2 and out2 == out
    s.cache.audit()
    assert s.cache.free_pages == [4] and s.cache.free_slots == s.cache.max_requests


def test_what_happens_when_pages_run_out():
    model = StandInModel()
    s = Scheduler(model, num_blocks=4, block_size=8)
    with pytest.raises(OversizedRequest):
        s.submit(Request(uid="big", prompt=[1] * 30, max_new_tokens=8))     # 5 pages > 4
    with pytest.raises(ValueError):
        s.submit(Request(uid="empty", prompt=[]))

    class Never(DefaultPolicy):
        def admit(self, state, uid, pages_needed):
            return False

    s = Scheduler(model, num_blocks=4, block_size=8, policy=Never())
    s.submit(Request(uid="a", prompt=[1, 2, 3]))
    with pytest.raises(OutOfPages, match="nothing running"):
        s.step()
    assert s.counters["out_of_pages"] == 1


def test_lazy_reservation_preempts_the_newest_and_recomputes():
    ps = prompts(20, 20, 20)
    want = {f"r{i}": expected_greedy(p, 12) for i, p in enumerate(ps)}

    class Eager(DefaultPolicy):                     # admit on the prompt alone; growth is found out later
        def admit(self, state, uid, pages_needed):
            return len(state.running) < self.max_running and state.free_pages >= 3

    out, s, model = run(reqs(ps, n=12), num_blocks=8, block_size=8, reserve="lazy", policy=Eager())
    assert out == want
    assert s.counters["preempt_for_pages"] > 0 and s.counters["resume"] > 0
    assert any(r.preemptions for r in s.done)
    s.cache.audit()
    assert s.cache.free_pages == [8]


def test_eos_stops_with_the_prefix_of_the_unbounded_run():
    p = prompts(11)[0]
    free = expected_greedy(p, 12)
    eos = free[4]
    cut = free[: free.index(eos) + 1]
    out, s, _ = run([Request(uid="r", prompt=p, max_new_tokens=12)], eos_token_ids={eos})
    assert out == {"r": cut} and s.counters["finish_eos"] == 1
    out, s, _ = run([Request(uid="r", prompt=p, max_new_tokens=12)])
    assert out == {"r": free} and s.counters["finish_limit"] == 1


def test_scripted_preemption_leaves_tokens_unchanged():
    ps = prompts(9, 23)
    want = {f"r{i}": expected_greedy(p, 8) for i, p in enumerate(ps)}
    for steps in ((2,), (2, 5), (2, 4, 6)):
        out, s, _ = run(reqs(ps, n=8), policy=PreemptAtStepsPolicy("r0", steps, chunk=7))
        assert out == want
        assert s.counters["preempt_fired"] == len(steps) and s.counters["resume"] == len(steps)
        assert [r.preemptions for r in s.done if r.uid == "r0"] == [len(steps)]
        assert Event.PREEMPT in s.lifecycle["r0"] and Event.RESUME in s.lifecycle["r0"]


def test_prefix_index_hits_trims_a_whole_prompt_hit_and_evicts_under_pressure():
    shared = prompts(32, seed=5)[0]
    a = Request(uid="a", prompt=shared + [1, 2, 3], max_new_tokens=4)
    model = StandInModel()
    s = Scheduler(model, num_blocks=12, block_size=8, enable_prefix_cache=True)
    for r in (a,):
        model.prompts[r.uid] = list(r.prompt); s.submit(r)
    s.run()
    assert s.counters["cache_miss"] == 1 and s.counters["cache_insert"] >= 4
    b = Request(uid="b", prompt=shared + [7, 8], max_new_tokens=4)
    c = Request(uid="c", prompt=shared, max_new_tokens=4)                 # the whole prompt is indexed
    for r in (b, c):
        model.prompts[r.uid] = list(r.prompt); s.submit(r)
    s.run()
    done = {r.uid: r for r in s.done}
    assert done["b"].reused == 32 and done["c"].reused == 24
    assert s.counters["cache_hit"] == 2 and s.counters["cache_full_prompt_trimmed"] == 1
    assert done["b"].generated == expected_greedy(b.prompt, 4)
    assert done["c"].generated == expected_greedy(c.prompt, 4)
    first_b = next(batch for batch in model.batches if any(u == "b" for u, _, _ in batch))
    assert ("b", 32, 2) in first_b                                         # only the tail was computed
    # pressure: a request that needs the indexed pages back
    held = s.num_pages - s.cache.free_pages[0]
    assert held > 0
    d = Request(uid="d", prompt=prompts(80, seed=9)[0], max_new_tokens=8)
    model.prompts["d"] = list(d.prompt); s.submit(d)
    s.run()
    assert s.counters["eviction_taken"] > 0 and s.evictions > 0
    assert {r.uid: r for r in s.done}["d"].generated == expected_greedy(d.prompt, 8)
    s.cache.audit()
    # refusing hits gives the same tokens
    s2 = Scheduler(model, num_blocks=12, block_size=8, enable_prefix_cache=True, policy=NoCacheHitPolicy())
    out = {}
    for uid, p in (("a2", a.prompt), ("b2", b.prompt)):      # one after the other: entries appear at finish
        model.prompts[uid] = list(p); s2.submit(Request(uid=uid, prompt=list(p), max_new_tokens=4))
        out.update(s2.run())
    assert out["b2"] == done["b"].generated and s2.counters["cache_hit_refused"] == 1


def test_sampled_tokens_depend_on_the_request_alone():
    # reference harness/mr/relations.py:184-223: removing, adding or reordering requests leaves survivors unchanged
    ps = prompts(5, 9, 14)

    def sampled(subset, order=1):
        rs = [Request(uid=f"r{i}", prompt=ps[i], seed=10 + i, max_new_tokens=10, temperature=0.8, top_p=0.95)
              for i in subset][::order]
        return run(rs)[0]

    everyone = sampled([0, 1, 2])
    assert sampled([1]) == {"r1": everyone["r1"]}
    assert sampled([0, 2], order=-1) == {"r0": everyone["r0"], "r2": everyone["r2"]}
    other_seed = run([Request(uid="r1", prompt=ps[1], seed=99, max_new_tokens=10, temperature=0.8, top_p=0.95)])[0]
    assert other_seed["r1"] != everyone["r1"]
    # position of the draw is the absolute index of the sampled row
    context = list(ps[1])
    want = []
    for _ in range(10):
        token = top_p(context_logits(context), 11, "r1", len(context) - 1, 0.95, 0.8)
        want.append(token); context.append(token)
    assert everyone["r1"] == want


def test_lifecycle_follows_the_state_machine():
    """Every life a run leaves walks the engine's own table (the scheduler checks each mark while
    auditing; here the whole lives again), the table is the reference's under full reservation
    (engine/sched/lifecycle.py:26-40), and a life that breaks it is refused."""
    from lockstep_amd.engine import lifecycle
    from lockstep_amd.engine.lifecycle import State

    reference = {
        ("waiting", Event.ADMIT): "admitted", ("admitted", Event.EVICT): "admitted",
        ("admitted", Event.CACHE_HIT): "prefilling", ("admitted", Event.CHUNK): "prefilling",
        ("admitted", Event.DECODE): "decoding", ("prefilling", Event.CHUNK): "prefilling",
        ("prefilling", Event.DECODE): "decoding", ("prefilling", Event.PREEMPT): "preempted",
        ("prefilling", Event.EVICT): "prefilling", ("decoding", Event.DECODE): "decoding",
        ("decoding", Event.PREEMPT): "preempted", ("decoding", Event.FINISH): "done",
        ("preempted", Event.RESUME): "admitted",
    }
    assert {(a.value, e): b.value for (a, e), b in lifecycle.STEPS.items()} == reference
    assert lifecycle.reachable() == set(State) and lifecycle.reachable(lazy=True) == set(State)
    ps = prompts(9, 23, 40)
    _, s, _ = run(reqs(ps, n=8), policy=PreemptAtStepsPolicy("r1", (3, 6), chunk=7), max_batched_tokens=20)
    for uid, events in s.lifecycle.items():
        assert lifecycle.follow(events) is State.DONE
    # what the run's lives contain is among what the table allows, and the table allows more than one run takes
    for n in (1, 2, 3):
        seen = lifecycle.observed_runs(s.lifecycle, n)
        assert seen and seen <= lifecycle.feasible_runs(n)
    assert len(lifecycle.feasible_runs(1)) == len(Event)
    assert (Event.PREEMPT, Event.RESUME) in lifecycle.feasible_runs(2)
    assert (Event.FINISH, Event.ADMIT) not in lifecycle.feasible_runs(2)
    assert lifecycle.feasible_runs(2) < lifecycle.feasible_runs(2, lazy=True)
    with pytest.raises(lifecycle.IllegalMark, match="not allowed in state waiting"):
        lifecycle.follow([Event.CHUNK])
    with pytest.raises(lifecycle.IllegalMark, match="marks decode first"):
        lifecycle.follow([Event.ADMIT, Event.FINISH])
    with pytest.raises(lifecycle.IllegalMark):
        lifecycle.follow([Event.ADMIT, Event.PREEMPT])                 # only lazy reservation does that
    assert lifecycle.follow([Event.ADMIT, Event.PREEMPT], lazy=True) is State.PREEMPTED
    a = run(reqs(ps, n=8))[1].trajectory
    b = run(reqs(ps, n=8))[1].trajectory
    c = run(reqs(ps, n=8), policy=FixedChunkPolicy(7))[1].trajectory
    assert a.hexdigest() == b.hexdigest() and a.first_divergence(b) is None
    assert a.hexdigest() != c.hexdigest() and a.first_divergence(c) == 0


def test_a_mark_the_table_forbids_stops_an_audited_run(monkeypatch):
    """Positive control of the walk: a scheduler that marks a finished request once more is caught at
    that mark when auditing, and not otherwise."""
    from lockstep_amd.engine import lifecycle

    original = Scheduler._retire

    def retire_and_mark_again(self):
        before = len(self.done)
        original(self)
        for seq in self.done[before:]:
            self._mark(seq.uid, Event.DECODE)

    monkeypatch.setattr(Scheduler, "_retire", retire_and_mark_again)
    with pytest.raises(lifecycle.IllegalMark, match="is done and was marked decode"):
        run(reqs(prompts(5), n=3))
    run(reqs(prompts(5), n=3), audit=False)


def test_lives_with_prefix_hits_evictions_and_lazy_preemption_follow_the_table():
    """The marks around a start (admit, then the prefix hit and the evictions it causes), and under lazy
    reservation the preemption of a request of which nothing has run yet."""
    from lockstep_amd.engine import lifecycle

    shared = prompts(32, seed=5)[0]
    model = StandInModel()
    s = Scheduler(model, num_blocks=12, block_size=8, enable_prefix_cache=True)

    def serve(uid, prompt, n=4):
        model.prompts[uid] = list(prompt)
        s.submit(Request(uid=uid, prompt=list(prompt), max_new_tokens=n))
        s.run()

    serve("a", shared + [1, 2, 3])
    serve("b", shared + [7, 8])
    serve("d", prompts(80, seed=9)[0], n=8)                    # needs the indexed pages back
    assert s.lifecycle["b"][:2] == [Event.ADMIT, Event.CACHE_HIT]
    assert s.lifecycle["d"][:2] == [Event.ADMIT, Event.EVICT]
    for events in s.lifecycle.values():
        assert lifecycle.follow(events) is lifecycle.State.DONE

    class Eager(DefaultPolicy):
        def admit(self, state, uid, pages_needed):
            return len(state.running) < self.max_running and state.free_pages >= 3

    ps = prompts(20, 20, 20)
    _, s, _ = run(reqs(ps, n=12), num_blocks=8, block_size=8, reserve="lazy", policy=Eager())
    s.counters.require_fired("preempt_for_pages", "resume")
    for events in s.lifecycle.values():
        assert lifecycle.follow(events, lazy=True) is lifecycle.State.DONE


def test_submit_refuses_before_anything_changes():
    """A uid in use (waiting, running, finished), fields out of range: a typed error from ``submit``,
    and the scheduler is as it was."""
    from lockstep_amd.engine.scheduler import InvalidRequest

    model = StandInModel()
    s = Scheduler(model, num_blocks=16)

    def state():
        return ([q.uid for q in s.waiting], [q.uid for q in s.running], [q.uid for q in s.done],
                s.cache.free_pages, s.cache.free_slots, dict(s.lifecycle))

    model.prompts["a"] = [1, 2, 3]
    s.submit(Request(uid="a", prompt=[1, 2, 3], max_new_tokens=3))
    before = state()
    with pytest.raises(InvalidRequest, match="it is waiting"):
        s.submit(Request(uid="a", prompt=[4, 5]))
    assert state() == before
    s.step()
    before = state()
    with pytest.raises(InvalidRequest, match="it is running"):
        s.submit(Request(uid="a", prompt=[4, 5]))
    assert state() == before
    s.run()
    with pytest.raises(InvalidRequest, match="it is finished"):
        s.submit(Request(uid="a", prompt=[4, 5]))
    bad = [dict(max_new_tokens=0), dict(max_new_tokens=-3), dict(max_new_tokens=2.5), dict(max_new_tokens=True),
           dict(temperature=-0.1), dict(temperature=float("nan")), dict(temperature=float("inf")),
           dict(temperature="hot"), dict(top_p=1.5), dict(top_p=-0.01), dict(top_p=float("nan")),
           dict(seed=-1), dict(seed=1 << 64), dict(seed=0.5), dict(prompt=[])]
    before = state()
    for i, fields in enumerate(bad):
        with pytest.raises(InvalidRequest):
            s.submit(Request(**{"uid": f"bad{i}", "prompt": [1, 2], **fields}))
    assert state() == before and s.counters["request_refused"] == 3 + len(bad)
    assert issubclass(InvalidRequest, ValueError)
    # the edges that are allowed: greedy, a nucleus of nothing but the best token, the whole distribution
    for i, fields in enumerate([dict(temperature=0), dict(temperature=0.0, top_p=0.0), dict(temperature=2.5, top_p=1),
                                dict(seed=(1 << 64) - 1, max_new_tokens=1)]):
        model.prompts[f"ok{i}"] = [1, 2]
        s.submit(Request(**{"uid": f"ok{i}", "prompt": [1, 2], **fields}))
    s.run()
    # a uid that was refused for its size or fields was never taken: it may come again
    with pytest.raises(OversizedRequest):
        s.submit(Request(uid="big", prompt=[1] * 300, max_new_tokens=8))
    model.prompts["big"] = [1] * 30
    s.submit(Request(uid="big", prompt=[1] * 30, max_new_tokens=2))
    s.submit(Request(uid="bad0", prompt=[1, 2]))
    model.prompts["bad0"] = [1, 2]
    assert set(s.run()) >= {"big", "bad0"}


def test_edge_counters_say_where_portions_ended():
    """Portions that end inside a page, on a page's edge and inside an attention split; contexts within one
    split and beyond it; second and third preemptions of one request: the run can show that it
    crossed them (the reference counts the same, engine/audit/counters.py:19-27)."""
    model = StandInModel()
    model.split_keys = 32
    p = prompts(70, seed=4)[0]
    model.prompts["r"] = p
    s = Scheduler(model, num_blocks=16, block_size=8, policy=ScriptedPolicy(chunk_plan=[8, 5, 19, 3]))
    s.submit(Request(uid="r", prompt=p, max_new_tokens=3))
    out = s.run()
    assert out["r"] == expected_greedy(p, 3)
    c = s.counters
    # ends at 8 (page edge), 13, 32 (page edge and split edge), 35, then the rest (the whole context: no edge)
    assert c["chunk_boundary_on_block"] == 2 and c["chunk_boundary_mid_block"] == 2
    assert c["chunk_boundary_mid_split"] == 3
    assert c["attention_single_split"] == 3 and c["attention_multi_split"] == 2 + 2     # 35, 70, and two decoded tokens
    c.require_fired("chunk_boundary_mid_block", "chunk_boundary_on_block", "chunk_boundary_mid_split",
                    "attention_multi_split", "attention_single_split")
    # a model that does not say how its attention is cut: the page counters only
    quiet = run(reqs([p], n=2), policy=FixedChunkPolicy(20))[1].counters
    assert quiet["chunk_boundary_mid_block"] == 3 and quiet["attention_multi_split"] == 0
    with pytest.raises(AssertionError, match="never took: attention_multi_split"):
        quiet.require_fired("chunk_boundary_mid_block", "attention_multi_split")
    # preemption depth
    ps = prompts(9, 23)
    for steps, second, third in (((2,), 0, 0), ((2, 5), 1, 0), ((2, 4, 6, 9), 1, 2)):
        _, s, _ = run(reqs(ps, n=10), policy=PreemptAtStepsPolicy("r0", steps, chunk=7))
        assert (s.counters["preempt_depth_2"], s.counters["preempt_depth_3_plus"]) == (second, third)
        assert s.counters["preempt_fired"] == len(steps)
    assert "preempt_depth_2" in s.counters.report() and not s.counters.never_taken("resume")


def test_a_prefix_cache_that_cannot_be_had_says_so():
    """A cache with a window (or state) cannot share pages: asking for the prefix cache then warns once,
    at construction, with the reason, and the scheduler records it."""
    from lockstep_amd.parts import StateSpec

    class Windowed(StandInModel):
        def make_cache(self, num_pages, page_size=16, max_requests=64, max_tokens_per_request=None, **_):
            return CacheManager([PagedKVSpec(1, 16, 24)], page_size, num_pages, max_requests,
                                max_tokens_per_request or num_pages * page_size)

    class Stateful(StandInModel):
        def make_cache(self, num_pages, page_size=16, max_requests=64, max_tokens_per_request=None, **_):
            return CacheManager([PagedKVSpec(1, 16, None), StateSpec((4,))], page_size, num_pages, max_requests,
                                max_tokens_per_request or num_pages * page_size)

    for model, reason in ((Windowed(), "window of keys"), (Stateful(), "per-request state")):
        with pytest.warns(RuntimeWarning, match=reason):
            s = Scheduler(model, num_blocks=16, block_size=8, enable_prefix_cache=True)
        assert s.prefix is None and reason in s.prefix_cache_refused
    import warnings

    with warnings.catch_warnings():
        warnings.simplefilter("error")
        s = Scheduler(StandInModel(), num_blocks=16, block_size=8, enable_prefix_cache=True)
        assert s.prefix is not None and s.prefix_cache_refused is None
        s = Scheduler(Windowed(), num_blocks=16, block_size=8)
        assert s.prefix_cache_refused is None


def test_decode_bursts_change_neither_tokens_nor_counts():
    """With decode_burst > 1 runs of decode steps go through the model's device-side loop: same
    tokens, same counters, same number of steps, same life cycle; a burst never runs past a
    request's last token, and not while something waits or samples (this stand-in model has no loop for
    that); a request that draws an end-of-sequence id inside a burst stops there."""
    ps = prompts(3, 20, 41)
    lengths = (5, 9, 14)

    def build():
        return [Request(uid=f"r{i}", prompt=p, max_new_tokens=n) for i, (p, n) in enumerate(zip(ps, lengths))]

    single, s1, m1 = run(build(), audit=False)
    burst, s2, m2 = run(build(), audit=False, decode_burst=4)
    assert burst == single == {f"r{i}": expected_greedy(p, n) for i, (p, n) in enumerate(zip(ps, lengths))}
    assert getattr(m2, "bursts", []) and max(m2.bursts) <= 4
    assert not hasattr(m1, "bursts")
    assert s2.counters["decode_burst"] == len(m2.bursts) and not s1.counters["decode_burst"]
    assert s1.counters.counts == {k: v for k, v in s2.counters.counts.items() if k != "decode_burst"}
    assert s1.step_index == s2.step_index and s1.lifecycle == s2.lifecycle
    # conditions that keep single steps: audit on, sampling with a model that has no loop for it, a waiting request
    for kw, requests in (({"audit": True}, build()),
                         ({"audit": False}, [Request(uid="t", prompt=ps[0], max_new_tokens=6, temperature=0.8, seed=3)])):
        _, _, m = run(requests, decode_burst=4, **kw)
        assert not hasattr(m, "bursts"), kw
    # end-of-sequence ids inside a burst: the request stops where single steps would stop it, the steps the
    # loop ran for it beyond that are dropped, and counters, steps and life cycles agree
    eos = [single["r1"][3], single["r2"][9]]
    stopped, s4, _ = run(build(), audit=False, eos_token_ids=eos)
    assert stopped == {f"r{i}": expected_greedy(p, n, eos) for i, (p, n) in enumerate(zip(ps, lengths))}
    assert any(len(stopped[u]) < len(single[u]) for u in stopped)
    bursting, s5, m5 = run(build(), audit=False, eos_token_ids=eos, decode_burst=4)
    assert bursting == stopped and getattr(m5, "bursts", [])
    assert s4.counters.counts == {k: v for k, v in s5.counters.counts.items() if k != "decode_burst"}
    assert s4.lifecycle == s5.lifecycle and s4.step_index == s5.step_index
    many = [Request(uid=f"w{i}", prompt=ps[0], max_new_tokens=8) for i in range(3)]
    out, s3, m3 = run(many, audit=False, decode_burst=16, policy=None, num_blocks=2)   # pages for two at a time
    assert out == {f"w{i}": expected_greedy(ps[0], 8) for i in range(3)}


def test_a_request_beyond_the_models_last_position_is_refused():
    class Bounded(StandInModel):
        class spec:                      # what the scheduler reads of a model
            max_positions = 40

    s = Scheduler(Bounded(), num_blocks=64)
    s.submit(Request(uid="fits", prompt=[1] * 30, max_new_tokens=10))
    with pytest.raises(OversizedRequest, match="positions end at 40"):
        s.submit(Request(uid="long", prompt=[1] * 30, max_new_tokens=11))
    assert s.counters["position_limit"] == 1 and [q.uid for q in s.waiting] == ["fits"]


def test_policies_are_put_together_from_rules():
    from lockstep_amd.engine.policy import AtSteps, EveryTokens, Listed, Policy

    ps = prompts(9, 23)
    want = {f"r{i}": expected_greedy(p, 8) for i, p in enumerate(ps)}
    rule = AtSteps([("r0", 3), ("r0", 7), ("r1", 1)])     # r1 has produced nothing at step 1: it is not asked about
    out, s, model = run(reqs(ps, n=8), policy=Policy(portion=EveryTokens(5), preemption=rule))
    assert out == want and rule.fired == [("r0", 3), ("r0", 7)] and s.counters["preempt_fired"] == 2
    assert all(n <= 5 for b in model.batches for _, _, n in b)
    assert not Policy(preemption=rule).same_answers_every_step()
    assert not Policy(portion=Listed([3])).same_answers_every_step()
    assert Policy(portion=EveryTokens(5)).same_answers_every_step() and FixedChunkPolicy(7).same_answers_every_step()

    class Own(DefaultPolicy):
        def chunk_boundary(self, view, uid, remaining):
            return 1

    assert not Own().same_answers_every_step()
    with pytest.raises(ValueError, match="between 1 and"):
        run(reqs(ps), policy=Policy(portion=lambda view, uid, remaining: remaining + 1))


def test_the_ledger_names_what_differs_between_two_runs():
    from lockstep_amd.engine.audit import StepLedger

    def ledger(logits=b"abc", state=(1, 2), steps=3):
        out = StepLedger()
        for i in range(steps):
            out.observe_step(i, [("r", [i], i)], [("r", i)], logits if i == 1 else b"same", state)
        return out

    a = ledger()
    assert a.first_difference(ledger()) is None and a.hexdigest() == ledger().hexdigest()
    assert a.first_difference(ledger(logits=b"abd")) == (1, ("logits",))
    assert a.first_difference(ledger(state=(1, 3))) == (0, ("state",))
    assert a.first_difference(ledger(steps=2)) == (2, ("length",)) and a.first_divergence(ledger(steps=2)) == 2
    assert len(set(a.per_step)) == 3


# -- positive controls on the host (the GPU ones are in test_controls_gpu.py) ------------------------

def test_a_draw_keyed_on_the_step_instead_of_the_position_is_caught(monkeypatch):
    """Sampled tokens must not depend on who else is served (reference harness/fuzz/faults.py:
    rng_keyed_on_global_step).  With the draw keyed on a running count of draws they do."""
    from lockstep_amd.sampling import philox

    ps = prompts(5, 9, 14)

    def sampled(subset):
        rs = [Request(uid=f"r{i}", prompt=ps[i], seed=10 + i, max_new_tokens=10, temperature=0.8, top_p=0.95)
              for i in subset]
        return run(rs)[0]

    def survivors_keep_their_tokens():
        everyone = sampled([0, 1, 2])
        return sampled([1]) == {"r1": everyone["r1"]} and sampled([0, 2]) == {k: everyone[k] for k in ("r0", "r2")}

    assert survivors_keep_their_tokens()
    original, count = philox.uniform, [0]

    def keyed_on_the_count(seed, uid, position, index=0):
        count[0] += 1
        return original(seed, uid, count[0], index)

    monkeypatch.setattr(philox, "uniform", keyed_on_the_count)
    assert not survivors_keep_their_tokens()
    monkeypatch.setattr(philox, "uniform", original)
    assert survivors_keep_their_tokens()


def test_a_page_given_back_without_its_count_going_down_is_caught(monkeypatch):
    """reference harness/fuzz/faults.py: refcount_decrement_missing_on_free -- the audit of every step sees it."""
    from lockstep_amd.cache import CacheAuditError
    from lockstep_amd.cache.manager import PagePool

    ps = prompts(20, 20)
    run(reqs(ps, n=4), num_blocks=8, block_size=8)                    # the unbroken run passes its audits
    original = PagePool.release

    def forgets_page_two(self, page):
        if page == 2:
            return False
        return original(self, page)

    monkeypatch.setattr(PagePool, "release", forgets_page_two)
    with pytest.raises(CacheAuditError):
        run(reqs(ps, n=4) + [Request(uid="late", prompt=ps[0], max_new_tokens=4)], num_blocks=8, block_size=8,
            policy=DefaultPolicy(max_running=1))
