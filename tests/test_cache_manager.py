"""The cache manager on the host: no page lost, held twice or freed twice,
under random orders of requests; windows give pages back; state slots."""

from __future__ import annotations

import random

import pytest

from lockstep_amd.cache import CacheAuditError, CacheManager, OutOfPages, PrefixIndex
from lockstep_amd.parts import PagedKVSpec, StateSpec

FULL = PagedKVSpec(2, 16, None)


def manager(num_pages=8, page_size=16, specs=(FULL, FULL), **kw):
    return CacheManager(list(specs), page_size, num_pages, max_requests=kw.pop("max_requests", 4),
                        max_tokens_per_request=kw.pop("max_tokens", num_pages * page_size), **kw)


def test_pages_are_taken_lowest_first_and_reused():
    # reference tests/test_paged_kv.py:50-64
    c = manager()
    c.open("a"); c.reserve("a", 33)
    c.open("b"); c.reserve("b", 16)
    assert c.request_pages("a") == [0, 1, 2] and c.request_pages("b") == [3]
    c.close("a")
    c.open("c"); c.reserve("c", 40)
    assert c.request_pages("c") == [0, 1, 2]
    c.audit()


def test_growth_is_on_demand_and_exhaustion_raises_without_taking_anything():
    c = manager(num_pages=4)
    c.open("a"); c.reserve("a", 16); c.commit("a", 16)
    c.reserve("a", 17)
    assert c.request_pages("a") == [0, 1]
    c.open("b")
    with pytest.raises(OutOfPages):
        c.reserve("b", 16 * 3)
    assert c.request_pages("b") == [] and c.free_pages == [2]
    with pytest.raises(ValueError):
        c.reserve("a", 16 * 5)        # more than a request may hold
    c.audit()


def test_unsupported_page_size_is_refused():
    with pytest.raises(ValueError):
        manager(page_size=48)         # reference tests/test_paged_kv.py:45-47


def test_groups_have_pages_of_their_own_and_windows_give_pages_back():
    window = PagedKVSpec(2, 16, 20)
    c = manager(num_pages=[8, 5], page_size=8, specs=(FULL, window, FULL, window), max_tokens=64)
    assert len(c.groups) == 2 and c.groups[0].units == [0, 2] and c.groups[1].units == [1, 3]
    c.open("a")
    pos = 0
    for step in (5, 8, 8, 8, 8, 8, 8, 3):      # 19 old keys + 8 new ones span at most five pages of 8
        c.reserve("a", pos + step)
        c.commit("a", pos + step)
        pos += step
        held = [p for p in c.request_pages("a", 1) if p >= 0]
        assert len(held) <= 5
        first_needed = max(0, pos - 20 + 1) // 8
        assert all(p == -1 for p in c.request_pages("a", 1)[:first_needed])
        assert all(p >= 0 for p in c.request_pages("a", 1)[first_needed:])
        c.audit()
    assert len([p for p in c.request_pages("a", 0) if p >= 0]) == 7       # the full group keeps everything
    c.close("a")
    assert c.free_pages == [8, 5]
    c.audit()


def test_a_long_first_portion_never_takes_pages_below_the_window():
    c = manager(num_pages=[32, 16], page_size=8, specs=(FULL, PagedKVSpec(2, 16, 10)), max_tokens=128)
    c.open("a"); c.reserve("a", 50)                             # prompt in one portion: needs all of its own keys
    assert [p >= 0 for p in c.request_pages("a", 1)] == [True] * 7
    c.commit("a", 50)                                           # the next query is at 50 and reads keys 41..
    assert [p >= 0 for p in c.request_pages("a", 1)] == [False] * 5 + [True] * 2
    c.reserve("a", 51); c.commit("a", 51)
    assert [p >= 0 for p in c.request_pages("a", 1)] == [False] * 5 + [True] * 2
    c.open("b"); c.commit("b", 0)
    c.reserve("b", 100, start=90)                                # resumed far into a sequence
    assert c.request_pages("b", 1)[:10] == [-1] * 10
    c.audit()


def test_state_slots_are_handed_out_lowest_first():
    c = manager(specs=(FULL, StateSpec((4, 2))), max_requests=2)
    assert c.open("a") == 0 and c.open("b") == 1
    with pytest.raises(OutOfPages):
        c.open("c")
    c.close("a")
    assert c.open("c") == 0 and c.state_units == {1: StateSpec((4, 2))}
    with pytest.raises(KeyError):
        c.open("c")
    c.audit()


def test_state_is_zeroed_when_taken_poisoned_when_given_back_and_in_the_ledger():
    import torch

    def build(**kw):
        return CacheManager([FULL, StateSpec((3,)), StateSpec((2, 2), dtype="int32")], 16, 4, max_requests=2,
                            max_tokens_per_request=64, torch_dtype=torch.float32, device=torch.device("cpu"), **kw)

    c = build(poison_on_free=True)
    assert c.unit_state(1).dtype is torch.float32 and c.unit_state(2).dtype is torch.int32
    c.open("a"); c.open("b")
    c.unit_state(1)[c.slot("a")] = torch.tensor([1.0, 2.0, 3.0])
    c.unit_state(2)[c.slot("b")] += 5
    c.audit()
    with_content = c.state_digest(content=True)
    c.unit_state(1)[c.slot("a"), 0] = 9.0
    assert c.state_digest(content=True) != with_content            # the rows of live requests are in the digest
    assert c.state_digest() == c.state_digest()                     # ... and only when asked for
    assert c.state_digest()[:2] == ((1, (3,), "float32"), (2, (2, 2), "int32"))
    c.close("a")
    assert bool(c.unit_state(1)[0].isnan().all()) and bool((c.unit_state(2)[0] == -(1 << 30)).all())
    c.audit()
    c.unit_state(1)[0] = 0.0                                        # someone wrote into a slot nobody owns
    with pytest.raises(CacheAuditError, match="not poisoned"):
        c.audit()
    assert c.open("c") == 0 and bool((c.unit_state(1)[0] == 0).all()) and bool((c.unit_state(2)[0] == 0).all())
    c.audit()
    c.unit_state(1)[c.slot("b"), 1] = float("nan")                  # a live request that read poison
    with pytest.raises(CacheAuditError, match="poisoned state"):
        c.audit()
    with pytest.raises(TypeError):
        CacheManager([StateSpec((3,), dtype="float64")], 16, 4, 2, 64, torch_dtype=torch.float32,
                     device=torch.device("cpu"))
    quiet = build()
    quiet.open("a"); quiet.unit_state(1)[0] = 4.0; quiet.close("a")
    assert bool((quiet.unit_state(1)[0] == 4.0).all())              # without poisoning the row is left as it was
    quiet.audit()


def test_audit_catches_a_lost_a_doubled_and_a_twice_freed_page():
    # reference tests/test_paged_kv.py:67-85
    c = manager()
    c.open("a"); c.reserve("a", 32)
    c.groups[0].pool.holders[0] += 1
    with pytest.raises(CacheAuditError):
        c.audit()
    c.groups[0].pool.holders[0] -= 1
    c.requests["a"].groups[0].pages[1] = 0
    with pytest.raises(CacheAuditError):
        c.audit()
    c.requests["a"].groups[0].pages[1] = 1
    c.audit()
    c.close("a")
    with pytest.raises(CacheAuditError):
        c.groups[0].pool.release(0)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_keep_the_ledger_balanced(seed):
    rng = random.Random(seed)
    window = PagedKVSpec(1, 16, 24)
    c = manager(num_pages=[24, 10], page_size=8, specs=(FULL, window), max_requests=5, max_tokens=96)
    live: dict[str, int] = {}
    digests = set()
    for step in range(400):
        action = rng.random()
        if live and action < 0.15:
            rid = rng.choice(sorted(live))
            c.close(rid); del live[rid]
        elif len(live) < 5 and action < 0.35:
            rid = f"r{step}"
            c.open(rid); live[rid] = 0
        elif live:
            rid = rng.choice(sorted(live))
            grow = rng.choice([1, 1, 1, 2, 7, 8, 9, 17])
            end = live[rid] + grow
            if end > 96:
                continue
            before = c.state_digest()
            try:
                c.reserve(rid, end)
            except OutOfPages:
                assert c.state_digest() == before          # nothing was taken
                continue
            c.commit(rid, end); live[rid] = end
        c.audit()
        digests.add(c.state_digest())
        for g in c.groups:
            held = sum(1 for r in c.requests.values() for p in r.groups[g.index].pages if p >= 0)
            assert held + g.pool.free_pages == g.pool.num_pages
    for rid in list(live):
        c.close(rid)
    c.audit()
    assert c.free_pages == [24, 10] and c.free_slots == 5 and len(digests) > 50


def test_prefix_index_shares_whole_pages_and_drops_only_unused_leaves():
    c = manager(num_pages=8, page_size=8, specs=(FULL,), max_tokens=64)
    index = PrefixIndex(8)
    tokens = list(range(22))
    c.open("a"); c.reserve("a", 22); c.commit("a", 22)
    assert index.remember(tokens, c.request_pages("a"), c) == 2       # two whole pages
    assert index.remember(tokens, c.request_pages("a"), c) == 0       # nothing new the second time
    c.close("a")
    assert c.free_pages == [6]                                        # the index still holds two
    pages = index.match(tokens[:16] + [99, 98])
    assert pages == [0, 1]
    assert index.match([0, 1, 2, 9] + tokens[4:16]) == []             # a changed first page: nothing after it counts
    assert index.match(tokens[:15]) == [0]                            # whole pages only
    c.open("b"); c.adopt("b", pages); c.commit("b", 16); c.reserve("b", 18)
    assert c.request_pages("b") == [0, 1, 2]
    c.audit()
    assert index.droppable(c) == [] and index.reclaimable(c) == 0     # b maps them
    with pytest.raises(CacheAuditError):
        c.assert_exclusive("b", 0, 0)                                 # a write into a shared page is refused
    c.assert_exclusive("b", 0, 2)
    # b finishes with a longer context: its third page joins the chain below the shared two
    c.commit("b", 24)
    assert index.remember(tokens[:16] + list(range(100, 108)), c.request_pages("b"), c) == 1
    c.close("b")
    assert index.reclaimable(c) == 3 and index.droppable(c) == [2]    # only the leaf may go
    assert not index.drop(0, c) and not index.drop(1, c)              # a page inside a chain stays
    assert index.drop(2, c) and index.droppable(c) == [1]
    assert index.drop(1, c) and index.drop(0, c) and c.free_pages == [8] and len(index) == 0
    c.audit()
    # two requests that computed the same first page on pages of their own share one node
    c.open("x"); c.reserve("x", 16); c.commit("x", 16)
    c.open("y"); c.reserve("y", 16); c.commit("y", 16)
    assert index.remember(tokens[:16], c.request_pages("x"), c) == 2
    assert index.remember(tokens[:8] + list(range(50, 58)), c.request_pages("y"), c) == 1
    assert sorted(index.by_page) == [0, 1, 3] and len(index.digest()) == 3
    c.close("x"); c.close("y")
    assert index.droppable(c) == [1, 3]                               # both leaves; their common parent stays
    c.audit()
    windowed = manager(specs=(FULL, PagedKVSpec(2, 16, 8)))
    assert not windowed.shareable()
