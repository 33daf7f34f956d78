"""Positive controls: the tests of batch independence and of the cache's bookkeeping must be
able to fail.  Every control states a relation that holds for the engine, breaks the engine in
one named way, shows that the relation now fails (and fails where the breakage says it should),
and shows that it holds again once the breakage is taken out.

Device-side breakages are wrong variants compiled into control libraries (``-DLS_MUTANTS``,
files of their own beside the product libraries) and switched on by a mask: K blocking that
depends on the rows of a launch, a norm whose summation order depends on the rows of a launch,
a sampler whose cut of a row depends on the rows of a call, the fold over the attention splits reversed.  Host-side breakages are patched in from here: a
block table that is not refreshed when a slot is used again, a recomputation that skips a token,
a prefix match rounded up past a page, a draw keyed on the step instead of the position, a page
given back without its holder count going down.  The list follows the reference's seeded faults
(harness/fuzz/faults.py:279-311) and ablations (harness/mr/ablation.py:145-166)."""

from __future__ import annotations

import contextlib

import pytest
import torch

from helpers import feed, random_tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def control_kernels():
    from lockstep_amd.ops.kernels import Kernels

    kernels = Kernels(mutants=True)
    yield kernels
    kernels.set_mutants(0, 0)


@contextlib.contextmanager
def mutant(kernels, core=0, attention=0):
    kernels.set_mutants(core, attention)
    try:
        yield
    finally:
        kernels.set_mutants(0, 0)


@contextlib.contextmanager
def patched(owner, name, replacement):
    original = getattr(owner, name)
    setattr(owner, name, replacement(original))
    try:
        yield
    finally:
        setattr(owner, name, original)


def holds_breaks_holds(relation, breakage):
    """The relation holds, fails under the breakage, and holds again afterwards."""
    assert relation(), "the relation does not hold for the unbroken engine"
    with breakage():
        assert not relation(), "the breakage went unnoticed: the test of this relation cannot fail"
    assert relation(), "the relation does not hold any more after the breakage was taken out"


# -- device side: kernels alone ----------------------------------------------------------------

def test_k_blocking_that_depends_on_the_rows_of_a_launch_is_caught(control_kernels):
    from lockstep_amd.ops import STORE_F32

    k = control_kernels
    g = torch.Generator().manual_seed(3)
    x = torch.randn(300, 1024, generator=g).to(torch.bfloat16).cuda()
    w = torch.randn(272, 1024, generator=g).to(torch.bfloat16).cuda()

    def product(rows):
        out = torch.empty(rows, 272, dtype=torch.float32, device="cuda")
        k.gemm(x[:rows], w, out, STORE_F32)
        return out

    def row_is_the_same_in_every_batch():
        full = product(300)
        return all(torch.equal(product(rows), full[:rows]) for rows in (1, 16, 17, 40, 64, 65))

    holds_breaks_holds(row_is_the_same_in_every_batch, lambda: mutant(k, core=k.MUTANT_KSLICE_BY_ROWS))
    with mutant(k, core=k.MUTANT_KSLICE_BY_ROWS):      # ... and only the launches of 17 to 64 rows are off
        full = product(300)
        assert torch.equal(product(16), full[:16]) and torch.equal(product(65), full[:65])
        assert not torch.equal(product(40), full[:40])
        assert (product(40) - full[:40]).abs().max() < 1e-2          # another order of the same sum, nothing else


def test_a_norm_whose_order_depends_on_the_rows_of_a_launch_is_caught(control_kernels):
    k = control_kernels
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(40, 1000, generator=g) * 3).cuda()
    weight = torch.ones(1000, device="cuda")

    def normed(lo, hi):
        out = torch.empty(hi - lo, 1000, dtype=torch.float32, device="cuda")
        k.rmsnorm(x[lo:hi], weight, out, 1e-6)
        return out

    def rows_alone_equal_rows_in_a_batch():
        together = normed(0, 40)
        return all(torch.equal(normed(lo, lo + 4), together[lo:lo + 4]) for lo in range(0, 40, 4))

    holds_breaks_holds(rows_alone_equal_rows_in_a_batch, lambda: mutant(k, core=k.MUTANT_NORM_BY_ROWS))


def test_a_sampler_whose_cut_depends_on_the_rows_of_a_call_is_caught(control_kernels):
    """Rows whose nucleus lies exactly on the boundary between two tokens get the same tokens alone
    and among 200 rows; a sampler that cuts a row into fewer chunks when the call has many rows adds
    its sums in another order there, and some boundary falls the other way."""
    from helpers import sampling_rows_on_boundaries
    from test_kernels_gpu import sample_among

    k = control_kernels
    logits, requests = sampling_rows_on_boundaries(151936, rows=24)
    dev = logits.cuda()

    def same_tokens_alone_and_in_company():
        alone = [sample_among(k, dev, [r], 1, 0)[0] for r in requests]
        return all(sample_among(k, dev, requests, n, n) == alone for n in (64, 200))

    holds_breaks_holds(same_tokens_alone_and_in_company, lambda: mutant(k, core=k.MUTANT_SAMPLE_CHUNKS_BY_ROWS))


# -- device side: through the model ---------------------------------------------------------------

def test_a_reversed_fold_over_the_splits_is_caught_where_there_are_three_splits(tiny_dirs, control_kernels):
    """A whole prompt (its workgroups walk the splits themselves) against the same tokens with the
    tail in steps of one and of two tokens (one split a workgroup; the sums of a single token are
    folded by the output product, those of two tokens by the combine kernel): equal bits.  With the
    folds running backwards they differ, and only at positions that have three splits of 128 keys and more
    (two partial results give the same sum in either order).  On the 32-bit path: the bfloat16 path rounds the
    attention output to eight bits, which hides a reordered 32-bit sum almost always."""
    from lockstep_amd.engine.model import load_model

    model = load_model(tiny_dirs[("B", "sharp")], dtype="float32")
    model.rt.kernels = control_kernels
    tokens = random_tokens(600, 1000, seed=21)
    head = 200

    def both_ways():
        cache = model.make_cache(num_pages=160, page_size=8, max_requests=2)
        whole = feed(model, cache, "w", tokens, [])
        tail = feed(model, cache, "t", tokens, [head] + [1, 2] * ((len(tokens) - head) // 3 + 1))
        return whole, tail

    def same_bits():
        whole, tail = both_ways()
        return torch.equal(whole, tail)

    # (decoded tokens with few splits are folded by the output product, longer ones by the combine launch:
    # both folds are reversed)
    reversed_folds = dict(core=control_kernels.MUTANT_REVERSED_FOLD_IN_PRODUCT,
                          attention=control_kernels.MUTANT_REVERSED_FOLD)
    holds_breaks_holds(same_bits, lambda: mutant(control_kernels, **reversed_folds))
    for one in ({"core": reversed_folds["core"]}, {"attention": reversed_folds["attention"]}):
        with mutant(control_kernels, **one):          # each of the two alone is noticed too: both folds are in use
            assert not same_bits(), one
    with mutant(control_kernels, **reversed_folds):
        whole, tail = both_ways()
        differs = (whole != tail).any(dim=1)
        assert not differs[:256].any(), "a position with one or two splits changed: the control fails for the wrong reason"
        assert differs[256:].any() and float((whole - tail).abs().max()) < 1e-3 * float(whole.abs().max())


def test_batch_dependent_k_blocking_is_caught_by_the_decode_test(tmp_path_factory, control_kernels):
    """Forty requests in one decode step against each of them alone (the relation of
    test_many_requests_decode_with_the_bits_of_one), at layer sizes whose products have four K slices."""
    from lockstep_amd.config import Qwen3Config
    from lockstep_amd.engine.batch import StepEntry
    from lockstep_amd.engine.model import load_model
    from lockstep_amd.weights import write_random_model

    config = Qwen3Config(hidden_size=1024, intermediate_size=3072, num_hidden_layers=1, num_attention_heads=16,
                         num_key_value_heads=8, head_dim=128, vocab_size=1031, rms_norm_eps=1e-6, rope_theta=1e6,
                         max_position_embeddings=512, tie_word_embeddings=True)
    folder = write_random_model(config, tmp_path_factory.mktemp("ctl"), seed=3, std=0.02, norm_std=0.1)
    model = load_model(folder, dtype="bfloat16")
    model.rt.kernels = control_kernels
    n_req = 40
    prompts = [random_tokens(6 + 7 * i % 50, 1031, seed=300 + i) for i in range(n_req)]

    def together_equals_alone():
        cache = model.make_cache(num_pages=4 * n_req, page_size=16, max_requests=n_req)
        for i, p in enumerate(prompts):
            cache.open(f"r{i}")
            model.step(cache, [StepEntry(f"r{i}", p[:-1], [])])
        together = model.step(cache, [StepEntry(f"r{i}", p[-1:], [0]) for i, p in enumerate(prompts)])
        for i in (0, 17, n_req - 1):
            alone = model.make_cache(num_pages=8, page_size=16, max_requests=1)
            want = feed(model, alone, "x", prompts[i], [len(prompts[i]) - 1, 1])[-1]
            if not torch.equal(together[i].cpu(), want):
                return False
        return True

    holds_breaks_holds(together_equals_alone, lambda: mutant(control_kernels, core=control_kernels.MUTANT_KSLICE_BY_ROWS))


# -- host side ---------------------------------------------------------------------------------------

def test_a_block_table_that_is_not_refreshed_is_caught(tiny_dirs):
    """Pages are used again by later requests in slots that earlier requests held.  If a slot's row
    of the device block table keeps what it got the first time, the kernels read pages that belong
    to someone else (or were poisoned when they were freed)."""
    from helpers import make_mixed_trace, max_live_tokens, replay_in_process
    from lockstep_amd.cache import CacheManager
    from lockstep_amd.engine.model import load_model

    model = load_model(tiny_dirs[("A", "sharp")], dtype="float32")
    requests = {f"q{i}": random_tokens(n, 512, seed=700 + i) for i, n in enumerate([70, 45, 33, 90, 21, 64])}
    steps = make_mixed_trace(requests, seed=5)
    roomy = model.make_cache(num_pages=64, page_size=16)
    whole = {rid: feed(model, roomy, rid, t, []) for rid, t in requests.items()}

    def mixed_equals_whole():
        pages = max_live_tokens(steps, round_to=16) // 16
        cache = model.make_cache(num_pages=pages, page_size=16, max_requests=4, max_tokens_per_request=96,
                                 poison_on_free=True)
        got = replay_in_process(model, cache, steps)
        return all(torch.equal(got[rid], whole[rid]) for rid in requests)

    def first_upload_only(original):
        def sync_tables(self):
            seen = self.__dict__.setdefault("_rows_uploaded_once", set())
            for group in self.groups:
                fresh = {row for row in group.dirty_rows if (group.index, row) not in seen}
                seen.update((group.index, row) for row in fresh)
                group.dirty_rows = fresh
            return original(self)
        return sync_tables

    holds_breaks_holds(mixed_equals_whole, lambda: patched(CacheManager, "sync_tables", first_upload_only))


def test_a_recomputation_that_skips_a_token_is_caught(tiny_dirs):
    from lockstep_amd import Request
    from lockstep_amd.engine.policy import PreemptAtStepsPolicy
    from lockstep_amd.engine.scheduler import Scheduler
    from test_scheduler_gpu import alone, serve

    model = load_tiny(tiny_dirs, "B", "float32")
    wave = [Request(uid="p0", prompt=random_tokens(19, 1000, seed=41), max_new_tokens=12),
            Request(uid="p1", prompt=random_tokens(30, 1000, seed=42), max_new_tokens=8)]
    want = {r.uid: alone(model, r, 8)[0] for r in wave}

    def preempted_equals_alone():
        out, s = serve(model, [[Request(**vars(r)) for r in wave]], 8, num_pages=24,
                       policy=PreemptAtStepsPolicy("p0", (4,), chunk=11))
        s.counters.require_fired("preempt_fired", "resume")
        return out == want

    def one_token_too_far(original):
        def start(self, seq, view):
            ok = original(self, seq, view)
            if ok and seq.preemptions:                  # a resumed request believes its first token is cached
                self.cache.reserve(seq.uid, 1, 0)
                self.cache.commit(seq.uid, 1)
                seq.cached = 1
            return ok
        return start

    holds_breaks_holds(preempted_equals_alone, lambda: patched(Scheduler, "_start", one_token_too_far))


def test_a_prefix_match_rounded_up_past_a_page_is_caught(tiny_dirs):
    from lockstep_amd import Request
    from lockstep_amd.cache import PrefixIndex
    from test_scheduler_gpu import alone, serve

    model = load_tiny(tiny_dirs, "A", "bfloat16")
    base = random_tokens(48, 512, seed=31)
    first = [Request(uid="a", prompt=base + random_tokens(20, 512, seed=32), max_new_tokens=4)]
    second = [Request(uid="b", prompt=base + random_tokens(20, 512, seed=33), max_new_tokens=6)]
    want = alone(model, second[0], 16)[0]

    def hit_equals_alone():
        out, s = serve(model, [[Request(**vars(r)) for r in first], [Request(**vars(r)) for r in second]], 16,
                       num_pages=20, enable_prefix_cache=True)
        s.counters.require_fired("cache_hit")
        return out["b"] == want

    def one_page_more(original):
        def match(self, tokens):
            pages = original(self, tokens)
            node = self.by_page.get(pages[-1]) if pages else None
            if node is not None and node.children and (len(pages) + 1) * self.page_size < len(tokens):
                pages = pages + [next(iter(node.children.values())).page]     # a page of other tokens
            return pages
        return match

    holds_breaks_holds(hit_equals_alone, lambda: patched(PrefixIndex, "match", one_page_more))


def load_tiny(tiny_dirs, name, dtype):
    from lockstep_amd.engine.model import load_model

    return load_model(tiny_dirs[(name, "gen")], dtype=dtype)
