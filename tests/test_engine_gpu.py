"""The engine against the plain implementation, under every way of cutting
the work, in float32 and in bfloat16, on the two tiny configurations."""

from __future__ import annotations

import pytest
import torch

from helpers import (BF16_EXACT_PREFIX_TOL, BF16_TOL, FP32_TOL, FP32_TOL_SOFT, feed, random_tokens, tol_for,
                     rel_err)

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
# what each path is held to on the sharpened weights: the 32-bit path against exact arithmetic, the
# bfloat16 path against the plain forward that stores in bfloat16 where the engine does


@pytest.fixture(scope="module")
def plain_logits(tiny_dirs):
    """Plain float64 logits of the test sequences, computed once.  ``[name]``: (folder, {n:
    (tokens, exact logits, logits with bfloat16 storage)}) on the sharpened weights; ``[(name,
    "soft")]``: (folder, {n: (tokens, exact logits)}) on the weights as drawn."""
    from plain.qwen3_plain import PlainModel, bf16

    out = {}
    for name in ("A", "B"):
        for variant in ("sharp", "soft"):
            folder = tiny_dirs[(name, variant)]
            plain = PlainModel(folder)
            vocab = plain.cfg["vocab_size"]
            seqs = {n: random_tokens(n, vocab, seed=100 + n) for n in (1, 7, 40, 333)}
            if variant == "sharp":
                out[name] = (folder, {n: (t, plain.logits(t), plain.logits(t, store=bf16)) for n, t in seqs.items()})
            else:
                out[(name, variant)] = (folder, {n: (t, plain.logits(t)) for n, t in seqs.items()})
    out["gen"] = {name: tiny_dirs[(name, "gen")] for name in ("A", "B")}
    return out


def want_for(entry, dtype):
    """The plain logits a path is compared with on the sharpened weights."""
    return entry[1] if dtype == "float32" else entry[2]


def plain_of(folder, dtype):
    """tokens -> plain logits as ``dtype`` is compared with them."""
    from plain.qwen3_plain import PlainModel, bf16

    plain = PlainModel(folder)
    return plain, (lambda tokens: plain.logits(tokens, store=None if dtype == "float32" else bf16))


def load(folder, dtype):
    from lockstep_amd.engine.model import load_model

    return load_model(folder, dtype=dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_whole_prompts_match_plain(plain_logits, dtype, name, page_size):
    folder, seqs = plain_logits[name]
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=64, page_size=page_size, poison_on_free=True)
    for n, entry in seqs.items():
        got = feed(model, cache, f"r{n}", entry[0], [])
        err = rel_err(got, want_for(entry, dtype))
        print(f"{name} {dtype} whole n={n}: rel err {err:.3e}")
        assert err < tol_for(dtype, name), f"n={n}"
        if dtype == "bfloat16" and n == 1:         # nothing can have flipped yet: the stored forward is exact
            assert err < BF16_EXACT_PREFIX_TOL
        cache.close(f"r{n}")
    cache.audit()
    # the weights as drawn: the 32-bit path at its tightest, the bfloat16 path against exact arithmetic
    folder, seqs = plain_logits[(name, "soft")]
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=64, page_size=page_size)
    for n, (tokens, want) in seqs.items():
        err = rel_err(feed(model, cache, f"s{n}", tokens, []), want)
        print(f"{name} {dtype} whole n={n}, weights as drawn: rel err {err:.3e}")
        assert err < (FP32_TOL_SOFT if dtype == "float32" else BF16_TOL), f"n={n}"
        cache.close(f"s{n}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_a_lost_far_page_or_key_would_show(plain_logits, dtype, name, page_size):
    """700 tokens (three splits of the keys) on the sharpened weights.  The plain forward states what
    a fault would give -- a far page hidden from the last 64 queries in every layer, the same in the
    first layer only, a single far key hidden -- and the engine has to lie far closer to the
    faultless logits than any of them does, in 32-bit and, against the forward that stores in
    bfloat16, in bfloat16."""
    folder, _ = plain_logits[name]
    plain, reference = plain_of(folder, dtype)
    store = None if dtype == "float32" else __import__("plain.qwen3_plain", fromlist=["bf16"]).bf16
    n, tail = 700, 64
    tokens = random_tokens(n, plain.cfg["vocab_size"], seed=100 + n)
    good = reference(tokens)
    layers = plain.cfg["num_hidden_layers"]
    page = {"A": 2, "B": 16}[name]                      # far behind the last queries, inside the first split

    def faulty(keys, where):
        hide = torch.zeros(n, n, dtype=torch.bool)
        hide[-tail:, keys] = True
        return rel_err(plain.logits(tokens, store=store, also_hidden={l: hide for l in where})[-tail:], good[-tail:])

    lost_page = faulty(slice(page * page_size, (page + 1) * page_size), range(layers))
    lost_page_one_layer = faulty(slice(page * page_size, (page + 1) * page_size), [0])
    lost_key = faulty(slice(page * page_size + 3, page * page_size + 4), range(layers))
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=-(-n // page_size) + 2, page_size=page_size, poison_on_free=True)
    got = feed(model, cache, "far", tokens, [n - tail] + [1] * tail)     # the last queries as decoded tokens
    err = rel_err(got[-tail:], good[-tail:])
    print(f"{name} {dtype}: engine {err:.2e}; a lost page {lost_page:.2e}, in one layer {lost_page_one_layer:.2e}, "
          f"a lost key {lost_key:.2e}")
    # every fault, the single key included, lies outside the bound that the engine is held to (and that every
    # other comparison of this configuration uses), by a factor of three
    bound = tol_for(dtype, name)
    assert err < bound
    assert lost_page > 3 * bound and lost_page_one_layer > 3 * bound and lost_key > 3 * bound


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_cuttings_give_the_same_bits(plain_logits, dtype, name, page_size):
    """Whole; most in one step and the last 32 one by one; portions of changing
    size down to two tokens; token by token: bitwise equal logits."""
    folder, seqs = plain_logits[name]
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=64, page_size=page_size, poison_on_free=True)
    tokens = seqs[333][0]
    whole = feed(model, cache, "whole", tokens, [])
    cache.close("whole")
    assert rel_err(whole, want_for(seqs[333], dtype)) < tol_for(dtype, name)
    cuttings = {
        "last32": [len(tokens) - 32] + [1] * 32,
        "ragged": [7, 17, 37, 2, 64, 3, 129, 2],
        "page_edges": [page_size - 1, 2, page_size, page_size + 1, 255 - 3 * page_size - 2, 2, 1, 2],
        "two_and_rest": [2, len(tokens) - 4, 2],
        "one_by_one": [1] * len(tokens),
    }
    for label, cuts in cuttings.items():
        got = feed(model, cache, label, tokens, cuts)
        cache.close(label)
        if not torch.equal(got, whole):
            bad = (got != whole).any(dim=1).nonzero()[0].item()
            pytest.fail(f"{name} {dtype} {label}: first differing position {bad}, "
                        f"max diff {float((got - whole).abs().max()):.3e}")
    cache.audit()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_mixed_batches_with_reused_pages(plain_logits, dtype, name, page_size):
    """Up to four live requests, portions of some beside decoded tokens of
    others, with so few pages that freed ones are used again (and poisoned in
    between): every request's logits equal its whole run bit for bit and the
    plain implementation within tolerance."""
    from helpers import make_mixed_trace, max_live_tokens, replay_in_process

    folder, _ = plain_logits[name]
    plain, reference = plain_of(folder, dtype)
    vocab = plain.cfg["vocab_size"]
    lengths = [70, 45, 33, 90, 21, 64, 130, 17]
    requests = {f"q{i}": random_tokens(n, vocab, seed=500 + i) for i, n in enumerate(lengths)}
    steps = make_mixed_trace(requests, seed=3)
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len(e["tokens"]) == 2 for s in steps for e in s["entries"])
    model = load(folder, dtype)
    num_pages = max_live_tokens(steps, round_to=page_size) // page_size
    cache = model.make_cache(num_pages=num_pages, page_size=page_size, max_requests=4,
                             max_tokens_per_request=max(lengths), poison_on_free=True)
    got = replay_in_process(model, cache, steps)
    assert cache.groups[0].pool.taken_total > 2 * num_pages, "pages were not used again"
    assert cache.free_pages == [num_pages]
    roomy = model.make_cache(num_pages=64, page_size=page_size, poison_on_free=True)
    for rid, tokens in requests.items():
        whole = feed(model, roomy, rid, tokens, [])
        roomy.close(rid)
        assert torch.equal(got[rid], whole), f"{rid}: mixed run differs from the whole run"
        assert rel_err(got[rid], reference(tokens)) < tol_for(dtype, name), rid


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_matches_plain(plain_logits, dtype):
    """Forty tokens at once, then three hundred one by one (past two splits of the keys)."""
    folder, _ = plain_logits["B"]
    plain, reference = plain_of(folder, dtype)
    tokens = random_tokens(340, plain.cfg["vocab_size"], seed=77)
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=48, page_size=8, poison_on_free=True)
    got = feed(model, cache, "long", tokens, [40] + [1] * 300)
    err = rel_err(got, reference(tokens))
    print(f"long decode {dtype}: rel err {err:.3e}")
    assert err < tol_for(dtype, "B")


@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_greedy_generation_through_the_entry_points(plain_logits, name, page_size):
    """Scheduler, LLM and generate_greedy against whole-sequence recomputation
    by the plain implementation (float32 for token equality); in bfloat16 the
    tokens do not depend on how the scheduler cuts the work."""
    from lockstep_amd import LLM, FixedChunkPolicy, Request, generate_greedy
    from plain.qwen3_plain import PlainModel

    folder = plain_logits["gen"][name]
    plain = PlainModel(folder)
    vocab = plain.cfg["vocab_size"]
    prompts = [random_tokens(n, vocab, seed=900 + n) for n in ((7, 13, 32) if name == "A" else (1, 9, 17, 40, 64))]
    new = 16 if name == "A" else 24
    want = {f"r{i}": plain.generate_greedy(p, new) for i, p in enumerate(prompts)}

    def requests():
        return [Request(uid=f"r{i}", prompt=p, max_new_tokens=new) for i, p in enumerate(prompts)]

    llm = LLM(folder, dtype="float32", num_pages=64, page_size=page_size, audit=True)
    assert llm.generate(requests()) == want
    assert llm.generate(requests(), policy=FixedChunkPolicy(12)) == want
    ids, step_logits = generate_greedy(llm.model, prompts[-1], new)
    assert ids == want[f"r{len(prompts) - 1}"] and len(step_logits) == new
    assert rel_err(step_logits[0].cpu(), plain.logits(prompts[-1])[-1]) < FP32_TOL

    half = LLM(folder, dtype="bfloat16", num_pages=64, page_size=page_size, audit=True)
    base = half.generate(requests())
    assert half.generate(requests(), policy=FixedChunkPolicy(12)) == base
    half.config = half.config.with_(max_batched_tokens=20)
    assert half.generate(requests(), policy=FixedChunkPolicy(5)) == base
    assert half.generate(requests()[1:2]) == {"r1": base["r1"]}
    # decode steps in bursts on the GPU (no audit, default policy): the same tokens, float32 and bfloat16
    for dtype, tokens in (("float32", want), ("bfloat16", base)):
        fast = LLM(folder, dtype=dtype, num_pages=64, page_size=page_size, audit=False, decode_burst=7)
        scheduler = fast.scheduler()
        for r in requests():
            scheduler.submit(r)
        assert scheduler.run() == tokens
        assert fast.model.graph_replays > 0 and scheduler.counters["decode_step"] == len(prompts) * (new - 1)


def test_sampled_generation_follows_the_plain_sampler(plain_logits):
    """Configuration B's workload: prompts of 1, 9, 17, 40 and 64 tokens as
    mixed portions of 12 beside decoded tokens, temperature 0.8 with a seed per
    request, 24 new tokens each; the sampled tokens equal what the plain
    implementation's sampler draws from the plain logits (float32)."""
    from lockstep_amd import LLM, FixedChunkPolicy, Request
    from plain import qwen3_plain as P

    folder = plain_logits["gen"]["B"]
    plain = P.PlainModel(folder)
    prompts = [random_tokens(n, plain.cfg["vocab_size"], seed=3000 + n) for n in (1, 9, 17, 40, 64)]
    llm = LLM(folder, dtype="float32", num_pages=96, page_size=8, audit=True)
    got = llm.generate([Request(uid=f"s{i}", prompt=p, seed=40 + i, max_new_tokens=24, temperature=0.8, top_p=0.95)
                        for i, p in enumerate(prompts)], policy=FixedChunkPolicy(12))
    for i, p in enumerate(prompts):
        context, want = list(p), []
        for _ in range(24):
            token = P.top_p(plain.logits(context)[-1].float(), 40 + i, f"s{i}", len(context) - 1, 0.95, 0.8)
            want.append(token); context.append(token)
        assert got[f"s{i}"] == want, f"s{i}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_steps_from_a_captured_graph_equal_eager_steps(plain_logits, dtype):
    """Decode steps are replayed from a HIP graph.  Replay it many times, with
    eager work (another request's prompt, a step of another batch size) between
    the replays, and compare every replay with the eager result."""
    from lockstep_amd.engine.batch import StepEntry

    folder, seqs = plain_logits["B"]
    tokens = seqs[333][0]
    other = random_tokens(50, 1000, seed=4)
    eager = load(folder, dtype)
    eager.use_graphs = False
    cache_e = eager.make_cache(num_pages=128, page_size=8)
    want_a = feed(eager, cache_e, "a", tokens, [200] + [1] * 133)
    want_b = feed(eager, cache_e, "b", other, [20] + [1] * 30)

    model = load(folder, dtype)
    assert model.use_graphs
    cache = model.make_cache(num_pages=128, page_size=8)
    cache.open("a"); cache.open("b")
    got_a = [model.step(cache, [StepEntry("a", tokens[:200], list(range(200)))]).cpu()]
    got_b = [model.step(cache, [StepEntry("b", other[:20], list(range(20)))]).cpu()]
    pos_b = 20
    for i in range(200, 333):
        if i % 4 == 0 and pos_b < 50:                # a two-request decode step: another graph shape
            both = model.step(cache, [StepEntry("a", tokens[i:i + 1], [0]), StepEntry("b", other[pos_b:pos_b + 1], [0])])
            got_a.append(both[:1].cpu()); got_b.append(both[1:].cpu())
            pos_b += 1
        else:
            got_a.append(model.step(cache, [StepEntry("a", tokens[i:i + 1], [0])]).cpu())
        if i % 50 == 0:                                # eager work in between
            cache.open(f"x{i}")
            model.step(cache, [StepEntry(f"x{i}", other[:13], [12])])
            cache.close(f"x{i}")
    while pos_b < 50:
        got_b.append(model.step(cache, [StepEntry("b", other[pos_b:pos_b + 1], [0])]).cpu())
        pos_b += 1
    assert model.graph_replays > 100
    assert torch.equal(torch.cat(got_a), want_a)
    assert torch.equal(torch.cat(got_b), want_b)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_large_decode_batch_gives_each_request_the_bits_it_gets_alone(plain_logits, dtype):
    """With many requests in a decode step the attention plan gives each
    (request, kv head) to one workgroup that walks all splits itself; a request
    alone is cut into splits and combined.  Same bits, also from the graph."""
    from lockstep_amd.engine.batch import StepEntry

    folder, _ = plain_logits["B"]
    model = load(folder, dtype)
    n_req, n_decode = 90, 5
    lengths = [3 + (37 * i) % 290 for i in range(n_req)]          # contexts on both sides of a split's edge
    prompts = [random_tokens(n + n_decode, 1000, seed=500 + i) for i, n in enumerate(lengths)]
    cache = model.make_cache(num_pages=sum(-(-(n + n_decode) // 8) for n in lengths) + 4, page_size=8,
                             max_requests=n_req + 1)
    for lo in range(0, n_req, 4):                                  # prompts, four requests a step
        group = range(lo, min(lo + 4, n_req))
        for i in group:
            cache.open(f"r{i}")
        model.step(cache, [StepEntry(f"r{i}", prompts[i][:lengths[i]], []) for i in group])
    together = []
    for k in range(n_decode):
        logits = model.step(cache, [StepEntry(f"r{i}", [prompts[i][lengths[i] + k]], [0]) for i in range(n_req)])
        together.append(logits.cpu())
    assert model.graph_replays >= n_decode - 2
    for i in (0, 7, 8, 33, 60, 89):
        alone = model.make_cache(num_pages=64, page_size=8)
        want = feed(model, alone, "x", prompts[i], [lengths[i]] + [1] * n_decode)[lengths[i]:]
        got = torch.stack([t[i] for t in together])
        assert torch.equal(got, want), f"request {i} (context {lengths[i]})"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_the_first_tokens_of_a_sequence(plain_logits, dtype, name, page_size):
    """A sequence decoded one by one from its very first token (position 0 has one key, the first
    page and the first tile are being filled): right against the plain implementation, and the
    same bits as the whole prompt in one step."""
    folder, seqs = plain_logits[name]
    tokens, want = seqs[40][0], want_for(seqs[40], dtype)
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=16, page_size=page_size, poison_on_free=True)
    whole = feed(model, cache, "whole", tokens, [])
    cache.close("whole")
    stepwise = feed(model, cache, "steps", tokens, [1] * len(tokens))
    cache.close("steps")
    pair = feed(model, cache, "pair", tokens, [2, 1, 1, 2])
    assert rel_err(stepwise[:3], want[:3]) < tol_for(dtype, name)
    assert rel_err(stepwise, want) < tol_for(dtype, name)
    assert torch.equal(stepwise, whole) and torch.equal(pair, whole)
    single, single_want = seqs[1][0], want_for(seqs[1], dtype)
    cache.close("pair")
    assert rel_err(feed(model, cache, "one", single, []), single_want) < tol_for(dtype, name)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_the_device_side_decode_loop_picks_the_tokens_of_stepwise_greedy_decoding(plain_logits, dtype, name, page_size):
    """Decode steps whose greedy picks are fed back on the device (no host in between) give the
    tokens of step-by-step decoding, leave the same cache behind, and can be called again;
    contexts cross pages, tiles and a split of the keys on the way."""
    from lockstep_amd.engine.batch import StepEntry

    folder = plain_logits["gen"][name]
    model = load(folder, dtype)
    vocab = model.spec.vocab_size
    prompts = [random_tokens(n, vocab, seed=900 + n) for n in (3, 120, 250)]
    steps = 140

    def prefill(cache):
        first = []
        for i, p in enumerate(prompts):
            cache.open(f"r{i}")
            logits = model.step(cache, [StepEntry(f"r{i}", p, [len(p) - 1])])
            first.append(int(logits[0].argmax()))
        return first

    ids = [f"r{i}" for i in range(len(prompts))]
    stepwise_cache = model.make_cache(num_pages=200, page_size=page_size)
    tokens = prefill(stepwise_cache)
    model.use_graphs = False                      # the reference: eager steps, picks read by the host
    want = model.decode_greedy(stepwise_cache, ids, tokens, steps)
    model.use_graphs = True
    assert model.graph_replays == 0

    loop_cache = model.make_cache(num_pages=200, page_size=page_size)
    tokens = prefill(loop_cache)
    got_a = model.decode_greedy(loop_cache, ids, tokens, 60)
    got_b = model.decode_greedy(loop_cache, ids, got_a[-1].tolist(), steps - 60)       # the captured loop again
    got = torch.cat([torch.as_tensor(got_a), torch.as_tensor(got_b)])
    assert torch.equal(got, torch.as_tensor(want))
    assert [loop_cache.length(r) for r in ids] == [stepwise_cache.length(r) for r in ids]
    probe = [StepEntry(r, [int(t)], [0]) for r, t in zip(ids, want[-1])]
    assert torch.equal(model.step(loop_cache, probe), model.step(stepwise_cache, probe))
    loop_cache.audit(); stepwise_cache.audit()


def test_a_width_that_is_no_multiple_of_four(tmp_path):
    """hidden_size 66: rows of the residual stream are not 16-byte aligned, so the products add to
    it in their own epilogue instead of leaving slice sums to the next norm.  Whole, cut and decoded
    one by one: the plain implementation's logits (float32), the same bits (both precisions)."""
    from lockstep_amd.config import Qwen3Config
    from lockstep_amd.weights import write_random_model
    from plain.qwen3_plain import PlainModel

    config = Qwen3Config(hidden_size=66, intermediate_size=100, num_hidden_layers=2, num_attention_heads=3,
                         num_key_value_heads=1, head_dim=16, vocab_size=301, rms_norm_eps=1e-6, rope_theta=10000.0,
                         max_position_embeddings=128, tie_word_embeddings=False)
    folder = write_random_model(config, tmp_path / "odd", seed=8, std=0.1, norm_std=0.1)
    tokens = random_tokens(90, 301, seed=4)
    want = PlainModel(folder).logits(tokens)
    for dtype in DTYPES:
        model = load(folder, dtype)
        cache = model.make_cache(num_pages=24, page_size=8, poison_on_free=True)
        whole = feed(model, cache, "w", tokens, [])
        if dtype == "float32":
            assert rel_err(whole, want) < FP32_TOL_SOFT
        else:
            assert rel_err(whole, want) < BF16_TOL
        cache.close("w")
        assert torch.equal(feed(model, cache, "c", tokens, [7, 2, 30, 1, 1, 17]), whole)
        cache.close("c")
        assert torch.equal(feed(model, cache, "d", tokens, [60] + [1] * 30), whole)
        cache.audit()
