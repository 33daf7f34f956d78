"""The engine at the layer sizes of real models (one or two layers of them):
head size 128, widths of 1,024 to 5,120, K cut into 4 to 100 slices.  These
sizes take other kernels and other paths inside the kernels than the tiny
configurations do (128 x 128 tiles, the streaming and the walking products,
the cooperative and the wide attention kernel at their full tile sizes), so
the cuttings are compared bit for bit here as well, and the 32-bit path with
the plain implementation."""

from __future__ import annotations

import pytest
import torch

from helpers import BF16_TOL, FP32_TOL_SOFT, feed, random_tokens, rel_err

pytestmark = pytest.mark.gpu

# width, query heads, kv heads, feed-forward width, layers, vocabulary (not a multiple of 16), tied head
SIZES = {
    "0.6b-like": dict(hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                      intermediate_size=3072, num_hidden_layers=2, vocab_size=4099, tie_word_embeddings=True,
                      rms_norm_eps=1e-6, rope_theta=1000000.0, max_position_embeddings=2048),
    "8b-like": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                    intermediate_size=12288, num_hidden_layers=1, vocab_size=5003, tie_word_embeddings=False,
                    rms_norm_eps=1e-6, rope_theta=1000000.0, max_position_embeddings=2048),
    # width 5,120 (K slices of 512), eight query heads a kv head (eight rows a decoded token), a feed-forward
    # width of 25,600 (gate/up over 51,200 columns; the down product over 100 K slices of 256 = 15 of 1,792)
    "32b-like": dict(hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                     intermediate_size=25600, num_hidden_layers=1, vocab_size=5011, tie_word_embeddings=False,
                     rms_norm_eps=1e-6, rope_theta=1000000.0, max_position_embeddings=2048),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """name -> (folder, config); weights as a real checkpoint has them in size (std 0.02), norm
    weights spread around one."""
    from lockstep_amd.config import Qwen3Config
    from lockstep_amd.weights import write_random_model

    out = {}
    for name, raw in SIZES.items():
        config = Qwen3Config.from_dict(raw)
        folder = tmp_path_factory.mktemp(name.replace(".", "_"))
        write_random_model(config, folder, seed=11, std=0.02, norm_std=0.1)
        out[name] = (folder, config)
    return out


def load(folder, dtype):
    from lockstep_amd.engine.model import load_model

    return load_model(folder, dtype=dtype)


@pytest.mark.parametrize("name", list(SIZES))
def test_cuttings_give_the_same_bits_at_real_layer_sizes(models, name):
    """bfloat16: a request whole; most of it in one step and the last 32 tokens one by one; in
    portions of changing size; and the tail decoded beside other requests, from the captured graph."""
    from lockstep_amd.engine.batch import StepEntry

    folder, config = models[name]
    model = load(folder, "bfloat16")
    vocab = config.vocab_size
    n = 620                                                       # three splits, the last tile partly filled
    tokens = random_tokens(n, vocab, seed=1)
    cache = model.make_cache(num_pages=3 * 48 + 8, page_size=16, max_requests=8)
    whole = feed(model, cache, "whole", tokens, [n])
    assert torch.isfinite(whole).all()
    cache.close("whole")
    tail = feed(model, cache, "tail", tokens, [n - 32] + [1] * 32)
    assert torch.equal(tail, whole), "prefix in one step, the last 32 tokens one by one"
    cache.close("tail")
    cut = feed(model, cache, "cut", tokens, [2, 37, 128, 3, 255, 64, 2, 100])
    assert torch.equal(cut, whole), "portions of changing size"
    cache.close("cut")

    # the last 24 tokens beside two other requests that decode too (different lengths), then beside a prompt portion
    others = {"o1": random_tokens(300, vocab, seed=2), "o2": random_tokens(77, vocab, seed=3)}
    for rid, toks in others.items():
        cache.open(rid)
        model.step(cache, [StepEntry(rid, toks[:-30], [])])
    cache.open("mix")
    model.step(cache, [StepEntry("mix", tokens[:n - 24], [])])
    rows = []
    for k in range(24):
        entries = [StepEntry("mix", [tokens[n - 24 + k]], [0])]
        for rid, toks in others.items():
            entries.append(StepEntry(rid, [toks[len(toks) - 30 + k]], []))
        if k == 20:                                               # a prompt portion joins the decode step
            cache.open("late")
            entries.append(StepEntry("late", random_tokens(50, vocab, seed=4), []))
        rows.append(model.step(cache, entries).cpu())
    assert torch.equal(torch.cat(rows), whole[n - 24:]), "decoded beside other requests"
    assert model.graph_replays > 10


@pytest.mark.parametrize("name", list(SIZES))
def test_many_requests_decode_with_the_bits_of_one(models, name):
    """Many requests in a decode step against each of them alone: 40 (three row tiles in the
    products, more than 256 (request, kv head) pairs in attention: one workgroup a pair, norm and
    rotation inside the attention kernel) and 66 (five row tiles, more than 512 pairs: norm and
    rotation as a launch of their own)."""
    from lockstep_amd.engine.batch import StepEntry

    folder, config = models[name]
    model = load(folder, "bfloat16")
    vocab = config.vocab_size
    n_req, n_decode = {"0.6b-like": 66, "8b-like": 40, "32b-like": 64}[name], 3
    lengths = [5 + (61 * i) % 400 for i in range(n_req)]
    prompts = [random_tokens(m + n_decode, vocab, seed=50 + i) for i, m in enumerate(lengths)]
    cache = model.make_cache(num_pages=sum(-(-(m + n_decode) // 16) for m in lengths) + 4, page_size=16,
                             max_requests=n_req + 1)
    for lo in range(0, n_req, 4):
        group = range(lo, min(lo + 4, n_req))
        for i in group:
            cache.open(f"r{i}")
        model.step(cache, [StepEntry(f"r{i}", prompts[i][:lengths[i]], []) for i in group])
    together = [model.step(cache, [StepEntry(f"r{i}", [prompts[i][lengths[i] + k]], [0]) for i in range(n_req)]).cpu()
                for k in range(n_decode)]
    for i in (0, 13, n_req - 1):
        alone = model.make_cache(num_pages=32, page_size=16)
        want = feed(model, alone, "x", prompts[i], [lengths[i]] + [1] * n_decode)[lengths[i]:]
        assert torch.equal(torch.stack([t[i] for t in together]), want), f"request {i} (context {lengths[i]})"


def test_requests_of_very_different_lengths_decode_with_the_bits_of_one(models):
    """Forty requests between 20 and 1,500 tokens in one decode step: there are so many splits that
    the long requests are cut into work items of several splits each (partial results and a fold),
    the short ones are walked whole, and the graph-replayed steps lay every request out for the
    longest; each request has the bits it has alone, eagerly and from the replayed graph."""
    from lockstep_amd.engine.batch import StepEntry

    folder, config = models["0.6b-like"]
    model = load(folder, "bfloat16")
    vocab = config.vocab_size
    n_req, n_decode = 40, 3
    lengths = [20 + (37 * i * i) % 1480 for i in range(n_req)]
    assert max(lengths) > 1300 and min(lengths) < 100
    prompts = [random_tokens(m + n_decode, vocab, seed=150 + i) for i, m in enumerate(lengths)]
    cache = model.make_cache(num_pages=sum(-(-(m + n_decode) // 16) for m in lengths) + 4, page_size=16,
                             max_requests=n_req)
    for i in range(n_req):
        cache.open(f"r{i}")
        model.step(cache, [StepEntry(f"r{i}", prompts[i][:lengths[i]], [])])
    replays = model.graph_replays
    together = [model.step(cache, [StepEntry(f"r{i}", [prompts[i][lengths[i] + k]], [0]) for i in range(n_req)]).cpu()
                for k in range(n_decode)]
    assert model.graph_replays > replays
    # the same step through the lists of a step that is not replayed (a portion of two tokens beside it)
    extra = random_tokens(300, vocab, seed=3)
    cache2 = model.make_cache(num_pages=sum(-(-(m + n_decode) // 16) for m in lengths) + 40, page_size=16,
                              max_requests=n_req + 1)
    for i in range(n_req):
        cache2.open(f"r{i}")
        model.step(cache2, [StepEntry(f"r{i}", prompts[i][:lengths[i]], [])])
    cache2.open("x")
    model.step(cache2, [StepEntry("x", extra[:298], [])])
    mixed = model.step(cache2, [StepEntry(f"r{i}", [prompts[i][lengths[i]]], [0]) for i in range(n_req)]
                       + [StepEntry("x", extra[298:], [1])]).cpu()
    assert torch.equal(mixed[:n_req], together[0])
    longest, shortest = lengths.index(max(lengths)), lengths.index(min(lengths))
    for i in (0, longest, shortest, n_req - 1):
        alone = model.make_cache(num_pages=100, page_size=16)
        want = feed(model, alone, "x", prompts[i], [lengths[i]] + [1] * n_decode)[lengths[i]:]
        assert torch.equal(torch.stack([t[i] for t in together]), want), f"request {i} (context {lengths[i]})"


def test_few_long_requests_are_cut_so_that_every_cu_has_work(tmp_path, monkeypatch):
    """Three requests of some 12,300 tokens in one decode step: walked whole they would be 24 workgroups;
    the planner cuts them into the longest items that still give every CU a set number (the test asks for
    two a CU, which makes items of two splits and so runs the kernel instance that leaves a partial result
    for each split of an item; the default of eight a CU makes items of one split here), the decode loop
    lays the same out for the lengths to come, and each request has the bits it has alone."""
    import lockstep_amd.parts.attention as attention_module
    from lockstep_amd.config import Qwen3Config
    from lockstep_amd.engine.batch import StepEntry
    from lockstep_amd.weights import write_random_model

    config = Qwen3Config.from_dict(dict(SIZES["0.6b-like"], num_hidden_layers=1, max_position_embeddings=16384))
    write_random_model(config, tmp_path, seed=12, std=0.02, norm_std=0.1)
    model = load(tmp_path, "bfloat16")
    vocab = config.vocab_size
    lengths, n_decode = [12300, 12290, 12310], 3
    prompts = [random_tokens(m + n_decode + 8, vocab, seed=170 + i) for i, m in enumerate(lengths)]
    cache = model.make_cache(num_pages=4 * 780, page_size=16, max_requests=4)

    def prefill(rid, tokens):
        cache.open(rid)
        for lo in range(0, len(tokens), 4096):
            part = tokens[lo:lo + 4096]
            logits = model.step(cache, [StepEntry(rid, part, [len(part) - 1])])
        return logits[0]

    for i, m in enumerate(lengths):
        prefill(f"r{i}", prompts[i][:m])
    seen = []
    original = attention_module.plan_attention

    def watching(ctx, *args):
        plan, ints = original(ctx, *args)
        seen.append(plan)
        return plan, ints

    attention_module.plan_attention = watching
    a_cu = attention_module.WORKGROUPS_A_CU
    monkeypatch.setattr(attention_module, "WORKGROUPS_A_CU", 2)
    try:
        together = [model.step(cache, [StepEntry(f"r{i}", [prompts[i][lengths[i] + k]], [0]) for i in range(3)]).cpu()
                    for k in range(n_decode)]
        assert seen and all(p.spans and p.n_combine >= 3 and 8 * p.n_coop >= 512 for p in seen), seen
        # ... and with the default, items of one split: the same bits
        monkeypatch.setattr(attention_module, "WORKGROUPS_A_CU", a_cu)
        cache_b = model.make_cache(num_pages=4 * 780, page_size=16, max_requests=4)
        for i, m in enumerate(lengths):
            cache_b.open(f"r{i}")
            for lo in range(0, m, 4096):
                model.step(cache_b, [StepEntry(f"r{i}", prompts[i][lo:min(lo + 4096, m)], [])])
        del seen[:]
        again = [model.step(cache_b, [StepEntry(f"r{i}", [prompts[i][lengths[i] + k]], [0]) for i in range(3)]).cpu()
                 for k in range(n_decode)]
        assert seen and all(not p.spans and p.single_tile for p in seen), seen
        assert all(torch.equal(a, b) for a, b in zip(together, again))
        del cache_b
        monkeypatch.setattr(attention_module, "WORKGROUPS_A_CU", 2)
    finally:
        attention_module.plan_attention = original
    prefill("alone", prompts[1][:lengths[1]])
    for k in range(n_decode):
        want = model.step(cache, [StepEntry("alone", [prompts[1][lengths[1] + k]], [0])]).cpu()
        assert torch.equal(together[k][1], want[0]), k
    # and through the device-side loop: the greedy continuation of one of three equals its own alone
    for rid in ("r0", "r1", "r2", "alone"):
        cache.close(rid)
    firsts = [int(prefill(f"q{i}", prompts[i][:m]).argmax()) for i, m in enumerate(lengths)]
    picked = model.decode_greedy(cache, ["q0", "q1", "q2"], firsts, 6)
    token = int(prefill("alone", prompts[1][:lengths[1]]).argmax())
    assert token == firsts[1]
    for k in range(6):
        token = int(model.step(cache, [StepEntry("alone", [token], [0])])[0].argmax())
        assert token == int(picked[k][1]), k


@pytest.mark.parametrize("name", list(SIZES))
def test_both_paths_match_plain_at_real_layer_sizes(models, name):
    """float32 against the plain float64 implementation, and bfloat16 within its tolerance: a whole
    prompt and a decoded tail; then the last rows again out of a step of 40 requests (the kernels
    that 17 to 64 rows take) and out of a portion of 200 tokens beside them."""
    from lockstep_amd.engine.batch import StepEntry
    from plain.qwen3_plain import PlainModel

    folder, config = models[name]
    n = 300 if name == "0.6b-like" else 130
    tokens = random_tokens(n, config.vocab_size, seed=9)
    want = PlainModel(folder).logits(tokens)
    others = [random_tokens(3 + (7 * i) % 30, config.vocab_size, seed=200 + i) for i in range(39)]
    for dtype, tol in (("float32", FP32_TOL_SOFT), ("bfloat16", BF16_TOL)):
        model = load(folder, dtype)
        cache = model.make_cache(num_pages=40 + 3 * 40, page_size=16, max_requests=42)
        got = feed(model, cache, "a", tokens, [n - 30] + [1] * 30)
        err = rel_err(got, want)
        print(f"{name} {dtype}: rel err {err:.3e}")
        assert err < tol
        # the last two tokens again, decoded in a step of 40 requests
        cache.close("a")
        for i, toks in enumerate(others):
            cache.open(f"o{i}")
        model.step(cache, [StepEntry(f"o{i}", toks[:-2], []) for i, toks in enumerate(others)])
        cache.open("b")
        model.step(cache, [StepEntry("b", tokens[:n - 2], [])])
        rows = []
        for k in range(2):
            entries = [StepEntry(f"o{i}", [toks[len(toks) - 2 + k]], []) for i, toks in enumerate(others)]
            entries.insert(17, StepEntry("b", [tokens[n - 2 + k]], [0]))
            rows.append(model.step(cache, entries).cpu())
        together = torch.cat(rows)
        assert rel_err(together, want[n - 2:]) < tol
        assert torch.equal(together, got[n - 2:]), "decoded among 40 requests: the bits of the request alone"
        del model, cache
        torch.cuda.empty_cache()


def test_the_device_side_loop_at_real_layer_sizes(models):
    """Greedy tokens from the device-side loop equal those of step-by-step decoding (logits well
    apart are not guaranteed with these weights, so the comparison is between the engine's two ways,
    which share every kernel)."""
    from lockstep_amd.engine.batch import StepEntry

    folder, config = models["0.6b-like"]
    model = load(folder, "bfloat16")
    prompts = {f"r{i}": random_tokens(40 + 90 * i, config.vocab_size, seed=70 + i) for i in range(3)}
    picked = {}
    for way in ("loop", "steps"):
        cache = model.make_cache(num_pages=96, page_size=16, max_requests=4)
        first = []
        for rid, toks in prompts.items():
            cache.open(rid)
            logits = model.step(cache, [StepEntry(rid, toks, [len(toks) - 1])])
            first.append(int(logits[0].argmax()))
        if way == "loop":
            picked[way] = model.decode_greedy(cache, list(prompts), first, 12).tolist()
        else:
            rows, cur = [], first
            for _ in range(12):
                logits = model.step(cache, [StepEntry(rid, [t], [0]) for rid, t in zip(prompts, cur)])
                cur = [int(row.argmax()) for row in logits]
                rows.append(cur)
            picked[way] = rows
    assert picked["loop"] == picked["steps"]


def test_a_captured_decode_loop_survives_a_large_argmax_in_between(models):
    """The arg-max inside the captured loop writes its partial results (this vocabulary has two
    chunks a row) to memory that must still be the loop's when the graph is replayed after an
    arg-max over many more rows."""
    from lockstep_amd.engine.batch import StepEntry

    folder, config = models["0.6b-like"]
    model = load(folder, "bfloat16")
    kernels = model.rt.kernels
    prompts = {f"r{i}": random_tokens(30 + 11 * i, config.vocab_size, seed=90 + i) for i in range(8)}

    def run(disturb: bool):
        cache = model.make_cache(num_pages=64, page_size=16, max_requests=8)
        first = []
        for rid, toks in prompts.items():
            cache.open(rid)
            logits = model.step(cache, [StepEntry(rid, toks, [len(toks) - 1])])
            first.append(int(logits[0].argmax()))
        a = model.decode_greedy(cache, list(prompts), first, 6)
        if disturb:
            for rows in (64, 9000):                 # 9,000 rows of two chunks: beyond the static scratch array
                big = torch.randn(rows, config.vocab_size, device="cuda")
                kernels.argmax(big, torch.empty(rows, dtype=torch.int32, device="cuda"))
                del big
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            filler = torch.full((1 << 22,), -1, dtype=torch.int32, device="cuda")    # takes freed blocks, if any
        replays = model.graph_replays
        b = model.decode_greedy(cache, list(prompts), a[-1].tolist(), 6)
        assert model.graph_replays > replays
        return a.tolist() + b.tolist()

    assert run(disturb=True) == run(disturb=False)


@pytest.mark.parametrize("name", list(SIZES))
def test_random_mixes_at_real_layer_sizes(models, name):
    """Random mixes of one to five requests (lengths on both sides of the tile, split and row-block
    edges), cut into portions of changing size beside decoded tokens, with a pool so small that
    pages are used again: every position has the bits of its request run whole and alone."""
    import random

    from helpers import make_mixed_trace
    from lockstep_amd.engine.batch import StepEntry

    folder, config = models[name]
    model = load(folder, "bfloat16")
    rng = random.Random(7)
    lengths = [2, 3, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 640, 1000, 1300]
    for it in range(25):
        n_req = rng.randint(1, 5)
        requests = {f"q{it}_{i}": random_tokens(rng.choice(lengths) + rng.randint(0, 40), config.vocab_size,
                                                seed=it * 10 + i) for i in range(n_req)}
        alone = model.make_cache(num_pages=96, page_size=16, max_requests=2)
        want = {}
        for rid, toks in requests.items():
            want[rid] = feed(model, alone, rid, toks, [len(toks)])
            alone.close(rid)
        steps = make_mixed_trace(requests, seed=it, max_live=4, decode_tail=rng.choice([0, 1, 8, 33]),
                                 max_portion=rng.choice([19, 64, 130, 700]))
        pages = [-(-len(t) // 16) for t in requests.values()]
        cache = model.make_cache(num_pages=max(sum(pages) * 2 // 3, max(pages) * min(4, n_req)) + 4, page_size=16,
                                 max_requests=5)
        got = {rid: [] for rid in requests}
        for st in steps:
            for e in st["entries"]:
                if e["id"] not in cache.requests:
                    cache.open(e["id"])
            logits = model.step(cache, [StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]]).cpu()
            at = 0
            for e in st["entries"]:
                got[e["id"]].append(logits[at:at + len(e["want"])])
                at += len(e["want"])
            for rid in st["end"]:
                cache.close(rid)
        for rid in requests:
            assert torch.equal(torch.cat(got[rid]), want[rid]), f"mix {it}, request {rid} ({len(requests[rid])} tokens)"
