"""The scheduler's mechanisms together, on random workloads with fixed seeds: prefix cache x decode
bursts x token budget x lazy reservation x sampled requests x end-of-sequence ids, in pools so small
that requests wait, are preempted and evict indexed pages.  Every request's tokens, and (where the
run keeps them) the logit rows they were picked from, equal those of the request served alone; the
first difference stops the test and names the workload.  At the end the counters of all workloads
together must show that every mechanism ran, a burst over adopted pages among them (reference
harness/mr/state.py:174-216: random states of the scheduler, each relation with its vacuity guard;
harness/mr/relations.py: outputs do not depend on cohabitants, cache hits or preemption).

The short form of longer runs of the same generator; bounded in time, not in what it asserts."""

from __future__ import annotations

import random
import time
from collections import Counter

import pytest
import torch

from helpers import random_tokens

pytestmark = pytest.mark.gpu

PAGE = 16
CONFIG = dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64, intermediate_size=768,
              num_hidden_layers=2, vocab_size=2003, tie_word_embeddings=True, rms_norm_eps=1e-6, rope_theta=1e6,
              max_position_embeddings=4096)
WORKLOADS = 160            # some ten seconds on an MI355X
TIME_LIMIT = 60.0          # seconds after which no further workload is started ...
MIN_WORKLOADS = 40         # ... unless fewer than this many have run


@pytest.fixture(scope="module")
def model():
    from lockstep_amd.config import Qwen3Config
    from lockstep_amd.engine.model import model_from_tensors
    from lockstep_amd.weights import random_tensors

    config = Qwen3Config.from_dict(CONFIG)
    return model_from_tensors(config, random_tensors(config, 5, 0.3, 0.1, torch.bfloat16), dtype="bfloat16")


def serve_alone(model, fields: dict):
    """The request by itself in a roomy pool, without end-of-sequence ids: tokens and their logit rows."""
    from lockstep_amd import Request, Scheduler

    pages = -(-(len(fields["prompt"]) + fields["max_new_tokens"]) // PAGE) + 1
    s = Scheduler(model, num_blocks=pages, block_size=PAGE, keep_logits=True, audit=False, max_requests=1)
    s.submit(Request(**fields))
    tokens = s.run()[fields["uid"]]
    return tokens, torch.stack(s.emitted_logits[fields["uid"]])


def cut_at_eos(tokens, eos):
    for i, t in enumerate(tokens):
        if t in eos:
            return tokens[: i + 1]
    return tokens


def draw_workload(rng: random.Random, number: int, vocab: int):
    """Two waves of requests; the second shares beginnings with the first (whole pages of them are in
    the index by then) and among itself."""
    shared = random_tokens(rng.choice([PAGE, 3 * PAGE, 8 * PAGE + 5, 17 * PAGE]), vocab, seed=1000 + number)
    waves, serial = [], 0
    for wave in range(2):
        requests = []
        for _ in range(rng.randint(2, 5)):
            own = random_tokens(rng.choice([1, 5, 30, 100, 260]) + rng.randint(0, 9), vocab, seed=number * 100 + serial)
            lead = rng.random()
            prompt = (shared + own if lead < 0.45 else list(shared) if lead < 0.55 and wave else
                      shared[: 2 * PAGE] + own if lead < 0.7 else own)
            sampled = rng.random() < 0.4
            requests.append(dict(uid=f"w{number}r{serial}", prompt=prompt, seed=number * 7 + serial,
                                 max_new_tokens=rng.choice([1, 4, 12, 30]),
                                 temperature=rng.choice([0.6, 0.9, 1.4]) if sampled else 0.0,
                                 top_p=rng.choice([1.0, 0.9, 0.5]) if sampled else 1.0))
            serial += 1
        waves.append(requests)
    return waves


def draw_options(rng: random.Random, need: list):
    """How the workload is served.  Runs that keep logits or audit take single steps; the others may
    burst, so both kinds are drawn."""
    lazy = rng.random() < 0.4
    quiet = rng.random() < 0.5                       # no audit, no kept logits: bursts possible
    options = dict(reserve="lazy" if lazy else "full", enable_prefix_cache=rng.random() < 0.7,
                   max_batched_tokens=rng.choice([None, None, 24, 100, 512]),
                   decode_burst=rng.choice([4, 32]) if quiet else rng.choice([1, 8]),
                   audit=not quiet, keep_logits=not quiet and rng.random() < 0.8)
    pool = max(need) + rng.randint(0, sum(need) // 2 if rng.random() < 0.6 else sum(need))
    slots = rng.choice([2, 3, 8])
    if rng.random() < 0.3:
        from lockstep_amd.engine.policy import FixedChunkPolicy

        options["policy"] = FixedChunkPolicy(rng.choice([7, 48, 130]), max_running=slots)
    elif lazy:
        from lockstep_amd.engine.policy import Policy

        # admit on what the prompt needs now; that the pool is too small for everyone's end is found out later
        options["policy"] = Policy(max_running=slots, admission=lambda view, uid, pages, slots=slots: len(
            view.running) < slots and view.obtainable_pages >= min(pages, 3))
    return options, pool + 1, slots


def test_random_workloads_give_every_request_the_tokens_and_logits_it_has_alone(model):
    from lockstep_amd import Request, Scheduler

    vocab = model.spec.vocab_size
    rng = random.Random(20260)
    totals: Counter = Counter()
    started = time.time()
    workloads = tokens_checked = rows_checked = bursts_seen = 0
    while workloads < MIN_WORKLOADS or (time.time() - started < TIME_LIMIT and workloads < WORKLOADS):
        workloads += 1
        waves = draw_workload(rng, workloads, vocab)
        everyone = [r for wave in waves for r in wave]
        alone = {r["uid"]: serve_alone(model, r) for r in everyone}
        # end-of-sequence ids out of the requests' own continuations, so that some stop early
        eos = set()
        if rng.random() < 0.5:
            for r in rng.sample(everyone, k=min(2, len(everyone))):
                tokens = alone[r["uid"]][0]
                eos.add(tokens[rng.randrange(len(tokens))])
        need = [-(-(len(r["prompt"]) + r["max_new_tokens"]) // PAGE) for r in everyone]
        options, pool, slots = draw_options(rng, need)
        what = f"workload {workloads}: {options}, pool {pool}, slots {slots}, eos {sorted(eos)}"
        cache = model.make_cache(num_pages=pool, page_size=PAGE, max_requests=slots, poison_on_free=True)
        replays = model.graph_replays
        s = Scheduler(model, num_blocks=pool, block_size=PAGE, cache=cache, eos_token_ids=eos, **options)
        got = {}
        for wave in waves:
            for r in wave:
                s.submit(Request(**r))
            got.update(s.run())
        for r in everyone:
            tokens, rows = alone[r["uid"]]
            want = cut_at_eos(tokens, eos)
            assert got[r["uid"]] == want, f"{what}: tokens of {r['uid']} ({len(r['prompt'])} prompt tokens)"
            tokens_checked += len(want)
            if options["keep_logits"]:
                kept = torch.stack(s.emitted_logits[r["uid"]])
                assert torch.equal(kept, rows[: len(want)]), f"{what}: logits of {r['uid']}"
                rows_checked += len(want)
        cache.audit()
        assert cache.free_slots == cache.max_requests, what
        if s.prefix is None:
            assert cache.free_pages == [pool], what
        if s.counters["decode_burst"]:
            assert model.graph_replays > replays, what
            bursts_seen += 1
        totals.update(s.counters.counts)
    print(f"{workloads} workloads in {time.time() - started:.0f} s: {tokens_checked} tokens and {rows_checked} "
          f"logit rows equal; {bursts_seen} workloads with bursts; counters {dict(totals)}")
    from lockstep_amd.engine.audit import Counters

    seen = Counters()
    seen.counts.update(totals)
    seen.require_fired(
        "admit", "admit_refused", "resume", "prefill_chunk", "prefill_complete", "decode_step", "budget_deferred",
        "chunk_boundary_mid_block", "chunk_boundary_on_block", "chunk_boundary_mid_split", "attention_multi_split",
        "attention_single_split", "preempt_for_pages", "cache_hit", "cache_miss", "cache_insert",
        "cache_full_prompt_trimmed", "eviction_taken", "finish_eos", "finish_limit", "decode_burst",
        "burst_on_shared_prefix", "preempt_depth_2", "preempt_depth_3_plus")
    assert rows_checked > 1000 and tokens_checked > 3000
