"""The engine's sampler against the plain implementation and the vectors the
reference's tests hold (tests/test_sampler.py:15-93)."""

from __future__ import annotations

import torch

from lockstep_amd.sampling import greedy, philox_4x32, top_p, uid_key, uniform
from plain import qwen3_plain as P


def test_philox_and_uniform_match_the_plain_implementation():
    assert philox_4x32((0, 0, 0, 0), (0, 0)) == (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)
    for seed, uid, pos in ((0, "a", 0), (7, "r01", 3), (2 ** 40 + 5, "long-uid", 2 ** 33 + 1)):
        assert uniform(seed, uid, pos) == P.uniform(seed, uid, pos)
    assert uid_key("r01") == int.from_bytes(__import__("hashlib").sha256(b"r01").digest()[:8], "big")
    interleaved = []
    for position in range(4):
        interleaved.append(uniform(0, "a", position))
        uniform(0, "b", position)
    assert interleaved == [uniform(0, "a", p) for p in range(4)]


def test_greedy_and_top_p_vectors():
    assert greedy(torch.tensor([1.0, 5.0, 5.0, 5.0, 2.0])) == 1
    assert top_p(torch.tensor([1.0, 9.0, 9.0, 3.0]), 1, "r", 0, temperature=0.0) == 1
    assert top_p(torch.tensor([0.0, 7.0, 7.0, 1.0]), 3, "r", 0, p=1e-9) == 1
    assert {top_p(torch.tensor([4.0, 4.0, 4.0, 4.0]), s, "r", 0, p=0.5) for s in range(50)} <= {0, 1}
    assert len({top_p(torch.tensor([1.0, 1.0, 1.0, 1.0]), s, "r", 0, p=1.0) for s in range(200)}) == 4


def test_top_p_agrees_with_the_plain_implementation():
    g = torch.Generator().manual_seed(4)
    for trial in range(60):
        row = torch.randn(300, generator=g) * 3
        row[trial % 300] = row[(trial * 7) % 300]            # a tie
        args = dict(seed=trial, uid=f"u{trial % 5}", position=trial * 3, p=[1.0, 0.9, 0.5, 0.05][trial % 4],
                    temperature=[1.0, 0.8, 0.3][trial % 3])
        assert top_p(row, **args) == P.top_p(row, **args)
        assert top_p(row.to(torch.bfloat16), **args) == P.top_p(row.to(torch.bfloat16), **args)
