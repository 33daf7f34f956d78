"""The engine against the plain implementation, under every way of cutting
the work, in float32 and in bfloat16, on the two tiny configurations."""

from __future__ import annotations

import pytest
import torch

from helpers import BF16_TOL, FP32_TOL, feed, random_tokens, rel_err

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
TOL = {"float32": FP32_TOL, "bfloat16": BF16_TOL}


@pytest.fixture(scope="module")
def plain_logits(tiny_a_dir, tiny_b_dir):
    """Plain float64 logits of the test sequences, computed once."""
    from plain.qwen3_plain import PlainModel

    out = {}
    for name, folder in (("A", tiny_a_dir), ("B", tiny_b_dir)):
        plain = PlainModel(folder)
        vocab = plain.cfg["vocab_size"]
        seqs = {n: random_tokens(n, vocab, seed=100 + n) for n in (1, 7, 40, 333)}
        out[name] = (folder, {n: (t, plain.logits(t)) for n, t in seqs.items()})
    return out


def load(folder, dtype):
    from lockstep_amd.engine.model import load_model

    return load_model(folder, dtype=dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_whole_prompts_match_plain(plain_logits, dtype, name, page_size):
    folder, seqs = plain_logits[name]
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=64, page_size=page_size, poison_on_free=True)
    for n, (tokens, want) in seqs.items():
        got = feed(model, cache, f"r{n}", tokens, [])
        err = rel_err(got, want)
        print(f"{name} {dtype} whole n={n}: rel err {err:.3e}")
        assert err < TOL[dtype], f"n={n}"
        cache.close(f"r{n}")
    cache.audit()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_cuttings_give_the_same_bits(plain_logits, dtype, name, page_size):
    """Whole; most in one step and the last 32 one by one; portions of changing
    size down to two tokens; token by token: bitwise equal logits."""
    folder, seqs = plain_logits[name]
    model = load(folder, dtype)
    cache = model.make_cache(num_pages=64, page_size=page_size, poison_on_free=True)
    tokens, want = seqs[333]
    whole = feed(model, cache, "whole", tokens, [])
    cache.close("whole")
    assert rel_err(whole, want) < TOL[dtype]
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
