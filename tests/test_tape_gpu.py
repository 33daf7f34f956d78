"""Layers that are alike repeat the launches of the second of them instead of running their
Python again (engine/tape.py): the logits are the same bits as with every layer run in Python,
the check mode agrees launch by launch, and it notices a part that says ``repeatable`` although
its launches depend on the layer in another way than through its tensors' addresses."""

from __future__ import annotations

import pytest
import torch

from helpers import FP32_TOL_SOFT, make_mixed_trace, random_tokens, rel_err, replay_in_process

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def deep_dirs(tmp_path_factory):
    from conftest import make_model_dir

    return {name: make_model_dir(tmp_path_factory, name, sharpen=1.5, overrides={"num_hidden_layers": 6})
            for name in ("A", "B")}


def load(folder, dtype, **flags):
    from lockstep_amd.engine.model import load_model

    model = load_model(folder, dtype=dtype)
    for name, value in flags.items():
        assert hasattr(model, name)
        setattr(model, name, value)
    return model


def trace_for(vocab):
    requests = {f"r{i}": random_tokens(n, vocab, seed=70 + i) for i, n in enumerate((45, 3, 130, 21, 77, 9))}
    return requests, make_mixed_trace(requests, seed=5, max_live=4, decode_tail=12)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page_size", [("A", 16), ("B", 8)])
def test_repeated_launches_give_the_bits_of_every_layer_run_in_python(deep_dirs, dtype, name, page_size):
    folder = deep_dirs[name]
    taped, checked = load(folder, dtype, use_tapes=True, verify_tapes=False), load(folder, dtype, verify_tapes=True)
    plainly = load(folder, dtype, use_tapes=False)
    requests, steps = trace_for(taped.spec.vocab_size)
    results = []
    for model in (taped, checked, plainly):
        cache = model.make_cache(num_pages=60, page_size=page_size, max_requests=4, poison_on_free=True)
        results.append(replay_in_process(model, cache, steps))
    # four of six layers a step are repeated (three in the very first step, whose third layer runs in Python
    # once more to be compared with the tape); graph-replayed decode steps launch nothing from the host
    assert taped.layers_repeated >= 4 * (len(steps) - taped.graph_replays) - 1 > 0 and taped.tapes_refused == 0
    assert checked.layers_repeated == 0 and plainly.layers_repeated == 0
    for rid in requests:
        assert torch.equal(results[0][rid], results[2][rid]), rid
        assert torch.equal(results[1][rid], results[2][rid]), rid
    if dtype == "float32":
        from plain.qwen3_plain import PlainModel

        plain = PlainModel(folder)
        for rid in ("r0", "r2"):
            assert rel_err(results[0][rid], plain.logits(requests[rid])) < FP32_TOL_SOFT, rid


def test_the_decode_loop_and_captured_steps_repeat_layers_too(deep_dirs):
    from lockstep_amd.engine.batch import StepEntry

    tokens = {}
    for flags in ({}, {"use_tapes": False}):
        model = load(deep_dirs["B"], "bfloat16", **(flags or {"use_tapes": True, "verify_tapes": False}))
        cache = model.make_cache(num_pages=64, page_size=8, max_requests=3)
        firsts = []
        for i, n in enumerate((5, 33, 18)):
            cache.open(i)
            logits = model.step(cache, [StepEntry(i, random_tokens(n, 1000, seed=90 + i), [n - 1])])
            firsts.append(int(logits[0].argmax()))
        tokens[bool(flags)] = model.decode_greedy(cache, [0, 1, 2], firsts, 24)
        if not flags:
            assert model.graph_replays > 0 and model.layers_repeated >= 5 * 4 - 1   # three prompts, first step, capture
    assert (tokens[False] == tokens[True]).all()


def test_the_check_mode_notices_a_number_that_differs_from_layer_to_layer(deep_dirs):
    """A part may hold per-layer numbers only in its specification (then the layers are of
    different kinds) or in device tensors; one that is set behind the specification's back makes
    the repeated launches wrong, and the check mode says which launch."""
    from lockstep_amd.engine.batch import StepEntry

    model = load(deep_dirs["A"], "float32", verify_tapes=True)
    model.layers[4].mixer_norm.eps = 2e-3
    cache = model.make_cache(num_pages=8, page_size=16, max_requests=1)
    cache.open("r")
    with pytest.raises(RuntimeError, match="layer run 4: launch 0 .* differs from the tape"):
        model.step(cache, [StepEntry("r", random_tokens(20, 512, seed=1), [19])])


def test_a_tensor_that_the_walk_does_not_find_switches_the_repetition_off(deep_dirs):
    """A part that says ``repeatable`` but keeps a per-layer tensor where the walk over its attributes
    does not look: the first layer a tape could stand for runs in Python as well, its launches name
    another tensor than the tape would, and the layers of that kind run in Python from then on --
    with the right logits, where repeating the tape would have run every layer on one layer's weight."""
    import types

    from lockstep_amd.parts.norm import RMSNorm

    class HiddenWeight(RMSNorm):
        weight = property(lambda self: self.box.tensor, lambda self, value: None)

    def hide(model):
        for layer in model.layers:
            norm = layer.mixer_norm
            box = types.SimpleNamespace(tensor=norm.__dict__.pop("weight"))
            norm.__class__, norm.box = HiddenWeight, box
        return model

    folder = deep_dirs["B"]
    hidden = hide(load(folder, "float32", use_tapes=True, verify_tapes=False))
    plainly = load(folder, "float32", use_tapes=False)
    requests, steps = trace_for(hidden.spec.vocab_size)
    results = []
    for model in (hidden, plainly):
        cache = model.make_cache(num_pages=60, page_size=8, max_requests=4, poison_on_free=True)
        results.append(replay_in_process(model, cache, steps))
    assert hidden.tapes_refused == 1 and hidden.layers_repeated == 0
    for rid in requests:
        assert torch.equal(results[0][rid], results[1][rid]), rid
    # under the check mode the same model raises, and says where
    checked = hide(load(folder, "float32", verify_tapes=True))
    cache = checked.make_cache(num_pages=8, page_size=8, max_requests=1)
    cache.open("r")
    from lockstep_amd.engine.batch import StepEntry

    with pytest.raises(RuntimeError, match="layer run 2: launch 0 .* differs from the tape"):
        checked.step(cache, [StepEntry("r", random_tokens(20, 1000, seed=1), [19])])


def test_launches_from_a_list_give_the_bits_of_launches_one_by_one(deep_dirs):
    """Repeated layers go to the library as one list of words (``ls_run_list``) or launch by launch
    from Python: the same logits, bit for bit, and the list really is what ran."""
    folder = deep_dirs["A"]
    listed = load(folder, "bfloat16", use_tapes=True, verify_tapes=False, list_launches=True)
    one_by_one = load(folder, "bfloat16", use_tapes=True, verify_tapes=False, list_launches=False)
    requests, steps = trace_for(listed.spec.vocab_size)
    calls = []
    kernels = listed.rt.kernels
    run_list = kernels.run_list
    kernels.run_list = lambda words, *a, **k: (calls.append(int(words.size)), run_list(words, *a, **k))[1]
    try:
        results = []
        for model in (listed, one_by_one):
            cache = model.make_cache(num_pages=60, page_size=16, max_requests=4, poison_on_free=True)
            results.append(replay_in_process(model, cache, steps))
    finally:
        kernels.run_list = run_list
    assert calls and listed.layers_repeated == one_by_one.layers_repeated > 0
    for rid in requests:
        assert torch.equal(results[0][rid], results[1][rid]), rid


def test_a_list_of_launches_that_is_wrong_is_refused_with_its_reason():
    """The runner checks a record before it calls: a record that runs past the list's end, an entry point
    that is not listed, and a call with the wrong number of arguments each end the run with a message."""
    import ctypes

    import numpy as np

    from lockstep_amd.ops import KernelError, kernels

    k = kernels()
    callee, index, lib = k.listed(k.core, k.core.ls_rmsnorm)
    assert k.listed(k.core, k.core.ls_argmax) is None                      # not among the listed entry points
    with pytest.raises(KernelError, match="runs past the end"):
        k.run_list(np.asarray([callee, index, 40, 1, 2], dtype=np.int64))
    with pytest.raises(KernelError, match="ls_rmsnorm takes 11 arguments, the list brings 2"):
        k.run_list(np.asarray([callee, index, 2, 0, 0], dtype=np.int64))
    with pytest.raises(KernelError, match="no listed entry point 99"):
        k.run_list(np.asarray([callee, 99, 0], dtype=np.int64))
    assert ctypes.cast(lib.ls_call_listed, ctypes.c_void_p).value == callee
