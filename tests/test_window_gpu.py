"""A toy architecture with a sliding window in one of its layers, registered from here, run
through the engine's own step function: the window logic of the step's work lists (first split,
first row block, the fixed-shape lists of graph-replayed decode steps that start at split 0 over
pages already given back) together with the cache manager handing pages back as the window
passes them.  Page size 8, a window of 150 keys (it crosses page, tile and split edges), freed
pages poisoned, and a pool so small that a second request takes the pages the first one released.
The weights are made so that attention is peaked: a key wrongly seen or wrongly dropped at the
window's edge changes the logits far beyond rounding."""

from __future__ import annotations

from dataclasses import dataclass

import pytest
import torch

from helpers import BF16_STORED_TOL_WINDOW_TOY, FP32_TOL, feed, random_tokens, rel_err
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu

WINDOW = 150
HIDDEN, HEADS, KV_HEADS, HEAD_DIM, VOCAB = 48, 4, 2, 16, 120


def _register():
    from lockstep_amd.config import (LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry,
                                     register_architecture)

    @register_architecture
    @dataclass(frozen=True)
    class WindowToy(ModelConfig):
        window: int
        architecture_names = ("toy-window",)

        def model_spec(self):
            h = HIDDEN
            norm = PartSpec("rmsnorm", {"size": h, "eps": 1e-5})
            ff = PartSpec("gated_mlp", {"hidden_size": h, "intermediate_size": 2 * h, "activation": "silu"})
            arr = PartSpec("prenorm_residual", {"mixer_prefix": "mixer", "feed_forward_prefix": "ff",
                                                "mixer_norm_name": "norm1", "feed_forward_norm_name": "norm2"})

            def attention(window):
                return PartSpec("attention", {
                    "hidden_size": h, "num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
                    "qk_norm": PartSpec("rmsnorm", {"size": HEAD_DIM, "eps": 1e-5}),
                    "position": PartSpec("rope_half", {"rotary_dim": HEAD_DIM, "theta": 10000.0}),
                    "window": window, "bias": False, "scale": HEAD_DIM ** -0.5})

            layers = (LayerSpec("layers.0", arr, attention(self.window), ff, norm, norm),
                      LayerSpec("layers.1", arr, attention(None), ff, norm, norm),
                      LayerSpec("layers.2", arr, attention(self.window), ff, norm, norm))
            return ModelSpec(
                hidden_size=h, vocab_size=VOCAB,
                embedding=PartSpec("token_embedding", {"name": "embed.weight", "vocab_size": VOCAB, "hidden_size": h}),
                layers=layers, schedule=tuple(ScheduleEntry(i, i) for i in range(3)),
                final_norm=PartSpec("rmsnorm", {"size": h, "eps": 1e-5, "name": "final_norm.weight"}),
                head=PartSpec("linear_head", {"name": "head.weight", "tied_to": None, "vocab_size": VOCAB,
                                              "hidden_size": h}))

    return WindowToy


def plain_logits(w, tokens, window, store=None):
    keep = store or (lambda x: x)
    t = len(tokens)
    positions = torch.arange(t)
    cfg = {"num_attention_heads": HEADS, "num_key_value_heads": KV_HEADS, "head_dim": HEAD_DIM,
           "rms_norm_eps": 1e-5, "rope_theta": 10000.0}
    h = w["embed.weight"][torch.tensor(tokens)]
    for layer in range(3):
        p = f"layers.{layer}"
        x = keep(P.rmsnorm(h, w[f"{p}.norm1.weight"], 1e-5))
        attn_cfg = dict(cfg)
        names = {f"a.{k}": w[f"{p}.mixer.{k}"] for k in ("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight",
                                                          "q_norm.weight", "k_norm.weight")}
        h = h + P.attention_block(attn_cfg, names, "a", x, positions, store, window=None if layer == 1 else window)
        h = h + P.mlp_block(w, f"{p}.ff", keep(P.rmsnorm(h, w[f"{p}.norm2.weight"], 1e-5)), store)
    return P.linear(keep(P.rmsnorm(h, w["final_norm.weight"], 1e-5)), w["head.weight"])


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from lockstep_amd.config import unregister_architecture
    from lockstep_amd.weights import random_tensors, save_file
    import json

    WindowToy = _register()
    cfg = WindowToy(window=WINDOW)
    folder = tmp_path_factory.mktemp("toy_window")
    tensors = random_tensors(cfg, seed=3, std=0.2, norm_std=0.1)
    for name in tensors:                         # peaked attention: large per-head norm weights
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            tensors[name] = (tensors[name].float() * 1.5).to(torch.bfloat16)
    (folder / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file(tensors, folder / "model.safetensors")
    w = {k: v.double() for k, v in tensors.items()}
    tokens = random_tokens(700, VOCAB, seed=9)          # three splits of 256 keys, the window inside and across them
    yield folder, w, tokens, {"float32": plain_logits(w, tokens, WINDOW),
                              "bfloat16": plain_logits(w, tokens, WINDOW, store=P.bf16)}
    unregister_architecture(WindowToy)


def test_the_window_matters_in_the_plain_forward(toy):
    _, w, tokens, wants = toy
    want = wants["float32"]
    full = plain_logits(w, tokens, None)
    assert rel_err(full[:WINDOW], want[:WINDOW]) < 1e-12          # below the window nothing is dropped
    assert rel_err(full[WINDOW + 20:], want[WINDOW + 20:]) > 1e-2  # beyond it the dropped keys show
    off_by_one = plain_logits(w, tokens, WINDOW + 1)
    shift = rel_err(off_by_one[WINDOW:], want[WINDOW:])
    print(f"a window one key too wide moves the plain logits by {shift:.2e}")
    assert shift > 3 * BF16_STORED_TOL_WINDOW_TOY                             # a window one key too wide shows as well


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windowed_layers_through_the_step_function(toy, dtype):
    from lockstep_amd.engine.batch import StepEntry
    from lockstep_amd.engine.model import load_model

    folder, w, tokens, wants = toy
    want = wants[dtype]
    model = load_model(folder, dtype=dtype)
    units = model.cache_unit_specs()
    assert [u.window for u in units] == [WINDOW, None, WINDOW]
    n = len(tokens)

    def cache_for(window_pages):
        cache = model.make_cache(num_pages=[window_pages if g == 0 else 200 for g in range(2)], page_size=8,
                                 max_requests=3, max_tokens_per_request=800, poison_on_free=True)
        assert [g.spec.window for g in cache.groups] == [WINDOW, None]
        return cache

    # whole, as one step: the windowed group needs every page of the prompt at once
    cache = cache_for(100)
    whole = feed(model, cache, "w", tokens, [])
    err = rel_err(whole, want)
    print(f"windowed toy, {dtype}: rel err of the whole prompt against plain {err:.3e}")
    # the bfloat16 path against the plain forward that stores in bfloat16 where the engine does; a window
    # one key too wide moves the plain logits by more than a tenth (test above)
    assert err < (FP32_TOL if dtype == "float32" else BF16_STORED_TOL_WINDOW_TOY)
    cache.close("w")
    cache.audit()

    # in portions of changing size with a windowed pool of 48 pages (384 keys): pages behind the window
    # go back while the request runs, are poisoned, and are taken again by the request itself
    cache = cache_for(48)
    cuts = [100, 37, 2, 64, 130, 3, 8, 150, 17]
    cut = feed(model, cache, "c", tokens, cuts)
    assert torch.equal(cut, whole)
    assert cache.groups[0].pool.taken_total > 48 and cache.groups[0].pool.freed_total > 0
    assert cache.request_pages("c", 0)[0] == -1 and cache.request_pages("c", 1)[0] >= 0
    cache.close("c")

    # most of it in portions, then the last 60 tokens one by one beside another request's decoded tokens:
    # those steps replay a captured graph whose work lists start at split 0, over pages given back
    cache = cache_for(100)
    head = n - 60
    feed(model, cache, "d", tokens[:head], [200, 200], want_all=False)
    other = random_tokens(300, VOCAB, seed=10)
    other_alone = feed(model, cache_for(100), "o", other, [])
    cache.open("o")
    model.step(cache, [StepEntry("o", other[:240], [])])
    replays = model.graph_replays
    rows_d, rows_o = [], []
    for i in range(60):
        logits = model.step(cache, [StepEntry("d", [tokens[head + i]], [0]), StepEntry("o", [other[240 + i]], [0])])
        rows_d.append(logits[0].cpu()); rows_o.append(logits[1].cpu())
        cache.audit()
    assert model.graph_replays - replays >= 50
    assert torch.equal(torch.stack(rows_d), whole[head:])
    assert torch.equal(torch.stack(rows_o), other_alone[240:300])
    # the device-side loop over the same layout: greedy tokens equal step-by-step greedy decoding
    cache.close("d"); cache.close("o")
    first = {}
    picked = {}
    for way in ("loop", "steps"):
        cache = cache_for(64)
        cache.open("g")
        logits = model.step(cache, [StepEntry("g", tokens[:400], [399])])
        cur = [int(logits[0].argmax())]
        if way == "loop":
            picked[way] = model.decode_greedy(cache, ["g"], cur, 30)[:, 0].tolist()
        else:
            got = []
            for _ in range(30):
                logits = model.step(cache, [StepEntry("g", cur, [0])])
                cur = [int(logits[0].argmax())]
                got.append(cur[0])
            picked[way] = got
        cache.audit()
    assert picked["loop"] == picked["steps"]
