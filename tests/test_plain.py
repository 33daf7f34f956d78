"""Pins for the plain implementation beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine,
and invariants -- each chosen so that a plausible mistake fails it."""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

from plain import qwen3_plain as P

torch.manual_seed(0)


def test_rmsnorm_equals_the_library_routine():
    x = torch.randn(5, 96, dtype=torch.float64)
    w = 1 + 0.1 * torch.randn(96, dtype=torch.float64)
    assert torch.allclose(P.rmsnorm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), atol=1e-12)


def test_rmsnorm_with_unit_weight_has_unit_mean_square_and_ignores_scale():
    x = torch.randn(3, 64, dtype=torch.float64) * 7
    y = P.rmsnorm(x, torch.ones(64, dtype=torch.float64), 1e-6)
    assert torch.allclose((y * y).mean(-1), torch.ones(3, dtype=torch.float64), atol=1e-6)
    assert torch.allclose(P.rmsnorm(3 * x, torch.ones(64, dtype=torch.float64), 1e-6), y, atol=1e-6)


def test_rope_position_zero_is_the_identity_and_pairs_are_half_apart():
    x = torch.randn(1, 2, 8, dtype=torch.float64)
    cos, sin = P.rope_tables(8, 10000.0, torch.tensor([0]))
    assert torch.equal(P.apply_rope(x, cos, sin), x)
    # rotate position 1: the pair of dim 0 is dim 4 (not dim 1), angle 1 radian for the first pair
    cos, sin = P.rope_tables(8, 10000.0, torch.tensor([1]))
    e0 = torch.zeros(1, 1, 8, dtype=torch.float64)
    e0[0, 0, 0] = 1.0
    out = P.apply_rope(e0, cos, sin)[0, 0]
    assert out[0] == pytest.approx(math.cos(1.0)) and out[4] == pytest.approx(math.sin(1.0))
    assert out[1] == 0 and out[5] == 0
    # the last pair turns by theta^(-2*3/8)
    e3 = torch.zeros(1, 1, 8, dtype=torch.float64)
    e3[0, 0, 7] = 1.0
    out = P.apply_rope(e3, cos, sin)[0, 0]
    ang = 10000.0 ** (-6 / 8)
    assert out[3] == pytest.approx(-math.sin(ang)) and out[7] == pytest.approx(math.cos(ang))


def test_rope_keeps_pair_norms_and_scores_depend_on_distance_only():
    d = 32
    q = torch.randn(1, 1, d, dtype=torch.float64)
    k = torch.randn(1, 1, d, dtype=torch.float64)

    def score(m, n):
        cq, sq = P.rope_tables(d, 1e6, torch.tensor([m]))
        ck, sk = P.rope_tables(d, 1e6, torch.tensor([n]))
        return float((P.apply_rope(q, cq, sq) * P.apply_rope(k, ck, sk)).sum())

    assert score(17, 5) == pytest.approx(score(112, 100), abs=1e-9)
    assert score(17, 5) != pytest.approx(score(17, 6), abs=1e-6)
    cos, sin = P.rope_tables(d, 1e6, torch.tensor([9]))
    r = P.apply_rope(q, cos, sin)
    half = d // 2
    assert torch.allclose(r[..., :half] ** 2 + r[..., half:] ** 2, q[..., :half] ** 2 + q[..., half:] ** 2)


def test_attention_equals_library_attention_for_whole_sequences():
    t, nq, nkv, d = 19, 6, 3, 16
    q = torch.randn(t, nq, d, dtype=torch.float64)
    k = torch.randn(t, nkv, d, dtype=torch.float64)
    v = torch.randn(t, nkv, d, dtype=torch.float64)
    got = P.causal_attention(q, k, v)
    g = nq // nkv
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat_interleave(g, 1).transpose(0, 1)[None],
        v.repeat_interleave(g, 1).transpose(0, 1)[None], is_causal=True, scale=d ** -0.5)[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-12)
    # a tiled GQA map (h % nkv) instead of h // group would differ
    wrong = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat(1, g, 1).transpose(0, 1)[None],
        v.repeat(1, g, 1).transpose(0, 1)[None], is_causal=True, scale=d ** -0.5)[0].transpose(0, 1)
    assert not torch.allclose(got, wrong, atol=1e-3)


def test_attention_special_cases():
    t, nq, nkv, d = 9, 2, 1, 8
    q = torch.randn(t, nq, d, dtype=torch.float64)
    k = torch.randn(t, nkv, d, dtype=torch.float64)
    v = torch.randn(t, nkv, d, dtype=torch.float64)
    out = P.causal_attention(q, k, v)
    assert torch.allclose(out[0], v[0].expand(nq, d))           # one key: the output is its value
    mean = P.causal_attention(torch.zeros_like(q), k, v)         # zero queries: running mean of the values
    assert torch.allclose(mean[4, 0], v[:5, 0].mean(0))
    k2, v2 = k.clone(), v.clone()
    k2[6:], v2[6:] = 0.0, 5.0                                    # the future does not reach the past
    assert torch.allclose(P.causal_attention(q, k2, v2)[:6], out[:6])
    tail = P.causal_attention(q[5:], k, v)                        # queries are the tail of the keys
    assert torch.allclose(tail, out[5:])
    win = P.causal_attention(q, k, v, window=1)
    assert torch.allclose(win, v.expand(t, nq, d))               # a window of one sees only itself


def test_swiglu_equals_silu_times_up():
    g = torch.randn(4, 10, dtype=torch.float64)
    u = torch.randn(4, 10, dtype=torch.float64)
    assert torch.allclose(P.swiglu(g, u), F.silu(g) * u, atol=1e-14)
    assert torch.count_nonzero(P.swiglu(torch.zeros(3), torch.ones(3))) == 0


def test_sampler_vectors_of_the_reference_tests():
    # reference tests/test_sampler.py:53-93
    assert P.greedy(torch.tensor([1.0, 5.0, 5.0, 5.0, 2.0])) == 1
    gen = torch.Generator().manual_seed(3)
    for _ in range(20):
        row = torch.randn(512, generator=gen)
        assert P.greedy(row) == int(row.argmax())
    assert P.top_p(torch.tensor([1.0, 9.0, 9.0, 3.0]), 1, "r", 0, temperature=0.0) == 1
    assert P.top_p(torch.tensor([0.0, 7.0, 7.0, 1.0]), 3, "r", 0, p=1e-9) == 1
    picks = {P.top_p(torch.tensor([4.0, 4.0, 4.0, 4.0]), s, "r", 0, p=0.5) for s in range(50)}
    assert picks <= {0, 1}
    picks = {P.top_p(torch.tensor([1.0, 1.0, 1.0, 1.0]), s, "r", 0, p=1.0) for s in range(200)}
    assert len(picks) == 4


def test_uniform_draws():
    # reference tests/test_sampler.py:15-50
    a = P.uniform(7, "r01", 3)
    assert a == P.uniform(7, "r01", 3) and 0.0 <= a < 1.0
    assert len({a, P.uniform(8, "r01", 3), P.uniform(7, "r02", 3), P.uniform(7, "r01", 4)}) == 4
    draws = [P.uniform(0, "r", i) for i in range(2000)]
    assert 0.45 < sum(draws) / len(draws) < 0.55 and len(set(draws)) > 1900
    assert min(draws) < 0.02 and max(draws) > 0.98
    # Philox-4x32-10 known answer (Random123 kat vectors): zero counter and key
    assert P.philox_4x32((0, 0, 0, 0), (0, 0)) == (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)
    assert P.philox_4x32((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2) == (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)


def _tiny(tmp_path, tie, zero_out=False):
    import json
    from safetensors.torch import save_file

    cfg = dict(model_type="qwen3", hidden_size=32, intermediate_size=48, num_hidden_layers=2,
               num_attention_heads=4, num_key_value_heads=2, head_dim=16, vocab_size=50, rms_norm_eps=1e-6,
               rope_theta=10000.0, max_position_embeddings=64, tie_word_embeddings=tie)
    g = torch.Generator().manual_seed(1)
    w = {"model.embed_tokens.weight": torch.randn(50, 32, generator=g) * 0.5,
         "model.norm.weight": 1 + 0.1 * torch.randn(32, generator=g)}
    if not tie:
        w["lm_head.weight"] = torch.randn(50, 32, generator=g) * 0.5
    for i in range(2):
        p = f"model.layers.{i}"
        w[f"{p}.input_layernorm.weight"] = 1 + 0.1 * torch.randn(32, generator=g)
        w[f"{p}.post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(32, generator=g)
        w[f"{p}.self_attn.q_proj.weight"] = torch.randn(64, 32, generator=g) * 0.3
        w[f"{p}.self_attn.k_proj.weight"] = torch.randn(32, 32, generator=g) * 0.3
        w[f"{p}.self_attn.v_proj.weight"] = torch.randn(32, 32, generator=g) * 0.3
        w[f"{p}.self_attn.o_proj.weight"] = torch.randn(32, 64, generator=g) * (0.0 if zero_out else 0.3)
        w[f"{p}.self_attn.q_norm.weight"] = 1 + 0.2 * torch.randn(16, generator=g)
        w[f"{p}.self_attn.k_norm.weight"] = 1 + 0.2 * torch.randn(16, generator=g)
        w[f"{p}.mlp.gate_proj.weight"] = torch.randn(48, 32, generator=g) * 0.3
        w[f"{p}.mlp.up_proj.weight"] = torch.randn(48, 32, generator=g) * 0.3
        w[f"{p}.mlp.down_proj.weight"] = torch.randn(32, 48, generator=g) * (0.0 if zero_out else 0.3)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file(w, str(tmp_path / "model.safetensors"))
    return tmp_path


def test_zero_output_projections_pass_the_embedding_through(tmp_path):
    model = P.PlainModel(_tiny(tmp_path, tie=True, zero_out=True))
    ids = [3, 9, 27]
    e = model.w["model.embed_tokens.weight"][ids]
    want = P.rmsnorm(e, model.w["model.norm.weight"], 1e-6) @ model.w["model.embed_tokens.weight"].T
    assert torch.allclose(model.logits(ids), want, atol=1e-12)


def test_causality_and_shift_of_all_positions(tmp_path):
    model = P.PlainModel(_tiny(tmp_path, tie=False))
    a = model.logits([1, 2, 3, 4, 5, 6])
    b = model.logits([1, 2, 3, 4, 9, 9])
    assert torch.allclose(a[:4], b[:4], atol=1e-12) and not torch.allclose(a[4:], b[4:], atol=1e-3)
    # only distances count: running the attention block at positions p+100 gives the same output
    cfg, w = model.cfg, model.w
    x = torch.randn(5, 32, dtype=torch.float64)
    at0 = P.attention_block(cfg, w, "model.layers.0.self_attn", x, torch.arange(5))
    at100 = P.attention_block(cfg, w, "model.layers.0.self_attn", x, torch.arange(100, 105))
    assert torch.allclose(at0, at100, atol=1e-9)


def test_q_norm_comes_before_the_rotation(tmp_path):
    """Swapping norm and rotation changes the result when the norm weight is not uniform."""
    model = P.PlainModel(_tiny(tmp_path, tie=False))
    w = model.w["model.layers.0.self_attn.q_norm.weight"]
    x = torch.randn(3, 4, 16, dtype=torch.float64)
    cos, sin = P.rope_tables(16, 10000.0, torch.arange(3) + 5)
    right = P.apply_rope(P.rmsnorm(x, w, 1e-6), cos, sin)
    wrong = P.rmsnorm(P.apply_rope(x, cos, sin), w, 1e-6)
    assert not torch.allclose(right, wrong, atol=1e-3)


def test_tied_head_refuses_a_differing_tensor(tmp_path):
    import json
    from safetensors.torch import load_file, save_file

    folder = _tiny(tmp_path, tie=True)
    w = load_file(str(folder / "model.safetensors"))
    w["lm_head.weight"] = w["model.embed_tokens.weight"] + 1
    save_file(w, str(folder / "model.safetensors"))
    with pytest.raises(ValueError):
        P.PlainModel(folder)


def test_bf16_rounds_to_nearest_even_and_stays_in_the_dtype():
    x = torch.tensor([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -7, -0.1, 3e38], dtype=torch.float64)
    y = P.bf16(x)
    assert y.dtype is torch.float64
    # 1 + 2^-8 lies halfway between 1 and 1 + 2^-7: the even neighbour (1) wins; 1 + 3*2^-8 goes up to 1 + 2^-6
    assert y[:4].tolist() == [1.0, 1.0, 1.0 + 2.0 ** -6, 1.0 + 2.0 ** -7]
    assert y[4] == torch.tensor(-0.1).to(torch.bfloat16).double() and torch.isfinite(y[5])


def test_stored_probabilities_multiply_the_values_and_unrounded_ones_form_the_sum():
    # reference engine/kernels/attention.py:111-112: l sums p, the product uses p in the value dtype
    q = torch.randn(6, 2, 8, dtype=torch.float64)
    k = torch.randn(6, 1, 8, dtype=torch.float64)
    v = torch.randn(6, 1, 8, dtype=torch.float64)
    exact = P.causal_attention(q, k, v)
    assert torch.equal(P.causal_attention(q, k, v, store=lambda t: t), exact) or \
        torch.allclose(P.causal_attention(q, k, v, store=lambda t: t), exact, atol=1e-15)
    stored = P.causal_attention(q, k, v, store=P.bf16)
    assert 0 < float((stored - exact).abs().max()) < 2.0 ** -7
    assert torch.equal(stored[0], v[0].expand(2, 8))              # one visible key: p = 1 is stored exactly
    # the rows of the stored probabilities do not sum to one; dividing by the stored sum instead would show
    scores = torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(2, 1)) / math.sqrt(8)
    scores = scores.masked_fill(torch.triu(torch.ones(6, 6, dtype=torch.bool), 1)[None], float("-inf"))
    e = (scores - scores.max(-1, keepdim=True).values).exp()
    wrong = torch.einsum("hqk,khd->qhd", P.bf16(e) / P.bf16(e).sum(-1, keepdim=True), v.repeat_interleave(2, 1))
    assert float((wrong - stored).abs().max()) > 1e-5


def test_hidden_keys_state_what_a_dropped_key_would_give():
    q = torch.randn(5, 2, 8, dtype=torch.float64)
    k = torch.randn(5, 2, 8, dtype=torch.float64)
    v = torch.randn(5, 2, 8, dtype=torch.float64)
    hide = torch.zeros(5, 5, dtype=torch.bool)
    hide[3:, 1] = True                                              # queries 3 and 4 do not see key 1
    out = P.causal_attention(q, k, v, also_hidden=hide)
    assert torch.equal(out[:3], P.causal_attention(q, k, v)[:3])
    keep = [0, 2, 3, 4]
    want = P.causal_attention(q[3:], k[keep], v[keep], q_positions=torch.tensor([2, 3]))
    assert torch.allclose(out[3:], want, atol=1e-14)


# --------------------------------------------------------------------------
# the wiring of a layer, composed by hand from library routines only
# --------------------------------------------------------------------------

def _one_layer(tmp_path, zero=()):
    """A one-layer model whose norm weights are far from one and from each other, so that a norm
    in the wrong place changes the logits; ``zero`` names projections whose weights are zeros."""
    import json
    from safetensors.torch import save_file

    cfg = dict(model_type="qwen3", hidden_size=24, intermediate_size=40, num_hidden_layers=1,
               num_attention_heads=6, num_key_value_heads=2, head_dim=8, vocab_size=37, rms_norm_eps=1e-5,
               rope_theta=100.0, max_position_embeddings=64, tie_word_embeddings=False)
    g = torch.Generator().manual_seed(5)
    p = "model.layers.0"
    w = {"model.embed_tokens.weight": torch.randn(37, 24, generator=g),
         "model.norm.weight": 1 + 0.5 * torch.rand(24, generator=g),
         "lm_head.weight": torch.randn(37, 24, generator=g) * 0.5,
         f"{p}.input_layernorm.weight": 0.5 + torch.rand(24, generator=g),
         f"{p}.post_attention_layernorm.weight": 1.5 + torch.rand(24, generator=g),
         f"{p}.self_attn.q_proj.weight": torch.randn(48, 24, generator=g) * 0.4,
         f"{p}.self_attn.k_proj.weight": torch.randn(16, 24, generator=g) * 0.4,
         f"{p}.self_attn.v_proj.weight": torch.randn(16, 24, generator=g) * 0.4,
         f"{p}.self_attn.o_proj.weight": torch.randn(24, 48, generator=g) * 0.4,
         f"{p}.self_attn.q_norm.weight": 0.5 + torch.rand(8, generator=g),
         f"{p}.self_attn.k_norm.weight": 1.5 + torch.rand(8, generator=g),
         f"{p}.mlp.gate_proj.weight": torch.randn(40, 24, generator=g) * 0.4,
         f"{p}.mlp.up_proj.weight": torch.randn(40, 24, generator=g) * 0.4,
         f"{p}.mlp.down_proj.weight": torch.randn(24, 40, generator=g) * 0.4}
    for name in zero:
        w[f"{p}.{name}.weight"] = torch.zeros_like(w[f"{p}.{name}.weight"])
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file(w, str(tmp_path / "model.safetensors"))
    return tmp_path


def _rotate_by_complex_product(x, theta):
    """The rotation as a product of complex numbers (no code of the plain implementation):
    dimension i of a head is the real part and dimension i + d/2 the imaginary part of one number,
    which turns by position * theta^(-2i/d)."""
    t, heads, d = x.shape
    half = d // 2
    freq = torch.tensor([theta ** (-2.0 * i / d) for i in range(half)], dtype=torch.float64)
    turn = torch.polar(torch.ones(t, half, dtype=torch.float64), torch.arange(t, dtype=torch.float64)[:, None] * freq)
    z = torch.complex(x[..., :half], x[..., half:]) * turn[:, None, :]
    return torch.cat([z.real, z.imag], dim=-1)


def _layer_by_hand(model, ids, norms=("input_layernorm", "post_attention_layernorm"), parallel=False):
    """One layer as the reference wires it (engine/model/qwen3.py:319-373), from library routines:
    ``h = E[ids]; h = h + O(attn(norm_1(h))); h = h + down(silu(gate(norm_2(h))) * up(norm_2(h)));
    logits = head(norm(h))``.  ``norms`` and ``parallel`` state the two plausible misreadings."""
    cfg, w = model.cfg, model.w
    p = "model.layers.0"
    eps = cfg["rms_norm_eps"]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    hidden = cfg["hidden_size"]
    t = len(ids)
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    x = F.rms_norm(h, (hidden,), w[f"{p}.{norms[0]}.weight"], eps)
    q = F.linear(x, w[f"{p}.self_attn.q_proj.weight"]).view(t, nq, d)
    k = F.linear(x, w[f"{p}.self_attn.k_proj.weight"]).view(t, nkv, d)
    v = F.linear(x, w[f"{p}.self_attn.v_proj.weight"]).view(t, nkv, d)
    q = _rotate_by_complex_product(F.rms_norm(q, (d,), w[f"{p}.self_attn.q_norm.weight"], eps), cfg["rope_theta"])
    k = _rotate_by_complex_product(F.rms_norm(k, (d,), w[f"{p}.self_attn.k_norm.weight"], eps), cfg["rope_theta"])
    g = nq // nkv
    attn = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat_interleave(g, 1).transpose(0, 1)[None],
        v.repeat_interleave(g, 1).transpose(0, 1)[None], is_causal=True, scale=d ** -0.5)[0].transpose(0, 1)
    after_attention = h + F.linear(attn.reshape(t, nq * d), w[f"{p}.self_attn.o_proj.weight"])
    x = F.rms_norm(h if parallel else after_attention, (hidden,), w[f"{p}.{norms[1]}.weight"], eps)
    mlp = F.linear(F.silu(F.linear(x, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(x, w[f"{p}.mlp.up_proj.weight"]),
                   w[f"{p}.mlp.down_proj.weight"])
    out = after_attention + mlp
    return F.linear(F.rms_norm(out, (hidden,), w["model.norm.weight"], eps), w["lm_head.weight"])


IDS = [3, 30, 7, 7, 19, 0, 36, 11, 2]


def test_one_layer_equals_its_composition_from_library_routines(tmp_path):
    """Pins the wiring: which norm feeds which part, and that the feed-forward reads the stream
    after the attention's addition.  The two misreadings are computed too and must differ."""
    model = P.PlainModel(_one_layer(tmp_path))
    got = model.logits(IDS)
    want = _layer_by_hand(model, IDS)
    assert torch.allclose(got, want, atol=1e-10)
    scale = float(want.abs().max())
    swapped = _layer_by_hand(model, IDS, norms=("post_attention_layernorm", "input_layernorm"))
    side_by_side = _layer_by_hand(model, IDS, parallel=True)
    assert float((swapped - got).abs().max()) > 1e-2 * scale
    assert float((side_by_side - got).abs().max()) > 1e-2 * scale


@pytest.mark.parametrize("zeroed", ["self_attn.o_proj", "mlp.down_proj"])
def test_half_zeroed_layers(tmp_path, zeroed):
    """Only the attention's output projection zero: the layer is the feed-forward on the embedding,
    under the second norm.  Only the down projection zero: the layer is the attention alone."""
    model = P.PlainModel(_one_layer(tmp_path, zero=(zeroed,)))
    cfg, w = model.cfg, model.w
    p = "model.layers.0"
    eps, hidden = cfg["rms_norm_eps"], cfg["hidden_size"]
    got = model.logits(IDS)
    assert torch.allclose(got, _layer_by_hand(model, IDS), atol=1e-10)
    h = F.embedding(torch.tensor(IDS), w["model.embed_tokens.weight"])
    if zeroed == "self_attn.o_proj":
        x = F.rms_norm(h, (hidden,), w[f"{p}.post_attention_layernorm.weight"], eps)
        h = h + F.linear(F.silu(F.linear(x, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(x, w[f"{p}.mlp.up_proj.weight"]),
                         w[f"{p}.mlp.down_proj.weight"])
    else:
        x = F.rms_norm(h, (hidden,), w[f"{p}.input_layernorm.weight"], eps)
        h = h + P.attention_block(cfg, w, f"{p}.self_attn", x, torch.arange(len(IDS)))
    want = F.linear(F.rms_norm(h, (hidden,), w["model.norm.weight"], eps), w["lm_head.weight"])
    assert torch.allclose(got, want, atol=1e-10)
    if zeroed == "self_attn.o_proj":
        # the first norm's weight in the second one's place would show
        x2 = F.rms_norm(F.embedding(torch.tensor(IDS), w["model.embed_tokens.weight"]), (hidden,),
                        w[f"{p}.input_layernorm.weight"], eps)
        h2 = F.embedding(torch.tensor(IDS), w["model.embed_tokens.weight"]) + F.linear(
            F.silu(F.linear(x2, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(x2, w[f"{p}.mlp.up_proj.weight"]),
            w[f"{p}.mlp.down_proj.weight"])
        wrong = F.linear(F.rms_norm(h2, (hidden,), w["model.norm.weight"], eps), w["lm_head.weight"])
        assert float((wrong - got).abs().max()) > 1e-2 * float(got.abs().max())
