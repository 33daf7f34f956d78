"""Each part of a layer alone against the plain implementation, a toy mixer
with state of its own registered from here, and schedules that name a layer
twice or share a cache -- all without touching the framework's files."""

from __future__ import annotations

import json
from dataclasses import dataclass

import pytest
import torch

from helpers import feed, random_tokens, rel_err
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu


class Harness:
    """A runtime, a cache for one unit spec and a way to make step contexts."""

    def __init__(self, dtype="float32", unit_specs=(None,), page_size=8, num_pages=32):
        from lockstep_amd.cache import CacheManager
        from lockstep_amd.engine.batch import Workspace
        from lockstep_amd.engine.runtime import Runtime

        self.rt = Runtime("cuda:0", dtype)
        self.cache = CacheManager(list(unit_specs), page_size, num_pages, 4, num_pages * page_size,
                                  torch_dtype=self.rt.dtype, device=self.rt.device, poison_on_free=True)
        self.workspace = Workspace(self.rt.device)

    def context(self, lengths: dict, mixers=()):
        from lockstep_amd.engine.batch import StepContext, StepEntry

        entries = []
        for rid, n in lengths.items():
            if rid not in self.cache.requests:
                self.cache.open(rid)
            self.cache.reserve(rid, self.cache.length(rid) + n)
            entries.append(StepEntry(rid, [0] * n, []))
        self.cache.sync_tables()
        ctx = StepContext(self.rt, self.cache, self.workspace, entries)
        for m in mixers:
            m.prepare(ctx)
        ctx.upload()
        return ctx

    def commit(self, ctx):
        for e, end in zip(ctx.entries, ctx.kv_len):
            self.cache.commit(e.request, int(end))


def store(tensors):
    from lockstep_amd.weights.store import DictWeightStore

    return DictWeightStore(tensors)


@dataclass
class Run:
    layer: int = 0
    cache: int = 0
    writes_cache: bool = True


def test_norm_part_alone():
    from lockstep_amd.config import PartSpec
    from lockstep_amd.parts import build_part

    h = Harness()
    part = build_part(PartSpec("rmsnorm", {"size": 72, "eps": 1e-3}), "n")
    w = 1 + 0.3 * torch.randn(72)
    part.load(store({"n.weight": w}), h.rt)
    x = torch.randn(5, 72) * 2
    ctx = h.context({"a": 5})
    out = torch.empty(5, 72, device="cuda")
    part.forward(ctx, x.cuda(), out)
    assert rel_err(out.cpu(), P.rmsnorm(x.double(), w.double(), 1e-3)) < 1e-6


def test_position_part_alone_matches_the_plain_tables():
    from lockstep_amd.config import PartSpec
    from lockstep_amd.parts import build_part

    h = Harness()
    part = build_part(PartSpec("rope_half", {"rotary_dim": 48, "theta": 5e5}))
    part.ensure(700, h.rt)
    cos, sin = P.rope_tables(48, 5e5, torch.arange(700))
    assert torch.equal(part.cos[:700].cpu(), cos.float()) and torch.equal(part.sin[:700].cpu(), sin.float())
    part.ensure(5000, h.rt)                                     # grows on demand
    assert part.cos.shape[0] >= 5000 and torch.equal(part.cos[:700].cpu(), cos.float())


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_attention_part_alone_in_portions(dtype, tol):
    from lockstep_amd.config import PartSpec
    from lockstep_amd.parts import build_part

    hidden, nq, nkv, d = 40, 6, 2, 48
    spec = PartSpec("attention", {
        "hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d,
        "qk_norm": PartSpec("rmsnorm", {"size": d, "eps": 1e-5}),
        "position": PartSpec("rope_half", {"rotary_dim": d, "theta": 1e4}),
        "window": None, "bias": False, "scale": d ** -0.5})
    part = build_part(spec, "att")
    g = torch.Generator().manual_seed(0)
    w = {"att.q_proj.weight": torch.randn(nq * d, hidden, generator=g) * 0.3,
         "att.k_proj.weight": torch.randn(nkv * d, hidden, generator=g) * 0.3,
         "att.v_proj.weight": torch.randn(nkv * d, hidden, generator=g) * 0.3,
         "att.o_proj.weight": torch.randn(hidden, nq * d, generator=g) * 0.3,
         "att.q_norm.weight": 1 + 0.2 * torch.randn(d, generator=g),
         "att.k_norm.weight": 1 + 0.2 * torch.randn(d, generator=g)}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    h = Harness(dtype, unit_specs=(part.cache_spec(),))
    part.load(store(w), h.rt)
    x = (torch.randn(29, hidden, generator=g)).to(torch.bfloat16)
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "rms_norm_eps": 1e-5,
           "rope_theta": 1e4}
    w64 = {k.replace("att.", "L."): v.double() for k, v in w.items()}
    want = P.attention_block(cfg, w64, "L", x.double(), torch.arange(29))
    got = []
    pos = 0
    for n in (11, 2, 15, 1):
        ctx = h.context({"a": n}, mixers=[part])
        out = torch.zeros(n, hidden, device="cuda")
        part.forward(ctx, Run(), x[pos:pos + n].to(h.rt.dtype).cuda(), out, accumulate=False)
        h.commit(ctx)
        got.append(out.cpu())
        pos += n
    assert rel_err(torch.cat(got), want) < tol


def test_a_position_encoding_that_pairs_neighbours_registers_without_a_kernel_of_its_own():
    """A toy rotary encoding whose pairs are the neighbours (2i, 2i + 1) of the first 32 of 48
    dimensions: it states the order that brings its pairs to (i, i + rotary_dim/2), the attention
    part reorders its query and key rows (and norm weights) at load, and the result equals a plain
    attention that rotates neighbours -- in portions, in float32."""
    from lockstep_amd.config import PartSpec
    from lockstep_amd.parts import build_part, register_part, unregister_part
    from lockstep_amd.parts.rope import RotaryHalf

    @register_part("toy_rope_neighbours")
    class NeighbourRotary(RotaryHalf):
        def share_key(self):
            return ("toy_rope_neighbours",) + super().share_key()

        def bind(self, rt):                       # tables of its own, not the half rotation's
            self._store = self.__dict__.setdefault("_own_tables", [None, None])

        def dim_order(self, head_dim):
            rot = self.rotary_dim
            return list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, head_dim))

    hidden, nq, nkv, d, rot, theta, eps = 40, 6, 2, 48, 32, 1e4, 1e-5
    try:
        spec = PartSpec("attention", {
            "hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d,
            "qk_norm": PartSpec("rmsnorm", {"size": d, "eps": eps}),
            "position": PartSpec("toy_rope_neighbours", {"rotary_dim": rot, "theta": theta}),
            "window": None, "bias": False, "scale": d ** -0.5})
        part = build_part(spec, "att")
        g = torch.Generator().manual_seed(4)
        w = {"att.q_proj.weight": torch.randn(nq * d, hidden, generator=g) * 0.3,
             "att.k_proj.weight": torch.randn(nkv * d, hidden, generator=g) * 0.3,
             "att.v_proj.weight": torch.randn(nkv * d, hidden, generator=g) * 0.3,
             "att.o_proj.weight": torch.randn(hidden, nq * d, generator=g) * 0.3,
             "att.q_norm.weight": 1 + 0.2 * torch.randn(d, generator=g),
             "att.k_norm.weight": 1 + 0.2 * torch.randn(d, generator=g)}
        w = {k: v.to(torch.bfloat16) for k, v in w.items()}
        h = Harness("float32", unit_specs=(part.cache_spec(),))
        part.load(store(w), h.rt)
        t = 27
        x = torch.randn(t, hidden, generator=g).to(torch.bfloat16)

        # the plain form: rotate neighbours of the first `rot` dimensions, in the checkpoint's own order
        w64 = {k: v.double() for k, v in w.items()}
        x64 = x.double()
        q = P.rmsnorm((x64 @ w64["att.q_proj.weight"].T).view(t, nq, d), w64["att.q_norm.weight"], eps)
        k = P.rmsnorm((x64 @ w64["att.k_proj.weight"].T).view(t, nkv, d), w64["att.k_norm.weight"], eps)
        v = (x64 @ w64["att.v_proj.weight"].T).view(t, nkv, d)
        inv_freq = theta ** (-torch.arange(0, rot, 2, dtype=torch.float64) / rot)
        angles = torch.arange(t, dtype=torch.float64)[:, None] * inv_freq[None, :]

        def rotate(z):
            out = z.clone()
            even, odd = z[..., 0:rot:2], z[..., 1:rot:2]
            c, s_ = angles.cos()[:, None, :], angles.sin()[:, None, :]
            out[..., 0:rot:2] = even * c - odd * s_
            out[..., 1:rot:2] = odd * c + even * s_
            return out

        attn = P.causal_attention(rotate(q), rotate(k), v, q_positions=torch.arange(t))
        want = attn.reshape(t, nq * d) @ w64["att.o_proj.weight"].T
        # a half rotation of the same weights is something else: the order matters
        cos, sin = P.rope_tables(rot, theta, torch.arange(t))
        assert rel_err(P.apply_rope(q[..., :rot], cos, sin), rotate(q)[..., :rot]) > 0.1

        got, pos = [], 0
        for n in (9, 2, 15, 1):
            ctx = h.context({"a": n}, mixers=[part])
            out = torch.zeros(n, hidden, device="cuda")
            part.forward(ctx, Run(), x[pos:pos + n].float().cuda(), out, accumulate=False)
            h.commit(ctx)
            got.append(out.cpu())
            pos += n
        assert rel_err(torch.cat(got), want) < 2e-5
    finally:
        unregister_part("toy_rope_neighbours")


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_parts_with_biases_and_another_activation(dtype, tol):
    """Attention with biases on all four projections and a gated feed-forward with the tanh form
    of GELU and biases, each alone in portions against the formulas in float64; the same rows in
    one step and in portions give the same bits."""
    from lockstep_amd.config import PartSpec
    from lockstep_amd.parts import build_part

    hidden, nq, nkv, d, inter, eps = 72, 6, 3, 32, 200, 1e-5
    g = torch.Generator().manual_seed(8)
    rnd = lambda *shape, scale=0.3: (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)
    att = build_part(PartSpec("attention", {
        "hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d,
        "qk_norm": PartSpec("rmsnorm", {"size": d, "eps": eps}),
        "position": PartSpec("rope_half", {"rotary_dim": d, "theta": 1e4}),
        "window": None, "bias": True, "out_bias": True, "scale": d ** -0.5}), "att")
    names = [w.name for w in att.weight_specs(att.spec, "att")]
    assert {"att.q_proj.bias", "att.k_proj.bias", "att.v_proj.bias", "att.o_proj.bias"} <= set(names)
    w = {"att.q_proj.weight": rnd(nq * d, hidden), "att.k_proj.weight": rnd(nkv * d, hidden),
         "att.v_proj.weight": rnd(nkv * d, hidden), "att.o_proj.weight": rnd(hidden, nq * d),
         "att.q_norm.weight": (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16),
         "att.k_norm.weight": (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16),
         "att.q_proj.bias": rnd(nq * d), "att.k_proj.bias": rnd(nkv * d), "att.v_proj.bias": rnd(nkv * d),
         "att.o_proj.bias": rnd(hidden)}
    h = Harness(dtype, unit_specs=(att.cache_spec(),))
    att.load(store(w), h.rt)
    t = 30
    x = rnd(t, hidden, scale=1.0)
    w64, x64 = {k: v.double() for k, v in w.items()}, x.double()
    q = P.rmsnorm((x64 @ w64["att.q_proj.weight"].T + w64["att.q_proj.bias"]).view(t, nq, d), w64["att.q_norm.weight"], eps)
    k = P.rmsnorm((x64 @ w64["att.k_proj.weight"].T + w64["att.k_proj.bias"]).view(t, nkv, d), w64["att.k_norm.weight"], eps)
    v = (x64 @ w64["att.v_proj.weight"].T + w64["att.v_proj.bias"]).view(t, nkv, d)
    cos, sin = P.rope_tables(d, 1e4, torch.arange(t))
    attn = P.causal_attention(P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin), v, q_positions=torch.arange(t))
    want = attn.reshape(t, nq * d) @ w64["att.o_proj.weight"].T + w64["att.o_proj.bias"]

    def run_attention(rid, cuts):
        got, pos = [], 0
        for n in cuts:
            ctx = h.context({rid: n}, mixers=[att])
            out = torch.zeros(n, hidden, device="cuda")
            att.forward(ctx, Run(), x[pos:pos + n].to(h.rt.dtype).cuda(), out, accumulate=False)
            h.commit(ctx)
            got.append(out.cpu())
            pos += n
        return torch.cat(got)

    whole, cut = run_attention("whole", (t,)), run_attention("cut", (11, 2, 16, 1))
    assert rel_err(whole, want) < tol and torch.equal(whole, cut)

    ff = build_part(PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter,
                                           "activation": "gelu_tanh", "bias": True}), "ff")
    wf = {"ff.gate_proj.weight": rnd(inter, hidden), "ff.up_proj.weight": rnd(inter, hidden),
          "ff.down_proj.weight": rnd(hidden, inter), "ff.gate_proj.bias": rnd(inter), "ff.up_proj.bias": rnd(inter),
          "ff.down_proj.bias": rnd(hidden)}
    ff.load(store(wf), h.rt)
    f64 = {k: v.double() for k, v in wf.items()}
    gate = x64 @ f64["ff.gate_proj.weight"].T + f64["ff.gate_proj.bias"]
    up = x64 @ f64["ff.up_proj.weight"].T + f64["ff.up_proj.bias"]
    stream = torch.randn(t, hidden, generator=g)
    want = stream.double() + (torch.nn.functional.gelu(gate, approximate="tanh") * up) @ f64["ff.down_proj.weight"].T \
        + f64["ff.down_proj.bias"]

    def run_ff(cuts):
        got, pos = [], 0
        for n in cuts:
            ctx = h.context({f"f{len(cuts)}": n})
            out = stream[pos:pos + n].cuda().clone()
            left = ff.forward(ctx, x[pos:pos + n].to(h.rt.dtype).cuda(), out, accumulate=True, defer=True)
            assert left is None                      # with biases the addition is not left to the next norm
            h.commit(ctx)
            got.append(out.cpu())
            pos += n
        return torch.cat(got)

    whole, cut = run_ff((t,)), run_ff((3, 20, 7))
    assert rel_err(whole, want) < tol and torch.equal(whole, cut)
    with pytest.raises(ValueError, match="not built"):
        build_part(PartSpec("gated_mlp", {"hidden_size": 8, "intermediate_size": 8, "activation": "swish7"}), "x")


def test_feed_forward_part_and_block_alone():
    from lockstep_amd.config import LayerSpec, PartSpec
    from lockstep_amd.parts import build_part, part_class

    hidden, inter = 56, 136
    g = torch.Generator().manual_seed(1)
    w = {"L.mlp.gate_proj.weight": torch.randn(inter, hidden, generator=g) * 0.3,
         "L.mlp.up_proj.weight": torch.randn(inter, hidden, generator=g) * 0.3,
         "L.mlp.down_proj.weight": torch.randn(hidden, inter, generator=g) * 0.3}
    ff_spec = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter, "activation": "silu"})
    h = Harness()
    part = build_part(ff_spec, "L.mlp")
    part.load(store(w), h.rt)
    x = torch.randn(9, hidden, generator=g)
    ctx = h.context({"a": 9})
    out = torch.ones(9, hidden, device="cuda")
    part.forward(ctx, x.cuda(), out, accumulate=True)
    want = 1 + P.mlp_block({k: v.double() for k, v in w.items()}, "L.mlp", x.double())
    assert rel_err(out.cpu(), want) < 2e-5
    with pytest.raises(ValueError):
        build_part(PartSpec("gated_mlp", {"hidden_size": 8, "intermediate_size": 8, "activation": "softsign"}), "m")

    # the whole arrangement: h += attn(norm(h)); h += mlp(norm(h))
    nq, nkv, d = 4, 4, 16
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6})
    layer = LayerSpec(
        prefix="L",
        arrangement=PartSpec("prenorm_residual", {"mixer_prefix": "self_attn", "feed_forward_prefix": "mlp",
                                                  "mixer_norm_name": "input_layernorm",
                                                  "feed_forward_norm_name": "post_attention_layernorm"}),
        mixer=PartSpec("attention", {"hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d,
                                     "qk_norm": None, "position": PartSpec("no_position", {}), "window": None,
                                     "bias": False, "scale": 0.2}),
        feed_forward=ff_spec, mixer_norm=norm, feed_forward_norm=norm)
    block = part_class("prenorm_residual")(layer)
    w.update({"L.input_layernorm.weight": 1 + 0.1 * torch.randn(hidden, generator=g),
              "L.post_attention_layernorm.weight": 1 + 0.1 * torch.randn(hidden, generator=g),
              "L.self_attn.q_proj.weight": torch.randn(nq * d, hidden, generator=g) * 0.3,
              "L.self_attn.k_proj.weight": torch.randn(nkv * d, hidden, generator=g) * 0.3,
              "L.self_attn.v_proj.weight": torch.randn(nkv * d, hidden, generator=g) * 0.3,
              "L.self_attn.o_proj.weight": torch.randn(hidden, nq * d, generator=g) * 0.3})
    names = sorted(s.name for s in part_class("prenorm_residual").weight_specs(layer))
    assert names == sorted(w)                                  # without q/k norm there are no norm tensors
    h2 = Harness(unit_specs=(block.mixer.cache_spec(),))
    block.load(store(w), h2.rt)
    hs = torch.randn(13, hidden, generator=g)
    ctx = h2.context({"a": 13}, mixers=[block.mixer])
    dev = hs.clone().cuda()
    left = block.forward(ctx, Run(), dev)
    if left is not None:                # a short step leaves its last addition to the next reader
        left.flush(ctx, dev)
    w64 = {k: v.double() for k, v in w.items()}
    x64 = hs.double()
    normed = P.rmsnorm(x64, w64["L.input_layernorm.weight"], 1e-6)
    q = P.linear(normed, w64["L.self_attn.q_proj.weight"]).view(13, nq, d)
    k = P.linear(normed, w64["L.self_attn.k_proj.weight"]).view(13, nkv, d)
    v = P.linear(normed, w64["L.self_attn.v_proj.weight"]).view(13, nkv, d)
    # plain attention without rotation; its score scale is 1/sqrt(d), the part's is 0.2: rescale q
    attn = P.causal_attention(q * (0.2 * d ** 0.5), k, v)
    x64 = x64 + P.linear(attn.reshape(13, nq * d), w64["L.self_attn.o_proj.weight"])
    x64 = x64 + P.mlp_block(w64, "L.mlp", P.rmsnorm(x64, w64["L.post_attention_layernorm.weight"], 1e-6))
    assert rel_err(dev.cpu(), x64) < 2e-5


# ---------------------------------------------------------------------------
# a toy architecture defined here: a mixer with a state of fixed size, a
# layer that runs twice, and a layer that reads another layer's keys/values
# ---------------------------------------------------------------------------

def _register_toy():
    from lockstep_amd.config import (LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry,
                                     register_architecture)
    from lockstep_amd.parts import Mixer, StateSpec, WeightSpec, register_part

    @register_part("toy_decay")
    class DecayMixer(Mixer):
        """s_t = decay * s_{t-1} + x_t / (1 + position_t % 5) (one state vector per request);
        out_t = s_t @ W^T.  The mixer owns device-side metadata of the step: a block of two ints
        a request (its state slot, the position of its token) whose positions move on by one with
        every token decoded without the host.  Steps of single decoded tokens read nothing on the
        host (torch operations indexed by that block, the engine's own matrix product), so the
        part is graph safe; prompt portions walk their rows on the host."""

        graph_safe = True

        def __init__(self, spec, prefix=""):
            super().__init__(spec, prefix)
            self.hidden, self.decay = int(spec["hidden_size"]), float(spec["decay"])

        @classmethod
        def weight_specs(cls, spec, prefix):
            return [WeightSpec(f"{prefix}.mix.weight", (int(spec["hidden_size"]),) * 2)]

        def cache_spec(self):
            return StateSpec((self.hidden,))

        def load(self, weights, rt):
            self.w = rt.vector(weights.get(f"{self.prefix}.mix.weight"))

        def prepare(self, ctx):
            if ctx.single_tokens and not ctx.declared("toy_decay"):
                ints = [v for slot, pos in zip(ctx.slots, ctx.q_start) for v in (int(slot), int(pos))]
                ctx.declare("toy_decay", ints, advance=[(1, 2, ctx.n_seqs)])

        def forward(self, ctx, run, x, out, accumulate):
            from lockstep_amd.ops import ADD_F32, STORE_F32

            state = ctx.cache.unit_state(run.cache)
            if ctx.single_tokens:                       # device side only: may be captured and replayed
                block = ctx.block("toy_decay").view(ctx.n_seqs, 2)
                slots, positions = block[:, 0].long(), block[:, 1]
                gain = 1.0 / (1 + positions % 5).to(torch.float32)
                fresh = self.decay * state.index_select(0, slots) + x.float() * gain[:, None]
                state.index_copy_(0, slots, fresh)
                ctx.rt.kernels.gemm(fresh.contiguous(), self.w, out, ADD_F32 if accumulate else STORE_F32)
                return
            for i in range(ctx.n_seqs):
                lo, n, slot, start = int(ctx.q_off[i]), int(ctx.q_len[i]), int(ctx.slots[i]), int(ctx.q_start[i])
                s = state[slot]
                rows = []
                for t in range(n):
                    s = self.decay * s + x[lo + t].float() / (1 + (start + t) % 5)
                    rows.append(s)
                state[slot] = s
                y = torch.stack(rows) @ self.w.T
                out[lo:lo + n] = out[lo:lo + n] + y if accumulate else y

    @register_architecture
    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        hidden_size: int
        vocab_size: int
        decay: float
        schedule: list
        architecture_names = ("toy-decay",)

        def model_spec(self):
            h = self.hidden_size
            norm = PartSpec("rmsnorm", {"size": h, "eps": 1e-5})
            ff = PartSpec("gated_mlp", {"hidden_size": h, "intermediate_size": 2 * h, "activation": "silu"})
            arr = PartSpec("prenorm_residual", {"mixer_prefix": "mixer", "feed_forward_prefix": "ff",
                                                "mixer_norm_name": "norm1", "feed_forward_norm_name": "norm2"})
            attn = PartSpec("attention", {"hidden_size": h, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                          "qk_norm": None,
                                          "position": PartSpec("rope_half", {"rotary_dim": 8, "theta": 100.0}),
                                          "window": None, "bias": False, "scale": 0.25})
            decay = PartSpec("toy_decay", {"hidden_size": h, "decay": self.decay})
            layers = (LayerSpec("layers.0", arr, decay, ff, norm, norm),
                      LayerSpec("layers.1", arr, attn, ff, norm, norm),
                      LayerSpec("layers.2", arr, attn, ff, norm, norm))
            return ModelSpec(
                hidden_size=h, vocab_size=self.vocab_size,
                embedding=PartSpec("token_embedding", {"name": "embed.weight", "vocab_size": self.vocab_size,
                                                       "hidden_size": h}),
                layers=layers,
                schedule=tuple(ScheduleEntry(*e) for e in self.schedule),
                final_norm=PartSpec("rmsnorm", {"size": h, "eps": 1e-5, "name": "final_norm.weight"}),
                head=PartSpec("linear_head", {"name": "head.weight", "tied_to": None,
                                              "vocab_size": self.vocab_size, "hidden_size": h}))

    return ToyConfig


def _toy_plain(cfg, w, tokens, schedule):
    """Plain float64 forward of the toy architecture, whole sequence."""
    t = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    positions = torch.arange(t)
    kv = {}
    for layer, unit, writes in schedule:
        p = f"layers.{layer}"
        x = P.rmsnorm(h, w[f"{p}.norm1.weight"], 1e-5)
        if layer == 0:
            s = torch.zeros(cfg["hidden_size"], dtype=torch.float64)
            rows = []
            for i in range(t):
                s = cfg["decay"] * s + x[i] / (1 + i % 5)
                rows.append(s)
            h = h + torch.stack(rows) @ w[f"{p}.mixer.mix.weight"].T
        else:
            q = P.linear(x, w[f"{p}.mixer.q_proj.weight"]).view(t, 2, 16)
            if writes:
                k = P.linear(x, w[f"{p}.mixer.k_proj.weight"]).view(t, 1, 16)
                v = P.linear(x, w[f"{p}.mixer.v_proj.weight"]).view(t, 1, 16)
                cos, sin = P.rope_tables(8, 100.0, positions)
                k = torch.cat([P.apply_rope(k[..., :8], cos, sin), k[..., 8:]], -1)
                kv[unit] = (k, v)
            cos, sin = P.rope_tables(8, 100.0, positions)
            q = torch.cat([P.apply_rope(q[..., :8], cos, sin), q[..., 8:]], -1)
            k, v = kv[unit]
            attn = P.causal_attention(q * (0.25 * 4.0), k, v)          # part scale 0.25, plain scale 1/sqrt(16)
            h = h + P.linear(attn.reshape(t, 32), w[f"{p}.mixer.o_proj.weight"])
        h = h + P.mlp_block({k_: v_ for k_, v_ in w.items()}, f"{p}.ff",
                            P.rmsnorm(h, w[f"{p}.norm2.weight"], 1e-5))
    return P.linear(P.rmsnorm(h, w["final_norm.weight"], 1e-5), w["head.weight"])


@pytest.mark.parametrize("schedule", [
    [(0, 0, True), (1, 1, True), (2, 2, True)],                      # state mixer, then two attention layers
    [(0, 0, True), (1, 1, True), (1, 2, True), (2, 3, True)],        # layer 1 runs twice, each run with its own cache
    [(0, 0, True), (1, 1, True), (2, 1, False)],                     # layer 2 reads the keys and values of layer 1
])
def test_toy_architecture_registers_builds_and_steps(tmp_path, schedule):
    from lockstep_amd.config import unregister_architecture
    from lockstep_amd.engine.model import load_model
    from lockstep_amd.parts import unregister_part
    from lockstep_amd.weights import write_random_model

    ToyConfig = _register_toy()
    try:
        cfg = ToyConfig(hidden_size=48, vocab_size=90, decay=0.9, schedule=[list(e) for e in schedule])
        folder = write_random_model(cfg, tmp_path / "toy", seed=5, std=0.2, norm_std=0.1)
        assert json.loads((folder / "config.json").read_text())["model_type"] == "toy-decay"
        model = load_model(folder, dtype="float32")
        units = model.cache_unit_specs()
        assert type(units[0]).__name__ == "StateSpec" and type(units[1]).__name__ == "PagedKVSpec"
        from safetensors.torch import load_file

        w = {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}
        tokens = random_tokens(50, 90, seed=1)
        want = _toy_plain({"hidden_size": 48, "decay": 0.9}, w, tokens, schedule)
        cache = model.make_cache(num_pages=16, page_size=8, max_requests=3, poison_on_free=True)
        whole = feed(model, cache, "w", tokens, [])
        assert rel_err(whole, want) < 5e-5
        other = feed(model, cache, "o", random_tokens(9, 90, seed=2), [])     # another request in between
        cut = feed(model, cache, "c", tokens, [7, 2, 17, 1, 1, 13])
        assert rel_err(cut, want) < 5e-5
        cache.close("w"); cache.close("o")
        again = feed(model, cache, "w2", tokens, [25])                          # a reused slot starts from zero state
        assert rel_err(again, want) < 5e-5
        cache.audit()
        cache.close("c"); cache.close("w2")
        # The mixer declared itself graph safe: steps of single decoded tokens are replayed from a captured
        # graph, with its block of slots and positions uploaded beside the attention layers' work lists ...
        replays = model.graph_replays
        tail = feed(model, cache, "t", tokens, [20] + [1] * 30)
        assert model.graph_replays - replays >= 25 and rel_err(tail, want) < 5e-5
        beside = random_tokens(50, 90, seed=3)                                  # ... two requests in a step
        want_beside = _toy_plain({"hidden_size": 48, "decay": 0.9}, w, beside, schedule)
        cache.close("t")
        feed(model, cache, "p", tokens[:30], [], want_all=False); feed(model, cache, "q", beside[:11], [], want_all=False)
        from lockstep_amd.engine.batch import StepEntry
        rows_p, rows_q = [], []
        for i in range(20):
            logits = model.step(cache, [StepEntry("p", [tokens[30 + i]], [0]), StepEntry("q", [beside[11 + i]], [0])])
            rows_p.append(logits[0].cpu()); rows_q.append(logits[1].cpu())
        assert rel_err(torch.stack(rows_p), want[30:50]) < 5e-5
        assert rel_err(torch.stack(rows_q), want_beside[11:31]) < 5e-5
        # ... and the device-side loop advances the mixer's positions itself: greedy tokens equal stepwise decoding
        picked = {}
        for way in ("loop", "steps"):
            cache.close("p"); cache.close("q")
            feed(model, cache, "p", tokens[:30], [], want_all=False); feed(model, cache, "q", beside[:11], [], want_all=False)
            cur = [tokens[30], beside[11]]
            if way == "loop":
                before = model.graph_replays
                picked[way] = model.decode_greedy(cache, ["p", "q"], cur, 12).tolist()
                assert model.graph_replays - before >= 10
            else:
                got = []
                for _ in range(12):
                    logits = model.step(cache, [StepEntry("p", cur[:1], [0]), StepEntry("q", cur[1:], [0])])
                    cur = [int(row.argmax()) for row in logits]
                    got.append(cur)
                picked[way] = got
        assert picked["loop"] == picked["steps"]
        cache.audit()
    finally:
        unregister_part("toy_decay")
        unregister_architecture(ToyConfig)


# ---------------------------------------------------------------------------
# a second toy architecture, defined here as well: a feed-forward that routes
# every token to one of several experts (it fetches the routing decision, so
# it may not run inside a captured graph), and a position encoding with
# frequencies and a stretch of its own behind the attention mixer
# ---------------------------------------------------------------------------

def _register_routed_toy():
    from lockstep_amd.config import (LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry,
                                     register_architecture)
    from lockstep_amd.parts import FeedForward, PositionEncoding, WeightSpec, bump_device_epoch, register_part

    @register_part("toy_linear_angles")
    class LinearAngles(PositionEncoding):
        """Pair i at position p turns by (p / stretch) * (i + 1) * step."""

        graph_safe = True

        def __init__(self, spec, prefix=""):
            super().__init__(spec, prefix)
            self.rotary_dim = int(spec["rotary_dim"])
            self.stretch, self.step = float(spec["stretch"]), float(spec["step"])
            self.cos = self.sin = None

        def ensure(self, max_position, rt):
            if self.cos is not None and self.cos.shape[0] >= max_position:
                return
            angles = _linear_angles(torch.arange(max(max_position, 24)), self.rotary_dim, self.stretch, self.step)
            self.cos = angles.cos().float().to(rt.device).contiguous()
            self.sin = angles.sin().float().to(rt.device).contiguous()
            bump_device_epoch()                      # a captured graph holds the old tables

    @register_part("toy_top1_experts")
    class Top1Experts(FeedForward):
        """logits = x R^T in float32; a token goes to the expert with the largest logit and its
        output is softmax(logits)[expert] * down_e(relu(up_e(x)))."""

        def __init__(self, spec, prefix=""):
            super().__init__(spec, prefix)
            self.hidden, self.experts, self.inter = (int(spec[k]) for k in ("hidden_size", "experts", "expert_size"))

        @classmethod
        def weight_specs(cls, spec, prefix):
            h, n, i = (int(spec[k]) for k in ("hidden_size", "experts", "expert_size"))
            out = [WeightSpec(f"{prefix}.router.weight", (n, h))]
            for e in range(n):
                out += [WeightSpec(f"{prefix}.experts.{e}.up.weight", (i, h)),
                        WeightSpec(f"{prefix}.experts.{e}.down.weight", (h, i))]
            return out

        def load(self, weights, rt):
            self.router = rt.vector(weights.get(f"{self.prefix}.router.weight"))
            self.up = [rt.vector(weights.get(f"{self.prefix}.experts.{e}.up.weight")) for e in range(self.experts)]
            self.down = [rt.vector(weights.get(f"{self.prefix}.experts.{e}.down.weight")) for e in range(self.experts)]

        def forward(self, ctx, x, out, accumulate):
            xf = x.float()
            logits = xf @ self.router.T
            choice = logits.argmax(-1)
            gate = torch.softmax(logits, -1).gather(1, choice[:, None])
            y = torch.zeros_like(xf)
            for e in choice.unique().tolist():       # read on the host
                rows = (choice == e).nonzero()[:, 0]
                y[rows] = torch.relu(xf[rows] @ self.up[e].T) @ self.down[e].T
            y = y * gate
            out[:] = out + y if accumulate else y

    @register_architecture
    @dataclass(frozen=True)
    class RoutedToyConfig(ModelConfig):
        hidden_size: int
        vocab_size: int
        experts: int
        routed: bool
        architecture_names = ("toy-routed",)

        def model_spec(self):
            h = self.hidden_size
            norm = PartSpec("rmsnorm", {"size": h, "eps": 1e-5})
            routed = PartSpec("toy_top1_experts", {"hidden_size": h, "experts": self.experts, "expert_size": 24})
            dense = PartSpec("gated_mlp", {"hidden_size": h, "intermediate_size": 2 * h, "activation": "silu"})
            arr = PartSpec("prenorm_residual", {"mixer_prefix": "mixer", "feed_forward_prefix": "ff",
                                                "mixer_norm_name": "norm1", "feed_forward_norm_name": "norm2"})
            attn = PartSpec("attention", {"hidden_size": h, "num_heads": 3, "num_kv_heads": 1, "head_dim": 16,
                                          "qk_norm": None,
                                          "position": PartSpec("toy_linear_angles",
                                                               {"rotary_dim": 12, "stretch": 4.0, "step": 0.3}),
                                          "window": None, "bias": False, "scale": 0.25})
            # layer 0 is dense, layer 1 routed (when asked for): parts are chosen layer by layer
            layers = (LayerSpec("layers.0", arr, attn, dense, norm, norm),
                      LayerSpec("layers.1", arr, attn, routed if self.routed else dense, norm, norm))
            return ModelSpec(
                hidden_size=h, vocab_size=self.vocab_size,
                embedding=PartSpec("token_embedding", {"name": "embed.weight", "vocab_size": self.vocab_size,
                                                       "hidden_size": h}),
                layers=layers, schedule=(ScheduleEntry(0, 0, True), ScheduleEntry(1, 1, True)),
                final_norm=PartSpec("rmsnorm", {"size": h, "eps": 1e-5, "name": "final_norm.weight"}),
                head=PartSpec("linear_head", {"name": "head.weight", "tied_to": None,
                                              "vocab_size": self.vocab_size, "hidden_size": h}))

    return RoutedToyConfig


def _linear_angles(positions, rotary_dim, stretch, step):
    pairs = torch.arange(1, rotary_dim // 2 + 1, dtype=torch.float64)
    return (positions.to(torch.float64) / stretch)[:, None] * (pairs * step)[None, :]


def _routed_toy_plain(w, tokens, hidden, experts, routed):
    """Plain float64 forward, whole sequence; also the smallest margin between a token's two best experts."""
    t = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    angles = _linear_angles(torch.arange(t), 12, 4.0, 0.3)
    cos, sin = angles.cos(), angles.sin()
    margin = float("inf")
    for layer in range(2):
        p = f"layers.{layer}"
        x = P.rmsnorm(h, w[f"{p}.norm1.weight"], 1e-5)
        q = P.linear(x, w[f"{p}.mixer.q_proj.weight"]).view(t, 3, 16)
        k = P.linear(x, w[f"{p}.mixer.k_proj.weight"]).view(t, 1, 16)
        v = P.linear(x, w[f"{p}.mixer.v_proj.weight"]).view(t, 1, 16)
        q = torch.cat([P.apply_rope(q[..., :12], cos, sin), q[..., 12:]], -1)
        k = torch.cat([P.apply_rope(k[..., :12], cos, sin), k[..., 12:]], -1)
        attn = P.causal_attention(q * (0.25 * 4.0), k, v)
        h = h + P.linear(attn.reshape(t, 48), w[f"{p}.mixer.o_proj.weight"])
        x = P.rmsnorm(h, w[f"{p}.norm2.weight"], 1e-5)
        if layer == 1 and routed:
            logits = x @ w[f"{p}.ff.router.weight"].T
            top = logits.topk(2, dim=-1).values
            margin = min(margin, float((top[:, 0] - top[:, 1]).min()))
            choice = logits.argmax(-1)
            gate = torch.softmax(logits, -1)
            rows = []
            for i in range(t):
                e = int(choice[i])
                mid = torch.relu(x[i] @ w[f"{p}.ff.experts.{e}.up.weight"].T)
                rows.append(gate[i, e] * (mid @ w[f"{p}.ff.experts.{e}.down.weight"].T))
            h = h + torch.stack(rows)
        else:
            h = h + P.mlp_block(w, f"{p}.ff", x)
    return P.linear(P.rmsnorm(h, w["final_norm.weight"], 1e-5), w["head.weight"]), margin


@pytest.mark.parametrize("routed", [True, False])
def test_toy_routed_feed_forward_and_toy_position_encoding(tmp_path, routed):
    """Parts of other kinds than the built-in ones, registered from outside: a routed feed-forward
    in one layer beside a dense one in the other, and a position encoding of its own behind the
    attention kernel.  The routed part reads its routing on the host, so the model must not
    capture decode steps; without it the steps are replayed from a graph, with the toy tables."""
    from lockstep_amd.config import unregister_architecture
    from lockstep_amd.engine.model import load_model
    from lockstep_amd.parts import unregister_part
    from lockstep_amd.weights import write_random_model
    from safetensors.torch import load_file

    RoutedToyConfig = _register_routed_toy()
    try:
        cfg = RoutedToyConfig(hidden_size=40, vocab_size=75, experts=3, routed=routed)
        folder = write_random_model(cfg, tmp_path / "routed", seed=8, std=0.25, norm_std=0.1)
        model = load_model(folder, dtype="float32")
        w = {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}
        assert ("layers.1.ff.experts.2.down.weight" in w) == routed and "layers.0.ff.gate_proj.weight" in w
        tokens = random_tokens(60, 75, seed=4)
        want, margin = _routed_toy_plain(w, tokens, 40, 3, routed)
        assert margin > 1e-3, "two experts nearly tie for a token: pick another seed"
        cache = model.make_cache(num_pages=24, page_size=8, max_requests=3, poison_on_free=True)
        whole = feed(model, cache, "w", tokens, [])
        assert rel_err(whole, want) < 5e-5
        cut = feed(model, cache, "c", tokens, [9, 2, 20] + [1] * 29)     # the tail as decode steps
        assert rel_err(cut, want) < 5e-5
        assert (model.graph_replays == 0) == routed, "a part that is not graph safe keeps the steps eager"
        cache.audit()
    finally:
        unregister_part("toy_linear_angles")
        unregister_part("toy_top1_experts")
        unregister_architecture(RoutedToyConfig)


# ---------------------------------------------------------------------------
# a third toy, for the shape of a layer itself: an arrangement with a norm in
# front of and behind each part (four norms), and one that is a feed-forward
# and nothing else -- parts beyond the common four travel in ``LayerSpec.parts``
# ---------------------------------------------------------------------------

def _register_sandwich_toy():
    from lockstep_amd.config import (LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry,
                                     register_architecture)
    from lockstep_amd.parts import Arrangement, build_part, part_class, register_part

    @register_part("toy_sandwich")
    class Sandwich(Arrangement):
        """``h += after_mixer(mixer(before_mixer(h))); h += after_ff(ff(before_ff(h)))``."""

        graph_safe = True
        NAMES = ("before_mixer", "mixer", "after_mixer", "before_ff", "ff", "after_ff")

        def __init__(self, layer_spec, prefix=""):
            super().__init__(layer_spec, build_part)
            for name in self.NAMES:
                setattr(self, f"p_{name}", build_part(layer_spec.part(name), self.join(layer_spec.prefix, name)))

        @classmethod
        def weight_specs(cls, layer_spec, prefix=""):
            return [w for name in cls.NAMES
                    for w in part_class(layer_spec.part(name).kind).weight_specs(layer_spec.part(name),
                                                                                 cls.join(layer_spec.prefix, name))]

        def parts(self):
            return tuple(getattr(self, f"p_{name}") for name in self.NAMES)

        mixer = property(lambda self: self.p_mixer)

        def load(self, weights, rt):
            for part in self.parts():
                part.load(weights, rt)

        def forward(self, ctx, run, h):
            rt, t, width = ctx.rt, ctx.n_tokens, h.shape[1]
            x = ctx.buf("sandwich.x", (t, width), rt.dtype)
            y = ctx.buf("sandwich.y", (t, width), torch.float32)
            z = ctx.buf("sandwich.z", (t, width), torch.float32)
            for before, part, after in ((self.p_before_mixer, self.p_mixer, self.p_after_mixer),
                                        (self.p_before_ff, self.p_ff, self.p_after_ff)):
                before.forward(ctx, h, x)
                if part is self.p_mixer:
                    part.forward(ctx, run, x, y, accumulate=False)
                else:
                    part.forward(ctx, x, y, accumulate=False)
                after.forward(ctx, y, z)                  # normalised into float32: the stream's own dtype
                h.add_(z)

    @register_part("toy_ff_only")
    class FeedForwardOnly(Arrangement):
        """``h += ff(norm(h))``: a layer that mixes nothing and keeps nothing."""

        graph_safe = True

        def __init__(self, layer_spec, prefix=""):
            super().__init__(layer_spec, build_part)
            self.norm = build_part(layer_spec.part("feed_forward_norm"), self.join(layer_spec.prefix, "norm"))
            self.ff = build_part(layer_spec.part("feed_forward"), self.join(layer_spec.prefix, "ff"))

        @classmethod
        def weight_specs(cls, layer_spec, prefix=""):
            norm, ff = layer_spec.part("feed_forward_norm"), layer_spec.part("feed_forward")
            return (part_class(norm.kind).weight_specs(norm, cls.join(layer_spec.prefix, "norm"))
                    + part_class(ff.kind).weight_specs(ff, cls.join(layer_spec.prefix, "ff")))

        def parts(self):
            return (self.norm, self.ff)

        mixer = property(lambda self: None)

        def load(self, weights, rt):
            self.norm.load(weights, rt)
            self.ff.load(weights, rt)

        def forward(self, ctx, run, h):
            x = ctx.buf("ff_only.x", (ctx.n_tokens, h.shape[1]), ctx.rt.dtype)
            self.norm.forward(ctx, h, x)
            self.ff.forward(ctx, x, h, accumulate=True)

    @register_architecture
    @dataclass(frozen=True)
    class SandwichConfig(ModelConfig):
        hidden_size: int
        vocab_size: int
        architecture_names = ("toy-sandwich",)

        def model_spec(self):
            h = self.hidden_size

            def norm(eps):
                return PartSpec("rmsnorm", {"size": h, "eps": eps})

            ff = PartSpec("gated_mlp", {"hidden_size": h, "intermediate_size": 3 * h, "activation": "silu"})
            attn = PartSpec("attention", {"hidden_size": h, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                          "qk_norm": None,
                                          "position": PartSpec("rope_half", {"rotary_dim": 16, "theta": 50.0}),
                                          "window": None, "bias": False, "scale": 0.25})
            sandwich = LayerSpec("layers.0", PartSpec("toy_sandwich"), mixer=attn,
                                 parts={"before_mixer": norm(1e-5), "after_mixer": norm(1e-4), "before_ff": norm(1e-3),
                                        "ff": ff, "after_ff": norm(1e-2)})
            ff_only = LayerSpec("layers.1", PartSpec("toy_ff_only"), feed_forward=ff, feed_forward_norm=norm(1e-5))
            return ModelSpec(
                hidden_size=h, vocab_size=self.vocab_size,
                embedding=PartSpec("token_embedding", {"name": "embed.weight", "vocab_size": self.vocab_size,
                                                       "hidden_size": h}),
                layers=(sandwich, ff_only),
                # the layer without a mixer names a cache unit like every run; it keeps nothing in it
                schedule=(ScheduleEntry(0, 0, True), ScheduleEntry(1, 1, True), ScheduleEntry(1, 1, True)),
                final_norm=PartSpec("rmsnorm", {"size": h, "eps": 1e-5, "name": "final_norm.weight"}),
                head=PartSpec("linear_head", {"name": "head.weight", "tied_to": None,
                                              "vocab_size": self.vocab_size, "hidden_size": h}))

    return SandwichConfig


def _sandwich_plain(w, tokens, hidden):
    t = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    cos, sin = P.rope_tables(16, 50.0, torch.arange(t))
    p = "layers.0"
    x = P.rmsnorm(h, w[f"{p}.before_mixer.weight"], 1e-5)
    q = P.apply_rope(P.linear(x, w[f"{p}.mixer.q_proj.weight"]).view(t, 4, 16), cos, sin)
    k = P.apply_rope(P.linear(x, w[f"{p}.mixer.k_proj.weight"]).view(t, 2, 16), cos, sin)
    v = P.linear(x, w[f"{p}.mixer.v_proj.weight"]).view(t, 2, 16)
    attn = P.causal_attention(q * (0.25 * 4.0), k, v)
    h = h + P.rmsnorm(P.linear(attn.reshape(t, 64), w[f"{p}.mixer.o_proj.weight"]), w[f"{p}.after_mixer.weight"], 1e-4)
    h = h + P.rmsnorm(P.mlp_block(w, f"{p}.ff", P.rmsnorm(h, w[f"{p}.before_ff.weight"], 1e-3)),
                      w[f"{p}.after_ff.weight"], 1e-2)
    for _ in range(2):                                       # the layer without a mixer runs twice
        h = h + P.mlp_block(w, "layers.1.ff", P.rmsnorm(h, w["layers.1.norm.weight"], 1e-5))
    return P.linear(P.rmsnorm(h, w["final_norm.weight"], 1e-5), w["head.weight"])


def test_layers_of_other_shapes_than_the_common_one(tmp_path):
    """A layer with four norms (two of them in ``LayerSpec.parts``, as is its feed-forward) and a layer
    that has no mixer at all, registered from outside: the weights are collected under the names the
    arrangements give them, the cache has one unit, and steps in portions and from replayed graphs
    equal the plain forward."""
    from lockstep_amd.config import ConfigError, LayerSpec, PartSpec, unregister_architecture
    from lockstep_amd.engine.model import load_model
    from lockstep_amd.parts import unregister_part
    from lockstep_amd.weights import write_random_model
    from safetensors.torch import load_file

    SandwichConfig = _register_sandwich_toy()
    try:
        cfg = SandwichConfig(hidden_size=48, vocab_size=90)
        spec = cfg.model_spec()
        assert set(spec.layers[0].named_parts()) == {"mixer", "before_mixer", "after_mixer", "before_ff", "ff", "after_ff"}
        assert spec.layers[1].mixer is None and not spec.layers[1].has("mixer")
        with pytest.raises(ConfigError, match="no part named 'gate'.*it has: feed_forward, feed_forward_norm"):
            spec.layers[1].part("gate")
        with pytest.raises(ConfigError, match="fields of the layer itself"):
            LayerSpec("x", PartSpec("toy_sandwich"), parts={"mixer": PartSpec("attention")})
        folder = write_random_model(cfg, tmp_path / "sandwich", seed=3, std=0.2, norm_std=0.2)
        w = {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}
        assert {"layers.0.after_ff.weight", "layers.0.before_mixer.weight", "layers.0.ff.down_proj.weight",
                "layers.1.norm.weight", "layers.1.ff.gate_proj.weight"} <= set(w)
        model = load_model(folder, dtype="float32")
        assert [type(u).__name__ for u in model.cache_unit_specs()] == ["PagedKVSpec", "NoneType"]
        tokens = random_tokens(50, 90, seed=6)
        want = _sandwich_plain(w, tokens, 48)
        cache = model.make_cache(num_pages=24, page_size=8, max_requests=3, poison_on_free=True)
        assert len(cache.groups) == 1 and not cache.state_units and cache.shareable()
        whole = feed(model, cache, "w", tokens, [])
        assert rel_err(whole, want) < 5e-5
        cut = feed(model, cache, "c", tokens, [7, 2, 21] + [1] * 20)
        assert rel_err(cut, want) < 5e-5
        assert model.graph_replays > 10
        cache.audit()
    finally:
        unregister_part("toy_sandwich")
        unregister_part("toy_ff_only")
        unregister_architecture(SandwichConfig)
