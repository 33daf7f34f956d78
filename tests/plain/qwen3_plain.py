"""Plain, slow implementation of the Qwen3 dense decoder: the oracle of the tests.

Whole sequences, no cache, one function for each part, CPU torch only.  It
shares no code with ``lockstep_amd``: it reads ``config.json`` and
``model.safetensors`` by itself (through the ``safetensors`` package, which
the engine does not use) and computes every formula directly from the
reference's text.  Every function cites the reference lines it was written
from (paths are relative to the reference checkout).

The default precision is float64; ``dtype=torch.float32`` gives the 32-bit
variant.  Weights are used at the values the checkpoint holds (bfloat16
values upcast exactly), as in bench/fp64_reference.py:76-80.

``store`` (optional, on the functions that take it) is applied wherever the
engine under test keeps a value in its 16-bit compute dtype between kernels:
the normalised rows that enter a projection, the projected q, k and v, q and
k after norm and rotation, the probabilities that multiply the values (the
row sum is formed from the unrounded ones, engine/kernels/attention.py:111-112),
the attention output, the activated feed-forward rows and the final
normalised rows.  The residual stream and the logits stay unrounded, which is
the engine's own contract (the reference rounds its residual stream too,
engine/model/qwen3.py:360,370).  With ``store=bf16`` the plain forward is the
exact-arithmetic model of the bfloat16 path: what is left between the two is
the order of sums and values that sit on a rounding boundary.
"""

from __future__ import annotations

import hashlib
import json
import math
from pathlib import Path

import torch

# --------------------------------------------------------------------------
# configuration and weights
# --------------------------------------------------------------------------

CONFIG_KEYS = (
    "hidden_size",
    "intermediate_size",
    "num_hidden_layers",
    "num_attention_heads",
    "num_key_value_heads",
    "head_dim",
    "vocab_size",
    "rms_norm_eps",
    "rope_theta",
    "max_position_embeddings",
    "tie_word_embeddings",
)


def read_config(model_dir) -> dict:
    """The eleven keys the model reads, no defaults (engine/model/qwen3.py:63-80)."""
    raw = json.loads((Path(model_dir) / "config.json").read_text())
    if raw.get("model_type") != "qwen3":
        raise ValueError(f"expected a qwen3 config, got {raw.get('model_type')!r}")
    return {key: raw[key] for key in CONFIG_KEYS}


def read_weights(model_dir, cfg: dict, dtype=torch.float64) -> dict:
    """Tensors by exact name, upcast; tied head aliases the embedding
    (engine/model/qwen3.py:153-174,201-202; bench/fp64_reference.py:59-80)."""
    from safetensors.torch import load_file

    tensors = load_file(str(Path(model_dir) / "model.safetensors"))
    if cfg["tie_word_embeddings"]:
        if "lm_head.weight" in tensors:
            if not torch.equal(tensors["lm_head.weight"], tensors["model.embed_tokens.weight"]):
                raise ValueError("tie_word_embeddings set but the two tensors differ")
        tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"]
    return {name: t.to(dtype) for name, t in tensors.items()}


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x @ W^T`` with ``W [out, in]``, no bias
    (engine/kernels/gemm.py:32,49-63; bench/fp64_reference.py:84-85)."""
    return x @ weight.T


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x * 1/sqrt(mean(x^2) + eps) * w`` over the last dimension
    (engine/kernels/rmsnorm.py:30-38; bench/fp64_reference.py:87-91)."""
    variance = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(variance + eps)) * weight


def rope_tables(head_dim: int, theta: float, positions: torch.Tensor):
    """cos and sin ``[len(positions), head_dim/2]``: ``inv_freq[i] = theta^(-2i/d)``,
    angle = position * inv_freq, computed in float64
    (engine/model/qwen3.py:117-129; bench/fp64_reference.py:93-98)."""
    half = head_dim // 2
    exponent = torch.arange(0, half, dtype=torch.float64) * 2.0 / head_dim
    inv_freq = 1.0 / (float(theta) ** exponent)
    angles = positions.to(torch.float64)[:, None] * inv_freq[None, :]
    return angles.cos(), angles.sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Half rotation over the whole head: pairs are (i, i + d/2);
    ``out_lo = lo*c - hi*s``, ``out_hi = hi*c + lo*s``.  ``x [T, heads, d]``
    (engine/kernels/rope.py:38-45; bench/fp64_reference.py:100-105)."""
    half = x.shape[-1] // 2
    lo, hi = x[..., :half], x[..., half:]
    c = cos[:, None, :].to(x.dtype)
    s = sin[:, None, :].to(x.dtype)
    return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1)


def bf16(x: torch.Tensor) -> torch.Tensor:
    """Round to the nearest bfloat16 (ties to even), kept in the input's dtype."""
    return x.to(torch.float32).to(torch.bfloat16).to(x.dtype)


def _keep(x: torch.Tensor) -> torch.Tensor:
    return x


def stable_softmax(scores: torch.Tensor) -> torch.Tensor:
    """Explicit max-subtract softmax over the last dimension
    (bench/fp64_reference.py:41-50)."""
    m = scores.max(dim=-1, keepdim=True).values
    e = (scores - m).exp()
    return e / e.sum(dim=-1, keepdim=True)


def causal_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    q_positions: torch.Tensor | None = None,
    window: int | None = None,
    store=None,
    also_hidden: torch.Tensor | None = None,
) -> torch.Tensor:
    """Grouped-query causal attention of whole sequences.

    ``q [Tq, nq, d]``, ``k, v [Tk, nkv, d]``; query head ``h`` reads kv head
    ``h // (nq/nkv)`` (repeat_interleave); scores are ``q.k`` times
    ``1/sqrt(d)``; key ``n`` is visible to the query at position ``p`` iff
    ``n <= p`` (engine/kernels/attention.py:74,96-99;
    bench/fp64_reference.py:136-142).  ``q_positions`` defaults to
    ``Tk - Tq + arange(Tq)``: the queries are the tail of the keys
    (engine/kernels/attention.py:224-227).  ``window`` is not in the
    reference: when given, a key is also dropped once ``p - n >= window``.
    ``also_hidden`` (bool ``[Tq, Tk]``, not in the reference either) hides further
    keys: tests use it to state what a fault (a dropped key, a lost page) would give.
    """
    tq, nq, d = q.shape
    tk, nkv, _ = k.shape
    group = nq // nkv
    if q_positions is None:
        q_positions = torch.arange(tk - tq, tk)
    k = k.repeat_interleave(group, dim=1)
    v = v.repeat_interleave(group, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * (1.0 / math.sqrt(d))
    key_positions = torch.arange(tk)
    hidden = key_positions[None, :] > q_positions[:, None]
    if window is not None:
        hidden = hidden | (q_positions[:, None] - key_positions[None, :] >= window)
    if also_hidden is not None:
        hidden = hidden | also_hidden
    scores = scores.masked_fill(hidden[None], float("-inf"))
    if store is None:
        return torch.einsum("hqk,khd->qhd", stable_softmax(scores), v)
    # the stored probabilities multiply the values, the unrounded ones form the row sum
    e = (scores - scores.max(dim=-1, keepdim=True).values).exp()
    return torch.einsum("hqk,khd->qhd", store(e), v) / e.sum(dim=-1).transpose(0, 1)[..., None]


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``gate * sigmoid(gate) * up`` (engine/kernels/swiglu.py:25-29;
    bench/fp64_reference.py:153)."""
    return gate * torch.sigmoid(gate) * up


def attention_block(cfg: dict, w: dict, prefix: str, x: torch.Tensor, positions: torch.Tensor, store=None,
                    window: int | None = None, also_hidden: torch.Tensor | None = None):
    """Projections, per-head q/k norm, rotation, attention, output projection
    (engine/model/qwen3.py:327-363; bench/fp64_reference.py:122-148).  The
    per-head norm uses one ``[d]`` weight for all heads, is applied to q and k
    only, and comes before the rotation."""
    keep = store or _keep
    t = x.shape[0]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = keep(linear(x, w[f"{prefix}.q_proj.weight"])).view(t, nq, d)
    k = keep(linear(x, w[f"{prefix}.k_proj.weight"])).view(t, nkv, d)
    v = keep(linear(x, w[f"{prefix}.v_proj.weight"])).view(t, nkv, d)
    q = rmsnorm(q, w[f"{prefix}.q_norm.weight"], cfg["rms_norm_eps"])
    k = rmsnorm(k, w[f"{prefix}.k_norm.weight"], cfg["rms_norm_eps"])
    cos, sin = rope_tables(d, cfg["rope_theta"], positions)
    q = keep(apply_rope(q, cos, sin))
    k = keep(apply_rope(k, cos, sin))
    attn = keep(causal_attention(q, k, v, q_positions=positions - positions[0], window=window, store=store,
                                 also_hidden=also_hidden))
    return linear(attn.reshape(t, nq * d), w[f"{prefix}.o_proj.weight"])


def mlp_block(w: dict, prefix: str, x: torch.Tensor, store=None) -> torch.Tensor:
    """``down(swiglu(gate(x), up(x)))`` (engine/model/qwen3.py:368-370;
    bench/fp64_reference.py:150-153)."""
    gate = linear(x, w[f"{prefix}.gate_proj.weight"])
    up = linear(x, w[f"{prefix}.up_proj.weight"])
    return linear((store or _keep)(swiglu(gate, up)), w[f"{prefix}.down_proj.weight"])


def hidden_states(cfg: dict, w: dict, token_ids, dtype=torch.float64, store=None, also_hidden=None) -> torch.Tensor:
    """Final normalised hidden states ``[T, H]`` of one whole sequence from
    position 0: embedding, then per layer ``h += attn(norm(h))`` and
    ``h += mlp(norm(h))``, then the final norm
    (engine/model/qwen3.py:319-372; bench/fp64_reference.py:107-155)."""
    ids = torch.as_tensor(list(token_ids), dtype=torch.long)
    positions = torch.arange(ids.shape[0])
    h = w["model.embed_tokens.weight"][ids].to(dtype)
    eps = cfg["rms_norm_eps"]
    keep = store or _keep
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        normed = keep(rmsnorm(h, w[f"{p}.input_layernorm.weight"], eps))
        h = h + attention_block(cfg, w, f"{p}.self_attn", normed, positions, store,
                                also_hidden=(also_hidden or {}).get(layer))
        normed = keep(rmsnorm(h, w[f"{p}.post_attention_layernorm.weight"], eps))
        h = h + mlp_block(w, f"{p}.mlp", normed, store)
    return keep(rmsnorm(h, w["model.norm.weight"], eps))


def logits(cfg: dict, w: dict, token_ids, dtype=torch.float64, store=None, also_hidden=None) -> torch.Tensor:
    """Logits ``[T, V]`` at every position: ``norm(h) @ lm_head^T``, no bias
    and no scaling (engine/model/qwen3.py:372-373;
    bench/fp64_reference.py:157-164)."""
    return linear(hidden_states(cfg, w, token_ids, dtype, store, also_hidden), w["lm_head.weight"])


class PlainModel:
    """A model folder opened by the plain implementation."""

    def __init__(self, model_dir, dtype=torch.float64):
        self.cfg = read_config(model_dir)
        self.dtype = dtype
        self.w = read_weights(model_dir, self.cfg, dtype)

    def logits(self, token_ids, store=None, also_hidden=None) -> torch.Tensor:
        """``also_hidden``: {layer: bool [T, T]} of keys to hide from queries in that layer."""
        return logits(self.cfg, self.w, token_ids, self.dtype, store, also_hidden)

    def generate_greedy(self, prompt, max_new_tokens: int, eos=()) -> list[int]:
        """Whole-sequence recomputation at every step, lowest-id tie-break
        (engine/model/qwen3.py:381-402 with engine/sampler/philox.py:64-68)."""
        context = list(prompt)
        out: list[int] = []
        for _ in range(max_new_tokens):
            token = greedy(self.logits(context)[-1])
            out.append(token)
            context.append(token)
            if token in eos:
                break
        return out


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------

_M32 = 0xFFFFFFFF


def philox_4x32(counter, key, rounds: int = 10):
    """Philox-4x32 with ten rounds on Python integers
    (engine/sampler/philox.py:9-47)."""
    c0, c1, c2, c3 = (x & _M32 for x in counter)
    k0, k1 = (x & _M32 for x in key)
    for r in range(rounds):
        p0 = 0xD2511F53 * c0
        p1 = 0xCD9E8D57 * c2
        hi0, lo0 = (p0 >> 32) & _M32, p0 & _M32
        hi1, lo1 = (p1 >> 32) & _M32, p1 & _M32
        c0, c1, c2, c3 = (hi1 ^ c1 ^ k0) & _M32, lo1, (hi0 ^ c3 ^ k1) & _M32, lo0
        if r < rounds - 1:
            k0 = (k0 + 0x9E3779B9) & _M32
            k1 = (k1 + 0xBB67AE85) & _M32
    return c0, c1, c2, c3


def uniform(seed: int, uid: str, position: int, index: int = 0) -> float:
    """A draw in [0, 1) that is a pure function of (seed, uid, position):
    counter (pos_lo, pos_hi, index, 0), key = seed XOR the first eight bytes
    (big-endian) of sha256(uid) (engine/sampler/philox.py:19-21,54-61)."""
    key64 = int.from_bytes(hashlib.sha256(uid.encode("utf-8")).digest()[:8], "big")
    mixed = seed ^ key64
    words = philox_4x32(
        (position & _M32, (position >> 32) & _M32, index & _M32, 0),
        (mixed & _M32, (mixed >> 32) & _M32),
    )
    return words[0] * 2.0**-32


def greedy(row: torch.Tensor) -> int:
    """Lowest index among the maxima of the row in float32
    (engine/sampler/philox.py:64-68)."""
    values = row.to(torch.float32)
    best = values.max()
    return int(torch.nonzero(values == best)[0].item())


def top_p(row: torch.Tensor, seed: int, uid: str, position: int, p: float = 1.0,
          temperature: float = 1.0) -> int:
    """Nucleus sampling (engine/sampler/philox.py:71-98): temperature <= 0 is
    greedy; else float32(row)/T in float64, softmax, order by (-prob, id),
    keep the shortest head whose cumulative sum reaches p, draw
    ``u * sum(head)`` and take the first index whose cumulative sum reaches it."""
    if temperature <= 0:
        return greedy(row)
    values = (row.to(torch.float32) / temperature).to(torch.float64)
    probs = stable_softmax(values)
    order = sorted(range(probs.numel()), key=lambda i: (-float(probs[i]), i))
    ordered = probs[torch.tensor(order)]
    cumulative = torch.cumsum(ordered, dim=0)
    keep = int(torch.searchsorted(cumulative, torch.tensor(p, dtype=torch.float64)).item()) + 1
    keep = min(keep, len(order))
    head = ordered[:keep]
    draw = uniform(seed, uid, position) * float(head.sum())
    chosen = int(torch.searchsorted(torch.cumsum(head, dim=0), torch.tensor(draw, dtype=torch.float64)).item())
    return order[min(chosen, keep - 1)]
