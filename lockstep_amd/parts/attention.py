"""Grouped-query attention over the paged cache.

Order of operations, as in the reference (engine/model/qwen3.py:327-363):
projections of the normalised hidden rows (no bias), optional RMSNorm per head
on q and k with one ``[d]`` weight for all heads, position encoding on q and
k, keys and values written to the request's pages, causal attention of the
step's queries over everything the request has cached (its own keys of this
step included), output projection added to the residual stream.

The three projections are one matrix product over the concatenation
``[Wq; Wk; Wv]`` (each output column keeps its own sum over the hidden size,
so this changes nothing in the result).  Norm, rotation and cache write are
one kernel; attention is one launch for all requests of the step.
"""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from ..ops import ADD_F32, STORE_F32
from .base import Mixer, PagedKVSpec, PendingAdd, WeightSpec, build_part, deferred_rows, register_part

import os

# Steps of single decoded tokens run norm, rotation and cache write inside the
# attention kernel (one launch less per layer); "0" keeps the separate kernel.
FUSE_DECODE = os.environ.get("LOCKSTEP_FUSE_DECODE", "1") not in ("", "0")
# From this many attention workgroups on (two a CU: the kernel is then bound by the cache it streams) the
# prologue of the fused kernel costs more than the separate norm/rotation launch; measured +2 % at batch 64.
FUSE_DECODE_BELOW = int(os.environ.get("LOCKSTEP_FUSE_DECODE_BELOW", "512"))


@register_part("attention")
class Attention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``,
    ``head_dim``, ``qk_norm`` (a norm ``PartSpec`` or None), ``position`` (a
    position-encoding ``PartSpec``), ``window`` (keys visible to a query,
    None for all), ``bias`` (must be False), ``scale`` (score multiplier)."""

    graph_safe = True

    def parts(self):
        return (self.position,)

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nq = int(p["num_heads"])
        self.nkv = int(p["num_kv_heads"])
        self.d = int(p["head_dim"])
        self.window = p.get("window")
        self.scale = float(p["scale"])
        if p.get("bias"):
            raise ValueError("attention with projection biases is not built")
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} kv heads")
        if self.d % 16 or not 16 <= self.d <= 256:
            raise ValueError(f"head size {self.d} is not supported: the attention kernels take "
                             "multiples of 16 from 16 to 256")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"window {self.window} must be positive")
        self.qk_norm_spec = p.get("qk_norm")
        self.position = build_part(p["position"], prefix)
        if self.position.rotary_dim > self.d:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head size {self.d}")
        self.w_qkv = self.w_q = self.w_o = self.q_norm = self.k_norm = None
        self.norm_eps = float(self.qk_norm_spec["eps"]) if self.qk_norm_spec else 0.0
        if self.qk_norm_spec is not None:
            if self.qk_norm_spec.kind != "rmsnorm" or int(self.qk_norm_spec["size"]) != self.d:
                raise ValueError("the per-head norm must be an rmsnorm over the head size")

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, nq, nkv, d = int(p["hidden_size"]), int(p["num_heads"]), int(p["num_kv_heads"]), int(p["head_dim"])
        out = [
            WeightSpec(f"{prefix}.q_proj.weight", (nq * d, h)),
            WeightSpec(f"{prefix}.k_proj.weight", (nkv * d, h)),
            WeightSpec(f"{prefix}.v_proj.weight", (nkv * d, h)),
            WeightSpec(f"{prefix}.o_proj.weight", (h, nq * d)),
        ]
        if p.get("qk_norm") is not None:
            out += [WeightSpec(f"{prefix}.q_norm.weight", (d,), kind="vector", init="norm"),
                    WeightSpec(f"{prefix}.k_norm.weight", (d,), kind="vector", init="norm")]
        return out

    def cache_spec(self):
        return PagedKVSpec(self.nkv, self.d, int(self.window) if self.window is not None else None)

    def load(self, weights, rt) -> None:
        q = weights.get(f"{self.prefix}.q_proj.weight")
        k = weights.get(f"{self.prefix}.k_proj.weight")
        v = weights.get(f"{self.prefix}.v_proj.weight")
        self.w_qkv = rt.matrix(torch.cat([q.to(torch.float32), k.to(torch.float32), v.to(torch.float32)], dim=0)
                               if len({q.dtype, k.dtype, v.dtype}) > 1 else torch.cat([q, k, v], dim=0))
        self.w_q = self.w_qkv[: self.nq * self.d]
        self.w_o = rt.matrix(weights.get(f"{self.prefix}.o_proj.weight"))
        if self.qk_norm_spec is not None:
            self.q_norm = rt.vector(weights.get(f"{self.prefix}.q_norm.weight"))
            self.k_norm = rt.vector(weights.get(f"{self.prefix}.k_norm.weight"))
        rt.kernels.attention_lib(self.d)
        if hasattr(self.position, "bind"):
            self.position.bind(rt)      # layers with equal constants share their tables

    def prepare_group(self):
        share = getattr(self.position, "share_key", None)
        if share is None:
            return None
        return ("attention", self.nq, self.nkv, self.d, self.window, share())

    def prepare(self, ctx) -> None:
        self.position.ensure(ctx.max_position + 1, ctx.rt)
        ctx.plan_attention(self.nq // self.nkv, self.nkv, self.d, int(self.window) if self.window is not None else 0)

    def forward(self, ctx, run, x, out, accumulate: bool, norm=None, defer: bool = False):
        """``norm``: when given, ``x`` is the float32 residual stream and ``norm``
        (an RMSNorm part) is applied inside the projection.  ``defer``: the addition
        of the output projection to ``out`` may be left to the caller (a ``PendingAdd``
        is returned)."""
        rt = ctx.rt
        k = rt.kernels
        t = ctx.n_tokens
        nq, nkv, d = self.nq, self.nkv, self.d
        group, key_pages, value_pages = ctx.cache.unit_pages(run.cache)
        width = (nq + 2 * nkv) * d
        qkv = ctx.buf("attention.qkv", (t, width), rt.dtype)
        fused = {} if norm is None else {"norm_weight": norm.weight, "eps": norm.eps}
        if run.writes_cache:
            k.gemm(x, self.w_qkv, qkv, **fused)
        else:
            k.gemm(x, self.w_q, qkv[:, : nq * d], **fused)
        attn = ctx.buf("attention.out", (t, nq * d), rt.dtype)
        window = int(self.window) if self.window is not None else 0
        plan = ctx.attention_plan(nq // nkv, nkv, d, window)
        if plan.decode_fused and FUSE_DECODE and plan.n_coop * nkv < FUSE_DECODE_BELOW:
            # single decoded tokens: norm, rotation and cache write happen inside the attention kernel
            k.attention_decode(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                               plan.coop_items, plan.n_coop, attn, plan.part_acc, plan.part_ml, self.scale, window,
                               self.q_norm, self.k_norm, self.norm_eps, self.position.cos, self.position.sin,
                               self.position.rotary_dim, ctx.max_position, run.writes_cache)
            if plan.n_combine:
                k.attention_combine(d, ctx.seqs, plan.combine_items, plan.n_combine, nq, nkv, plan.part_acc,
                                    plan.part_ml, attn)
            return self._project_out(ctx, attn, out, accumulate, defer)
        k.qk_rope_kv(qkv, t, nq, nkv, d, self.q_norm, self.k_norm, self.norm_eps, self.position.cos,
                     self.position.sin, self.position.rotary_dim, ctx.tok_seq, ctx.tok_pos, ctx.seqs,
                     ctx.max_position, group.table, key_pages, value_pages, group.page_size, run.writes_cache)
        if plan.n_items:
            k.attention(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                        plan.items, plan.n_items, attn, plan.part_acc, plan.part_ml, self.scale, window)
        if plan.n_coop:
            k.attention(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                        plan.coop_items, plan.n_coop, attn, plan.part_acc, plan.part_ml, self.scale, window,
                        variant=3, max_rows=plan.coop_max_rows)
        if plan.n_wide:
            k.attention(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                        plan.wide_items, plan.n_wide, attn, plan.part_acc, plan.part_ml, self.scale, window,
                        variant=plan.wide_variant)
        if plan.n_combine:
            k.attention_combine(d, ctx.seqs, plan.combine_items, plan.n_combine, nq, nkv, plan.part_acc,
                                plan.part_ml, attn)
        return self._project_out(ctx, attn, out, accumulate, defer)

    def _project_out(self, ctx, attn, out, accumulate: bool, defer: bool):
        k = ctx.rt.kernels
        if defer and accumulate and 0 < ctx.n_tokens <= deferred_rows(ctx, self.nq * self.d, out.shape[1]):
            slices = k.gemm_slices_count(self.nq * self.d)
            partials = ctx.buf("attention.out_slices", (slices * ctx.n_tokens, out.shape[1]), torch.float32)
            partials = partials.view(slices, ctx.n_tokens, out.shape[1])
            k.gemm_slices(attn, self.w_o, partials)
            return PendingAdd(partials)
        k.gemm(attn, self.w_o, out, ADD_F32 if accumulate else STORE_F32)
        return None
