"""Gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases; with the
SiLU activation this is the reference's SwiGLU MLP
(engine/model/qwen3.py:368-370, engine/kernels/swiglu.py:25-29).  Gate and up
are one matrix product over their rows interleaved in tiles of 16, whose
epilogue applies the activation, so the two projections never leave the
kernel."""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from ..ops import ADD_F32, STORE_F32, SWIGLU, interleave_gate_up
from .base import FeedForward, PendingAdd, WeightSpec, deferred_rows, register_part


@register_part("gated_mlp")
class GatedMLP(FeedForward):
    """Parameters: ``hidden_size``, ``intermediate_size``, ``activation``."""

    graph_safe = True
    repeatable = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        if spec["activation"] != "silu":
            raise ValueError(f"activation {spec['activation']!r} is not built; known: silu")
        self.w_gate_up = self.w_down = None

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
        return [WeightSpec(f"{prefix}.gate_proj.weight", (i, h)),
                WeightSpec(f"{prefix}.up_proj.weight", (i, h)),
                WeightSpec(f"{prefix}.down_proj.weight", (h, i))]

    def load(self, weights, rt) -> None:
        gate = weights.get(f"{self.prefix}.gate_proj.weight")
        up = weights.get(f"{self.prefix}.up_proj.weight")
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        self.w_gate_up = rt.matrix(interleave_gate_up(gate, up))
        self.w_down = rt.matrix(weights.get(f"{self.prefix}.down_proj.weight"))

    def forward(self, ctx, x, out, accumulate: bool, norm=None, defer: bool = False):
        """``norm``: when given, ``x`` is the float32 residual stream and ``norm``
        (an RMSNorm part) is applied inside the first matrix product.  ``defer``: the
        addition to ``out`` may be left to the caller (a ``PendingAdd`` is returned)."""
        rt = ctx.rt
        act = ctx.buf("mlp.act", (ctx.n_tokens, self.inter), rt.dtype)
        if norm is None:
            rt.kernels.gemm(x, self.w_gate_up, act, SWIGLU)
        else:
            rt.kernels.gemm(x, self.w_gate_up, act, SWIGLU, norm_weight=norm.weight, eps=norm.eps)
        if defer and accumulate and 0 < ctx.n_tokens <= deferred_rows(ctx, self.inter, out.shape[1]):
            slices = rt.kernels.gemm_slices_count(self.inter)
            partials = ctx.buf("mlp.down_slices", (slices * ctx.n_tokens, out.shape[1]), torch.float32)
            partials = partials.view(slices, ctx.n_tokens, out.shape[1])
            rt.kernels.gemm_slices(act, self.w_down, partials)
            return PendingAdd(partials)
        rt.kernels.gemm(act, self.w_down, out, ADD_F32 if accumulate else STORE_F32)
        return None
