"""Gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases; with the
SiLU activation this is the reference's SwiGLU MLP
(engine/model/qwen3.py:368-370, engine/kernels/swiglu.py:25-29).  Gate and up
are one matrix product over ``[Wg; Wu]``."""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from ..ops import ADD_F32, STORE_F32
from .base import FeedForward, WeightSpec, register_part


@register_part("gated_mlp")
class GatedMLP(FeedForward):
    """Parameters: ``hidden_size``, ``intermediate_size``, ``activation``."""

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
        self.w_gate_up = rt.matrix(torch.cat([gate, up], dim=0))
        self.w_down = rt.matrix(weights.get(f"{self.prefix}.down_proj.weight"))

    def forward(self, ctx, x, out, accumulate: bool) -> None:
        rt = ctx.rt
        t = ctx.n_tokens
        gate_up = ctx.buf("mlp.gate_up", (t, 2 * self.inter), rt.dtype)
        rt.kernels.gemm(x, self.w_gate_up, gate_up)
        act = ctx.buf("mlp.act", (t, self.inter), rt.dtype)
        rt.kernels.swiglu(gate_up, act)
        rt.kernels.gemm(act, self.w_down, out, ADD_F32 if accumulate else STORE_F32)
