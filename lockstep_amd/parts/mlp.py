"""Gated feed-forward: ``down(act(gate(x)) * up(x))``, with biases if asked for; with the
SiLU activation and without biases this is the reference's SwiGLU MLP
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
    """Parameters: ``hidden_size``, ``intermediate_size``, ``activation`` (``silu``, ``gelu``,
    ``gelu_tanh``, ``relu``), ``bias`` (optional, default False: ``gate_proj.bias``, ``up_proj.bias``
    and ``down_proj.bias``).

    SiLU without biases is the fast path (the activation is the product's epilogue).  Anything else
    stores the gate/up product in float32 and applies biases and activation in a pass of its own,
    and adds the down projection to the residual stream at once rather than leaving it to the next
    norm, so that the order of the additions (stream + product, then + bias) is the same at every
    batch size."""

    graph_safe = True
    repeatable = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = str(spec["activation"])
        self.bias = bool(spec.params.get("bias", False))
        if self.activation not in ("silu", "gelu", "gelu_tanh", "relu"):
            raise ValueError(f"activation {self.activation!r} is not built; known: silu, gelu, gelu_tanh, relu")
        self.fused = self.activation == "silu" and not self.bias
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
        out = [WeightSpec(f"{prefix}.gate_proj.weight", (i, h)),
               WeightSpec(f"{prefix}.up_proj.weight", (i, h)),
               WeightSpec(f"{prefix}.down_proj.weight", (h, i))]
        if spec.params.get("bias", False):
            out += [WeightSpec(f"{prefix}.gate_proj.bias", (i,), kind="vector"),
                    WeightSpec(f"{prefix}.up_proj.bias", (i,), kind="vector"),
                    WeightSpec(f"{prefix}.down_proj.bias", (h,), kind="vector")]
        return out

    def load(self, weights, rt) -> None:
        gate = weights.get(f"{self.prefix}.gate_proj.weight")
        up = weights.get(f"{self.prefix}.up_proj.weight")
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        self.w_gate_up = rt.matrix(interleave_gate_up(gate, up) if self.fused else torch.cat([gate, up], dim=0))
        self.w_down = rt.matrix(weights.get(f"{self.prefix}.down_proj.weight"))
        if self.bias:
            self.b_gate_up = rt.vector(torch.cat([weights.get(f"{self.prefix}.gate_proj.bias").to(torch.float32),
                                                  weights.get(f"{self.prefix}.up_proj.bias").to(torch.float32)]))
            self.b_down = rt.vector(weights.get(f"{self.prefix}.down_proj.bias"))

    def forward(self, ctx, x, out, accumulate: bool, norm=None, defer: bool = False):
        """``norm``: when given, ``x`` is the float32 residual stream and ``norm``
        (an RMSNorm part) is applied inside the first matrix product.  ``defer``: the
        addition to ``out`` may be left to the caller (a ``PendingAdd`` is returned)."""
        rt = ctx.rt
        k = rt.kernels
        act = ctx.buf("mlp.act", (ctx.n_tokens, self.inter), rt.dtype)
        fused_norm = {} if norm is None else {"norm_weight": norm.weight, "eps": norm.eps}
        if not self.fused:
            wide = ctx.buf("mlp.gate_up", (ctx.n_tokens, 2 * self.inter), torch.float32)
            k.gemm(x, self.w_gate_up, wide, STORE_F32, **fused_norm)
            k.bias_act(wide, self.b_gate_up, act, self.activation, gated=True)
            k.gemm(act, self.w_down, out, ADD_F32 if accumulate else STORE_F32)
            if self.b_down is not None:
                k.bias_act(out, self.b_down, out)
            return None
        k.gemm(x, self.w_gate_up, act, SWIGLU, **fused_norm)
        if defer and accumulate and 0 < ctx.n_tokens <= deferred_rows(ctx, self.inter, out.shape[1]):
            slices = k.gemm_slices_count(self.inter)
            partials = ctx.buf("mlp.down_slices", (slices * ctx.n_tokens, out.shape[1]), torch.float32)
            partials = partials.view(slices, ctx.n_tokens, out.shape[1])
            k.gemm_slices(act, self.w_down, partials)
            return PendingAdd(partials)
        k.gemm(act, self.w_down, out, ADD_F32 if accumulate else STORE_F32)
        return None
