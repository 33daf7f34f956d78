"""RMSNorm: ``y = x * 1/sqrt(mean(x^2) + eps) * w`` in 32-bit
(reference engine/kernels/rmsnorm.py:30-38)."""

from __future__ import annotations

from ..config.base import PartSpec
from .base import Norm, WeightSpec, register_part


@register_part("rmsnorm")
class RMSNorm(Norm):
    """Parameters: ``size``, ``eps``; ``name`` overrides the tensor name."""

    graph_safe = True
    repeatable = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.weight = None

    @staticmethod
    def tensor_name(spec: PartSpec, prefix: str) -> str:
        return spec.params.get("name") or f"{prefix}.weight"

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        return [WeightSpec(cls.tensor_name(spec, prefix), (int(spec["size"]),), kind="vector", init="norm")]

    def load(self, weights, rt) -> None:
        self.weight = rt.vector(weights.get(self.tensor_name(self.spec, self.prefix)))

    def forward(self, ctx, x, out, rows=None, pending=None) -> None:
        """``pending`` (a ``PendingAdd``): added to ``x`` first, in the same launch."""
        if pending is not None:
            ctx.rt.kernels.add_rmsnorm(x, pending.partials, self.weight, out, self.eps, rows)
        else:
            ctx.rt.kernels.rmsnorm(x, self.weight, out, self.eps, rows)
