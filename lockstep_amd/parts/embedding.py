"""Token embedding and output head."""

from __future__ import annotations

from ..config.base import PartSpec
from ..ops import STORE_F32
from .base import Part, WeightSpec, register_part


@register_part("token_embedding")
class TokenEmbedding(Part):
    """``h[t] = E[token[t]]``, no scaling (reference engine/model/qwen3.py:319).
    Parameters: ``name``, ``vocab_size``, ``hidden_size``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.table = None

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        return [WeightSpec(spec["name"], (int(spec["vocab_size"]), int(spec["hidden_size"])))]

    def load(self, weights, rt) -> None:
        self.table = rt.matrix(weights.get(self.spec["name"]), share_key=weights.source_name(self.spec["name"]))

    def forward(self, ctx, tokens, out) -> None:
        ctx.rt.kernels.embed(tokens, self.table, out)


@register_part("linear_head")
class LinearHead(Part):
    """``logits = x @ W^T`` in float32, no bias and no scaling (reference
    engine/model/qwen3.py:373).  Parameters: ``name``, ``tied_to`` (a tensor
    name the head aliases when the checkpoint does not hold its own, or None),
    ``vocab_size``, ``hidden_size``."""

    graph_safe = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.weight = None
        self.vocab = int(spec["vocab_size"])

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        return [WeightSpec(spec["name"], (int(spec["vocab_size"]), int(spec["hidden_size"])))]

    @classmethod
    def ties(cls, spec: PartSpec) -> dict[str, str]:
        return {spec["name"]: spec["tied_to"]} if spec.params.get("tied_to") else {}

    def load(self, weights, rt) -> None:
        self.weight = rt.matrix(weights.get(self.spec["name"]), share_key=weights.source_name(self.spec["name"]))

    def forward(self, ctx, x, logits) -> None:
        ctx.rt.kernels.gemm(x, self.weight, logits, STORE_F32)
