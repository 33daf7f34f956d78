"""Qwen3 dense decoder: config.json keys and their meaning as parts.

The eleven keys are the ones the reference reads, all without defaults
(reference engine/model/qwen3.py:49-80); any other key is ignored there and
here.  ``max_position_embeddings``, which the reference stores and never uses,
bounds a request here: no token may sit at a position beyond it.  ``model_spec`` states the architecture once, as data: token embedding,
``num_hidden_layers`` pre-norm residual layers of grouped-query attention
(per-head q/k RMSNorm, half-rotation RoPE over the whole head, full causal
mask) and a SwiGLU MLP, a final RMSNorm and an untied or tied head
(reference engine/model/qwen3.py:319-373).
"""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry
from .registry import register_architecture


@register_architecture
@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool

    architecture_names = ("qwen3", "Qwen3ForCausalLM")

    def validate(self) -> None:
        for name in ("hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim",
                     "vocab_size", "max_position_embeddings"):
            value = getattr(self, name)
            if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
                raise ConfigError(f"{name} must be a positive integer, got {value!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} is odd; the rotation pairs (i, i + d/2)")
        if not float(self.rms_norm_eps) > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps!r}")
        if not float(self.rope_theta) > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta!r}")

    def model_spec(self) -> ModelSpec:
        eps = float(self.rms_norm_eps)
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": eps})
        mixer = PartSpec("attention", {
            "hidden_size": self.hidden_size,
            "num_heads": self.num_attention_heads,
            "num_kv_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "qk_norm": PartSpec("rmsnorm", {"size": self.head_dim, "eps": eps}),
            "position": PartSpec("rope_half", {
                "rotary_dim": self.head_dim, "theta": float(self.rope_theta)}),
            "window": None,
            "bias": False,
            "scale": self.head_dim ** -0.5,
        })
        feed_forward = PartSpec("gated_mlp", {
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "activation": "silu",
        })
        layers = tuple(
            LayerSpec(
                prefix=f"model.layers.{i}",
                arrangement=PartSpec("prenorm_residual", {
                    "mixer_prefix": "self_attn", "feed_forward_prefix": "mlp",
                    "mixer_norm_name": "input_layernorm",
                    "feed_forward_norm_name": "post_attention_layernorm"}),
                mixer=mixer, feed_forward=feed_forward,
                mixer_norm=norm, feed_forward_norm=norm,
            )
            for i in range(self.num_hidden_layers)
        )
        schedule = tuple(ScheduleEntry(layer=i, cache=i) for i in range(self.num_hidden_layers))
        return ModelSpec(
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            embedding=PartSpec("token_embedding", {
                "name": "model.embed_tokens.weight",
                "vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
            layers=layers,
            schedule=schedule,
            final_norm=PartSpec("rmsnorm", {
                "size": self.hidden_size, "eps": eps, "name": "model.norm.weight"}),
            head=PartSpec("linear_head", {
                "name": "lm_head.weight", "tied_to": "model.embed_tokens.weight"
                if self.tie_word_embeddings else None,
                "vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
            max_positions=self.max_position_embeddings,
        )
