"""Rotary position encoding with half rotation: the pair of dimension ``i`` is
``i + rotary_dim/2``.  Tables are built in float64 on the host and kept in
float32, ``inv_freq[i] = theta^(-2i/rotary_dim)``, ``angle = position *
inv_freq`` (reference engine/model/qwen3.py:117-129).  The mixer applies them
inside its fused kernel."""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from .base import PositionEncoding, bump_device_epoch, register_part

# Layers with the same constants share one pair of tables per device.
_TABLES: dict[tuple, list] = {}


@register_part("rope_half")
class RotaryHalf(PositionEncoding):
    """Parameters: ``rotary_dim`` (even, at most the head size), ``theta``."""

    graph_safe = True
    repeatable = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.rotary_dim = int(spec["rotary_dim"])
        self.theta = float(spec["theta"])
        if self.rotary_dim % 2 or self.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be a positive even number")
        self._store = None

    @property
    def cos(self):
        return None if self._store is None else self._store[0]

    @property
    def sin(self):
        return None if self._store is None else self._store[1]

    def share_key(self):
        return (self.rotary_dim, self.theta)

    def tables(self, positions: torch.Tensor):
        half = self.rotary_dim // 2
        exponent = torch.arange(0, half, dtype=torch.float64) * 2.0 / self.rotary_dim
        inv_freq = 1.0 / (self.theta ** exponent)
        angles = positions.to(torch.float64)[:, None] * inv_freq[None, :]
        return angles.cos().to(torch.float32), angles.sin().to(torch.float32)

    def bind(self, rt) -> None:
        """Attach to the tables that all layers with these constants share on this device."""
        self._store = _TABLES.setdefault((self.rotary_dim, self.theta, str(rt.device)), [None, None])

    def ensure(self, max_position: int, rt) -> None:
        if self._store is None:
            self.bind(rt)
        have = 0 if self._store[0] is None else self._store[0].shape[0]
        if max_position <= have:
            return
        size = max(max_position, 2 * have, 256)
        cos, sin = self.tables(torch.arange(size))
        self._store[0] = cos.to(rt.device).contiguous()
        self._store[1] = sin.to(rt.device).contiguous()
        bump_device_epoch()


@register_part("no_position")
class NoPosition(PositionEncoding):
    """Leaves queries and keys as they are."""

    graph_safe = True
    repeatable = True

    rotary_dim = 0
    cos = None
    sin = None

    def share_key(self):
        return ("none",)
