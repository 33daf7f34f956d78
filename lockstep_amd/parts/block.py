"""Arrangements: how a layer's parts are wired around the residual stream."""

from __future__ import annotations

from .base import Arrangement, PendingAdd, build_part, register_part, takes


@register_part("prenorm_residual")
class PreNormResidual(Arrangement):
    """``h += mixer(norm_1(h)); h += feed_forward(norm_2(h))``
    (reference engine/model/qwen3.py:324-370).

    Parameters name the parts' tensor prefixes below the layer's prefix:
    ``mixer_prefix``, ``feed_forward_prefix``, ``mixer_norm_name``,
    ``feed_forward_norm_name``.
    """

    graph_safe = True
    repeatable = True

    def __init__(self, layer_spec, prefix: str = ""):
        super().__init__(layer_spec, build_part)
        p = layer_spec.arrangement.params
        base = layer_spec.prefix
        self.mixer_norm = build_part(layer_spec.part("mixer_norm"), self.join(base, p["mixer_norm_name"]))
        self._mixer = build_part(layer_spec.part("mixer"), self.join(base, p["mixer_prefix"]))
        self.feed_forward_norm = build_part(layer_spec.part("feed_forward_norm"),
                                            self.join(base, p["feed_forward_norm_name"]))
        self.feed_forward = build_part(layer_spec.part("feed_forward"), self.join(base, p["feed_forward_prefix"]))
        self._fuse_mixer = self._fuses(self._mixer, self.mixer_norm)
        self._fuse_ff = self._fuses(self.feed_forward, self.feed_forward_norm)
        # parts that can leave their residual addition to the next norm (see PendingAdd)
        self._defer_mixer = takes(self._mixer.forward, "defer")
        self._defer_ff = takes(self.feed_forward.forward, "defer")
        self._norm1_pending = takes(self.mixer_norm.forward, "pending")
        self._norm2_pending = takes(self.feed_forward_norm.forward, "pending")

    @classmethod
    def weight_specs(cls, layer_spec, prefix: str = ""):
        from .base import part_class

        p = layer_spec.arrangement.params
        base = layer_spec.prefix
        out = []
        for spec, name in ((layer_spec.part("mixer_norm"), p["mixer_norm_name"]),
                           (layer_spec.part("mixer"), p["mixer_prefix"]),
                           (layer_spec.part("feed_forward_norm"), p["feed_forward_norm_name"]),
                           (layer_spec.part("feed_forward"), p["feed_forward_prefix"])):
            out += part_class(spec.kind).weight_specs(spec, cls.join(base, name))
        return out

    def parts(self):
        return (self.mixer_norm, self._mixer, self.feed_forward_norm, self.feed_forward)

    @property
    def mixer(self):
        return self._mixer

    def load(self, weights, rt) -> None:
        for part in self.parts():
            part.load(weights, rt)

    #: a step of at most this many tokens lets the consumer's first matrix
    #: product normalise its input itself (one launch less per norm).  Off by
    #: default: on MI355X the longer dependent chain inside the product costs
    #: more than the launch it saves (Qwen3-0.6B sizes, batch 1 and 8: 7 % slower).
    FUSE_NORM_ROWS = int(__import__("os").environ.get("LOCKSTEP_FUSE_NORM_ROWS", "0"))

    @staticmethod
    def _fuses(part, norm) -> bool:
        import inspect

        return (getattr(norm, "kind", "") == "rmsnorm"
                and "norm" in inspect.signature(part.forward).parameters)

    def forward(self, ctx, run, h, pending=None):
        """``pending``: an addition to ``h`` that the previous layer left to its reader.  Returns
        the one this layer leaves (or None)."""
        rt = ctx.rt
        small = ctx.n_tokens <= self.FUSE_NORM_ROWS
        if pending is not None and (small and self._fuse_mixer or not self._norm1_pending):
            pending.flush(ctx, h)
            pending = None
        if small and self._fuse_mixer:
            mixed = self._mixer.forward(ctx, run, h, h, accumulate=True, norm=self.mixer_norm)
        else:
            x = ctx.buf("block.normed", (ctx.n_tokens, h.shape[1]), rt.dtype)
            if pending is not None:
                self.mixer_norm.forward(ctx, h, x, pending=pending)
            else:
                self.mixer_norm.forward(ctx, h, x)
            if self._defer_mixer:
                mixed = self._mixer.forward(ctx, run, x, h, accumulate=True, defer=True)
            else:
                mixed = self._mixer.forward(ctx, run, x, h, accumulate=True)
        mixed = mixed if isinstance(mixed, PendingAdd) else None
        if mixed is not None and (small and self._fuse_ff or not self._norm2_pending):
            mixed.flush(ctx, h)
            mixed = None
        if small and self._fuse_ff:
            left = self.feed_forward.forward(ctx, h, h, accumulate=True, norm=self.feed_forward_norm)
        else:
            x = ctx.buf("block.normed", (ctx.n_tokens, h.shape[1]), rt.dtype)
            if mixed is not None:
                self.feed_forward_norm.forward(ctx, h, x, pending=mixed)
            else:
                self.feed_forward_norm.forward(ctx, h, x)
            if self._defer_ff:
                left = self.feed_forward.forward(ctx, x, h, accumulate=True, defer=True)
            else:
                left = self.feed_forward.forward(ctx, x, h, accumulate=True)
        return left if isinstance(left, PendingAdd) else None
