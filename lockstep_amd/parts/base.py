"""Interfaces of the parts a layer is put together from.

A *part* is built from a ``PartSpec`` (its kind and constants) and a tensor
name prefix.  It states which tensors it needs (``weight_specs``), takes them
(``load``) and runs on a packed batch (``forward``).  Parts never look at the
model configuration and never know which model they are in; every size and
constant arrives through the spec.

Kinds of part and what each must provide:

``Norm``            ``forward(ctx, x, out, rows=None)``: normalise rows of the
                    32-bit residual stream ``x [T, H]`` into ``out`` in the
                    compute dtype; ``rows`` optionally selects input rows.
``PositionEncoding`` tables or constants a mixer applies at absolute
                    positions; ``ensure(max_position)`` grows them.
``Mixer``           ``cache_spec()`` says what it keeps between steps (paged
                    keys/values, a fixed-size state, or nothing) and
                    ``forward(ctx, run, x, out, accumulate)`` mixes tokens of
                    the same request: it reads what earlier steps left in the
                    cache, writes this step's part of it, and writes (or adds)
                    ``[T, H]`` into the 32-bit ``out``.
``FeedForward``     ``forward(ctx, x, out, accumulate)``: token-wise.
                    A mixer or feed-forward whose ``forward`` also takes
                    ``norm=None`` may be handed the residual stream itself and
                    the norm part to apply inside its first kernel (the
                    arrangement does so for small steps); it must give the
                    bits it would give on the separately normalised input.
``Arrangement``     owns one layer's parts and the order they run in.

Rule for every ``forward``: a row's result depends on rows of the same
request at earlier positions only, and not on how the request's tokens were
cut into steps or on what else is in the batch.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Optional, Sequence

from ..config.base import PartSpec


@dataclass(frozen=True)
class WeightSpec:
    """A tensor a part expects in the checkpoint.

    ``kind``: ``matrix`` tensors are operands of matrix products and live in
    the compute dtype; ``vector`` tensors (norm weights, biases) are used in
    32-bit arithmetic and are kept in float32; ``int`` tensors are integer
    tables kept as int32.  ``init`` steers the random-weights mode: ``normal``
    is N(0, std), ``norm`` is 1 + N(0, norm_std), ``zeros`` is 0.
    """

    name: str
    shape: tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"
    optional: bool = False


@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values of every token, or of the last ``window`` tokens."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    """A state of fixed size per request: ``shape`` elements of ``dtype`` ("float32",
    "bfloat16" or "int32"), all zero when a request starts."""

    shape: tuple[int, ...]
    dtype: str = "float32"


class Part:
    """Base of all parts."""

    kind: str = ""

    #: True if the part's ``forward`` only launches kernels that read the step's metadata and its
    #: data from device memory, so a decode step may be captured in a HIP graph and replayed with
    #: new metadata.  A part that reads sizes, slots or values on the host while it runs (a state
    #: update in Python, a routing decision fetched from the device) must leave this False; one
    #: such part anywhere in the model switches the graphs off for the model.
    graph_safe = False

    #: True if all that ``forward`` does is launch kernels through ``ctx.rt.kernels``, with arguments
    #: that depend on the layer only through the addresses of device tensors the part holds in its
    #: attributes (weights) and of its unit of the cache.  The engine then runs ``forward`` for the
    #: first two layers of a kind in a step and repeats the second one's launches, with each layer's
    #: own addresses, for the others.  A part that launches in another way (torch operations), keeps
    #: per-layer state on the host or passes per-layer numbers to a kernel leaves this False, and
    #: every layer that contains it runs its ``forward`` every time.
    repeatable = False

    def __init__(self, spec: PartSpec, prefix: str = ""):
        self.spec = spec
        self.prefix = prefix

    def parts(self) -> Sequence["Part"]:
        """The parts this part is built from (none for a leaf)."""
        return ()

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        return []

    def load(self, weights, rt) -> None:
        """Take tensors from ``weights`` (name -> CPU tensor) onto ``rt.device``."""

    @staticmethod
    def join(prefix: str, name: str) -> str:
        return f"{prefix}.{name}" if prefix else name


class Norm(Part):
    def forward(self, ctx, x, out, rows=None) -> None:
        raise NotImplementedError


class PositionEncoding(Part):
    """What the attention mixer asks of a position encoding: ``rotary_dim`` (the leading
    dimensions of a head that are rotated, 0 for none; dimension ``i`` is paired with
    ``i + rotary_dim/2``) and ``cos`` / ``sin``, float32 device tables ``[positions,
    rotary_dim/2]`` of the angle of each pair at each absolute position (None while
    ``rotary_dim`` is 0).  The frequencies, and any scaling of the positions, are the
    part's own business.  Optional: ``share_key()`` (layers with equal keys use one set of
    tables and are prepared once a step) and ``bind(rt)`` (called at load)."""

    rotary_dim = 0
    cos = None
    sin = None

    def dim_order(self, head_dim: int):
        """An encoding that pairs other dimensions than ``i`` with ``i + rotary_dim/2`` (neighbours,
        for instance) says here in which order a head's dimensions have to stand for its pairs to be
        those: a permutation of ``range(head_dim)``, ``order[j]`` being the dimension that comes to
        place ``j``.  The mixer reorders the rows of its query and key projections (and the
        per-head norm weights) that way when it loads them; scores do not change, because queries
        and keys are reordered alike.  None: as they are."""
        return None

    def ensure(self, max_position: int, rt) -> None:
        """Make the tables cover positions ``< max_position``; a part that replaces a table
        a captured graph may hold calls ``bump_device_epoch()``."""


class Mixer(Part):
    def cache_spec(self):
        """``PagedKVSpec``, ``StateSpec`` or ``None``."""
        return None

    def prepare(self, ctx) -> None:
        """Declare per-step needs (work lists) before the step's metadata is uploaded."""

    def prepare_group(self):
        """Mixers that return the same hashable value here need ``prepare`` only once a step
        (one of them is called); None: always call this one."""
        return None

    def mixing_flops(self, tokens: int, start: int) -> float:
        """Multiply-adds times two that mixing ``tokens`` new tokens of one request at positions
        ``start``.. costs beyond the part's matrix products (measurements price a step with it)."""
        return 0.0

    def forward(self, ctx, run, x, out, accumulate: bool) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, x, out, accumulate: bool) -> None:
        raise NotImplementedError


class Arrangement(Part):
    """One layer: builds its parts from a ``LayerSpec`` and runs them."""

    def __init__(self, layer_spec, build_part: Callable[..., Part]):
        super().__init__(layer_spec.arrangement, layer_spec.prefix)
        self.layer_spec = layer_spec

    def parts(self) -> Sequence[Part]:
        raise NotImplementedError

    @property
    def mixer(self):
        """The part that owns the layer's unit of the cache and prepares its steps: a ``Mixer``,
        or None for a layer that mixes nothing."""
        raise NotImplementedError

    def forward(self, ctx, run, h) -> None:
        raise NotImplementedError


# --------------------------------------------------------------------------
# registry of part kinds
# --------------------------------------------------------------------------

_PARTS: dict[str, type] = {}


def register_part(kind: str):
    """Class decorator: make a part class buildable from ``PartSpec(kind, ...)``."""

    def decorate(cls):
        known = _PARTS.get(kind)
        if known is not None and known is not cls:
            raise ValueError(f"part kind {kind!r} is already registered by {known.__name__}")
        cls.kind = kind
        _PARTS[kind] = cls
        return cls

    return decorate


def unregister_part(kind: str) -> None:
    _PARTS.pop(kind, None)


def part_class(kind: str) -> type:
    try:
        return _PARTS[kind]
    except KeyError:
        raise KeyError(
            f"no part of kind {kind!r} is registered; known: {', '.join(sorted(_PARTS))}"
        ) from None


def build_part(spec: PartSpec, prefix: str = "", **extra: Any) -> Part:
    return part_class(spec.kind)(spec, prefix, **extra)


class PendingAdd:
    """A matrix product that still has to be added to the residual stream, left as the sums of
    its K slices: ``stream += partials[0] + partials[1] + ...`` (in this order).  A part that is
    called with ``defer=True`` may return one instead of adding itself; the next reader of the
    stream (a norm that takes ``pending``, or ``flush``) does the addition on its way."""

    def __init__(self, partials):
        self.partials = partials        # [slices, rows, width] float32

    def flush(self, ctx, stream, rows=None) -> None:
        ctx.rt.kernels.add_rmsnorm(stream, self.partials, None, None, 0.0, rows)


#: steps of at most this many tokens leave the residual additions of the output products to the
#: following norm (their work is then cut over K as well, which fills the GPU); 0 switches it off.
#: Up to 64 rows every product is left so; beyond, up to this bound, a product whose slice length
#: has a many-row kernel and whose slice sums stay small (``deferred_rows``).
DEFER_ADD_ROWS = int(__import__("os").environ.get("LOCKSTEP_DEFER_ADD_ROWS", "256"))

#: slices x output width up to which more than 64 rows are left as slice sums: the sums are that
#: many floats a row, written and read once, which beyond this outweighs what cutting K gains
#: (measured: 8 to 12 slices of 1,024 columns gain, 16 slices of 4,096 columns lose)
DEFER_MANY_ROWS_SUMS = 16384


def deferred_rows(ctx, k: int, n: int) -> int:
    """The most tokens of a step for which a product over ``k`` with ``n`` outputs is left as
    K-slice sums (0: never; the kernel that adds the sums moves four columns at a time)."""
    kernels = ctx.rt.kernels
    if n % 4:
        return 0
    if kernels.gemm_slices_count(k) * n > DEFER_MANY_ROWS_SUMS:
        return min(DEFER_ADD_ROWS, 64)
    return min(DEFER_ADD_ROWS, kernels.gemm_slices_max_rows(k, ctx.rt.dtype))


def graph_safe_tree(part: Part) -> bool:
    """Whether ``part`` and every part below it may run inside a captured graph."""
    return bool(part.graph_safe) and all(graph_safe_tree(p) for p in part.parts())


def takes(function, name: str) -> bool:
    """Whether a part's method accepts the optional keyword ``name``."""
    import inspect

    return name in inspect.signature(function).parameters


# Captured graphs hold the addresses of device tensors that parts own (tables that grow with
# the longest position, for instance).  A part that replaces such a tensor bumps the epoch;
# the model keys its graphs on it.
_DEVICE_EPOCH = 0


def device_epoch() -> int:
    return _DEVICE_EPOCH


def bump_device_epoch() -> None:
    global _DEVICE_EPOCH
    _DEVICE_EPOCH += 1
