"""Parts a layer is put together from, and the registry of their kinds."""

from .base import (Arrangement, FeedForward, Mixer, Norm, PagedKVSpec, Part, PositionEncoding,
                   StateSpec, WeightSpec, build_part, bump_device_epoch, part_class, register_part,
                   unregister_part)
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401 - register the built-in kinds

__all__ = ["Arrangement", "FeedForward", "Mixer", "Norm", "PagedKVSpec", "Part", "PositionEncoding",
           "StateSpec", "WeightSpec", "build_part", "bump_device_epoch", "part_class", "register_part",
           "unregister_part"]
