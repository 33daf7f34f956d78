"""What parts need from their surroundings: device, compute dtype, kernels."""

from __future__ import annotations

import torch

from ..ops import kernels as load_kernels
from ..weights.cast import CastLedger

DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}; use bfloat16 or float32") from None


class Runtime:
    """Device, compute dtype and the loaded kernels.

    ``dtype`` is the type of everything that enters a matrix product and of
    the cache: bfloat16 for serving, float32 for the true 32-bit path (the
    kernels then use full 32-bit MFMA, never a reduced-precision mode).
    Softmax, norms, rotation and the residual stream are float32 in both.
    """

    def __init__(self, device="cuda:0", dtype="bfloat16"):
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise RuntimeError(
                "lockstep_amd runs on an AMD GPU through its HIP kernels; no GPU is visible to torch "
                "and there is no CPU fallback")
        torch.cuda.set_device(self.device)
        self.dtype = parse_dtype(dtype)
        self.kernels = load_kernels()
        self._shared: dict[str, torch.Tensor] = {}
        self.casts = CastLedger(self.dtype)     # what casting stored tensors to their working dtypes cost

    def matrix(self, tensor: torch.Tensor, share_key: str | None = None) -> torch.Tensor:
        """An operand of a matrix product: compute dtype, contiguous, on the device.
        Tensors loaded under the same ``share_key`` share one buffer (tied weights)."""
        if share_key is not None and share_key in self._shared:
            return self._shared[share_key]
        out = self._cast(tensor, self.dtype).to(device=self.device).contiguous()
        if share_key is not None:
            self._shared[share_key] = out
        return out

    def vector(self, tensor: torch.Tensor) -> torch.Tensor:
        """A tensor used in 32-bit arithmetic (norm weights): float32 on the device."""
        return self._cast(tensor, torch.float32).to(device=self.device).contiguous()

    def _cast(self, tensor: torch.Tensor, target: torch.dtype) -> torch.Tensor:
        return self.casts.cast(tensor, target)

    @property
    def cast_report(self) -> dict:
        return self.casts.report

    def element_size(self) -> int:
        return 2 if self.dtype is torch.bfloat16 else 4
