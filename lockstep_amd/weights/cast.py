"""The record of what casting a checkpoint's tensors to the dtypes they are used in cost.

A bfloat16 checkpoint goes into the bfloat16 path bit for bit and widens into the 32-bit path
exactly, so its record stays at zero.  A float16 or float32 checkpoint on the bfloat16 path loses
bits; how many elements changed and by how much is measured the way the reference measures its
own checkpoint cast (engine/model/qwen3.py:176-216): element count, inexact count, largest
absolute and relative error.
"""

from __future__ import annotations

import torch

EXACT = {(torch.bfloat16, torch.float32), (torch.float16, torch.float32), (torch.float32, torch.float64)}


class CastLedger:
    CHUNK = 1 << 24          # elements compared at a time

    def __init__(self, compute_dtype: torch.dtype):
        self.report = {"compute_dtype": str(compute_dtype), "elements": 0, "lossy_tensors": 0,
                       "inexact_elements": 0, "max_abs_error": 0.0, "max_rel_error": 0.0}

    def cast(self, tensor: torch.Tensor, target: torch.dtype) -> torch.Tensor:
        """``tensor`` in ``target``; a floating tensor that changes dtype is counted."""
        if tensor.dtype == target or not tensor.dtype.is_floating_point:
            return tensor
        out = tensor.to(target)
        report = self.report
        report["elements"] += tensor.numel()
        if (tensor.dtype, target) in EXACT:
            return out
        report["lossy_tensors"] += 1
        tiny = torch.finfo(torch.float32).tiny
        before, after = tensor.reshape(-1), out.reshape(-1)
        for lo in range(0, before.numel(), self.CHUNK):
            a = before[lo:lo + self.CHUNK].to(torch.float32)
            diff = (a - after[lo:lo + self.CHUNK].to(torch.float32)).abs()
            if diff.numel():
                report["inexact_elements"] += int((diff > 0).sum())
                report["max_abs_error"] = max(report["max_abs_error"], float(diff.max()))
                report["max_rel_error"] = max(report["max_rel_error"],
                                              float((diff / a.abs().clamp_min(tiny)).max()))
        return out
