"""ReLU on E5M2-packed input, FP32 output (reference feather/routines/activations.py)."""
from __future__ import annotations

import torch

from .. import _native as N

__all__ = ["relu1d_fp8_ret_fp32_feather_gpu"]


def relu1d_fp8_ret_fp32_feather_gpu(x: torch.Tensor, n: int) -> torch.Tensor:
    """``max(0, dec5(x))`` for the first ``n`` elements packed in ``x`` (reference
    activations.py:33-42); float32 ``[n]`` on the device."""
    x = N.as_words(x, "x")
    n = int(n)
    if n < 0 or n > 4 * x.numel():
        raise ValueError(f"n={n} exceeds the {4 * x.numel()} elements packed in x")
    full = torch.empty(4 * x.numel(), dtype=torch.float32, device=x.device)
    N.call(x.device, "feather_unpack_fp8", N.ptr(x), N.ptr(full), x.numel(), N.E5M2, N.SEM_KERNEL, N.OUT_F32, 1)
    return full[:n]
