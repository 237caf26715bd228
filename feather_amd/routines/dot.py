"""Packed dot products with FP32 accumulation (reference feather/routines/dot.py).

All variants run in ``csrc/dot.hip``.  Unlike the reference, which adds
per-block sums with fp32 atomics (dot.py:142, :189-192), the result is
deterministic: partial sums are combined in a fixed order.
"""
from __future__ import annotations

import numpy as np
import torch

from .. import _native as N

__all__ = ["dot_fp16_acc_fp32_vec", "dot_fp16_acc_fp32_numba", "dot_fp16_acc_fp32_gpu",
           "dot_fp8_e5m2_acc_fp32_gpu", "dot_fp8_e4m3_acc_fp32_gpu", "dot_fp8_acc_fp32_gpu"]


def _operands(x1: torch.Tensor, x2: torch.Tensor):
    x1 = N.as_words(x1, "x1")
    x2 = N.as_words(x2, "x2")
    if x1.numel() != x2.numel():
        raise ValueError(f"x1 and x2 must hold the same number of words, got {x1.numel()} and {x2.numel()}")
    if x1.device != x2.device:
        raise ValueError("x1 and x2 must be on the same device")
    return x1, x2


_SCRATCH_BYTES = None


def _scratch_bytes() -> int:
    global _SCRATCH_BYTES
    if _SCRATCH_BYTES is None:
        _SCRATCH_BYTES = int(N.lib().feather_dot_scratch_bytes())
    return _SCRATCH_BYTES


def _scratch(dev: torch.device) -> torch.Tensor:
    return N.scratch(dev, _scratch_bytes(), "dot")


def dot_fp8_acc_fp32_gpu(x1: torch.Tensor, x2: torch.Tensor, mode: str = "E5M2") -> torch.Tensor:
    """``sum_k dec(x1[k]) * dec(x2[k])`` as a 0-dim float32 tensor on the device."""
    code = N.mode_code(mode)
    x1, x2 = _operands(x1, x2)
    out = torch.empty((), dtype=torch.float32, device=x1.device)
    N.call(x1.device, "feather_dot_fp8", N.ptr(x1), N.ptr(x2), N.ptr(out), N.ptr(_scratch(x1.device)), x1.numel(), code)
    return out


def dot_fp8_e5m2_acc_fp32_gpu(x1: torch.Tensor, x2: torch.Tensor) -> torch.Tensor:
    """Reference feather/routines/dot.py:220-260."""
    return dot_fp8_acc_fp32_gpu(x1, x2, "E5M2")


def dot_fp8_e4m3_acc_fp32_gpu(x1: torch.Tensor, x2: torch.Tensor) -> torch.Tensor:
    """E4M3 counterpart (none in the reference); decode as in the E4M3 GEMV kernel."""
    return dot_fp8_acc_fp32_gpu(x1, x2, "E4M3")


def _dot_fp16(x1: torch.Tensor, x2: torch.Tensor, fp16_products: bool) -> torch.Tensor:
    x1, x2 = _operands(x1, x2)
    out = torch.empty((), dtype=torch.float32, device=x1.device)
    N.call(x1.device, "feather_dot_fp16", N.ptr(x1), N.ptr(x2), N.ptr(out), N.ptr(_scratch(x1.device)), x1.numel(), int(fp16_products))
    return out


def dot_fp16_acc_fp32_gpu(x1: torch.Tensor, x2: torch.Tensor) -> torch.Tensor:
    """Reference feather/routines/dot.py:194-218: per word the two products and their
    sum are rounded to fp16 (dot.py:134-141), the rest accumulates in fp32."""
    return _dot_fp16(x1, x2, True)


def _np_words_to_device(x) -> torch.Tensor:
    dev = N.require_gpu()
    a = np.ascontiguousarray(np.asarray(x)).reshape(-1)
    if a.dtype.itemsize != 4:
        raise ValueError(f"packed words must be a 4-byte container, got {a.dtype}")
    return torch.from_numpy(a.view(np.int32)).to(dev)


def dot_fp16_acc_fp32_vec(x1: np.ndarray, x2: np.ndarray) -> np.float32:
    """Reference feather/routines/dot.py:9-50 (numpy in, exact fp32 products);
    the arrays are staged to the device and reduced there."""
    return np.float32(_dot_fp16(_np_words_to_device(x1), _np_words_to_device(x2), False).item())


def dot_fp16_acc_fp32_numba(x1: np.ndarray, x2: np.ndarray, lut: np.ndarray = None) -> np.float32:
    """Reference feather/routines/dot.py:53-106.  ``lut`` (the fp16 -> fp32 table
    numba needed) is accepted and ignored."""
    return dot_fp16_acc_fp32_vec(x1, x2)
