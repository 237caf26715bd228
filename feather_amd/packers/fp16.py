"""FP16 packers: two fp16 values per 32-bit word, first value in the low half
(``hi << 16 | lo``, reference feather/packers/fp16.py:39), odd tail padded with
+0 (fp16.py:110-113).  Same names as the reference plus tensor variants; the
repacking runs in the HIP kernels of ``csrc/pack.hip``.
"""
from __future__ import annotations

import logging

import numpy as np
import torch

from .. import _native as N
from .fp8 import _half_on_device, _words_on_device

__all__ = ["pack_fp16_into_fp32", "unpack_fp32_into_fp16", "pack_fp16_ndarray", "unpack_into_fp16_ndarray",
           "pack_fp16_tensor", "unpack_fp16_tensor"]


def _pack_device(x: torch.Tensor) -> torch.Tensor:
    x = x.contiguous().view(-1)
    n = x.numel()
    out = torch.empty((n + 1) // 2, dtype=torch.int32, device=x.device)
    N.call(x.device, "feather_pack_fp16", N.ptr(x), N.ptr(out), n)
    return out.view(torch.uint32)


def _unpack_device(w: torch.Tensor) -> torch.Tensor:
    w = w.contiguous().view(-1)
    out = torch.empty(w.numel() * 2, dtype=torch.float16, device=w.device)
    N.call(w.device, "feather_unpack_fp16", N.ptr(w), N.ptr(out), w.numel())
    return out


def pack_fp16_tensor(x: torch.Tensor) -> torch.Tensor:
    """fp16 tensor (flattened) -> ``torch.uint32`` words on the input's device."""
    was_cpu = not x.is_cuda
    out = _pack_device(_half_on_device(x, "x"))
    return out.cpu() if was_cpu else out


def unpack_fp16_tensor(x: torch.Tensor) -> torch.Tensor:
    """Packed words -> fp16 tensor of twice the length on the input's device."""
    was_cpu = not x.is_cuda
    out = _unpack_device(_words_on_device(x, "x"))
    return out.cpu() if was_cpu else out


def pack_fp16_into_fp32(a, b):
    """Two fp16 values (or equally shaped arrays) -> float32 container(s)
    (reference fp16.py:8-43)."""
    a, b = np.asarray(a), np.asarray(b)
    if a.dtype != np.float16 or b.dtype != np.float16:
        logging.warning(f"PARAM a ({a}) or b ({b}) was not float16, routine is undefined!")
    if a.ndim > 1 or b.ndim > 1:
        logging.warning(f"PARAM a ({a}) and b ({b}) had more than 1 element to pack")
    shape = a.shape
    cols = np.stack([np.asarray(t, dtype=np.float16).reshape(-1) for t in (a, b)], axis=-1)
    res = _pack_device(_half_on_device(cols, "a")).view(torch.int32).cpu().numpy().view(np.float32).reshape(shape)
    return res[()] if res.ndim == 0 else res


def unpack_fp32_into_fp16(a) -> np.ndarray:
    """One float32 container -> float16[2] (low half first) (reference fp16.py:46-80)."""
    arr = np.asarray(a)
    if arr.dtype != np.float32:
        logging.warning(f"PARAM a ({a}) was not float32, routine is undefined!")
        arr = arr.astype(np.float32)
    if arr.ndim > 1:
        logging.warning(f"PARAM a ({a}) had more than 1 element to pack")
    flat = np.atleast_1d(arr).reshape(-1)[:1]
    return _unpack_device(_words_on_device(flat, "a")).cpu().numpy()


def pack_fp16_ndarray(x: np.ndarray) -> np.ndarray:
    """fp16 array -> float32 container array of ``ceil(n/2)`` words (reference fp16.py:83-116)."""
    out = _pack_device(_half_on_device(np.asarray(x).reshape(-1), "x"))
    return out.view(torch.int32).cpu().numpy().view(np.float32)


def unpack_into_fp16_ndarray(x: np.ndarray) -> np.ndarray:
    """float32 container array -> fp16 array of ``2 * len(x)`` values (reference fp16.py:119-151)."""
    return _unpack_device(_words_on_device(np.asarray(x).reshape(-1), "x")).cpu().numpy()
