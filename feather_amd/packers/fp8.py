"""FP8 packers: four FP8 codes (E5M2 or E4M3) per 32-bit word.

Same names, arguments and layout as the reference's ``feather/packers/fp8.py``;
every conversion runs in the HIP pack/unpack kernels (``csrc/pack.hip``).  The
reference packs on the CPU with numpy + ml_dtypes; here host inputs are staged
through the device, so a HIP device is required even for numpy arguments.

Layout (reference fp8.py:134): element ``4j+i`` of the flattened input is bits
``[8i, 8i+8)`` of word ``j``; the tail is padded with +0 (fp8.py:201-204).

One deliberate difference: ``pack_fp8_tensor`` returns its result on the
device of the input (the reference always returns a CPU tensor, fp8.py:280-281,
which callers then move with ``.to("cuda")``; that call still works and is a
no-op here).
"""
from __future__ import annotations

import logging

import numpy as np
import torch

from .. import _native as N

__all__ = [
    "pack_fp8_into_fp32_legacy", "pack_fp8_into_fp32", "pack_fp8_ndarray_legacy", "pack_fp8_ndarray",
    "pack_fp8_tensor_legacy", "pack_fp8_tensor", "unpack_fp8_from_fp32_legacy", "unpack_fp8_from_fp32",
    "unpack_into_fp8_ndarray", "unpack_fp8_tensor",
]


# ------------------------------------------------------------------ device plumbing

def _pack_device(x: torch.Tensor, mode: int, rounding: int) -> torch.Tensor:
    """fp16 tensor on a HIP device (any shape) -> uint32[ceil(n/4)] on the same device."""
    x = x.contiguous().view(-1)
    n = x.numel()
    out = torch.empty((n + 3) // 4, dtype=torch.int32, device=x.device)
    N.call(x.device, "feather_pack_fp8", N.ptr(x), N.ptr(out), n, mode, rounding)
    return out.view(torch.uint32)


def _unpack_device(w: torch.Tensor, mode: int, semantics: int, out_f16: bool, relu: bool = False) -> torch.Tensor:
    w = w.contiguous().view(-1)
    out = torch.empty(w.numel() * 4, dtype=torch.float16 if out_f16 else torch.float32, device=w.device)
    N.call(w.device, "feather_unpack_fp8", N.ptr(w), N.ptr(out), w.numel(), mode, semantics, N.OUT_F16 if out_f16 else N.OUT_F32, int(relu))
    return out


def _half_on_device(x, what: str) -> torch.Tensor:
    """numpy array / tensor -> contiguous fp16 tensor on the current HIP device.
    Non-fp16 input is warned about like the reference (fp8.py:95-103) and rounded
    to fp16 first."""
    dev = N.require_gpu()
    if isinstance(x, torch.Tensor):
        t = x
    else:
        a = np.asarray(x)
        if a.dtype != np.float16:
            logging.warning(f"PARAM {what} was not float16, routine is undefined!")
            a = a.astype(np.float16)
        t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype != torch.float16:
        logging.warning(f"PARAM {what} was not float16, routine is undefined!")
        t = t.to(torch.float16)
    if not t.is_cuda:
        t = t.to(dev)
    return t.contiguous()


def _words_on_device(x, what: str) -> torch.Tensor:
    """float32/uint32 container (numpy or tensor) -> int32 words on the device."""
    dev = N.require_gpu()
    if isinstance(x, torch.Tensor):
        t = x
        if t.dtype not in (torch.float32, torch.uint32, torch.int32):
            raise ValueError(f"{what}: packed words must be a 4-byte container, got {t.dtype}")
        t = t.contiguous().view(torch.int32)
    else:
        a = np.ascontiguousarray(np.asarray(x))
        if a.dtype != np.float32:
            if a.dtype.itemsize != 4:
                raise ValueError(f"{what}: packed words must be a 4-byte container, got {a.dtype}")
            if a.dtype not in (np.uint32, np.int32):
                logging.warning(f"PARAM {what} was not float32, routine is undefined!")
        t = torch.from_numpy(a.view(np.int32))
    if not t.is_cuda:
        t = t.to(dev)
    return t.view(-1)


# ------------------------------------------------------------------ pack

def pack_fp8_tensor(x: torch.Tensor, mode: str = "E5M2") -> torch.Tensor:
    """Pack a tensor of fp16 values into uint32 words, four FP8 codes each, rounding
    to nearest even (reference fp8.py:260-281).  Returns a 1-D ``torch.uint32``
    tensor of ``ceil(numel/4)`` words on the input's device."""
    m = N.mode_code(mode)
    if not isinstance(x, torch.Tensor):
        raise ValueError("pack_fp8_tensor expects a torch.Tensor")
    was_cpu = not x.is_cuda
    out = _pack_device(_half_on_device(x, "x"), m, N.ROUND_RNE)
    return out.cpu() if was_cpu else out


def pack_fp8_tensor_legacy(x: torch.Tensor, mode: str = "E5M2") -> torch.Tensor:
    """Truncating E5M2 pack, returned as a float32 container (reference
    fp8.py:213-257).  Unlike the reference (whose ``F.pad`` call fails), inputs
    whose size is not a multiple of 4 are zero-padded."""
    if mode != "E5M2":
        N.mode_code(mode)
        raise NotImplementedError(f"PARAM mode {mode} is not supported")
    was_cpu = not x.is_cuda
    out = _pack_device(_half_on_device(x, "x"), N.E5M2, N.ROUND_TRUNC).view(torch.float32)
    return out.cpu() if was_cpu else out


def pack_fp8_ndarray(x: np.ndarray, mode: str = "E5M2") -> np.ndarray:
    """numpy fp16 array (flattened row-major) -> float32 container of
    ``ceil(n/4)`` packed words (reference fp8.py:178-210)."""
    m = N.mode_code(mode)
    out = _pack_device(_half_on_device(np.asarray(x).reshape(-1), "x"), m, N.ROUND_RNE)
    return out.view(torch.int32).cpu().numpy().view(np.float32)


def pack_fp8_ndarray_legacy(x: np.ndarray, mode: str = "E5M2") -> np.ndarray:
    """Reference fp8.py:139-175: the per-group loop calls the rounding packer, so
    the result equals :func:`pack_fp8_ndarray` on a 1-D input."""
    return pack_fp8_ndarray(np.asarray(x).reshape(-1), mode)


def _pack_columns(a, b, c, d, mode: int, rounding: int):
    a, b, c, d = (np.asarray(t) for t in (a, b, c, d))
    if a.dtype != np.float16 or b.dtype != np.float16 or c.dtype != np.float16 or d.dtype != np.float16:
        logging.warning(f"PARAM a ({a}) or b ({b}) or c({c}) or d ({d}) was not float16, routine is undefined!")
    if a.ndim > 1 or b.ndim > 1 or c.ndim > 1 or d.ndim > 1:
        logging.warning(f"PARAM a ({a}) or b ({b}) or c({c}) or d ({d}) had more than 1 element to pack")
    shape = a.shape
    cols = np.stack([np.asarray(t, dtype=np.float16).reshape(-1) for t in (a, b, c, d)], axis=-1)
    out = _pack_device(_half_on_device(cols, "a"), mode, rounding)
    res = out.view(torch.int32).cpu().numpy().view(np.float32).reshape(shape)
    return res[()] if res.ndim == 0 else res


def pack_fp8_into_fp32(a, b, c, d, mode: str = "E5M2"):
    """Pack four fp16 values (or four equally shaped arrays, element-wise) into
    float32 containers: ``a | b<<8 | c<<16 | d<<24`` (reference fp8.py:69-136)."""
    return _pack_columns(a, b, c, d, N.mode_code(mode), N.ROUND_RNE)


def pack_fp8_into_fp32_legacy(a, b, c, d, mode: str = "E5M2"):
    """Truncating E5M2 variant (reference fp8.py:8-66)."""
    if mode != "E5M2":
        raise NotImplementedError(f"PARAM mode {mode} is not supported")
    return _pack_columns(a, b, c, d, N.E5M2, N.ROUND_TRUNC)


# ------------------------------------------------------------------ unpack

def unpack_fp8_tensor(x: torch.Tensor, mode: str = "E5M2", semantics: str = "ieee",
                      dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Packed words -> ``4 * n_words`` values on the input's device.

    ``semantics="ieee"`` is the exact value of each code (what the reference's
    CPU ``unpack_*`` functions return, fp8.py:381-391); ``semantics="kernel"``
    is the decode of the GPU kernels (gemv.py:83-88), which differs for E4M3
    codes with a zero exponent field and for 0x7F/0xFF."""
    m = N.mode_code(mode)
    if semantics not in ("ieee", "kernel"):
        raise ValueError(f"semantics must be 'ieee' or 'kernel', got {semantics!r}")
    if dtype not in (torch.float32, torch.float16):
        raise ValueError("dtype must be torch.float32 or torch.float16")
    was_cpu = isinstance(x, torch.Tensor) and not x.is_cuda
    out = _unpack_device(_words_on_device(x, "x"), m, N.SEM_IEEE if semantics == "ieee" else N.SEM_KERNEL,
                         dtype == torch.float16)
    return out.cpu() if was_cpu else out


def unpack_fp8_from_fp32(a, mode: str = "E5M2") -> np.ndarray:
    """One packed float32 container -> its four values as float32, shape
    ``(4, 1)`` for a scalar (reference fp8.py:336-392)."""
    m = N.mode_code(mode)
    arr = np.asarray(a)
    if arr.dtype != np.float32:
        logging.warning(f"PARAM a ({a}) was not float32, routine is undefined!")
        arr = arr.astype(np.float32)
    if arr.ndim > 1:
        logging.warning(f"PARAM a ({a}) had more than 1 element to pack")
    flat = np.atleast_1d(arr).reshape(-1)
    vals = _unpack_device(_words_on_device(flat, "a"), m, N.SEM_IEEE, False).cpu().numpy()
    return np.ascontiguousarray(vals.reshape(-1, 4).T)


def unpack_fp8_from_fp32_legacy(a, mode: str = "E5M2") -> np.ndarray:
    """E5M2 by ``byte << 8`` (reference fp8.py:284-333); returns float32[4]."""
    if mode != "E5M2":
        raise NotImplementedError(f"Mode {mode} not supported")
    arr = np.asarray(a)
    if arr.dtype != np.float32:
        logging.warning(f"PARAM a ({a}) was not float32, routine is undefined!")
        arr = arr.astype(np.float32)
    flat = np.atleast_1d(arr).reshape(-1)[:1]
    return _unpack_device(_words_on_device(flat, "a"), N.E5M2, N.SEM_KERNEL, False).cpu().numpy()


def unpack_into_fp8_ndarray(x: np.ndarray, mode: str = "E5M2") -> np.ndarray:
    """float32 container array -> float16 array of ``4 * len(x)`` values
    (reference fp8.py:395-432)."""
    m = N.mode_code(mode)
    return _unpack_device(_words_on_device(np.asarray(x).reshape(-1), "x"), m, N.SEM_IEEE, True).cpu().numpy()
