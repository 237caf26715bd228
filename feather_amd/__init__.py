"""feather_amd: MI355X (gfx950) implementation of the packed-low-precision
routines of SuriyaaMM/feather behind the reference's Python API.

Top-level names follow the reference README (README.md:95-107):

    m_packed = feather.pack_fp8_tensor(matrix, mode="E5M2")
    v_packed = feather.pack_fp8_tensor(vector, mode="E5M2")
    result = feather.gemv(m_packed, v_packed, original_shape=matrix.shape)

Every routine runs in hand-written HIP kernels loaded from
``feather_amd/lib/libfeather_hip.so``; there is no CPU fallback.
"""
from __future__ import annotations

from . import packers, routines  # noqa: F401
from .packers.fp8 import pack_fp8_tensor, unpack_fp8_tensor  # noqa: F401
from .packers.fp16 import pack_fp16_tensor, unpack_fp16_tensor  # noqa: F401
from .routines.attention import (flash_attention_fp8_acc_fp32_gpu, flash_attention_fp8_e4m3_acc_fp32_gpu,  # noqa: F401
                                 flash_attention_fp8_e5m2_acc_fp32_gpu)
from .routines.paged_attention import paged_attention_fp8_acc_fp32_gpu  # noqa: F401
from .routines import dot as _dot, gemv as _gemv

__version__ = "0.1.0"


def gemv(m, v, original_shape=None, mode: str = "E5M2", *, m_shape=None):
    """``feather.gemv(m_packed, v_packed, original_shape=matrix.shape)`` (reference
    README.md:107; the routines' own spelling ``m_shape`` is accepted too)."""
    shape = original_shape if original_shape is not None else m_shape
    if shape is None:
        raise ValueError("gemv needs original_shape (the matrix shape before packing)")
    return _gemv.gemv_fp8_acc_fp32_gpu(m, v, shape, mode)


def dot(x1, x2, mode: str = "E5M2"):
    """Packed dot product; ``mode`` is "E5M2", "E4M3" or "FP16"."""
    if mode == "FP16":
        return _dot.dot_fp16_acc_fp32_gpu(x1, x2)
    return _dot.dot_fp8_acc_fp32_gpu(x1, x2, mode)
