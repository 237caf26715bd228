"""Packed-FP8 GEMV with FP32 accumulation (reference feather/routines/gemv.py).

``out[r] = sum_k dec(m[r, k]) * dec(v[k])`` on operands packed by
``feather_amd.packers.fp8``; the work runs in ``csrc/gemv.hip``.
"""
from __future__ import annotations

import torch

from .. import _native as N

__all__ = ["gemv_fp8_e5m2_acc_fp32_gpu", "gemv_fp8_e4m3_acc_fp32_gpu", "gemv_fp8_acc_fp32_gpu",
           "gemv_fp8_batched_acc_fp32_gpu"]


def _shape2(m_shape) -> tuple[int, int]:
    try:
        M, K = (int(s) for s in m_shape)
    except Exception as e:  # noqa: BLE001
        raise ValueError(f"m_shape must be the (rows, cols) of the matrix before packing, got {m_shape!r}") from e
    if M < 0 or K < 0:
        raise ValueError(f"m_shape must be non-negative, got {m_shape!r}")
    if K % 4 != 0:
        raise ValueError(f"m_shape[1]={K} must be a multiple of 4: the packer flattens the matrix, so rows of "
                         "other lengths straddle packed words")
    return M, K


def gemv_fp8_acc_fp32_gpu(m: torch.Tensor, v: torch.Tensor, m_shape, mode: str = "E5M2") -> torch.Tensor:
    """GEMV on FP8-packed operands; ``m_shape`` is the matrix shape before packing.
    Returns float32 ``[m_shape[0]]`` on the operands' device."""
    code = N.mode_code(mode)
    M, K = _shape2(m_shape)
    m = N.as_words(m, "m")
    v = N.as_words(v, "v")
    if m.numel() != M * K // 4:
        raise ValueError(f"m holds {m.numel()} words, expected {M * K // 4} for shape {(M, K)}")
    if v.numel() < K // 4:
        raise ValueError(f"v holds {v.numel()} words, expected {K // 4} for {K} columns")
    if v.device != m.device:
        raise ValueError("m and v must be on the same device")
    out = torch.empty((M,), dtype=torch.float32, device=m.device)
    N.call(m.device, "feather_gemv_fp8", N.ptr(m), N.ptr(v), N.ptr(out), M, K, code)
    return out


def gemv_fp8_e5m2_acc_fp32_gpu(m: torch.Tensor, v: torch.Tensor, m_shape: tuple) -> torch.Tensor:
    """Reference feather/routines/gemv.py:136-184."""
    return gemv_fp8_acc_fp32_gpu(m, v, m_shape, "E5M2")


def gemv_fp8_e4m3_acc_fp32_gpu(m: torch.Tensor, v: torch.Tensor, m_shape: tuple) -> torch.Tensor:
    """Reference feather/routines/gemv.py:187-235 (kernel decode: rebias only when
    the exponent field is non-zero, gemv.py:83-88)."""
    return gemv_fp8_acc_fp32_gpu(m, v, m_shape, "E4M3")


def gemv_fp8_batched_acc_fp32_gpu(w: torch.Tensor, x: torch.Tensor, w_shape, nvec: int,
                                  mode: str = "E4M3") -> torch.Tensor:
    """``out[b, r] = sum_k dec(w[r, k]) * dec(x[b, k])`` for ``nvec`` packed vectors
    stacked in ``x`` (``[nvec, K/4]`` words): the weights stream once for the whole
    batch.  No reference counterpart (one vector per launch there)."""
    code = N.mode_code(mode)
    M, K = _shape2(w_shape)
    nvec = int(nvec)
    if not 1 <= nvec <= 64:
        raise ValueError(f"nvec must be in [1, 64], got {nvec}")
    w = N.as_words(w, "w")
    x = N.as_words(x, "x")
    if w.numel() != M * K // 4:
        raise ValueError(f"w holds {w.numel()} words, expected {M * K // 4} for shape {(M, K)}")
    if x.numel() != nvec * K // 4:
        raise ValueError(f"x holds {x.numel()} words, expected {nvec * K // 4} for {nvec} vectors of {K}")
    out = torch.empty((nvec, M), dtype=torch.float32, device=w.device)
    N.call(w.device, "feather_gemv_fp8_batched", N.ptr(w), N.ptr(x), N.ptr(out), M, K, nvec, code)
    return out
