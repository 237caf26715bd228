"""Producers that emit the packed operand of the next GEMV directly: the callers' side of the
packed routines.  The reference quantises on the CPU (``pack_fp8_tensor``,
feather/packers/fp8.py:260-281) and has no device-side producer; here the rounding chain
fp32 -> fp16 -> FP8 (round to nearest even twice, i.e. ``pack_fp8_tensor(x.half())``) and the
packing run inside the kernel that computes the values (``csrc/pack.hip``,
``csrc/decode_step.hip``, the SwiGLU epilogue of ``csrc/gemv_batched.hip``).
"""
from __future__ import annotations

import torch

from .. import _native as N

__all__ = ["quant_pack_f32", "add_rmsnorm_pack", "rope_append", "gemv_fp8_batched_swiglu"]


def _f32(t: torch.Tensor, name: str, shape=None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor) or t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous float32 tensor on the device")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t


def _i32(t: torch.Tensor, name: str, shape=None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor) or t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous int32 tensor on the device")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t


def _same_device(ref: torch.Tensor, *others) -> None:
    for t in others:
        if t is not None and t.device != ref.device:
            raise ValueError("all tensors must be on the same device")


def quant_pack_f32(x: torch.Tensor, mode: str = "E4M3") -> torch.Tensor:
    """float32 tensor (any shape, flattened row-major) -> ``uint32[ceil(n / 4)]`` packed FP8 words,
    bit-identical to ``pack_fp8_tensor(x.half(), mode)``."""
    code = N.mode_code(mode)
    x = _f32(x.contiguous() if isinstance(x, torch.Tensor) else x, "x")
    n = x.numel()
    out = torch.empty(((n + 3) // 4,), dtype=torch.int32, device=x.device)
    N.call(x.device, "feather_quant_pack_f32", N.ptr(x), N.ptr(out), n, code)
    return out.view(torch.uint32)


def add_rmsnorm_pack(h: torch.Tensor, gain: torch.Tensor, delta: torch.Tensor | None = None, *, eps: float = 1e-5,
                     mode: str = "E4M3", return_f32: bool = False):
    """In place ``h += delta.sum(0)`` (``delta`` is ``[n_part, batch, hidden]`` partial sums added in
    index order, or None), then ``y = h * rsqrt(mean(h^2) + eps) * gain``.  Returns the packed FP8
    words of ``y`` (``[batch, hidden / 4]``), and with ``return_f32`` also ``y`` itself."""
    code = N.mode_code(mode)
    _f32(h, "h")
    if h.dim() != 2 or h.shape[1] % 4 != 0:
        raise ValueError("h must be [batch, hidden] with hidden a multiple of 4")
    batch, hidden = h.shape
    _f32(gain, "gain", (hidden,))
    n_part, stride, dptr = 0, 0, None
    if delta is not None:
        _f32(delta, "delta")
        if delta.dim() != 3 or tuple(delta.shape[1:]) != (batch, hidden) or not 1 <= delta.shape[0] <= 64:
            raise ValueError("delta must be [n_part, batch, hidden] with 1 <= n_part <= 64")
        n_part, stride, dptr = delta.shape[0], batch * hidden, N.ptr(delta)
    _same_device(h, gain, delta)
    xq = torch.empty((batch, hidden // 4), dtype=torch.int32, device=h.device)
    y = torch.empty((batch, hidden), dtype=torch.float32, device=h.device) if return_f32 else None
    N.call(h.device, "feather_add_rmsnorm_pack", N.ptr(h), dptr, n_part, stride, N.ptr(gain), N.ptr(xq),
           N.ptr(y) if y is not None else None, batch, hidden, float(eps), code)
    return (xq.view(torch.uint32), y) if return_f32 else xq.view(torch.uint32)


def rope_append(qkv: torch.Tensor, ctx_lens: torch.Tensor, block_tables: torch.Tensor, k_cache: torch.Tensor,
                v_cache: torch.Tensor, *, n_q_heads: int, rope_theta: float = 10000.0, mode: str = "E4M3",
                return_f32: bool = False):
    """Rotary embedding of the q and k heads of ``qkv`` (``[batch, (n_q + 2 n_kv) * d]`` float32, or
    ``[n_part, batch, ...]`` partial sums) at position ``ctx_lens[b]``, q packed to FP8, k and v
    encoded and appended to the paged cache at that position.  Returns ``(q_packed [batch, n_q, d/4],
    ctx_after [batch], status [batch])`` and with ``return_f32`` also the rotated fp32 values
    ``[batch, n_q + 2 n_kv, d]``.  ``status``: 0 appended, 1 no room or bad position, 2 bad block id."""
    code = N.mode_code(mode)
    k_cache, v_cache = N.as_words(k_cache, "k_cache"), N.as_words(v_cache, "v_cache")
    if k_cache.dim() != 4 or v_cache.shape != k_cache.shape:
        raise ValueError("expected k_cache/v_cache [n_blocks, n_kv_heads, block_size, d/4]")
    n_blocks, n_kv, block_size, dw = k_cache.shape
    d, heads = 4 * dw, int(n_q_heads) + 2 * n_kv
    _f32(qkv, "qkv")
    if qkv.dim() == 2:
        qkv = qkv.unsqueeze(0)
    if qkv.dim() != 3 or qkv.shape[2] != heads * d or not 1 <= qkv.shape[0] <= 64:
        raise ValueError(f"qkv must be [batch, {heads * d}] or [n_part <= 64, batch, {heads * d}]")
    n_part, batch = qkv.shape[0], qkv.shape[1]
    _i32(ctx_lens, "ctx_lens", (batch,))
    _i32(block_tables, "block_tables")
    if block_tables.dim() != 2 or block_tables.shape[0] != batch or block_tables.shape[1] < 1:
        raise ValueError("block_tables must be [batch, max_blocks >= 1]")
    _same_device(qkv, ctx_lens, block_tables, k_cache, v_cache)
    dev = qkv.device
    qp = torch.empty((batch, int(n_q_heads), dw), dtype=torch.int32, device=dev)
    ctx_after = torch.empty((batch,), dtype=torch.int32, device=dev)
    status = torch.empty((batch,), dtype=torch.int32, device=dev)
    rot = torch.empty((batch, heads, d), dtype=torch.float32, device=dev) if return_f32 else None
    N.call(dev, "feather_rope_append", N.ptr(qkv), n_part, batch * heads * d, N.ptr(ctx_lens), N.ptr(block_tables),
           N.ptr(qp), N.ptr(k_cache), N.ptr(v_cache), N.ptr(ctx_after), N.ptr(status),
           N.ptr(rot) if rot is not None else None, batch, int(n_q_heads), n_kv, d, block_size, block_tables.shape[1],
           n_blocks, float(rope_theta), code)
    res = (qp.view(torch.uint32), ctx_after, status)
    return res + (rot,) if return_f32 else res


def gemv_fp8_batched_swiglu(w_gate_up: torch.Tensor, x: torch.Tensor, inter: int, K: int, nvec: int, *,
                            mode: str = "E4M3", return_f32: bool = False):
    """``silu(W_gate x) * (W_up x)`` for ``nvec`` packed vectors, emitted as packed FP8 words
    ``[nvec, inter / 4]`` by the GEMV's own epilogue (``w_gate_up`` is ``[2 * inter, K]`` packed, gate rows
    first).  With ``return_f32`` also the fp32 values ``[nvec, inter]`` the codes were rounded from."""
    code = N.mode_code(mode)
    inter, K, nvec = int(inter), int(K), int(nvec)
    if K <= 0 or K % 256 != 0 or inter % 4 != 0 or inter < 0:
        raise ValueError("K must be a positive multiple of 256 and inter a multiple of 4")
    if not 1 <= nvec <= 64:
        raise ValueError(f"nvec must be in [1, 64], got {nvec}")
    w_gate_up, x = N.as_words(w_gate_up, "w_gate_up"), N.as_words(x, "x")
    if w_gate_up.numel() != 2 * inter * K // 4 or x.numel() != nvec * K // 4:
        raise ValueError("w_gate_up must hold 2 * inter * K / 4 words and x nvec * K / 4 words")
    _same_device(w_gate_up, x)
    act = torch.empty((nvec, inter // 4), dtype=torch.int32, device=x.device)
    f = torch.empty((nvec, inter), dtype=torch.float32, device=x.device) if return_f32 else None
    N.call(x.device, "feather_gemv_fp8_batched_swiglu", N.ptr(w_gate_up), N.ptr(x), N.ptr(act),
           N.ptr(f) if f is not None else None, inter, K, nvec, code)
    return (act.view(torch.uint32), f) if return_f32 else act.view(torch.uint32)
