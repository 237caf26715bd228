"""Single-query attention over a paged FP8 KV cache (decode step).  The reference
has no paged attention; numerics follow its flash-attention kernel (decode by
mode, fp32 scores and softmax, P rounded to fp16, fp32 output) and the kernel is
``csrc/paged_attention.hip``.
"""
from __future__ import annotations

import math

import torch

from .. import _native as N

__all__ = ["paged_attention_fp8_acc_fp32_gpu", "paged_cache_write"]


def paged_attention_fp8_acc_fp32_gpu(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                     block_tables: torch.Tensor, context_lens: torch.Tensor, *, mode: str = "E5M2",
                                     scale: float | None = None, max_context_len: int | None = None,
                                     return_packed: bool = False):
    """
    q             ``[n_seq, n_q_heads, d/4]`` packed words
    k_cache       ``[n_blocks, n_kv_heads, block_size, d/4]`` packed words (``v_cache`` alike)
    block_tables  ``[n_seq, max_blocks]`` int32, physical block of each logical block
    context_lens  ``[n_seq]`` int32
    Returns float32 ``[n_seq, n_q_heads, d]``.  Query head ``h`` reads KV head
    ``h // (n_q_heads // n_kv_heads)``.  ``max_context_len`` (default
    ``max_blocks * block_size``) bounds the context split count without a
    device-to-host copy of ``context_lens``.  With ``return_packed`` the result is also returned as
    packed FP8 words ``[n_seq, n_q_heads * d / 4]`` of ``mode`` (rounded fp32 -> fp16 -> FP8 in the
    kernel's epilogue: the operand of a following packed GEMV).  Table entries that are not blocks of
    the cache are read as the last block (never outside the cache)."""
    code = N.mode_code(mode)
    q, k_cache, v_cache = N.as_words(q, "q"), N.as_words(k_cache, "k_cache"), N.as_words(v_cache, "v_cache")
    if q.dim() != 3 or k_cache.dim() != 4 or v_cache.shape != k_cache.shape:
        raise ValueError("expected q [n_seq, n_q_heads, d/4] and k_cache/v_cache [n_blocks, n_kv_heads, block_size, d/4]")
    n_seq, n_q_heads, dw = q.shape
    n_blocks, n_kv_heads, block_size, dw2 = k_cache.shape
    if dw != dw2:
        raise ValueError(f"head dim mismatch: q has {dw} words per head, cache has {dw2}")
    d = 4 * dw
    if d not in (64, 128, 256, 512):
        raise ValueError(f"head dim {d} not supported: 64, 128, 256 or 512")
    if n_q_heads % n_kv_heads != 0 or n_q_heads // n_kv_heads > 16:
        raise ValueError(f"n_q_heads={n_q_heads} must be a multiple of n_kv_heads={n_kv_heads} with ratio <= 16")
    if block_tables.dtype != torch.int32 or context_lens.dtype != torch.int32:
        raise ValueError("block_tables and context_lens must be int32")
    if block_tables.dim() != 2 or block_tables.shape[0] != n_seq or context_lens.shape != (n_seq,):
        raise ValueError("block_tables must be [n_seq, max_blocks] and context_lens [n_seq]")
    if not (block_tables.is_cuda and context_lens.is_cuda):
        raise ValueError("block_tables and context_lens must live on the device")
    if n_blocks < 1:
        raise ValueError("the cache must hold at least one block")
    for t in (k_cache, v_cache, block_tables, context_lens):
        if t.device != q.device:
            raise ValueError("q, the caches, block_tables and context_lens must be on the same device")
    if scale is not None and not scale > 0:
        raise ValueError(f"scale must be positive, got {scale}")
    block_tables, context_lens = block_tables.contiguous(), context_lens.contiguous()
    max_blocks = block_tables.shape[1]
    max_ctx = max_blocks * block_size if max_context_len is None else int(max_context_len)
    if max_ctx > max_blocks * block_size or max_ctx < 0:
        raise ValueError(f"max_context_len={max_ctx} exceeds the block table ({max_blocks} x {block_size})")
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.empty((n_seq, n_q_heads, d), dtype=torch.float32, device=q.device)
    nbytes = int(N.lib().feather_paged_attn_scratch_bytes(n_seq, n_q_heads, d, max_ctx))
    scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
    packed = torch.empty((n_seq, n_q_heads * dw), dtype=torch.int32, device=q.device) if return_packed else None
    N.call(q.device, "feather_paged_attn_fp8", N.ptr(q), N.ptr(k_cache), N.ptr(v_cache), N.ptr(block_tables),
           N.ptr(context_lens), N.ptr(out), N.ptr(packed) if packed is not None else None, N.ptr(scratch), n_seq,
           n_q_heads, n_kv_heads, d, block_size, max_blocks, n_blocks, max_ctx, code, float(scale))
    return (out, packed.view(torch.uint32)) if return_packed else out


def paged_cache_write(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, cu_seqlens: torch.Tensor, start_pos: torch.Tensor | None = None, *,
                      mode: str = "E5M2") -> None:
    """Write the K and V rows of packed variable-length sequences into a paged cache, in place.

    k, v          ``[n_kv_heads, total_rows, d/4]`` packed words, or ``[n_kv_heads, total_rows, d]`` float16
                  (then encoded to ``mode`` on the device, as ``pack_fp8_tensor``)
    k_cache       ``[n_blocks, n_kv_heads, block_size, d/4]`` packed words (``v_cache`` alike)
    block_tables  ``[n_seq, max_blocks]`` int32; ``cu_seqlens`` ``[n_seq + 1]`` int32
    start_pos     ``[n_seq]`` int32 cache position of each sequence's first row (default 0)
    Row ``cu[s] + i`` lands at position ``start_pos[s] + i`` of sequence ``s``; positions past the block
    table, and rows whose table entry is not a block of the cache, are dropped."""
    code = N.mode_code(mode)
    k_cache, v_cache = N.as_words(k_cache, "k_cache"), N.as_words(v_cache, "v_cache")
    if k_cache.dim() != 4 or v_cache.shape != k_cache.shape:
        raise ValueError("expected k_cache/v_cache [n_blocks, n_kv_heads, block_size, d/4]")
    n_blocks, n_kv, block_size, dw = k_cache.shape
    d = 4 * dw
    f16 = k.dtype == torch.float16
    if f16:
        if not isinstance(v, torch.Tensor) or v.dtype != torch.float16:
            raise ValueError("k and v must both be float16 or both packed words")
        if not (k.is_cuda and v.is_cuda):
            raise ValueError(f"k and v must live on a HIP device ('cuda'), got {k.device} and {v.device}")
        k, v = k.contiguous(), v.contiguous()
        want = (n_kv, k.shape[1] if k.dim() == 3 else -1, d)
    else:
        k, v = N.as_words(k, "k"), N.as_words(v, "v")
        want = (n_kv, k.shape[1] if k.dim() == 3 else -1, dw)
    if k.dim() != 3 or tuple(k.shape) != want or v.shape != k.shape:
        raise ValueError(f"expected k and v of shape [n_kv_heads={n_kv}, total_rows, {want[2]}], got {tuple(k.shape)} and {tuple(v.shape)}")
    if d % 16 != 0:
        raise ValueError(f"head dim {d} is not a multiple of 16")
    total = k.shape[1]
    for name, t in (("block_tables", block_tables), ("cu_seqlens", cu_seqlens), ("start_pos", start_pos)):
        if t is not None and (t.dtype != torch.int32 or not t.is_cuda):
            raise ValueError(f"{name} must be an int32 tensor on the device")
    n_seq = cu_seqlens.numel() - 1
    if cu_seqlens.dim() != 1 or n_seq < 0 or block_tables.dim() != 2 or block_tables.shape[0] != n_seq:
        raise ValueError("cu_seqlens must be [n_seq + 1] and block_tables [n_seq, max_blocks]")
    if start_pos is not None and start_pos.shape != (n_seq,):
        raise ValueError("start_pos must be [n_seq]")
    for name, t in (("k", k), ("v", v), ("v_cache", v_cache), ("block_tables", block_tables), ("cu_seqlens", cu_seqlens),
                    ("start_pos", start_pos)):
        if t is not None and t.device != k_cache.device:
            raise ValueError(f"{name} is on {t.device}, the cache on {k_cache.device}")
    block_tables, cu_seqlens = block_tables.contiguous(), cu_seqlens.contiguous()
    sp = N.ptr(start_pos.contiguous()) if start_pos is not None else None
    N.call(k_cache.device, "feather_paged_cache_write", N.ptr(k), N.ptr(v), 1 if f16 else 0, N.ptr(k_cache),
           N.ptr(v_cache), N.ptr(block_tables), N.ptr(cu_seqlens), sp, n_seq, total, n_kv, d, block_size,
           block_tables.shape[1], n_blocks, code)
