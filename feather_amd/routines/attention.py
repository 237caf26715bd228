"""Flash attention on FP8-packed Q/K/V, FP32 accumulate and output (reference
feather/routines/attention.py).  The kernel is ``csrc/attention.hip``: packed
K/V tiles staged through LDS, decoded to fp16, QK^T and PV on MFMA.

The reference handles one head of shape ``[seq_len, d]`` packed along ``d``
(``h_dim = d // 4`` words per row).  Leading batch/head dimensions are an
extension: any tensor holding ``n * seq_len * h_dim`` words is treated as ``n``
independent heads laid out back to back.
"""
from __future__ import annotations

import math

import torch

from .. import _native as N

__all__ = ["flash_attention_fp8_e5m2_acc_fp32_gpu", "flash_attention_fp8_e4m3_acc_fp32_gpu",
           "flash_attention_fp8_acc_fp32_gpu", "flash_attention_fp8_varlen_acc_fp32_gpu"]

_TAILS = {"mask": N.TAIL_MASK, "reference": N.TAIL_REFERENCE}


def flash_attention_fp8_acc_fp32_gpu(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_len: int, h_dim: int, *,
                                     mode: str = "E5M2", scale: float | None = None, tail: str = "mask",
                                     kv_group: int = 1, causal: bool = False, workspace: bool = True) -> torch.Tensor:
    """``softmax(Q K^T * scale) V`` per head; non-causal unless ``causal=True``
    (query ``i`` then sees keys ``0..i``; needs ``tail="mask"``).  ``workspace=False`` keeps the call from
    allocating the scratch tensor that short sequences of few wide heads use to spread over the whole GPU.

    ``q`` holds ``n_heads * seq_len * h_dim`` packed words (``h_dim = d // 4``);
    ``k``/``v`` hold ``n_heads // kv_group`` heads.  Returns float32
    ``[seq_len, d]`` for one head, else ``[n_heads, seq_len, d]`` (or ``q``'s
    leading dimensions when it is given as ``[..., seq_len, h_dim]``).
    ``tail="reference"`` reproduces the reference's handling of
    ``seq_len % 64 != 0`` (keys past the end of the last 64-key tile count as
    zero rows, attention.py:57-59); ``tail="mask"`` excludes them."""
    code = N.mode_code(mode)
    if tail not in _TAILS:
        raise ValueError(f"tail must be 'mask' or 'reference', got {tail!r}")
    seq_len, h_dim, kv_group = int(seq_len), int(h_dim), int(kv_group)
    if seq_len < 0 or h_dim <= 0:
        raise ValueError(f"bad shape: seq_len={seq_len}, h_dim={h_dim}")
    d = 4 * h_dim
    if d not in (32, 64, 128, 256, 512):
        raise ValueError(f"head dim {d} (h_dim={h_dim} words) not supported: 32, 64, 128, 256 or 512")
    q, k, v = N.as_words(q, "q"), N.as_words(k, "k"), N.as_words(v, "v")
    per_head = seq_len * h_dim
    if per_head == 0 or q.numel() % per_head != 0:
        raise ValueError(f"q holds {q.numel()} words, not a multiple of seq_len * h_dim = {per_head}")
    n_heads = q.numel() // per_head
    if kv_group < 1 or n_heads % kv_group != 0:
        raise ValueError(f"n_heads={n_heads} is not a multiple of kv_group={kv_group}")
    if k.numel() != (n_heads // kv_group) * per_head or v.numel() != k.numel():
        raise ValueError(f"k/v must hold {(n_heads // kv_group) * per_head} words, got {k.numel()} and {v.numel()}")
    if not (q.device == k.device == v.device):
        raise ValueError("q, k and v must be on the same device")
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if not scale > 0:
        raise ValueError(f"scale must be positive, got {scale}")
    out = torch.empty((n_heads, seq_len, d), dtype=torch.float32, device=q.device)
    if causal:
        if tail != "mask":
            raise ValueError("causal attention needs tail='mask'")
        cu = torch.arange(2, dtype=torch.int32, device=q.device) * seq_len   # [0, L], built on the device (graph-capturable)
        N.call(q.device, "feather_flash_attn_fp8_varlen", N.ptr(q), N.ptr(k), N.ptr(v), N.ptr(out), N.ptr(cu), 1, seq_len, seq_len, n_heads, d, kv_group, code, float(scale), 1)
    else:
        # few short wide heads: the library cuts the key loop over more workgroups if it is given room for the partial results
        ws_bytes = int(N.lib().feather_flash_attn_workspace_bytes(n_heads, seq_len, d)) if workspace else 0
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        N.call(q.device, "feather_flash_attn_fp8_ws", N.ptr(q), N.ptr(k), N.ptr(v), N.ptr(out), N.ptr(ws) if ws_bytes else None, ws_bytes, n_heads, seq_len, d, kv_group, code, float(scale), _TAILS[tail])
    if q.dim() >= 2 and q.shape[-2:] == (seq_len, h_dim):
        return out.view(*q.shape[:-2], seq_len, d)
    return out[0] if n_heads == 1 else out


def flash_attention_fp8_e5m2_acc_fp32_gpu(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_len: int,
                                          h_dim: int, *, scale: float | None = None, tail: str = "reference",
                                          kv_group: int = 1) -> torch.Tensor:
    """Reference feather/routines/attention.py:110-179.  ``h_dim`` is the head
    dimension divided by 4 (packed words per row), as in the reference."""
    return flash_attention_fp8_acc_fp32_gpu(q, k, v, seq_len, h_dim, mode="E5M2", scale=scale, tail=tail,
                                            kv_group=kv_group)


def flash_attention_fp8_e4m3_acc_fp32_gpu(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_len: int,
                                          h_dim: int, *, scale: float | None = None, tail: str = "mask",
                                          kv_group: int = 1) -> torch.Tensor:
    """E4M3 counterpart (none in the reference); decode as in the E4M3 GEMV kernel
    (gemv.py:83-88)."""
    return flash_attention_fp8_acc_fp32_gpu(q, k, v, seq_len, h_dim, mode="E4M3", scale=scale, tail=tail,
                                            kv_group=kv_group)


def flash_attention_fp8_varlen_acc_fp32_gpu(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor,
                                            max_seqlen: int, *, mode: str = "E5M2", scale: float | None = None,
                                            causal: bool = False) -> torch.Tensor:
    """Attention over variable-length sequences packed back to back (no counterpart in
    the reference).

    q            ``[n_heads, total_rows, d/4]`` packed words
    k, v         ``[n_kv_heads, total_rows, d/4]`` (query head ``h`` reads KV head ``h // (n_heads // n_kv_heads)``)
    cu_seqlens   ``[n_seq + 1]`` int32 on the device: sequence ``s`` is rows ``cu[s] .. cu[s+1]-1``
    max_seqlen   upper bound of the sequence lengths (sizes the grid, no device-to-host copy)
    Returns float32 ``[n_heads, total_rows, d]``; rows outside every sequence are zero."""
    code = N.mode_code(mode)
    q, k, v = N.as_words(q, "q"), N.as_words(k, "k"), N.as_words(v, "v")
    if q.dim() != 3 or k.dim() != 3 or v.shape != k.shape or k.shape[1:] != q.shape[1:]:
        raise ValueError("expected q [n_heads, total_rows, d/4] and k, v [n_kv_heads, total_rows, d/4]")
    n_heads, total, dw = q.shape
    n_kv = k.shape[0]
    d = 4 * dw
    if d not in (32, 64, 128, 256, 512):
        raise ValueError(f"head dim {d} not supported: 32, 64, 128, 256 or 512")
    if n_kv == 0 or n_heads % n_kv != 0:
        raise ValueError(f"n_heads={n_heads} is not a multiple of n_kv_heads={n_kv}")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.numel() < 1 or not cu_seqlens.is_cuda:
        raise ValueError("cu_seqlens must be a 1-D int32 tensor of n_seq + 1 offsets on the device")
    max_seqlen = int(max_seqlen)
    if max_seqlen < 0 or max_seqlen > total:
        raise ValueError(f"max_seqlen={max_seqlen} outside [0, total_rows={total}]")
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if not scale > 0:
        raise ValueError(f"scale must be positive, got {scale}")
    out = torch.zeros((n_heads, total, d), dtype=torch.float32, device=q.device)
    cu_seqlens = cu_seqlens.contiguous()
    N.call(q.device, "feather_flash_attn_fp8_varlen", N.ptr(q), N.ptr(k), N.ptr(v), N.ptr(out), N.ptr(cu_seqlens), cu_seqlens.numel() - 1, max_seqlen, total, n_heads, d, n_heads // n_kv, code, float(scale), 1 if causal else 0)
    return out
