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
           "flash_attention_fp8_acc_fp32_gpu"]

_TAILS = {"mask": N.TAIL_MASK, "reference": N.TAIL_REFERENCE}


def flash_attention_fp8_acc_fp32_gpu(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_len: int, h_dim: int, *,
                                     mode: str = "E5M2", scale: float | None = None, tail: str = "mask",
                                     kv_group: int = 1) -> torch.Tensor:
    """``softmax(Q K^T * scale) V`` per head, non-causal.

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
    if d not in (64, 128, 256, 512):
        raise ValueError(f"head dim {d} (h_dim={h_dim} words) not supported: 64, 128, 256 or 512")
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
    out = torch.empty((n_heads, seq_len, d), dtype=torch.float32, device=q.device)
    N.call(q.device, "feather_flash_attn_fp8", N.ptr(q), N.ptr(k), N.ptr(v), N.ptr(out), n_heads, seq_len, d, kv_group, code, float(scale), _TAILS[tail])
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
