"""One decode step of a Llama-shaped model on FP8-packed weights and a paged FP8 KV cache.

The reference has no model code.  This module holds the packed weights and caches of such a
model and runs one token step for a batch through a single C-ABI call
(``feather_decode_step``, ``csrc/decode_step.hip``), which strings together the batched
packed GEMV, the paged attention and small fused glue kernels (RMSNorm + quantise + pack,
rotary embedding + cache append, SwiGLU + pack) on the current stream.
"""
from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass

import torch

from .. import _native as N
from ..packers.fp8 import pack_fp8_tensor

__all__ = ["DecoderConfig", "PackedDecoder", "TINYLLAMA_1_1B"]


@dataclass(frozen=True)
class DecoderConfig:
    n_layers: int
    hidden: int
    n_q_heads: int
    n_kv_heads: int
    head_dim: int
    inter: int
    vocab: int
    block_size: int = 16
    rms_eps: float = 1e-5
    rope_theta: float = 10000.0

    @property
    def qkv_rows(self) -> int:
        return (self.n_q_heads + 2 * self.n_kv_heads) * self.head_dim


TINYLLAMA_1_1B = DecoderConfig(n_layers=22, hidden=2048, n_q_heads=32, n_kv_heads=4, head_dim=64, inter=5632,
                               vocab=32000)


class PackedDecoder:
    """Packed weights + paged KV caches of one model instance on one device.

    ``weights`` maps names to fp16 tensors of the usual Llama shapes:
    ``embed [vocab, hidden]``, ``norm_final [hidden]``, ``lm_head [vocab, hidden]`` and per
    layer ``l``: ``l.wq [n_q*d, hidden]``, ``l.wk``, ``l.wv [n_kv*d, hidden]``,
    ``l.wo [hidden, n_q*d]``, ``l.w_gate``, ``l.w_up [inter, hidden]``,
    ``l.w_down [hidden, inter]``, ``l.norm_attn``, ``l.norm_mlp [hidden]``.
    Linear weights are packed with ``pack_fp8_tensor`` (q/k/v and gate/up fused row-wise)."""

    def __init__(self, cfg: DecoderConfig, weights: dict, n_blocks: int, max_blocks: int, mode: str = "E4M3",
                 device=None):
        self.cfg, self.mode, self.code = cfg, mode, N.mode_code(mode)
        self.device = torch.device(device) if device is not None else N.require_gpu()
        if self.device.type == "cuda" and self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        if cfg.hidden != cfg.n_q_heads * cfg.head_dim:
            raise ValueError("hidden must equal n_q_heads * head_dim")
        self.n_blocks, self.max_blocks = int(n_blocks), int(max_blocks)
        dev = self.device
        pk = lambda t: pack_fp8_tensor(t.to(dev, torch.float16), mode=mode)
        f32 = lambda t: t.to(dev, torch.float32).contiguous()
        self.embed = weights["embed"].to(dev, torch.float16).contiguous()
        self.norm_final = f32(weights["norm_final"])
        self.lm_head = pk(weights["lm_head"])
        self.layers = []
        dw = cfg.head_dim // 4
        for l in range(cfg.n_layers):
            g = lambda n: weights[f"{l}.{n}"]
            lay = {
                "w_qkv": pk(torch.cat([g("wq"), g("wk"), g("wv")], dim=0)),
                "w_o": pk(g("wo")),
                "w_gate_up": pk(torch.cat([g("w_gate"), g("w_up")], dim=0)),
                "w_down": pk(g("w_down")),
                "norm_attn": f32(g("norm_attn")),
                "norm_mlp": f32(g("norm_mlp")),
                "k_cache": torch.zeros((n_blocks, cfg.n_kv_heads, cfg.block_size, dw), dtype=torch.int32, device=dev),
                "v_cache": torch.zeros((n_blocks, cfg.n_kv_heads, cfg.block_size, dw), dtype=torch.int32, device=dev),
            }
            self.layers.append(lay)
        self._c_layers = (N.DecoderLayer * max(cfg.n_layers, 1))()
        for i, lay in enumerate(self.layers):
            for name in ("w_qkv", "w_o", "w_gate_up", "w_down", "norm_attn", "norm_mlp", "k_cache", "v_cache"):
                setattr(self._c_layers[i], name, lay[name].data_ptr())
        self._c = N.Decoder(cfg.n_layers, cfg.hidden, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.inter, cfg.vocab,
                            cfg.block_size, self.max_blocks, self.n_blocks, self.code, cfg.rms_eps, cfg.rope_theta,
                            ctypes.cast(self._c_layers, ctypes.POINTER(N.DecoderLayer)), self.embed.data_ptr(),
                            self.norm_final.data_ptr(), self.lm_head.data_ptr())
        self._scratch = {}

    def weight_bytes(self) -> int:
        """Packed weight bytes one step streams (each linear layer once, embedding rows aside)."""
        n = self.lm_head.numel() * 4
        for lay in self.layers:
            n += 4 * (lay["w_qkv"].numel() + lay["w_o"].numel() + lay["w_gate_up"].numel() + lay["w_down"].numel())
        return n

    def attention_path(self, batch: int, max_ctx: int | None = None) -> str:
        """Which attention path a step of this shape takes: ``"fused"`` (rotary embedding, query packing and the
        K/V append inside the attention kernel; the new token is scored after the cached ones) or ``"generic"``
        (separate rotary / append kernel, then paged attention in position order)."""
        max_ctx = self.max_blocks * self.cfg.block_size if max_ctx is None else int(max_ctx)
        r = int(N.lib().feather_decode_step_attention_path(ctypes.byref(self._c), int(batch), max_ctx))
        if r < 0:
            raise ValueError(N.lib().feather_last_error().decode())
        return "fused" if r == 1 else "generic"

    def step(self, token_ids: torch.Tensor, block_tables: torch.Tensor, ctx_lens: torch.Tensor,
             max_ctx: int | None = None, out: torch.Tensor | None = None,
             status: torch.Tensor | None = None) -> torch.Tensor:
        """Run one token for every sequence of the batch; returns float32 logits ``[batch, vocab]``.
        ``ctx_lens[b]`` is the number of tokens already cached for sequence ``b`` (the new token is
        written at that position; the caller adds 1 afterwards).  ``max_ctx`` bounds
        ``ctx_lens + 1`` (default: the whole block table).  ``status`` (optional int32 ``[batch]``)
        receives 0 for every sequence whose token was appended, 1 where the block table is full or the
        length negative, 2 where the table entry is not a block of the cache; those sequences are not
        written and their logits are meaningless."""
        cfg = self.cfg
        for t, name in ((token_ids, "token_ids"), (block_tables, "block_tables"), (ctx_lens, "ctx_lens"),
                        (status, "status")):
            if t is None:
                continue
            if not isinstance(t, torch.Tensor) or t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous int32 tensor on the device")
            if t.device != self.device:
                raise ValueError(f"{name} is on {t.device}, the decoder on {self.device}")
        batch = token_ids.numel()
        if not 1 <= batch <= 64:
            raise ValueError(f"batch must be in [1, 64], got {batch}")
        if block_tables.shape != (batch, self.max_blocks) or ctx_lens.shape != (batch,):
            raise ValueError("block_tables must be [batch, max_blocks] and ctx_lens [batch]")
        if status is not None and status.shape != (batch,):
            raise ValueError("status must be [batch]")
        if out is not None:
            if (not isinstance(out, torch.Tensor) or out.dtype != torch.float32 or not out.is_cuda
                    or out.device != self.device or not out.is_contiguous() or tuple(out.shape) != (batch, cfg.vocab)):
                raise ValueError(f"out must be a contiguous float32 [batch={batch}, vocab={cfg.vocab}] tensor on {self.device}")
        max_ctx = self.max_blocks * cfg.block_size if max_ctx is None else int(max_ctx)
        # one scratch buffer per (shape, stream): steps on different streams may run concurrently
        key = (batch, max_ctx, N.stream_ptr(self.device))
        if key not in self._scratch:
            nbytes = int(N.lib().feather_decode_step_scratch_bytes(ctypes.byref(self._c), batch, max_ctx))
            if nbytes < 0:
                raise ValueError(N.lib().feather_last_error().decode())
            if len(self._scratch) >= 8:
                self._scratch.clear()
            self._scratch[key] = torch.empty(nbytes + 256, dtype=torch.uint8, device=self.device)
        sptr = (self._scratch[key].data_ptr() + 255) // 256 * 256
        if out is None:
            out = torch.empty((batch, cfg.vocab), dtype=torch.float32, device=self.device)
        N.call(self.device, "feather_decode_step", ctypes.addressof(self._c), N.ptr(token_ids), N.ptr(block_tables),
               N.ptr(ctx_lens), batch, max_ctx, sptr, N.ptr(out), N.ptr(status) if status is not None else None)
        return out


def random_weights(cfg: DecoderConfig, seed: int = 5, device="cpu") -> dict:
    """Random-init fp16 weights of the architecture (N(0, 1/fan_in) linears, unit norms)."""
    g = torch.Generator(device=device).manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, device=device)
    w = {"embed": rn(cfg.vocab, cfg.hidden).half(), "norm_final": torch.ones(cfg.hidden, device=device),
         "lm_head": (rn(cfg.vocab, cfg.hidden) / math.sqrt(cfg.hidden)).half()}
    for l in range(cfg.n_layers):
        qd, kd = cfg.n_q_heads * cfg.head_dim, cfg.n_kv_heads * cfg.head_dim
        w[f"{l}.wq"] = (rn(qd, cfg.hidden) / math.sqrt(cfg.hidden)).half()
        w[f"{l}.wk"] = (rn(kd, cfg.hidden) / math.sqrt(cfg.hidden)).half()
        w[f"{l}.wv"] = (rn(kd, cfg.hidden) / math.sqrt(cfg.hidden)).half()
        w[f"{l}.wo"] = (rn(cfg.hidden, qd) / math.sqrt(qd)).half()
        w[f"{l}.w_gate"] = (rn(cfg.inter, cfg.hidden) / math.sqrt(cfg.hidden)).half()
        w[f"{l}.w_up"] = (rn(cfg.inter, cfg.hidden) / math.sqrt(cfg.hidden)).half()
        w[f"{l}.w_down"] = (rn(cfg.hidden, cfg.inter) / math.sqrt(cfg.inter)).half()
        w[f"{l}.norm_attn"] = 1.0 + 0.1 * rn(cfg.hidden)
        w[f"{l}.norm_mlp"] = 1.0 + 0.1 * rn(cfg.hidden)
    return w
