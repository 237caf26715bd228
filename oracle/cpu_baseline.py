"""CPU baseline for bench.py: the reference's CPU path restated with torch-CPU ops
(the reference packer itself needs ml_dtypes, which this image lacks).

    pack    : x.to(torch.float8_*)  -> bytes          (reference fp8.py:109-136, RNE casts)
    decode  : 256-entry LUT gather to fp32 with the kernel decode (gemv.py:31-58, :83-88)
    compute : fp32 torch.mv / torch.dot / scaled_dot_product_attention

This is test/bench infrastructure (a reported baseline), never part of the product path.
"""
from __future__ import annotations

import os
import time

import numpy as np
import torch

from . import dec_table

_DT = {"E5M2": torch.float8_e5m2, "E4M3": torch.float8_e4m3fn}


def _median_time(fn, repeats):
    ts = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return float(np.median(ts))


def gemv_baseline(M: int, K: int, mode: str, sample_rows: int, repeats: int = 3, seed: int = 2) -> dict:
    """Times pack / decode / fp32 matvec on `sample_rows` rows of an M x K problem and scales
    the row-proportional parts to M rows."""
    g = torch.Generator().manual_seed(seed)
    rows = min(sample_rows, M)
    x = torch.randn(rows, K, generator=g)
    x[torch.rand(rows, K, generator=g) < 0.01] *= 1e-3
    x = x.half()
    v = torch.randn(K, generator=g).half()
    lut = torch.from_numpy(dec_table(mode))
    state = {}

    def pack():
        state["codes"] = x.to(_DT[mode]).view(torch.uint8)
        state["vcodes"] = v.to(_DT[mode]).view(torch.uint8)

    def decode():
        state["a"] = lut[state["codes"].long()] if rows * K <= (1 << 24) else _lut_chunks(lut, state["codes"])
        state["b"] = lut[state["vcodes"].long()]

    def compute():
        state["y"] = torch.mv(state["a"], state["b"])

    t_pack = _median_time(pack, repeats)
    t_dec = _median_time(decode, repeats)
    t_mv = _median_time(compute, repeats)
    f = M / rows
    return {
        "pack_s": t_pack * f, "decode_s": t_dec * f, "compute_s": t_mv * f,
        "total_s": (t_pack + t_dec + t_mv) * f,  # pack, decode and compute are reported separately and summed
        "cores": torch.get_num_threads(), "cpu_count": os.cpu_count(),
        "sample": f"{rows} of {M} rows x {K} cols, {mode}, median of {repeats}; scaled x{f:g}",
    }


def _lut_chunks(lut, codes, chunk=1 << 24):
    flat = codes.reshape(-1)
    out = torch.empty(flat.numel(), dtype=torch.float32)
    for i in range(0, flat.numel(), chunk):
        out[i:i + chunk] = lut[flat[i:i + chunk].long()]
    return out.view(codes.shape)


def attention_baseline(heads: int, L: int, d: int, mode: str, sample_heads: int = 1, repeats: int = 1,
                       seed: int = 3) -> dict:
    """decode + fp32 SDPA looped per head on `sample_heads` heads, scaled to `heads`."""
    g = torch.Generator().manual_seed(seed)
    lut = torch.from_numpy(dec_table(mode))
    n = min(sample_heads, heads)
    src = [torch.randn(n, L, d, generator=g).half() for _ in range(3)]
    state = {}

    def pack():
        state["qkv"] = [t.to(_DT[mode]).view(torch.uint8) for t in src]

    def run():
        for h in range(n):
            q, k, v = (lut[t[h].long()] for t in state["qkv"])
            torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None])

    t_pack = _median_time(pack, repeats)
    t = _median_time(run, repeats)
    return {"total_s": (t_pack + t) * heads / n, "pack_s": t_pack * heads / n, "compute_s": t * heads / n,
            "cores": torch.get_num_threads(),
            "sample": f"{n} of {heads} heads, L={L}, d={d}, {mode}; scaled x{heads / n:g}"}


def dot_baseline(n: int, mode: str, repeats: int = 5, seed: int = 2) -> dict:
    """pack (both operands) + LUT decode + fp32 torch.dot on the whole problem of n elements."""
    g = torch.Generator().manual_seed(seed)
    a, b = (torch.randn(n, generator=g).half() for _ in range(2))
    lut = torch.from_numpy(dec_table(mode))
    state = {}

    def pack():
        state["ca"], state["cb"] = a.to(_DT[mode]).view(torch.uint8), b.to(_DT[mode]).view(torch.uint8)

    def decode():
        state["fa"], state["fb"] = _lut_chunks(lut, state["ca"]), _lut_chunks(lut, state["cb"])

    def compute():
        state["y"] = torch.dot(state["fa"], state["fb"])

    t_pack, t_dec, t_dot = _median_time(pack, repeats), _median_time(decode, repeats), _median_time(compute, repeats)
    return {"pack_s": t_pack, "decode_s": t_dec, "compute_s": t_dot, "total_s": t_pack + t_dec + t_dot,
            "cores": torch.get_num_threads(), "sample": f"whole problem, n = {n}, {mode}, median of {repeats}"}


def decode_step_baseline(cfg, batch: int, ctx_lens, mode: str, sample_layers: int = 2, repeats: int = 3, seed: int = 5) -> dict:
    """One decode step of a Llama-shaped model on packed weights as the same decode-then-fp32 chain per layer:
    weight codes -> LUT decode -> fp32 matmul for the batch, K/V codes of every context token gathered per sequence
    -> LUT decode -> fp32 SDPA (grouped-query), activations re-quantised (float8 cast + LUT) in front of every
    matmul.  `sample_layers` layers and the lm_head are timed; the layers are scaled to cfg.n_layers."""
    g = torch.Generator().manual_seed(seed)
    lut = torch.from_numpy(dec_table(mode))
    H, nq, nkv, d, I = cfg.hidden, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.inter
    rnd_codes = lambda *shape: torch.randint(0, 120, shape, generator=g, dtype=torch.uint8)   # finite codes of either mode
    layer = {"qkv": rnd_codes((nq + 2 * nkv) * d, H), "o": rnd_codes(H, nq * d), "gu": rnd_codes(2 * I, H), "down": rnd_codes(H, I)}
    lm_head = rnd_codes(cfg.vocab, H)
    ctx = [int(c) for c in ctx_lens]
    kv = [(rnd_codes(c, nkv, d), rnd_codes(c, nkv, d)) for c in ctx]    # the gathered rows of each sequence
    quant = lambda x: lut[x.half().to(_DT[mode]).view(torch.uint8).long()]
    dec = lambda codes: _lut_chunks(lut, codes)
    x0 = torch.randn(batch, H, generator=g)

    def one_layer(x):
        h = quant(torch.nn.functional.rms_norm(x, (H,)))
        qkv = h @ dec(layer["qkv"]).T
        q = quant(qkv[:, : nq * d]).view(batch, nq, d)
        outs = []
        for b in range(batch):
            k, v = dec(kv[b][0]), dec(kv[b][1])                              # [ctx, nkv, d]
            k = k.permute(1, 0, 2).repeat_interleave(nq // nkv, dim=0)       # [nq, ctx, d]
            v = v.permute(1, 0, 2).repeat_interleave(nq // nkv, dim=0)
            outs.append(torch.nn.functional.scaled_dot_product_attention(q[b][:, None, :], k, v).reshape(nq * d))
        x = x + quant(torch.stack(outs)) @ dec(layer["o"]).T
        h = quant(torch.nn.functional.rms_norm(x, (H,)))
        gu = h @ dec(layer["gu"]).T
        act = quant(torch.nn.functional.silu(gu[:, :I]) * gu[:, I:])
        return x + act @ dec(layer["down"]).T

    def layers():
        x = x0
        for _ in range(sample_layers):
            x = one_layer(x)
        return x

    def head():
        return quant(torch.nn.functional.rms_norm(x0, (H,))) @ dec(lm_head).T

    t_layers, t_head = _median_time(layers, repeats), _median_time(head, repeats)
    f = cfg.n_layers / sample_layers
    return {"total_s": t_layers * f + t_head, "layers_s": t_layers * f, "lm_head_s": t_head,
            "cores": torch.get_num_threads(),
            "sample": f"{sample_layers} of {cfg.n_layers} layers (scaled x{f:g}) + lm_head, batch {batch}, "
                      f"{sum(ctx)} context tokens, {mode}, median of {repeats}"}
