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
