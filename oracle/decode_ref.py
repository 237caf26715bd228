"""numpy restatement of the packed decode step (csrc/decode_step.hip) for the tests.
TEST INFRASTRUCTURE ONLY.  The step is build-defined (the reference has no model code);
this file fixes its meaning: float32 element-wise math, every GEMV operand rounded
fp32 -> fp16 -> FP8 (RNE) and decoded with the kernel decode, GEMV sums in float64.
Parity status: the pieces (quant, rmsnorm, rope, online_attention) are pinned by closed forms
in tests/test_oracle.py.  The composition (layer order, residual placement, q/k/v row split of the
fused projection, grouped-query head mapping, cache position and block addressing, gate/up split) is
pinned there too: with ``mode=None`` (no quantiser, float caches) decode_step_ref must equal an
independent float64 Llama step assembled from torch library routines on separate q/k/v/o/gate/up/down
weights, and that check is shown to fail for swapped k/v rows, a shifted head mapping and a dropped
residual."""
from __future__ import annotations

import numpy as np

from . import decode_np, pack_fp8


def quant(x: np.ndarray, mode) -> np.ndarray:
    """fp32 array -> decoded values after fp16 + FP8 rounding (same shape, float64); mode None: no rounding."""
    if mode is None:
        return np.asarray(x, dtype=np.float64)
    with np.errstate(over="ignore"):
        words = pack_fp8(x.astype(np.float32).astype(np.float16), mode)
    return decode_np(words, mode)[: x.size].reshape(x.shape)


def quant_codes(x: np.ndarray, mode: str) -> np.ndarray:
    with np.errstate(over="ignore"):
        return pack_fp8(x.astype(np.float32).astype(np.float16), mode)


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    x = x.astype(np.float32)
    ms = np.mean(x.astype(np.float64) ** 2, axis=-1, keepdims=True).astype(np.float32)
    r = (np.float32(1.0) / np.sqrt(ms + np.float32(eps))).astype(np.float32)
    return (x * r) * w.astype(np.float32)


def rope(x: np.ndarray, pos: int, theta: float) -> np.ndarray:
    """x [heads, d] float32, rotate-half convention."""
    d = x.shape[-1]
    j = np.arange(d // 2, dtype=np.float32)
    inv = np.exp2(-(np.float32(2.0) * j / np.float32(d)) * np.log2(np.float32(theta))).astype(np.float32)
    ang = (np.float32(pos) * inv).astype(np.float32)
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    lo, hi = x[..., : d // 2], x[..., d // 2:]
    return np.concatenate([lo * c - hi * s, hi * c + lo * s], axis=-1).astype(np.float32)


def online_attention(dots: np.ndarray, V: np.ndarray, scale: float, chunk: int = 32, split: int = 512,
                     waves: int = 4, new_token_separate: bool = False) -> np.ndarray:
    """Single-query attention with the evaluation order of csrc/paged_attention.hip: tokens in
    splits of 512; the 32-token chunks of a split are dealt round robin to 4 waves, each of which
    keeps a running maximum (log2 domain), rounds P to fp16 relative to it for P.V, sums the
    denominator from the unrounded P and rescales O when the maximum moves; the waves of a
    split, then the splits, are merged by their maxima.  (Rounding P relative to a running
    instead of the global maximum moves results by ~2^-12, which is enough to flip an FP8 code
    downstream, hence the same order here.)  With new_token_separate the last token is not part of the
    chunks: wave 0 of the split that holds it takes it as one more chunk of one token after its own chunks,
    which is how the decode step's attention scores the token it has just appended."""
    c = np.float32(scale * 1.4426950408889634)
    x = (dots.astype(np.float32) * c).astype(np.float32)
    n, d = V.shape

    def merge(parts):
        parts = [p_ for p_ in parts if np.isfinite(p_[0])]
        mg = max(p_[0] for p_ in parts)
        num, den = np.zeros(d, dtype=np.float64), np.float32(0)
        for m, l, o in parts:
            w = np.float32(np.exp2(np.float32(m - mg)))
            num += float(w) * o
            den = np.float32(den + w * l)
        return mg, den, num

    n_chunked = n - 1 if new_token_separate else n
    split_parts = []
    for s0 in range(0, n, split):
        s1 = min(s0 + split, n_chunked)
        wave_parts = []
        for w in range(waves):
            m, l, o = -np.inf, np.float32(0), np.zeros(d, dtype=np.float64)
            starts = list(range(s0 + w * chunk, s1, waves * chunk))
            if new_token_separate and w == 0 and s0 <= n - 1 < s0 + split:
                starts.append(n - 1)                                  # the new token: one more chunk of one token
            for c0 in starts:
                if c0 == n - 1 and new_token_separate:
                    s1_ = n
                else:
                    s1_ = s1
                xs = x[c0:min(c0 + chunk, s1_)]
                m_new = max(m, float(xs.max()))
                alpha = np.float32(np.exp2(np.float32(m - m_new))) if np.isfinite(m) else np.float32(0)
                # the kernel evaluates 2^(s * c - m) with one fused multiply-add per score
                raw = dots[c0:min(c0 + chunk, s1_)].astype(np.float32).astype(np.float64)
                p = np.exp2((raw * float(c) - m_new).astype(np.float32)).astype(np.float32)
                l = np.float32(l * alpha + p.sum(dtype=np.float32))
                o = o * float(alpha) + p.astype(np.float16).astype(np.float64) @ V[c0:c0 + len(xs)]
                m = m_new
            wave_parts.append((m, l, o))
        split_parts.append(merge(wave_parts))
    _, den, num = merge(split_parts)
    return (num / float(den)).astype(np.float32)


def decode_step_ref(cfg, weights: dict, k_caches, v_caches, tokens, block_tables, ctx_lens, mode,
                    new_token_separate: bool = True):
    """weights: fp16 numpy arrays under the names of PackedDecoder; k_caches / v_caches: per-layer
    uint32 arrays [n_blocks, n_kv, block_size, d/4], updated in place.  Returns logits [B, vocab] float32.
    mode None runs the same composition without any FP8 rounding on float caches
    [n_blocks, n_kv, block_size, d] (used to pin the composition against library routines).
    new_token_separate: evaluation order of the attention (see online_attention): True for the step's
    fused attention kernel (head dim 64, power-of-two blocks), False for its generic path."""
    store = (lambda a: quant_codes(a, mode)) if mode is not None else (lambda a: np.asarray(a, dtype=np.float32))
    load = (lambda w_, n_, d_: decode_np(w_, mode).reshape(n_, d_)) if mode is not None else \
        (lambda w_, n_, d_: np.asarray(w_, dtype=np.float64).reshape(n_, d_))
    H, nq, nkv, d, I = cfg.hidden, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.inter
    B = len(tokens)
    Wq = lambda a: quant(np.asarray(a, dtype=np.float32), mode)                  # packed weight values
    h = np.asarray(weights["embed"], dtype=np.float32)[np.asarray(tokens)]        # [B, H]
    scale = np.float32(1.0 / np.sqrt(d))
    for l in range(cfg.n_layers):
        g = lambda n: weights[f"{l}.{n}"]
        xq = quant(rmsnorm(h, g("norm_attn"), cfg.rms_eps), mode)
        wqkv = Wq(np.concatenate([g("wq"), g("wk"), g("wv")], axis=0))
        qkv = (xq @ wqkv.T).astype(np.float32)                                    # [B, (nq + 2 nkv) d]
        attn = np.zeros((B, nq * d), dtype=np.float32)
        for b in range(B):
            pos = int(ctx_lens[b])
            heads = qkv[b].reshape(nq + 2 * nkv, d)
            q = rope(heads[:nq], pos, cfg.rope_theta)
            k = rope(heads[nq:nq + nkv], pos, cfg.rope_theta)
            v = heads[nq + nkv:]
            blk, slot = int(block_tables[b][pos // cfg.block_size]), pos % cfg.block_size
            for kvh in range(nkv):
                k_caches[l][blk, kvh, slot] = store(k[kvh])
                v_caches[l][blk, kvh, slot] = store(v[kvh])
            qd = quant(q, mode)
            n = pos + 1
            t = np.arange(n)
            blocks, slots = np.asarray(block_tables[b])[t // cfg.block_size], t % cfg.block_size
            for kvh in range(nkv):
                Kd = load(k_caches[l][blocks, kvh, slots], n, d)
                Vd = load(v_caches[l][blocks, kvh, slots], n, d)
                for hq in range(kvh * (nq // nkv), (kvh + 1) * (nq // nkv)):     # query head hq reads KV head hq // group
                    attn[b, hq * d:(hq + 1) * d] = online_attention(Kd @ qd[hq], Vd, float(scale),
                                                                      new_token_separate=new_token_separate)
        o = (quant(attn, mode) @ Wq(g("wo")).T).astype(np.float32)
        h = h + o
        xq = quant(rmsnorm(h, g("norm_mlp"), cfg.rms_eps), mode)
        gu = (xq @ Wq(np.concatenate([g("w_gate"), g("w_up")], axis=0)).T).astype(np.float32)
        gate, up = gu[:, :I], gu[:, I:]
        act = (gate / (np.float32(1.0) + np.exp(-gate))) * up
        dn = (quant(act, mode) @ Wq(g("w_down")).T).astype(np.float32)
        h = h + dn
    xq = quant(rmsnorm(h, weights["norm_final"], cfg.rms_eps), mode)
    return (xq @ Wq(weights["lm_head"]).T).astype(np.float32)
