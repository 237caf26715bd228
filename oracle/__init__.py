"""CPU oracle for the packed-low-precision path.  TEST INFRASTRUCTURE ONLY.

Loads ``oracle/libfeather_oracle.so`` (plain-C restatement of the reference's
algorithms, built by ``oracle/Makefile``) and adds numpy helpers that reduce the
same semantics to textbook routines (LUT decode followed by a float64 matmul or
an explicit softmax).  Only tests, the smoke check and the bench's CPU-baseline
leg may import this package; the product package never does.

Parity status of the numpy helpers defined here (the C functions list theirs in
feather_oracle.c): ``decode_np``, ``gemv_f64_np``, ``attention_f64_np`` are the textbook
reductions the C oracle is pinned against; ``attention_varlen_f64_np`` (build-defined: the
reference has no variable-length or causal attention) is pinned by reduction to
``attention_f64_np`` per sequence and by the prefix property of the causal mask;
``paged_cache_write_np`` (build-defined) by gathering back through the block table.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfeather_oracle.so")

E5M2, E4M3 = 0, 1
RNE, TRUNC = 0, 1
SEM_KERNEL, SEM_IEEE = 0, 1
_MODES = {"E5M2": E5M2, "E4M3": E4M3}


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (a few hundred ms)."""
    src = os.path.join(_HERE, "feather_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B", "libfeather_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        L.fo_half_bits_to_float.restype = f32
        L.fo_half_bits_to_float.argtypes = [ctypes.c_uint16]
        L.fo_float_to_half_bits.restype = ctypes.c_uint16
        L.fo_float_to_half_bits.argtypes = [f32]
        for name in ("fo_enc_e5m2", "fo_enc_e5m2_trunc", "fo_enc_e4m3"):
            getattr(L, name).restype = ctypes.c_uint8
            getattr(L, name).argtypes = [ctypes.c_uint16]
        L.fo_dec.restype = ctypes.c_uint16
        L.fo_dec.argtypes = [ctypes.c_uint8, i32, i32]
        L.fo_dec_table.argtypes = [vp, i32, i32]
        L.fo_pack_fp8.argtypes = [vp, i64, vp, i32, i32]
        L.fo_unpack_fp8.argtypes = [vp, i64, vp, i32, i32]
        L.fo_pack_fp16.argtypes = [vp, i64, vp]
        L.fo_unpack_fp16.argtypes = [vp, i64, vp]
        L.fo_gemv_fp8.argtypes = [vp, vp, vp, i64, i64, i32, i32]
        L.fo_gemv_fp8_batched.argtypes = [vp, vp, vp, i64, i64, i64, i32]
        L.fo_dot_fp8.argtypes = [vp, vp, i64, i32, i32, vp]
        L.fo_dot_fp16.argtypes = [vp, vp, i64, i32, vp]
        L.fo_flash_attn_fp8.argtypes = [vp, vp, vp, vp, i64, i64, i32, f32, i32]
        L.fo_paged_attn_fp8.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i32, f32]
        L.fo_relu_fp8_e5m2.argtypes = [vp, i64, vp]
        _lib = L
    return _lib


def _mode(mode) -> int:
    if isinstance(mode, str):
        if mode not in _MODES:
            raise NotImplementedError(f"Mode {mode} not supported")
        return _MODES[mode]
    return int(mode)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _u32(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype != np.uint32:
        a = a.view(np.uint32)
    return a.reshape(-1)


# ----------------------------------------------------------------- scalar tables

def enc_table(mode, rounding: int = RNE) -> np.ndarray:
    """uint8[65536]: fp16 bit pattern -> fp8 code."""
    L = lib()
    m = _mode(mode)
    f = L.fo_enc_e5m2_trunc if rounding == TRUNC else (L.fo_enc_e5m2 if m == E5M2 else L.fo_enc_e4m3)
    return np.array([f(h) for h in range(65536)], dtype=np.uint8)


def dec_table_bits(mode, semantics: int = SEM_KERNEL) -> np.ndarray:
    """uint16[256]: fp8 code -> fp16 bit pattern."""
    L = lib()
    m = _mode(mode)
    return np.array([L.fo_dec(c, m, semantics) for c in range(256)], dtype=np.uint16)


def dec_table(mode, semantics: int = SEM_KERNEL) -> np.ndarray:
    """float32[256]: fp8 code -> value."""
    out = np.empty(256, dtype=np.float32)
    lib().fo_dec_table(_ptr(out), _mode(mode), semantics)
    return out


# ----------------------------------------------------------------- pack / unpack

def pack_fp8(x: np.ndarray, mode="E5M2", rounding: int = RNE) -> np.ndarray:
    """fp16 array (any shape, flattened row-major) -> uint32[ceil(n/4)]."""
    x = np.ascontiguousarray(x, dtype=np.float16).reshape(-1)
    out = np.empty((x.size + 3) // 4, dtype=np.uint32)
    rc = lib().fo_pack_fp8(_ptr(x), x.size, _ptr(out), _mode(mode), rounding)
    if rc != 0:
        raise NotImplementedError(f"mode/rounding not supported: {mode}/{rounding}")
    return out


def unpack_fp8(words, mode="E5M2", semantics: int = SEM_KERNEL) -> np.ndarray:
    w = _u32(words)
    out = np.empty(w.size * 4, dtype=np.float32)
    rc = lib().fo_unpack_fp8(_ptr(w), w.size, _ptr(out), _mode(mode), semantics)
    if rc != 0:
        raise NotImplementedError(f"Mode {mode} not supported")
    return out


def pack_fp16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float16).reshape(-1)
    out = np.empty((x.size + 1) // 2, dtype=np.uint32)
    lib().fo_pack_fp16(_ptr(x), x.size, _ptr(out))
    return out


def unpack_fp16(words) -> np.ndarray:
    w = _u32(words)
    out = np.empty(w.size * 2, dtype=np.float16)
    lib().fo_unpack_fp16(_ptr(w), w.size, _ptr(out))
    return out


def codes(words) -> np.ndarray:
    """uint32 words -> uint8 codes in element order (little-endian byte view)."""
    return _u32(words).view(np.uint8)


# ----------------------------------------------------------------- routines (C, reference structure)

def gemv(m, v, M: int, K: int, mode="E5M2", acc64: bool = False) -> np.ndarray:
    m, v = _u32(m), _u32(v)
    assert m.size == M * K // 4 and v.size == K // 4
    out = np.empty(M, dtype=np.float32)
    rc = lib().fo_gemv_fp8(_ptr(m), _ptr(v), _ptr(out), M, K, _mode(mode), int(acc64))
    if rc != 0:
        raise ValueError("K must be a multiple of 4")
    return out


def gemv_batched(w, x, M: int, K: int, nvec: int, mode="E4M3") -> np.ndarray:
    w, x = _u32(w), _u32(x)
    assert w.size == M * K // 4 and x.size == nvec * K // 4
    out = np.empty((nvec, M), dtype=np.float32)
    rc = lib().fo_gemv_fp8_batched(_ptr(w), _ptr(x), _ptr(out), M, K, nvec, _mode(mode))
    if rc != 0:
        raise ValueError("K must be a multiple of 4")
    return out


def dot_fp8(x1, x2, mode="E5M2", acc64: bool = False) -> np.float32:
    x1, x2 = _u32(x1), _u32(x2)
    assert x1.size == x2.size
    out = np.zeros(1, dtype=np.float32)
    rc = lib().fo_dot_fp8(_ptr(x1), _ptr(x2), x1.size, _mode(mode), int(acc64), _ptr(out))
    if rc != 0:
        raise NotImplementedError(mode)
    return out[0]


def dot_fp16(x1, x2, acc64: bool = False) -> np.float32:
    x1, x2 = _u32(x1), _u32(x2)
    assert x1.size == x2.size
    out = np.zeros(1, dtype=np.float32)
    lib().fo_dot_fp16(_ptr(x1), _ptr(x2), x1.size, int(acc64), _ptr(out))
    return out[0]


def flash_attn(q, k, v, L: int, d: int, mode="E5M2", scale=None, tail_reference: bool = False) -> np.ndarray:
    """q,k,v: [..., L, d/4] words; returns [..., L, d] fp32 (loops over leading heads)."""
    q, k, v = _u32(q), _u32(k), _u32(v)
    per = L * d // 4
    heads = q.size // per
    assert q.size == heads * per == k.size == v.size
    if scale is None:
        scale = 1.0 / np.sqrt(np.float32(d))
    out = np.empty((heads, L, d), dtype=np.float32)
    for h in range(heads):
        sl = slice(h * per, (h + 1) * per)
        qq, kk, vv = (np.ascontiguousarray(t[sl]) for t in (q, k, v))
        rc = lib().fo_flash_attn_fp8(_ptr(qq), _ptr(kk), _ptr(vv), _ptr(out[h]), L, d, _mode(mode),
                                     float(scale), int(tail_reference))
        if rc != 0:
            raise ValueError("bad attention arguments")
    return out


def paged_attn(q, k_cache, v_cache, block_tables, ctx_lens, n_q_heads, n_kv_heads, d, block_size,
               mode="E5M2", scale=None) -> np.ndarray:
    q, kc, vc = _u32(q), _u32(k_cache), _u32(v_cache)
    bt = np.ascontiguousarray(block_tables, dtype=np.int32)
    cl = np.ascontiguousarray(ctx_lens, dtype=np.int32)
    n_seq, max_blocks = bt.shape
    if scale is None:
        scale = 1.0 / np.sqrt(np.float32(d))
    out = np.empty((n_seq, n_q_heads, d), dtype=np.float32)
    rc = lib().fo_paged_attn_fp8(_ptr(q), _ptr(kc), _ptr(vc), _ptr(bt), _ptr(cl), _ptr(out), n_seq, n_q_heads,
                                 n_kv_heads, d, block_size, max_blocks, _mode(mode), float(scale))
    if rc != 0:
        raise ValueError("bad paged-attention arguments")
    return out


def relu_fp8_e5m2(words) -> np.ndarray:
    w = _u32(words)
    out = np.empty(w.size * 4, dtype=np.float32)
    lib().fo_relu_fp8_e5m2(_ptr(w), w.size, _ptr(out))
    return out


# ----------------------------------------------------------------- numpy reductions to textbook routines

def decode_np(words, mode="E5M2", semantics: int = SEM_KERNEL, dtype=np.float64) -> np.ndarray:
    """LUT decode, vectorised (for sizes the scalar C loops would take long on)."""
    return dec_table(mode, semantics).astype(dtype)[codes(words)]


def gemv_f64_np(m, v, M: int, K: int, mode="E5M2") -> np.ndarray:
    """Decode with the kernel semantics, then a float64 BLAS matvec."""
    A = decode_np(m, mode).reshape(M, K)
    x = decode_np(v, mode)[:K]
    return A @ x


def attention_f64_np(q, k, v, L: int, d: int, mode="E5M2", scale=None) -> np.ndarray:
    """Decode, then softmax(Q K^T * scale) V in float64 per head (closed form, no tiling,
    no fp16 rounding of P)."""
    per = L * d
    Q = decode_np(q, mode)
    heads = Q.size // per
    Q = Q.reshape(heads, L, d)
    Kd = decode_np(k, mode).reshape(heads, L, d)
    Vd = decode_np(v, mode).reshape(heads, L, d)
    if scale is None:
        scale = 1.0 / np.sqrt(d)
    out = np.empty((heads, L, d), dtype=np.float64)
    for h in range(heads):
        S = (Q[h] @ Kd[h].T) * scale
        S -= S.max(axis=1, keepdims=True)
        P = np.exp(S)
        out[h] = (P @ Vd[h]) / P.sum(axis=1, keepdims=True)
    return out


def attention_varlen_f64_np(q, k, v, cu_seqlens, d: int, mode="E5M2", scale=None, causal: bool = False) -> np.ndarray:
    """Variable-length attention in float64 (closed form): q words [n_heads, total, d/4], k/v words
    [n_kv_heads, total, d/4]; sequence s is rows cu[s]..cu[s+1]-1 and attends only to itself; with
    `causal`, query i of a sequence sees keys 0..i.  Rows outside every sequence stay zero."""
    q, k, v = (np.asarray(a) for a in (q, k, v))
    n_heads, total = q.shape[0], q.shape[1]
    n_kv = k.shape[0]
    group = n_heads // n_kv
    Q = decode_np(q.reshape(-1), mode).reshape(n_heads, total, d)
    Kd = decode_np(k.reshape(-1), mode).reshape(n_kv, total, d)
    Vd = decode_np(v.reshape(-1), mode).reshape(n_kv, total, d)
    if scale is None:
        scale = 1.0 / np.sqrt(d)
    out = np.zeros((n_heads, total, d), dtype=np.float64)
    cu = [int(c) for c in cu_seqlens]
    for h in range(n_heads):
        for a, b in zip(cu[:-1], cu[1:]):
            if b <= a:
                continue
            S = (Q[h, a:b] @ Kd[h // group, a:b].T) * scale
            if causal:
                S = np.where(np.tril(np.ones((b - a, b - a), dtype=bool)), S, -np.inf)
            S = S - S.max(axis=1, keepdims=True)
            P = np.exp(S)
            out[h, a:b] = (P @ Vd[h // group, a:b]) / P.sum(axis=1, keepdims=True)
    return out


def paged_cache_write_np(k_words, v_words, k_cache, v_cache, block_tables, cu_seqlens, start_pos=None) -> None:
    """Scatter packed rows [n_kv_heads, total, d/4] into caches [n_blocks, n_kv_heads, block_size, d/4]
    in place: row cu[s] + i goes to position start_pos[s] + i of sequence s; positions without a
    block-table entry are dropped."""
    n_seq = len(cu_seqlens) - 1
    block_size, max_blocks = k_cache.shape[2], block_tables.shape[1]
    for s in range(n_seq):
        p0 = 0 if start_pos is None else int(start_pos[s])
        for i, t in enumerate(range(int(cu_seqlens[s]), int(cu_seqlens[s + 1]))):
            pos = p0 + i
            if pos < 0 or pos >= max_blocks * block_size:
                continue
            blk = int(block_tables[s, pos // block_size])
            k_cache[blk, :, pos % block_size, :] = k_words[:, t, :]
            v_cache[blk, :, pos % block_size, :] = v_words[:, t, :]

