"""Pins the CPU oracle (oracle/) before anything is compared against it.

Every check here is independent of the oracle's own formulas: golden tables made
with torch-CPU float8 casts, a brute-force nearest-representable search, the
reference's docstring known answers, exact-integer invariants, float64 textbook
reductions and closed-form special cases of attention.
"""
import numpy as np
import pytest
import torch


# ---------------------------------------------------------------- encode

@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_encode_matches_golden_table(orc, tables, mode):
    got = orc.enc_table(mode)
    ref = tables["enc_e5m2" if mode == "E5M2" else "enc_e4m3"]
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("mode,dt", [("E5M2", torch.float8_e5m2), ("E4M3", torch.float8_e4m3fn)])
def test_encode_matches_torch_cpu_live(orc, mode, dt):
    h = np.arange(65536, dtype=np.uint16)
    ref = torch.from_numpy(h.view(np.float16).copy()).to(dt).view(torch.uint8).numpy()
    assert np.array_equal(orc.enc_table(mode), ref)


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_encode_is_nearest_even_brute_force(orc, tables, mode):
    """For every finite fp16 value: the code is the nearest representable value,
    ties go to the code with an even mantissa; past the largest finite + half an
    ulp it is inf (E5M2) or the NaN code (E4M3fn)."""
    dec = tables["dec_e5m2_ieee" if mode == "E5M2" else "dec_e4m3_ieee"].astype(np.float64)
    pos_codes = np.array([c for c in range(128) if np.isfinite(dec[c])])
    pos_vals = dec[pos_codes]
    assert np.all(np.diff(pos_vals) > 0)           # codes are monotone in value
    h = np.arange(0x7C00, dtype=np.uint16)          # all non-negative finite fp16
    x = h.view(np.float16).astype(np.float64)
    idx = np.searchsorted(pos_vals, x)              # first value >= x
    lo = np.clip(idx - 1, 0, len(pos_vals) - 1)
    hi = np.clip(idx, 0, len(pos_vals) - 1)
    dlo, dhi = np.abs(x - pos_vals[lo]), np.abs(pos_vals[hi] - x)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (pos_codes[hi] % 2 == 0))
    want = np.where(pick_hi, pos_codes[hi], pos_codes[lo]).astype(np.uint8)
    # overflow: the step above the largest finite value is (max + next), where next is 2 * 2^emax
    vmax = pos_vals[-1]
    ulp = pos_vals[-1] - pos_vals[-2]
    over = x >= vmax + ulp / 2                      # tie at max + ulp/2 goes to the even neighbour = overflow
    if mode == "E4M3":
        # largest finite 448 = 0x7E is even, so the tie at 464 stays finite
        over = x > vmax + ulp / 2
    want = np.where(over, 0x7C if mode == "E5M2" else 0x7F, want).astype(np.uint8)
    got = orc.enc_table(mode)
    assert np.array_equal(got[:0x7C00], want)
    # sign symmetry
    assert np.array_equal(got[0x8000:0x8000 + 0x7C00], want | 0x80)


def test_encode_edge_values(orc):
    L = orc.lib()
    f = lambda v: int(np.float16(v).view(np.uint16))
    # E4M3fn: tie at 464 -> 448, anything larger -> NaN code; 2^-10 tie -> 0
    assert L.fo_enc_e4m3(f(448.0)) == 0x7E and L.fo_enc_e4m3(f(464.0)) == 0x7E
    assert L.fo_enc_e4m3(f(464.25)) == 0x7F and L.fo_enc_e4m3(f(65504.0)) == 0x7F
    assert L.fo_enc_e4m3(0x7C00) == 0x7F and L.fo_enc_e4m3(0xFC00) == 0xFF
    assert L.fo_enc_e4m3(f(2.0 ** -10)) == 0x00 and L.fo_enc_e4m3(f(2.0 ** -10 * 1.01)) == 0x01
    assert L.fo_enc_e4m3(f(2.0 ** -9)) == 0x01 and L.fo_enc_e4m3(f(2.0 ** -6)) == 0x08
    # E5M2: 61440 is the tie between 57344 and inf -> inf; fp16 max -> inf
    assert L.fo_enc_e5m2(f(57344.0)) == 0x7B and L.fo_enc_e5m2(f(61440.0)) == 0x7C
    assert L.fo_enc_e5m2(f(65504.0)) == 0x7C and L.fo_enc_e5m2(0x7C00) == 0x7C
    # truncation (legacy packers) is the high byte
    for h in (0x3C00, 0x3CFF, 0xBFFF, 0x7BFF):
        assert L.fo_enc_e5m2_trunc(h) == h >> 8


def test_rne_and_truncation_differ_where_expected(orc):
    rne, tr = orc.enc_table("E5M2"), orc.enc_table("E5M2", orc.TRUNC)
    nan = np.isnan(np.arange(65536, dtype=np.uint16).view(np.float16))
    # rounding up happens when the dropped byte is > 0x80 (127 patterns per high byte) or == 0x80
    # with an odd high byte; 124 finite high bytes per sign: 2 * (124 * 127 + 62)
    assert int(((rne != tr) & ~nan).sum()) == 2 * (124 * 127 + 62)


# ---------------------------------------------------------------- decode

def test_decode_e5m2_is_byte_shift(orc, tables):
    bits = orc.dec_table_bits("E5M2")
    assert np.array_equal(bits, (np.arange(256, dtype=np.uint16) << 8))
    got = orc.dec_table("E5M2")
    ref = tables["dec_e5m2_ieee"]
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(got[~np.isnan(ref)], ref[~np.isnan(ref)])


def test_decode_e4m3_kernel_formula_and_exceptions(orc, tables, kats):
    kern_bits = orc.dec_table_bits("E4M3", orc.SEM_KERNEL)
    assert np.array_equal(kern_bits, tables["dec_e4m3_kernel_bits"])
    kern = orc.dec_table("E4M3", orc.SEM_KERNEL)
    ieee = orc.dec_table("E4M3", orc.SEM_IEEE)
    ref = tables["dec_e4m3_ieee"]
    assert np.array_equal(np.isnan(ieee), np.isnan(ref))
    assert np.array_equal(ieee[~np.isnan(ref)], ref[~np.isnan(ref)])
    diff = [c for c in range(256) if not (kern[c] == ieee[c])]
    assert diff == kats["e4m3_decode_exceptions"]
    for m in range(1, 8):                               # zero exponent field: m * 2^-17, not m * 2^-9
        assert kern[m] == m * 2.0 ** -17 and ieee[m] == m * 2.0 ** -9
        assert kern[0x80 | m] == -m * 2.0 ** -17
    assert kern[0x7F] == 480.0 and kern[0xFF] == -480.0 and np.isnan(ieee[0x7F])


def test_half_conversions_roundtrip(orc):
    L = orc.lib()
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    for i in range(0, 65536, 7):
        v = L.fo_half_bits_to_float(int(h[i]))
        assert (np.isnan(v) and np.isnan(f[i])) or v == f[i]
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4000).astype(np.float32) * s for s in (1e-7, 1e-4, 1.0, 300.0, 7e4)])
    want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.fo_float_to_half_bits(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- layout

def test_pack_layout_and_padding(orc):
    x = np.array([1.0, -2.0, 0.5, 448.0, 3.0], dtype=np.float16)
    w = orc.pack_fp8(x, "E4M3")
    enc = orc.enc_table("E4M3")
    c = enc[x.view(np.uint16)]
    assert w.dtype == np.uint32 and w.size == 2
    assert w[0] == int(c[0]) | int(c[1]) << 8 | int(c[2]) << 16 | int(c[3]) << 24
    assert w[1] == int(c[4])                           # tail padded with +0
    assert np.array_equal(orc.codes(w)[:5], c)
    # 2-D input is flattened row-major
    m = np.arange(8, dtype=np.float16).reshape(2, 4)
    assert np.array_equal(orc.pack_fp8(m, "E5M2"), orc.pack_fp8(m.reshape(-1), "E5M2"))
    assert orc.pack_fp8(np.zeros(0, np.float16)).size == 0


def test_unknown_mode_raises(orc):
    with pytest.raises(NotImplementedError):
        orc.pack_fp8(np.zeros(4, np.float16), "E3M4")
    with pytest.raises(NotImplementedError):
        orc.pack_fp8(np.zeros(4, np.float16), "E4M3", orc.TRUNC)


def test_fp16_container_roundtrip_all_patterns(orc):
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    w = orc.pack_fp16(h)
    assert np.array_equal(w, h.view(np.uint32))        # little-endian identity: lo | hi << 16
    assert np.array_equal(orc.unpack_fp16(w).view(np.uint16), h.view(np.uint16))
    odd = orc.pack_fp16(h[:5])
    assert odd.size == 3 and odd[2] == int(h[4:5].view(np.uint16)[0])


def test_unpack_roundtrip_is_projection(orc):
    """decode(encode(decode(c))) == decode(c) for every finite code (IEEE semantics)."""
    for mode in ("E5M2", "E4M3"):
        w = np.arange(256, dtype=np.uint8).view(np.uint32)
        vals = orc.unpack_fp8(w, mode, orc.SEM_IEEE)
        fin = np.isfinite(vals)
        again = orc.unpack_fp8(orc.pack_fp8(np.where(fin, vals, 0).astype(np.float16), mode), mode, orc.SEM_IEEE)
        assert np.array_equal(again[fin], vals[fin])


# ---------------------------------------------------------------- GEMV / dot

@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_gemv_docstring_known_answer(orc, kats, mode):
    k = kats["gemv"]
    a = np.array(k["matrix"], dtype=np.float16)
    b = np.array(k["vector"], dtype=np.float16)
    got = orc.gemv(orc.pack_fp8(a, mode), orc.pack_fp8(b, mode), 4, 4, mode)
    assert got.tolist() == k["expected"]


def test_gemv_docstring_e4m3_kernel_on_e5m2_packed_ints(orc, kats):
    """gemv.py:214-225 packs with E5M2 and runs the E4M3 kernel; the documented answer only
    holds if both operands are packed for the kernel that reads them -- record what the
    mismatch computes so the quirk is pinned, not silently 'fixed'."""
    k = kats["gemv"]
    a = np.array(k["matrix"], dtype=np.float16)
    b = np.array(k["vector"], dtype=np.float16)
    mixed = orc.gemv(orc.pack_fp8(a, "E5M2"), orc.pack_fp8(b, "E5M2"), 4, 4, "E4M3")
    lut4 = orc.dec_table("E4M3").astype(np.float64)
    A = lut4[orc.codes(orc.pack_fp8(a, "E5M2"))].reshape(4, 4)
    x = lut4[orc.codes(orc.pack_fp8(b, "E5M2"))]
    assert np.allclose(mixed, A @ x, rtol=1e-6)


def test_dot_docstring_known_answers(orc, kats):
    k = kats["dot_fp8_e5m2"]
    x1, x2 = (np.array(k[n], dtype=np.float16) for n in ("x1", "x2"))
    assert orc.dot_fp8(orc.pack_fp8(x1), orc.pack_fp8(x2), "E5M2") == k["expected"]
    assert orc.dot_fp8(orc.pack_fp8(x1, "E4M3"), orc.pack_fp8(x2, "E4M3"), "E4M3") == k["expected"]
    k = kats["dot_fp16"]
    x1, x2 = (np.array(k[n], dtype=np.float16) for n in ("x1", "x2"))
    assert orc.dot_fp16(orc.pack_fp16(x1), orc.pack_fp16(x2)) == k["expected"]


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_gemv_integer_inputs_are_exact(orc, mode):
    """Inputs as in the reference harness (bench_gemv.py:53-57): integers in [-3, 3) are exact
    in both formats and the sums stay below 2^24, so every summation order gives the integer
    matvec exactly."""
    rng = np.random.default_rng(1)
    M, K = 37, 2052
    a = rng.integers(-3, 3, size=(M, K)).astype(np.float16)
    b = rng.integers(-3, 3, size=K).astype(np.float16)
    want = a.astype(np.int64) @ b.astype(np.int64)
    for acc64 in (False, True):
        got = orc.gemv(orc.pack_fp8(a, mode), orc.pack_fp8(b, mode), M, K, mode, acc64)
        assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_gemv_matches_float64_textbook(orc, mode):
    rng = np.random.default_rng(2)
    M, K = 64, 4096
    a = rng.standard_normal((M, K)).astype(np.float32)
    a[rng.random((M, K)) < 0.01] *= 1e-3                    # exercises the E4M3 zero-exponent codes
    b = rng.standard_normal(K).astype(np.float32)
    mp, vp = orc.pack_fp8(a.astype(np.float16), mode), orc.pack_fp8(b.astype(np.float16), mode)
    want = orc.gemv_f64_np(mp, vp, M, K, mode)
    scale = np.abs(want).max()
    for acc64 in (False, True):
        got = orc.gemv(mp, vp, M, K, mode, acc64)
        assert np.abs(got - want).max() / scale < (1e-6 if acc64 else 2e-5)
    if mode == "E4M3":                                      # the two decodes really differ on this data
        lut = orc.dec_table("E4M3", orc.SEM_IEEE).astype(np.float64)
        ieee = lut[orc.codes(mp)].reshape(M, K) @ lut[orc.codes(vp)]
        assert np.abs(ieee - want).max() > 0


def test_gemv_rejects_ragged_k(orc):
    with pytest.raises((ValueError, AssertionError)):
        orc.gemv(np.zeros(3, np.uint32), np.zeros(2, np.uint32), 2, 6, "E5M2")


def test_dot_fp16_follows_fp16_rounding(orc):
    rng = np.random.default_rng(3)
    n = 4096
    a = (rng.standard_normal(n) * 3).astype(np.float16)
    b = (rng.standard_normal(n) * 3).astype(np.float16)
    pl = (a[0::2] * b[0::2])                                # numpy rounds each fp16 op to fp16
    ph = (a[1::2] * b[1::2])
    per_word = (pl + ph).astype(np.float32)
    want = np.float32(per_word.astype(np.float64).sum())
    got = orc.dot_fp16(orc.pack_fp16(a), orc.pack_fp16(b), acc64=True)
    assert got == want
    got32 = orc.dot_fp16(orc.pack_fp16(a), orc.pack_fp16(b))
    assert abs(got32 - want) <= 1e-4 * abs(want) + 1e-3


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_dot_fp8_matches_float64(orc, mode):
    rng = np.random.default_rng(4)
    n = 10_000                                              # bench_dot.py:15 smallest size (100_00)
    a, b = (rng.standard_normal(n).astype(np.float16) for _ in range(2))
    x1, x2 = orc.pack_fp8(a, mode), orc.pack_fp8(b, mode)
    want = float(orc.decode_np(x1, mode) @ orc.decode_np(x2, mode))
    assert abs(orc.dot_fp8(x1, x2, mode, acc64=True) - want) < 1e-4
    assert abs(orc.dot_fp8(x1, x2, mode) - want) < 1e-2
    assert orc.dot_fp8(np.zeros(0, np.uint32), np.zeros(0, np.uint32), mode) == 0.0


# ---------------------------------------------------------------- attention

def _qkv(rng, heads, L, d, mode, orc, ints=False):
    def one():
        if ints:                                            # bench_attention.py:52-59
            return rng.integers(-2, 2, size=(heads, L, d)).astype(np.float16)
        return rng.standard_normal((heads, L, d)).astype(np.float16)
    return [orc.pack_fp8(one(), mode) for _ in range(3)]


@pytest.mark.parametrize("mode,L,d", [("E5M2", 128, 64), ("E4M3", 64, 128), ("E5M2", 100, 64)])
def test_attention_matches_float64_closed_form(orc, mode, L, d):
    rng = np.random.default_rng(5)
    q, k, v = _qkv(rng, 2, L, d, mode, orc)
    got = orc.flash_attn(q, k, v, L, d, mode)
    want = orc.attention_f64_np(q, k, v, L, d, mode)
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-3     # P -> fp16 costs ~2^-11


def test_attention_invariants(orc):
    rng = np.random.default_rng(6)
    L, d = 96, 64
    q, k, v = _qkv(rng, 1, L, d, "E5M2", orc)
    # constant V -> output is that constant
    vc = orc.pack_fp8(np.full((L, d), 1.5, np.float16), "E5M2")
    assert np.allclose(orc.flash_attn(q, k, vc, L, d), 1.5, rtol=2e-3)
    # all keys equal -> uniform weights -> column mean of V
    k1 = orc.pack_fp8(np.tile(rng.standard_normal((1, d)).astype(np.float16), (L, 1)), "E5M2")
    mean_v = orc.decode_np(v, "E5M2").reshape(L, d).mean(axis=0)
    out = orc.flash_attn(q, k1, v, L, d)[0]
    assert np.abs(out - mean_v).max() < 2e-3
    # permuting the keys together with the values changes nothing (up to fp32 reassociation)
    perm = rng.permutation(L)
    kp = k.reshape(L, d // 4)[perm].reshape(-1)
    vp = v.reshape(L, d // 4)[perm].reshape(-1)
    a, b = orc.flash_attn(q, k, v, L, d), orc.flash_attn(q, kp, vp, L, d)
    assert np.abs(a - b).max() < 2e-3


def test_attention_tail_modes(orc):
    """L % 64 != 0: 'reference' scores the zero rows of the last tile (attention.py:57-59),
    which equals appending explicit zero keys/values; 'mask' is the exact softmax over L keys."""
    rng = np.random.default_rng(7)
    L, d = 70, 64
    q, k, v = _qkv(rng, 1, L, d, "E5M2", orc)
    ref_mode = orc.flash_attn(q, k, v, L, d, tail_reference=True)[0]
    Lp = 128
    pad = np.zeros((Lp - L) * d // 4, np.uint32)
    qd, kd, vd = (orc.decode_np(t, "E5M2").reshape(L, d) for t in (q, k, v))
    kz = np.vstack([kd, np.zeros((Lp - L, d))])
    vz = np.vstack([vd, np.zeros((Lp - L, d))])
    S = qd @ kz.T / 8.0
    P = np.exp(S - S.max(axis=1, keepdims=True))
    want = (P @ vz) / P.sum(axis=1, keepdims=True)
    assert np.abs(ref_mode - want).max() / np.abs(want).max() < 1e-3
    masked = orc.flash_attn(q, k, v, L, d)[0]
    exact = orc.attention_f64_np(q, k, v, L, d)[0]
    assert np.abs(masked - exact).max() / np.abs(exact).max() < 1e-3
    assert np.abs(masked - ref_mode).max() > 1e-3          # the two really differ
    assert pad.size > 0


def test_attention_integer_inputs(orc):
    rng = np.random.default_rng(8)
    L, d = 64, 64
    q, k, v = _qkv(rng, 1, L, d, "E5M2", orc, ints=True)
    got = orc.flash_attn(q, k, v, L, d)
    want = orc.attention_f64_np(q, k, v, L, d)
    assert np.abs(got - want).max() < 2e-3


def test_paged_attention_matches_contiguous(orc):
    """Build-defined: gathering the blocks of a sequence and running the contiguous
    closed form must give the paged result."""
    rng = np.random.default_rng(9)
    n_seq, Hq, Hkv, d, bs = 3, 8, 2, 64, 16
    ctx = np.array([5, 48, 33], np.int32)
    max_blocks = 4
    n_blocks = n_seq * max_blocks + 2
    mode = "E4M3"
    kc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode)
    vc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode)
    q = orc.pack_fp8(rng.standard_normal((n_seq, Hq, d)).astype(np.float16), mode)
    bt = rng.permutation(n_blocks)[: n_seq * max_blocks].reshape(n_seq, max_blocks).astype(np.int32)
    got = orc.paged_attn(q, kc, vc, bt, ctx, Hq, Hkv, d, bs, mode)
    K = orc.decode_np(kc, mode).reshape(n_blocks, Hkv, bs, d)
    V = orc.decode_np(vc, mode).reshape(n_blocks, Hkv, bs, d)
    Q = orc.decode_np(q, mode).reshape(n_seq, Hq, d)
    for s in range(n_seq):
        for h in range(Hq):
            kvh = h // (Hq // Hkv)
            ks = np.concatenate([K[b, kvh] for b in bt[s]])[: ctx[s]]
            vs = np.concatenate([V[b, kvh] for b in bt[s]])[: ctx[s]]
            sc = ks @ Q[s, h] / np.sqrt(d)
            p = np.exp(sc - sc.max())
            want = p @ vs / p.sum()
            assert np.abs(got[s, h] - want).max() < 1e-4


def test_relu_oracle(orc):
    x = np.array([-4, -1, 0, 2, 3, -0.5, 4, 1], np.float16)   # bench_activations.py:28 range
    got = orc.relu_fp8_e5m2(orc.pack_fp8(x, "E5M2"))
    assert np.array_equal(got, np.maximum(x.astype(np.float32), 0))


# ---------------------------------------------------------------- decode-step pieces (build-defined)

def test_decode_ref_rmsnorm_and_rope_match_library_forms(orc):
    from oracle import decode_ref
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x), (64,), torch.from_numpy(w), 1e-5).numpy()
    assert np.abs(decode_ref.rmsnorm(x, w, 1e-5) - ref).max() < 1e-6
    d, pos = 64, 37
    q = rng.standard_normal((2, d)).astype(np.float32)
    inv = 1.0 / (10000.0 ** (np.arange(0, d, 2) / d))                   # rotate-half form used by Llama code
    cos, sin = np.concatenate([np.cos(pos * inv)] * 2), np.concatenate([np.sin(pos * inv)] * 2)
    rot = np.concatenate([-q[:, d // 2:], q[:, : d // 2]], axis=-1)
    assert np.abs(decode_ref.rope(q, pos, 10000.0) - (q * cos + rot * sin)).max() < 2e-5
    assert np.array_equal(decode_ref.rope(q, 0, 10000.0), q)           # position 0 is the identity


def test_decode_ref_quant_is_pack_then_decode(orc):
    from oracle import decode_ref
    x = np.array([0.3, -1.7, 500.0, 1e-4, 0.0, 3.14159], np.float32)
    for mode in ("E5M2", "E4M3"):
        want = orc.decode_np(orc.pack_fp8(x.astype(np.float16), mode), mode)[: x.size]
        assert np.array_equal(decode_ref.quant(x, mode), want)


def test_decode_ref_online_attention_matches_exact_softmax(orc):
    """The chunked evaluation order (running maximum, P rounded to fp16) is the exact softmax
    average up to the fp16 rounding of P."""
    from oracle import decode_ref
    rng = np.random.default_rng(11)
    for n in (1, 3, 31, 32, 33, 100, 256, 257, 700):
        dots = (rng.standard_normal(n) * 8).astype(np.float32)
        V = rng.standard_normal((n, 64))
        sc = dots.astype(np.float64) * 0.125
        p = np.exp(sc - sc.max())
        want = p @ V / p.sum()
        got = decode_ref.online_attention(dots, V, 0.125)
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-3
    V = np.full((50, 64), 2.5)
    assert np.allclose(decode_ref.online_attention(rng.standard_normal(50).astype(np.float32), V, 1.0), 2.5, rtol=1e-3)


# ---------------------------------------------------------------- variable-length / causal attention, cache writer

def test_attention_varlen_oracle_reduces_to_fixed_length_and_prefix(orc):
    """Pins attention_varlen_f64_np: (a) without a mask each sequence equals the fixed-length closed
    form on its own rows; (b) causal row i equals NON-causal attention over the prefix 0..i (the
    definition of the mask, evaluated by the already pinned routine); (c) row 0 of a causal sequence
    is V[0]; (d) rows outside every sequence stay zero."""
    rng = np.random.default_rng(5)
    d, mode, total = 64, "E5M2", 40
    cu = [3, 12, 12, 33]                                    # a gap in front, an empty sequence, a tail gap
    q = orc.pack_fp8(rng.standard_normal((2, total, d)).astype(np.float16), mode).reshape(2, total, d // 4)
    k = orc.pack_fp8(rng.standard_normal((1, total, d)).astype(np.float16), mode).reshape(1, total, d // 4)
    v = orc.pack_fp8(rng.standard_normal((1, total, d)).astype(np.float16), mode).reshape(1, total, d // 4)
    full = orc.attention_varlen_f64_np(q, k, v, cu, d, mode)
    caus = orc.attention_varlen_f64_np(q, k, v, cu, d, mode, causal=True)
    for h in range(2):
        for a, b in ((3, 12), (12, 33)):
            want = orc.attention_f64_np(q[h, a:b].reshape(-1), k[0, a:b].reshape(-1), v[0, a:b].reshape(-1), b - a, d, mode)[0]
            assert np.allclose(full[h, a:b], want, rtol=1e-12, atol=1e-14)
            for i in (0, 1, (b - a) // 2, b - a - 1):
                pre = orc.attention_f64_np(q[h, a + i:a + i + 1].repeat(i + 1, axis=0).reshape(-1), k[0, a:a + i + 1].reshape(-1),
                                           v[0, a:a + i + 1].reshape(-1), i + 1, d, mode)[0]
                assert np.allclose(caus[h, a + i], pre[0], rtol=1e-12, atol=1e-14)
            assert np.allclose(caus[h, a], orc.decode_np(v[0, a], mode))
    for o in (full, caus):
        assert not o[:, :3].any() and not o[:, 33:].any()


def test_paged_cache_write_oracle_places_rows(orc):
    """Pins paged_cache_write_np by reading the cache back through the block table (gather is the
    inverse of the scatter), untouched slots and dropped positions included."""
    rng = np.random.default_rng(6)
    n_kv, dw, bs, max_blocks, n_blocks = 2, 4, 4, 3, 8
    cu = np.array([0, 5, 5, 14], dtype=np.int32)
    start = np.array([2, 0, 6], dtype=np.int32)             # sequence 2 runs past 3 blocks x 4 slots: 3 rows dropped
    bt = np.array([[5, 1, 7], [0, 0, 0], [2, 6, 3]], dtype=np.int32)
    k = rng.integers(1, 2**32, (n_kv, 14, dw), dtype=np.uint64).astype(np.uint32)
    v = rng.integers(1, 2**32, (n_kv, 14, dw), dtype=np.uint64).astype(np.uint32)
    kc = np.zeros((n_blocks, n_kv, bs, dw), dtype=np.uint32)
    vc = np.zeros_like(kc)
    orc.paged_cache_write_np(k, v, kc, vc, bt, cu, start)
    written = 0
    for s in range(3):
        for i in range(cu[s + 1] - cu[s]):
            pos = start[s] + i
            if pos >= bs * max_blocks:
                continue
            assert (kc[bt[s, pos // bs], :, pos % bs] == k[:, cu[s] + i]).all()
            assert (vc[bt[s, pos // bs], :, pos % bs] == v[:, cu[s] + i]).all()
            written += 1
    assert written == 5 + 6 and (kc.reshape(-1, dw).any(axis=1).sum() == written * n_kv)


# ---------------------------------------------------------------- decode step: the composition

def _llama_step_f64(cfg, w, k_cache, v_cache, tokens, bt, ctx, bug=None):
    """One Llama decode step in float64 from torch library routines only, on SEPARATE q/k/v/o/gate/up/down
    weights and float caches [n_blocks, n_kv, block_size, d] per layer (updated in place).  Written
    independently of oracle/decode_ref.py: complex-multiplication RoPE, F.rms_norm, F.silu,
    F.scaled_dot_product_attention over the gathered cache with repeated KV heads.  `bug` plants one
    composition mistake, to show that the comparison would catch it."""
    F = torch.nn.functional
    t = lambda a: torch.as_tensor(np.asarray(a, dtype=np.float64))
    H, nq, nkv, d, bs = cfg.hidden, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.block_size
    inv = cfg.rope_theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)          # theta^(-2j/d)

    def rot(x, pos):                                   # rotate-half: (x_j, x_{j+d/2}) is one complex number
        z = torch.complex(x[..., : d // 2], x[..., d // 2:]) * torch.polar(torch.ones_like(inv), pos * inv)
        return torch.cat([z.real, z.imag], dim=-1)

    h = t(w["embed"])[torch.as_tensor(np.asarray(tokens, dtype=np.int64))]
    for l in range(cfg.n_layers):
        g = lambda n: t(w[f"{l}.{n}"])
        x = F.rms_norm(h, (H,), g("norm_attn"), cfg.rms_eps)
        q, k, v = x @ g("wq").T, x @ g("wk").T, x @ g("wv").T
        if bug == "swap_kv":
            k, v = v, k
        att = torch.zeros_like(q)
        for b in range(len(tokens)):
            pos = int(ctx[b]) + (1 if bug == "position" else 0)
            qb = rot(q[b].view(nq, d), pos)
            kb = rot(k[b].view(nkv, d), pos)
            blk, slot = int(bt[b][int(ctx[b]) // bs]), int(ctx[b]) % bs
            k_cache[l][blk, :, slot] = kb
            v_cache[l][blk, :, slot] = v[b].view(nkv, d)
            n = int(ctx[b]) + 1
            blocks = torch.as_tensor(np.asarray(bt[b][: (n + bs - 1) // bs], dtype=np.int64))
            K = k_cache[l][blocks].permute(1, 0, 2, 3).reshape(nkv, -1, d)[:, :n]      # [nkv, n, d]
            V = v_cache[l][blocks].permute(1, 0, 2, 3).reshape(nkv, -1, d)[:, :n]
            if bug == "head_map":                      # query head h -> KV head h % nkv instead of h // group
                K, V = K.repeat(nq // nkv, 1, 1), V.repeat(nq // nkv, 1, 1)
            else:
                K, V = K.repeat_interleave(nq // nkv, dim=0), V.repeat_interleave(nq // nkv, dim=0)
            att[b] = F.scaled_dot_product_attention(qb[:, None, :], K, V).reshape(-1)
        o = att @ g("wo").T
        h = o if bug == "residual" else h + o
        x = F.rms_norm(h, (H,), g("norm_mlp"), cfg.rms_eps)
        gate, up = x @ g("w_gate").T, x @ g("w_up").T
        if bug == "gate_up":
            gate, up = up, gate
        h = h + (F.silu(gate) * up) @ g("w_down").T
    return (F.rms_norm(h, (H,), t(w["norm_final"]), cfg.rms_eps) @ t(w["lm_head"]).T).numpy()


def test_decode_step_ref_composition_matches_library_llama_step(orc):
    """Pins the composition of decode_step_ref (which the GPU decode step is checked against): without
    the quantiser it is an ordinary Llama decode step, so it must agree with a float64 step built from
    torch library routines; only the fp16 rounding of P inside online_attention separates them
    (<= 2^-11 relative per term).  Planted composition mistakes must break the agreement."""
    import types
    from oracle import decode_ref
    cfg = types.SimpleNamespace(n_layers=2, hidden=128, n_q_heads=4, n_kv_heads=2, head_dim=32, inter=192, vocab=50,
                                block_size=4, rms_eps=1e-5, rope_theta=10000.0)
    rng = np.random.default_rng(12)
    rn = lambda *s: rng.standard_normal(s).astype(np.float32)
    H, nq, nkv, d, I = cfg.hidden, cfg.n_q_heads, cfg.n_kv_heads, cfg.head_dim, cfg.inter
    w = {"embed": rn(cfg.vocab, H), "norm_final": 1 + 0.1 * rn(H), "lm_head": rn(cfg.vocab, H) / np.sqrt(H)}
    for l in range(cfg.n_layers):
        w.update({f"{l}.wq": rn(nq * d, H) / np.sqrt(H), f"{l}.wk": rn(nkv * d, H) / np.sqrt(H),
                  f"{l}.wv": rn(nkv * d, H) / np.sqrt(H), f"{l}.wo": rn(H, nq * d) / np.sqrt(H),
                  f"{l}.w_gate": rn(I, H) / np.sqrt(H), f"{l}.w_up": rn(I, H) / np.sqrt(H),
                  f"{l}.w_down": rn(H, I) / np.sqrt(I), f"{l}.norm_attn": 1 + 0.1 * rn(H), f"{l}.norm_mlp": 1 + 0.1 * rn(H)})
    B, max_blocks = 3, 5
    n_blocks = B * max_blocks + 1
    bt = rng.permutation(n_blocks)[: B * max_blocks].reshape(B, max_blocks).astype(np.int32)
    ctx = np.array([0, 7, 18], dtype=np.int32)                 # empty cache, mid-block, first slot of a later block... (18 % 4 = 2)
    tokens = np.array([3, 11, 42], dtype=np.int32)
    caches = [rn(n_blocks, nkv, cfg.block_size, d) for _ in range(2 * cfg.n_layers)]
    fresh = lambda as_torch: [torch.as_tensor(c.astype(np.float64)) if as_torch else c.copy() for c in caches]

    kc, vc = fresh(False)[: cfg.n_layers], fresh(False)[cfg.n_layers:]
    got = decode_ref.decode_step_ref(cfg, w, kc, vc, tokens, bt, ctx, None)
    tk, tv = fresh(True)[: cfg.n_layers], fresh(True)[cfg.n_layers:]
    want = _llama_step_f64(cfg, w, tk, tv, tokens, bt, ctx)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() / scale < 5e-4
    for l in range(cfg.n_layers):                               # the appended rows, and nothing else, changed
        tol = 1e-5 if l == 0 else 1e-3                          # layer 0 has no attention (fp16 P) upstream
        assert np.abs(kc[l] - tk[l].numpy()).max() < tol and np.abs(vc[l] - tv[l].numpy()).max() < tol
        changed = np.argwhere(np.any(kc[l] != caches[l], axis=-1))
        assert sorted(map(tuple, changed)) == sorted((int(bt[b][ctx[b] // 4]), kv, int(ctx[b] % 4)) for b in range(B) for kv in range(nkv))
    for bug in ("swap_kv", "head_map", "residual", "gate_up", "position"):
        tk, tv = fresh(True)[: cfg.n_layers], fresh(True)[cfg.n_layers:]
        wrong = _llama_step_f64(cfg, w, tk, tv, tokens, bt, ctx, bug=bug)
        assert np.abs(got - wrong).max() / scale > 2e-2, f"planted mistake '{bug}' would go unnoticed"
