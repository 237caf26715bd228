"""GPU parity: flash attention (prefill) and paged attention (decode) against the CPU oracle.

Tolerance: max |o - o_ref| / max |o_ref| <= 1e-3 against (a) the oracle's restatement of the
reference tile algorithm (fp32, P rounded to fp16) and (b) decode + float64 softmax; the
budget is dominated by rounding P to fp16 (2^-11 per weight)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _dev_words(a, dev, shape=None):
    t = torch.from_numpy(a.view(np.int32).copy()).to(dev).view(torch.uint32)
    return t if shape is None else t.view(*shape)


def _nerr(got, want):
    return float(np.abs(got - want).max() / np.abs(want).max())


def _qkv(rng, heads, L, d, mode, orc, ints=False):
    def one():
        if ints:
            return rng.integers(-2, 2, size=(heads, L, d)).astype(np.float16)
        return rng.standard_normal((heads, L, d)).astype(np.float16)
    return [orc.pack_fp8(one(), mode) for _ in range(3)]


@pytest.mark.parametrize("mode,heads,L,d", [
    ("E5M2", 1, 128, 64), ("E5M2", 3, 256, 64), ("E4M3", 2, 128, 64), ("E5M2", 2, 128, 128),
    ("E4M3", 1, 64, 256), ("E4M3", 1, 96, 512), ("E5M2", 1, 64, 512), ("E5M2", 8, 1024, 64),
    # d = 256 below 256 workgroups: two wave groups take one half of every key tile each; the last tile
    # leaves the second group nothing (200, 330), a few keys (100, 300), everything (128), and a sequence
    # shorter than the first group's half
    ("E4M3", 2, 200, 256), ("E5M2", 1, 330, 256), ("E4M3", 1, 128, 256), ("E5M2", 2, 100, 256),
    ("E4M3", 1, 300, 256), ("E4M3", 1, 7, 256),
    # the same split at d = 512 (32-key tiles, 16 keys per group on the 16x16x16 MFMA)
    ("E4M3", 2, 100, 512), ("E5M2", 1, 200, 512), ("E4M3", 1, 50, 512), ("E5M2", 2, 81, 512), ("E4M3", 1, 3, 512),
    # d = 32: narrower than the reference's tl.dot takes; one MFMA k-step per score, half a tile of staging threads
    ("E5M2", 3, 300, 32), ("E4M3", 2, 257, 32), ("E5M2", 1, 64, 32), ("E4M3", 1, 5, 32), ("E5M2", 8, 1024, 32),
])
def test_flash_attention_vs_oracle(dev, orc, mode, heads, L, d):
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(heads * 1000 + L + d)
    q, k, v = _qkv(rng, heads, L, d, mode, orc)
    out = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(k, dev), _dev_words(v, dev), L, d // 4,
                                           mode=mode)
    got = out.cpu().numpy().reshape(heads, L, d)
    want64 = orc.attention_f64_np(q, k, v, L, d, mode)
    assert _nerr(got, want64) <= TOL
    if heads * L * L * d <= 1 << 26:
        assert _nerr(got, orc.flash_attn(q, k, v, L, d, mode)) <= TOL


@pytest.mark.parametrize("mode,heads,L,d,tail", [
    ("E4M3", 2, 512, 256, "mask"), ("E5M2", 1, 1000, 256, "mask"), ("E4M3", 1, 1000, 256, "reference"),
    ("E4M3", 1, 300, 512, "mask"), ("E5M2", 2, 530, 512, "mask"), ("E4M3", 1, 530, 512, "reference"),
    ("E5M2", 2, 1100, 128, "mask"), ("E4M3", 3, 600, 128, "mask"), ("E4M3", 8, 1024, 512, "mask"),
    # d = 64: the reference's own call shape, one head (bench_attention.py:13-14: one head of 128 .. 8192 rows) -- 32
    # workgroups without the key ranges
    ("E5M2", 1, 8192, 64, "mask"), ("E4M3", 2, 3000, 64, "mask"), ("E5M2", 1, 1000, 64, "reference"),
    ("E4M3", 1, 2100, 64, "reference"), ("E5M2", 16, 1024, 64, "mask"),
])
def test_flash_attention_key_ranges_over_workgroups(dev, orc, mode, heads, L, d, tail):
    """Few short wide heads, or one head of any length: with a workspace the key loop of every query tile is cut into
    2, 4 or 8 ranges that run as separate workgroups and are combined by a second kernel.  Same result as the oracle,
    and as the plain kernel up to the rounding of P (the ranges have other reference points) and of the fp32 additions;
    ragged last ranges, both tail modes, and what a missing or short workspace does."""
    from feather_amd import _native as N
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    lib = N.lib()
    need = int(lib.feather_flash_attn_workspace_bytes(heads, L, d))
    ranges = need // (heads * L * (d + 2) * 4)
    assert ranges in (2, 4, 8) and need == ranges * heads * L * (d + 2) * 4
    rng = np.random.default_rng(heads * 1000 + L + d)
    q, k, v = _qkv(rng, heads, L, d, mode, orc)
    qd, kd, vd = (_dev_words(t, dev) for t in (q, k, v))
    got = flash_attention_fp8_acc_fp32_gpu(qd, kd, vd, L, d // 4, mode=mode, tail=tail).cpu().numpy().reshape(heads, L, d)
    plain = flash_attention_fp8_acc_fp32_gpu(qd, kd, vd, L, d // 4, mode=mode, tail=tail, workspace=False)
    plain = plain.cpu().numpy().reshape(heads, L, d)
    if tail == "mask":
        assert _nerr(got, orc.attention_f64_np(q, k, v, L, d, mode)) <= TOL
    else:
        assert _nerr(got, orc.flash_attn(q, k, v, L, d, mode, tail_reference=True)) <= TOL
    assert _nerr(got, plain) <= 8e-4               # two roundings of P against two sets of reference points
    assert not np.array_equal(got, plain)          # the ranges did run
    # through the C ABI: a workspace too small for two ranges runs the plain kernel (bit-identical), one that holds
    # half of what was asked for runs half the ranges
    code, scale = N.mode_code(mode), 1.0 / float(np.sqrt(d))      # the wrapper's default, to the bit
    tl = N.TAIL_MASK if tail == "mask" else N.TAIL_REFERENCE
    for ws_bytes, same_as_plain in ((2 * heads * L * (d + 2) * 4 - 16, True), (need // 2, ranges == 2), (need, False)):
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        out = torch.full((heads, L, d), float("nan"), dtype=torch.float32, device=dev)
        N.check(lib.feather_flash_attn_fp8_ws(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), ws.data_ptr(),
                                              ws_bytes, heads, L, d, 1, code, scale, tl, N.stream_ptr(dev)))
        torch.cuda.synchronize()
        o = out.cpu().numpy()
        assert np.isfinite(o).all()
        assert np.array_equal(o, plain) == same_as_plain
        assert _nerr(o, plain) <= 8e-4


@pytest.mark.parametrize("mode,d,L", [("E4M3", 128, 700), ("E5M2", 64, 1500), ("E4M3", 512, 400)])
def test_flash_attention_key_ranges_with_grouped_kv_heads(dev, orc, mode, d, L):
    """Key ranges over workgroups with four query heads on two K/V heads: the partial results are indexed by query
    head, the K/V rows by the shared head."""
    from feather_amd import _native as N
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    heads, group = 4, 2
    assert int(N.lib().feather_flash_attn_workspace_bytes(heads, L, d)) > 0
    rng = np.random.default_rng(d + L)
    q, _, _ = _qkv(rng, heads, L, d, mode, orc)
    _, k, v = _qkv(rng, heads // group, L, d, mode, orc)
    got = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(k, dev), _dev_words(v, dev), L, d // 4, mode=mode,
                                           kv_group=group).cpu().numpy().reshape(heads, L, d)
    per = L * d // 4
    k_rep = np.concatenate([k.reshape(-1)[(h // group) * per:(h // group + 1) * per] for h in range(heads)])
    v_rep = np.concatenate([v.reshape(-1)[(h // group) * per:(h // group + 1) * per] for h in range(heads)])
    assert _nerr(got, orc.attention_f64_np(q, k_rep, v_rep, L, d, mode)) <= TOL


@pytest.mark.parametrize("mode", ["E4M3", "E5M2"])
@pytest.mark.parametrize("heads,L,d", [(8, 1024, 512), (1, 300, 512), (2, 530, 512), (8, 1024, 256), (8, 1024, 128),
                                         (8, 2048, 64), (4, 600, 32)])
def test_flash_attention_is_identical_from_call_to_call(dev, mode, heads, L, d):
    """Six calls on the same operands give the same bits.  (An asm statement that was the first reader of the score
    MFMA's result did not get the wait states the compiler inserts for its own instructions, and in the shape with 16
    keys per wave group -- d = 512 below 256 workgroups -- the row maximum was now and then taken from accumulators
    that the last MFMA had not updated yet: a valid result with another reference point, but another one from call to
    call.)  With and without the workspace for key ranges."""
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    import feather_amd as feather
    g = torch.Generator(device=dev).manual_seed(heads + L + d)
    q, k, v = (feather.pack_fp8_tensor(torch.randn(heads, L, d, generator=g, device=dev).half(), mode=mode).view(heads, L, d // 4)
               for _ in range(3))
    for ws in (False, True):
        first = flash_attention_fp8_acc_fp32_gpu(q, k, v, L, d // 4, mode=mode, workspace=ws)
        for _ in range(5):
            assert torch.equal(flash_attention_fp8_acc_fp32_gpu(q, k, v, L, d // 4, mode=mode, workspace=ws), first)


def test_flash_attention_reference_signature_and_ints(dev, orc):
    """Reference call shape: 2-D [L, d/4] words, h_dim = d // 4, E5M2, integer inputs as in
    bench_attention.py:52-59, output [L, d] fp32 in the original column order."""
    from feather_amd.routines.attention import flash_attention_fp8_e5m2_acc_fp32_gpu
    rng = np.random.default_rng(11)
    L, d = 512, 64
    q, k, v = _qkv(rng, 1, L, d, "E5M2", orc, ints=True)
    out = flash_attention_fp8_e5m2_acc_fp32_gpu(_dev_words(q, dev, (L, d // 4)), _dev_words(k, dev, (L, d // 4)),
                                                _dev_words(v, dev, (L, d // 4)), L, d // 4)
    assert out.shape == (L, d) and out.dtype == torch.float32
    want = orc.attention_f64_np(q, k, v, L, d)[0]
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3
    sd = torch.nn.functional.scaled_dot_product_attention(
        *[torch.from_numpy(orc.decode_np(t, "E5M2", dtype=np.float32).reshape(1, L, d)) for t in (q, k, v)])[0]
    assert np.abs(out.cpu().numpy() - sd.numpy()).max() <= 2e-3


@pytest.mark.parametrize("L,d", [(1, 32), (65, 32), (1, 64), (5, 64), (63, 64), (65, 64), (70, 64), (130, 64),
                                 (70, 256), (100, 256), (40, 512), (81, 512)])   # wide heads: two key groups per tile
def test_flash_attention_ragged_tails(dev, orc, L, d):
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(L)
    q, k, v = _qkv(rng, 2, L, d, "E5M2", orc)
    args = (_dev_words(q, dev), _dev_words(k, dev), _dev_words(v, dev), L, d // 4)
    masked = flash_attention_fp8_acc_fp32_gpu(*args, tail="mask").cpu().numpy()
    assert _nerr(masked, orc.attention_f64_np(q, k, v, L, d)) <= TOL
    ref = flash_attention_fp8_acc_fp32_gpu(*args, tail="reference").cpu().numpy()
    assert _nerr(ref, orc.flash_attn(q, k, v, L, d, tail_reference=True)) <= TOL
    if L % 64 == 0:
        assert np.array_equal(ref, masked)


def test_flash_attention_invariants_and_gqa(dev, orc):
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    import feather_amd as feather
    rng = np.random.default_rng(12)
    L, d = 320, 64
    q, k, v = _qkv(rng, 4, L, d, "E4M3", orc)
    vc = feather.pack_fp8_tensor(torch.full((4, L, d), 1.5, dtype=torch.float16, device=dev), mode="E4M3")
    out = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(k, dev), vc, L, d // 4, mode="E4M3")
    assert torch.allclose(out, torch.full_like(out, 1.5), rtol=2e-3)
    # grouped KV: 4 query heads on 2 KV heads == explicit repetition
    k2, v2 = k.reshape(4, -1)[:2], v.reshape(4, -1)[:2]
    grouped = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(np.ascontiguousarray(k2), dev),
                                               _dev_words(np.ascontiguousarray(v2), dev), L, d // 4, mode="E4M3",
                                               kv_group=2)
    rep = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(np.repeat(k2, 2, axis=0), dev),
                                           _dev_words(np.repeat(v2, 2, axis=0), dev), L, d // 4, mode="E4M3")
    assert torch.equal(grouped, rep)


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("d", [64, 128, 256, 512])
@pytest.mark.parametrize("ramp", ["steps", "creep", "fall"])
def test_flash_attention_rising_scores(dev, orc, mode, d, ramp):
    """The kernels raise the reference point of their exponentials lazily (only when a score exceeds it by
    more than 2^8): scores that jump by ~2^30 every 48 keys (inside and across key tiles), that creep up by
    a few binary orders per tile, or that start at their maximum and fall, must all give the closed-form
    softmax (float64, of the decoded operands)."""
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(d + len(ramp))
    heads, L = 2, 400
    j = np.arange(L, dtype=np.float64)
    c = 1.4426950408889634 / np.sqrt(d)                # exponent units per raw score unit
    if ramp == "steps":
        lift = np.floor(j / 48) * 30.0                 # binary orders of magnitude
    elif ramp == "creep":
        lift = j * (5.0 / 64)
    else:
        lift = (L - j) * (20.0 / 64)
    # q = 0.5 in every dim (+ noise), k_j = kval_j in every dim (+ noise): raw score ~ d * 0.5 * kval_j
    kval = lift / c / (0.5 * d)
    q = (0.5 + 0.05 * rng.standard_normal((heads, L, d))).astype(np.float16)
    k = (kval[None, :, None] + 0.05 * rng.standard_normal((heads, L, d))).astype(np.float16)
    v = rng.standard_normal((heads, L, d)).astype(np.float16)
    qp, kp, vp = (orc.pack_fp8(a, mode) for a in (q, k, v))
    out = flash_attention_fp8_acc_fp32_gpu(_dev_words(qp, dev), _dev_words(kp, dev), _dev_words(vp, dev), L, d // 4,
                                           mode=mode)
    got = out.cpu().numpy().reshape(heads, L, d)
    assert np.isfinite(got).all()
    want64 = orc.attention_f64_np(qp, kp, vp, L, d, mode)
    assert _nerr(got, want64) <= TOL


@pytest.mark.parametrize("mode,d", [("E5M2", 64), ("E4M3", 64), ("E4M3", 256)])
def test_flash_attention_denominator_of_rounded_p(dev, orc, mode, d):
    """The one deliberate deviation from the reference's arithmetic, bounded by itself: the kernels divide by the
    sum of the fp16-rounded P (the values that multiply V), the reference by the sum of P before rounding
    (feather/routines/attention.py:80-82 against :90).  Both quotients are formed here in float64 from the decoded
    operands: they differ by at most 2^-11 of the output scale (the rounding errors of a row's weights mostly
    cancel: measured ~1e-5); the kernel -- whose exponentials refer to another point than the row maximum, so its
    P round differently -- agrees with both to half the stated tolerance or better."""
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(7 + d)
    heads, L = 2, 512
    q, k, v = _qkv(rng, heads, L, d, mode, orc)
    out = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(k, dev), _dev_words(v, dev), L, d // 4,
                                           mode=mode)
    got = out.cpu().numpy().reshape(heads, L, d).astype(np.float64)
    Q, K, V = (orc.decode_np(a, mode).reshape(heads, L, d) for a in (q, k, v))
    S = np.einsum("hqd,hkd->hqk", Q, K) / np.sqrt(d)
    P = np.exp(S - S.max(axis=-1, keepdims=True))
    P16 = P.astype(np.float16).astype(np.float64)
    num = np.einsum("hqk,hkd->hqd", P16, V)
    ref_variant = num / P.sum(axis=-1, keepdims=True)        # the reference: l sums P before rounding
    own_variant = num / P16.sum(axis=-1, keepdims=True)      # the kernels: l sums the rounded P
    scale = np.abs(ref_variant).max()
    assert np.abs(own_variant - ref_variant).max() / scale <= 2.0 ** -11
    assert np.abs(got - own_variant).max() / scale <= 5e-4
    assert np.abs(got - ref_variant).max() / scale <= TOL


@pytest.mark.parametrize("d", [64, 128, 256])
def test_flash_attention_e4m3_kernel_decode_codes(dev, orc, d):
    """E4M3 operands are decoded as the reference kernel does (gemv.py:83-88), not as OCP FP8: a zero-exponent
    code c is m * 2^-17 (OCP: m * 2^-9) and 0x7F / 0xFF are +-480 (OCP: NaN).  Keys made of 0x7F against keys
    made of 0x7E (448) and of zero-exponent codes: an OCP decode would give NaN, and 256 x larger scores for
    the zero-exponent keys."""
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(d)
    L = 192
    K = np.zeros((L, d), np.uint8)
    K[0::3] = 0x7F                                     # 480 in every dim
    K[1::3] = 0x7E                                     # 448
    K[2::3] = rng.integers(1, 8, size=(L // 3, d))     # zero-exponent codes 0x01..0x07
    Q = np.full((L, d), 0x18, np.uint8)                # 2^-4: raw scores 30 d, 28 d and ~0
    Q[1::2] = 0x98                                     # and -2^-4 for the odd queries
    V = rng.integers(0x30, 0x48, size=(L, d)).astype(np.uint8)   # values around 1
    V[0::3] |= 0x80
    q, k, v = (np.ascontiguousarray(a).view(np.uint32) for a in (Q, K, V))
    out = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(k, dev), _dev_words(v, dev), L, d // 4,
                                           mode="E4M3").cpu().numpy()
    assert np.isfinite(out).all()
    want = orc.attention_f64_np(q, k, v, L, d, "E4M3")[0]
    assert _nerr(out, want) <= TOL
    # even queries attend to the 480-keys (negative V), odd queries to the zero-exponent keys (scores ~0 against
    # -30 d and -28 d): the two groups of rows must differ the way the closed form says
    assert want[0].mean() < 0 < want[1].mean()


def test_flash_attention_repeatable_and_graph_replay(dev, orc):
    """Same inputs, same bits: across calls and across replays of a captured HIP graph (the kernels hold no state
    between calls and have no atomics)."""
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    import feather_amd as feather
    g = torch.Generator(device=dev).manual_seed(7)
    for mode, H, L, d in (("E5M2", 8, 1024, 64), ("E4M3", 8, 1024, 64), ("E4M3", 2, 512, 256)):
        qkv = [feather.pack_fp8_tensor(torch.randn(H, L, d, generator=g, device=dev).half(), mode=mode).view(H, L, d // 4)
               for _ in range(3)]
        ref = flash_attention_fp8_acc_fp32_gpu(*qkv, L, d // 4, mode=mode).clone()
        again = flash_attention_fp8_acc_fp32_gpu(*qkv, L, d // 4, mode=mode)
        assert torch.equal(ref, again)
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            flash_attention_fp8_acc_fp32_gpu(*qkv, L, d // 4, mode=mode)
        torch.cuda.current_stream().wait_stream(s)
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            out = flash_attention_fp8_acc_fp32_gpu(*qkv, L, d // 4, mode=mode)
        for _ in range(3):
            out.zero_()
            gr.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, ref)


@pytest.mark.parametrize("d", [64, 128])
def test_flash_attention_e5m2_subnormal_codes_count(dev, orc, d):
    """E5M2 scores must keep subnormal codes exact: keys of code 0x01 (2^-16) against queries of
    code 0x7B (57344) give a raw score of 0.875 * d, against 0 for the zero keys;
    flushing the subnormals would leave a uniform softmax (output -0.5 instead of ~1)."""
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    L = 64
    K = np.zeros((L, d), np.uint8)
    K[:32] = 0x01
    Q = np.full((L, d), 0x7B, np.uint8)
    V = np.zeros((L, d), np.uint8)
    V[:32], V[32:] = 0x3C, 0xC0  # 1.0 and -2.0
    q, k, v = (np.ascontiguousarray(a).view(np.uint32) for a in (Q, K, V))
    out = flash_attention_fp8_acc_fp32_gpu(_dev_words(q, dev), _dev_words(k, dev), _dev_words(v, dev), L, d // 4,
                                           mode="E5M2").cpu().numpy()
    want = orc.attention_f64_np(q, k, v, L, d, "E5M2")[0]
    assert want[0, 0] > 0.9
    assert np.abs(out - want).max() <= 1e-5


def test_flash_attention_config_sized_property(dev, orc):
    """B4 H16 L4096 d64 E5M2: too big for the scalar oracle; compare with torch SDPA (fp32 math) of the
    operands decoded on the host by the oracle's table (the first two heads of every batch entry) and check
    determinism."""
    import feather_amd as feather
    g = torch.Generator().manual_seed(3)
    B, H, L, d = 4, 16, 4096, 64
    qkv = [torch.randn(B, H, L, d, generator=g).half().to(dev) for _ in range(3)]
    p = [feather.pack_fp8_tensor(t, mode="E5M2").view(B, H, L, d // 4) for t in qkv]
    out = feather.flash_attention_fp8_e5m2_acc_fp32_gpu(p[0], p[1], p[2], L, d // 4)
    assert out.shape == (B, H, L, d)
    dec = [torch.from_numpy(orc.decode_np(t[:, :2].contiguous().view(torch.int32).cpu().numpy().view(np.uint32).reshape(-1),
                                          "E5M2", dtype=np.float32).reshape(B, 2, L, d)).to(dev) for t in p]
    with torch.backends.cuda.sdp_kernel(enable_flash=False, enable_mem_efficient=False, enable_math=True):
        want = torch.nn.functional.scaled_dot_product_attention(dec[0], dec[1], dec[2])
    err = (out[:, :2] - want).abs().max() / want.abs().max()
    assert err.item() <= TOL
    again = feather.flash_attention_fp8_e5m2_acc_fp32_gpu(p[0], p[1], p[2], L, d // 4)
    assert torch.equal(out, again)


@pytest.mark.parametrize("mode,B,H,L,d,causal", [
    ("E5M2", 4, 16, 8192, 64, False), ("E4M3", 1, 8, 4096, 256, False), ("E4M3", 1, 8, 8192, 512, False),
    ("E4M3", 1, 8, 1024, 256, True), ("E5M2", 2, 4, 8192, 64, True),
    # eight-wave workgroups: d = 128 and d = 512 switch to them once the coarser grid covers 256 CUs
    ("E5M2", 4, 16, 4096, 128, False), ("E4M3", 4, 16, 1024, 128, True), ("E4M3", 1, 8, 4100, 512, True),
    ("E5M2", 1, 8, 4096, 256, False), ("E4M3", 1, 8, 1024, 256, False),
    # d = 256 with >= 256 workgroups of 256 queries: 32 queries per wave
    ("E4M3", 2, 16, 2048, 256, False), ("E5M2", 2, 16, 2048, 256, True), ("E4M3", 1, 8, 8192, 256, False),
    # the wide-head benchmark configuration (B1 H8, E4M3) at its two remaining lengths
    ("E4M3", 1, 8, 1024, 512, False), ("E4M3", 1, 8, 4096, 512, False),
    ("E5M2", 4, 16, 4096, 64, False),
])
def test_flash_attention_full_size_rows_vs_fp32_math(dev, orc, mode, B, H, L, d, causal):
    """The remaining attention shapes of the benchmark configurations, too big for the scalar oracle:
    a sample of query rows of two heads against explicit softmax(q K^T / sqrt(d)) V in float64 of the
    operands, whose packed words are copied to the host and decoded there by the oracle's table."""
    import feather_amd as feather
    g = torch.Generator(device=dev).manual_seed(L + d)
    qkv = [torch.randn(B, H, L, d, generator=g, device=dev).half() for _ in range(3)]
    p = [feather.pack_fp8_tensor(t, mode=mode).view(B, H, L, d // 4) for t in qkv]
    out = feather.flash_attention_fp8_acc_fp32_gpu(p[0], p[1], p[2], L, d // 4, mode=mode, causal=causal)
    assert out.shape == (B, H, L, d) and bool(torch.isfinite(out).all())
    rows = np.array([0, 1, 63, 64, L // 2 - 1, L // 2, L - 2, L - 1])
    for b, h in ((0, 0), (B - 1, H - 1)):
        qd, kd, vd = (orc.decode_np(t[b, h].contiguous().view(torch.int32).cpu().numpy().view(np.uint32).reshape(-1), mode)
                      .reshape(L, d) for t in p)                         # float64, on the host
        s = qd[rows] @ kd.T / np.sqrt(d)                                   # [rows, L]
        if causal:
            s = np.where(np.arange(L)[None, :] > rows[:, None], -np.inf, s)
        w = np.exp(s - s.max(axis=-1, keepdims=True))
        want = (w / w.sum(axis=-1, keepdims=True)) @ vd
        got = out[b, h][torch.from_numpy(rows).to(dev)].double().cpu().numpy()
        assert np.abs(got - want).max() / np.abs(want).max() <= TOL


@pytest.mark.parametrize("seed", range(12))
def test_varlen_attention_random_shapes(dev, orc, seed):
    """Seeded random (mode, head dim, head counts, lengths, causal) draws: the launcher picks between
    four- and eight-wave workgroups and the key-split shape from the grid size, so cover its choices
    with lengths that land on and around every tile size."""
    from feather_amd.routines.attention import flash_attention_fp8_varlen_acc_fp32_gpu
    rng = np.random.default_rng(1000 + seed)
    mode = ("E5M2", "E4M3")[seed % 2]
    d = (64, 128, 256, 512)[(seed // 2) % 4]
    n_kv = int(rng.integers(1, 5))
    n_heads = n_kv * int(rng.integers(1, 5))
    edges = np.array([0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513])
    n_seq = int(rng.integers(1, 7)) if seed % 3 else int(rng.integers(20, 40))
    lens = [int(x) for x in rng.choice(edges[edges <= (513 if d <= 128 else 257)], size=n_seq)]
    if max(lens) == 0:
        lens[0] = 33
    causal = bool(seed % 4 < 2)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    total = int(cu[-1])
    q = orc.pack_fp8(rng.standard_normal((n_heads, total, d)).astype(np.float16), mode).reshape(n_heads, total, d // 4)
    k = orc.pack_fp8(rng.standard_normal((n_kv, total, d)).astype(np.float16), mode).reshape(n_kv, total, d // 4)
    v = orc.pack_fp8(rng.standard_normal((n_kv, total, d)).astype(np.float16), mode).reshape(n_kv, total, d // 4)
    out = flash_attention_fp8_varlen_acc_fp32_gpu(_dev_words(q, dev, q.shape), _dev_words(k, dev, k.shape),
                                                  _dev_words(v, dev, v.shape), torch.from_numpy(cu).to(dev), max(lens),
                                                  mode=mode, causal=causal).cpu().numpy()
    want = orc.attention_varlen_f64_np(q, k, v, cu, d, mode, causal=causal)
    assert np.isfinite(out).all() and _nerr(out, want) <= TOL


# ---------------------------------------------------------------- paged decode

@pytest.mark.parametrize("mode,n_seq,Hq,Hkv,d,bs,max_ctx", [
    ("E5M2", 3, 8, 2, 64, 16, 100), ("E4M3", 4, 32, 4, 64, 16, 700), ("E4M3", 2, 4, 4, 128, 16, 300),
    ("E5M2", 2, 16, 1, 64, 8, 90), ("E4M3", 1, 2, 1, 256, 32, 257),
    # d = 512 (one step in flight per wave, 96 KB of LDS for the wave merge): one split, three splits, odd block size
    ("E4M3", 2, 4, 2, 512, 16, 200), ("E5M2", 3, 8, 1, 512, 16, 1300), ("E4M3", 2, 2, 2, 512, 12, 100),
])
def test_paged_attention_vs_oracle(dev, orc, mode, n_seq, Hq, Hkv, d, bs, max_ctx):
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(n_seq * 7 + Hq + d + max_ctx)
    max_blocks = (max_ctx + bs - 1) // bs
    n_blocks = n_seq * max_blocks + 3
    ctx = rng.integers(1, max_ctx + 1, size=n_seq).astype(np.int32)
    ctx[0] = max_ctx
    kc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode)
    vc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode)
    q = orc.pack_fp8(rng.standard_normal((n_seq, Hq, d)).astype(np.float16), mode)
    bt = rng.permutation(n_blocks)[: n_seq * max_blocks].reshape(n_seq, max_blocks).astype(np.int32)
    want = orc.paged_attn(q, kc, vc, bt, ctx, Hq, Hkv, d, bs, mode)
    out = paged_attention_fp8_acc_fp32_gpu(
        _dev_words(q, dev, (n_seq, Hq, d // 4)), _dev_words(kc, dev, (n_blocks, Hkv, bs, d // 4)),
        _dev_words(vc, dev, (n_blocks, Hkv, bs, d // 4)), torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev),
        mode=mode, max_context_len=max_ctx)
    assert out.shape == (n_seq, Hq, d)
    assert _nerr(out.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("mode,n_seq,Hq,Hkv,d,bs,max_ctx", [
    ("E4M3", 70, 4, 2, 64, 16, 1100),      # more sequences than lanes of a wave, three splits
    ("E5M2", 5, 8, 2, 64, 12, 700),        # block size that is not a power of two, two splits
    ("E4M3", 3, 6, 3, 128, 4, 1030),       # smallest power-of-two block, three splits, d = 128
])
def test_paged_attention_split_bookkeeping(dev, orc, mode, n_seq, Hq, Hkv, d, bs, max_ctx):
    """Contexts of every kind under one context bound: empty, one token, exactly one split, one token
    more, the bound itself.  Empty sequences give zero rows."""
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(n_seq + bs + max_ctx)
    max_blocks = (max_ctx + bs - 1) // bs
    n_blocks = n_seq * max_blocks + 1
    ctx = rng.integers(0, max_ctx + 1, size=n_seq).astype(np.int32)
    ctx[: 5] = [0, 1, 512, 513, max_ctx][: min(5, n_seq)]
    if n_seq > 5:
        ctx[-1] = 0
    kc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode).reshape(n_blocks, -1)
    vc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode).reshape(n_blocks, -1)
    poison = n_blocks - 1                                      # a block of NaN codes: using it shows in the result
    kc[poison] = vc[poison] = 0x7F7F7F7F
    q = orc.pack_fp8(rng.standard_normal((n_seq, Hq, d)).astype(np.float16), mode)
    bt = rng.permutation(n_blocks - 1)[: n_seq * max_blocks].reshape(n_seq, max_blocks).astype(np.int32)
    for i in range(n_seq):                                     # entries past a context must never be used
        bt[i, (ctx[i] + bs - 1) // bs:] = poison
    out = paged_attention_fp8_acc_fp32_gpu(
        _dev_words(q, dev, (n_seq, Hq, d // 4)), _dev_words(kc, dev, (n_blocks, Hkv, bs, d // 4)),
        _dev_words(vc, dev, (n_blocks, Hkv, bs, d // 4)), torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev),
        mode=mode, max_context_len=max_ctx).cpu().numpy()
    live = np.flatnonzero(ctx > 0)
    want = orc.paged_attn(q.reshape(n_seq, -1)[live], kc, vc, bt[live], ctx[live], Hq, Hkv, d, bs, mode)
    assert np.isfinite(want).all()
    assert _nerr(out[live], want) <= TOL
    assert not out[ctx == 0].any()


@pytest.mark.parametrize("seed", range(12))
def test_paged_attention_random_shapes(dev, orc, seed):
    """Random head groupings, head dims, block sizes (powers of two and not), context bounds around the
    512-token split and contexts from empty to the bound, against the oracle."""
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(1000 + seed)
    mode = ("E5M2", "E4M3")[seed % 2]
    d = int(rng.choice([64, 64, 128, 256]))
    group = int(rng.choice([1, 2, 3, 4, 8, 16]))
    Hkv = int(rng.integers(1, 4))
    Hq = group * Hkv
    bs = int(rng.choice([4, 8, 16, 32, 5, 12, 24]))
    max_ctx = int(rng.choice([1, 31, 200, 512, 513, 1024, 1025, 1400]))
    n_seq = int(rng.integers(1, 7))
    max_blocks = (max_ctx + bs - 1) // bs
    n_blocks = n_seq * max_blocks + 2
    ctx = rng.integers(0, max_ctx + 1, size=n_seq).astype(np.int32)
    ctx[rng.integers(0, n_seq)] = max_ctx
    kc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode).reshape(n_blocks, -1)
    vc = orc.pack_fp8(rng.standard_normal((n_blocks, Hkv, bs, d)).astype(np.float16), mode).reshape(n_blocks, -1)
    poison = n_blocks - 1
    kc[poison] = vc[poison] = 0x7F7F7F7F
    q = orc.pack_fp8((2.0 * rng.standard_normal((n_seq, Hq, d))).astype(np.float16), mode)
    bt = rng.permutation(n_blocks - 1)[: n_seq * max_blocks].reshape(n_seq, max_blocks).astype(np.int32)
    for i in range(n_seq):
        bt[i, (ctx[i] + bs - 1) // bs:] = poison
    print(f"seed {seed}: {mode} n_seq {n_seq} Hq {Hq} Hkv {Hkv} d {d} bs {bs} max_ctx {max_ctx} ctx {ctx.tolist()}", flush=True)
    out = paged_attention_fp8_acc_fp32_gpu(
        _dev_words(q, dev, (n_seq, Hq, d // 4)), _dev_words(kc, dev, (n_blocks, Hkv, bs, d // 4)),
        _dev_words(vc, dev, (n_blocks, Hkv, bs, d // 4)), torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev),
        mode=mode, max_context_len=max_ctx).cpu().numpy()
    live = np.flatnonzero(ctx > 0)
    want = orc.paged_attn(q.reshape(n_seq, -1)[live], kc, vc, bt[live], ctx[live], Hq, Hkv, d, bs, mode)
    assert np.isfinite(want).all()
    assert _nerr(out[live], want) <= TOL
    assert not out[ctx == 0].any()


def test_paged_attention_config_shape(dev, orc):
    """TinyLlama-shaped decode attention: batch 32, 32 query / 4 KV heads, d 64, block 16,
    contexts uniform in [512, 4096], permuted block table."""
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
    import feather_amd as feather
    g = torch.Generator().manual_seed(5)
    n_seq, Hq, Hkv, d, bs = 32, 32, 4, 64, 16
    ctx = torch.randint(512, 4097, (n_seq,), generator=g, dtype=torch.int32)
    max_blocks = 4096 // bs
    n_blocks = n_seq * max_blocks
    bt = torch.randperm(n_blocks, generator=g).to(torch.int32).view(n_seq, max_blocks)
    kc = feather.pack_fp8_tensor(torch.randn(n_blocks, Hkv, bs, d, generator=g).half().to(dev), mode="E4M3")
    vc = feather.pack_fp8_tensor(torch.randn(n_blocks, Hkv, bs, d, generator=g).half().to(dev), mode="E4M3")
    q = feather.pack_fp8_tensor(torch.randn(n_seq, Hq, d, generator=g).half().to(dev), mode="E4M3")
    out = paged_attention_fp8_acc_fp32_gpu(q.view(n_seq, Hq, d // 4), kc.view(n_blocks, Hkv, bs, d // 4),
                                           vc.view(n_blocks, Hkv, bs, d // 4), bt.to(dev), ctx.to(dev), mode="E4M3")
    to_np = lambda t: t.view(torch.int32).cpu().numpy().view(np.uint32)
    seqs = [0, 7, 31]                                          # the oracle is scalar C: check three sequences
    want = orc.paged_attn(to_np(q).reshape(n_seq, -1)[seqs], to_np(kc), to_np(vc), bt.numpy()[seqs], ctx.numpy()[seqs],
                          Hq, Hkv, d, bs, "E4M3")
    assert _nerr(out.cpu().numpy()[seqs], want) <= TOL


# ---------------------------------------------------------------- variable length, causal, cache writer

@pytest.mark.parametrize("mode,n_heads,n_kv,d,lens,causal", [
    ("E5M2", 2, 1, 64, [70, 0, 300, 1], True), ("E5M2", 2, 2, 64, [70, 0, 300, 1], False),
    ("E4M3", 4, 2, 64, [513, 255], True), ("E5M2", 1, 1, 128, [129, 64], True),
    ("E4M3", 1, 1, 256, [100, 37], True), ("E5M2", 1, 1, 512, [65], True), ("E4M3", 2, 1, 128, [200], False),
    # enough (head, sequence, tile) groups for the eight-wave d = 128 shape; lengths straddle its 256-query tile
    ("E4M3", 8, 4, 128, [257, 31, 0, 256] * 4, True), ("E5M2", 16, 16, 128, [300, 90] * 4, False),
    # the eight-wave d = 64 shape (non-causal, >= 256 groups of 512 queries), lengths around its tile
    ("E5M2", 16, 8, 64, [513, 100, 512, 0] * 4, False),
    ("E4M3", 2, 1, 256, [130, 64, 0, 257], False),           # d = 256 with the key tiles split between wave groups
    ("E4M3", 16, 8, 256, [257, 100] * 8, True),              # d = 256, 32 queries per wave (>= 256 workgroups)
    ("E5M2", 4, 2, 32, [70, 0, 300, 1], True), ("E4M3", 2, 1, 32, [129, 64], False),     # d = 32
])
def test_varlen_attention_vs_oracle(dev, orc, mode, n_heads, n_kv, d, lens, causal):
    from feather_amd.routines.attention import flash_attention_fp8_varlen_acc_fp32_gpu
    rng = np.random.default_rng(sum(lens) + d + n_heads)
    gap = 3                                                  # rows in front of the first sequence belong to no one
    cu = np.concatenate([[gap], gap + np.cumsum(lens)]).astype(np.int32)
    total = int(cu[-1]) + 2
    q = orc.pack_fp8(rng.standard_normal((n_heads, total, d)).astype(np.float16), mode).reshape(n_heads, total, d // 4)
    k = orc.pack_fp8(rng.standard_normal((n_kv, total, d)).astype(np.float16), mode).reshape(n_kv, total, d // 4)
    v = orc.pack_fp8(rng.standard_normal((n_kv, total, d)).astype(np.float16), mode).reshape(n_kv, total, d // 4)
    out = flash_attention_fp8_varlen_acc_fp32_gpu(_dev_words(q, dev, q.shape), _dev_words(k, dev, k.shape),
                                                  _dev_words(v, dev, v.shape), torch.from_numpy(cu).to(dev), max(lens),
                                                  mode=mode, causal=causal).cpu().numpy()
    want = orc.attention_varlen_f64_np(q, k, v, cu, d, mode, causal=causal)
    assert _nerr(out, want) <= TOL
    assert not out[:, :gap].any() and not out[:, int(cu[-1]):].any()      # rows outside every sequence untouched


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_causal_fixed_length_rows_equal_prefix_attention(dev, orc, mode):
    """causal=True of the fixed-length entry: row i equals the non-causal kernel run on keys 0..i
    (L = 1000: ragged last tile, several query tiles)."""
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(21)
    heads, L, d = 2, 1000, 64
    q, k, v = _qkv(rng, heads, L, d, mode, orc)
    qd, kd, vd = (_dev_words(a, dev, (heads, L, d // 4)) for a in (q, k, v))
    caus = flash_attention_fp8_acc_fp32_gpu(qd, kd, vd, L, d // 4, mode=mode, causal=True)
    assert caus.shape == (heads, L, d)
    for i in (0, 63, 64, 255, 256, 700, 999):
        pre = flash_attention_fp8_acc_fp32_gpu(qd[:, i:i + 1].expand(heads, i + 1, d // 4).contiguous(),
                                               kd[:, :i + 1].contiguous(), vd[:, :i + 1].contiguous(), i + 1, d // 4, mode=mode)
        err = (caus[:, i] - pre[:, 0]).abs().max() / pre[:, 0].abs().max()
        assert err.item() <= TOL
    with pytest.raises(ValueError):
        flash_attention_fp8_acc_fp32_gpu(qd, kd, vd, L, d // 4, mode=mode, causal=True, tail="reference")


@pytest.mark.parametrize("mode,f16", [("E5M2", False), ("E4M3", False), ("E4M3", True), ("E5M2", True)])
def test_paged_cache_write_bit_exact(dev, orc, mode, f16):
    from feather_amd.routines.paged_attention import paged_cache_write
    rng = np.random.default_rng(8)
    n_kv, d, bs, max_blocks = 2, 64, 16, 6
    lens, start = [40, 0, 77, 5], np.array([3, 0, 30, 95], dtype=np.int32)   # sequence 2 overruns 96 slots: rows dropped
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    total, n_blocks = int(cu[-1]) + 4, 4 * max_blocks + 1
    bt = rng.permutation(n_blocks - 1)[:4 * max_blocks].reshape(4, max_blocks).astype(np.int32)
    k16, v16 = (rng.standard_normal((n_kv, total, d)).astype(np.float16) * 20 for _ in range(2))
    k16[0, 1, :4] = [np.inf, -np.inf, 500.0, 1e-4]                            # saturating and tiny values through the encoder
    kw, vw = (orc.pack_fp8(a, mode).reshape(n_kv, total, d // 4) for a in (k16, v16))
    fill = rng.integers(0, 2**32, (n_blocks, n_kv, bs, d // 4), dtype=np.uint64).astype(np.uint32)
    kc, vc = fill.copy(), fill[::-1].copy()
    kcd, vcd = _dev_words(kc, dev, kc.shape), _dev_words(vc, dev, vc.shape)
    src = (torch.from_numpy(k16).to(dev), torch.from_numpy(v16).to(dev)) if f16 else \
        (_dev_words(kw, dev, kw.shape), _dev_words(vw, dev, vw.shape))
    paged_cache_write(src[0], src[1], kcd, vcd, torch.from_numpy(bt).to(dev), torch.from_numpy(cu).to(dev),
                      torch.from_numpy(start).to(dev), mode=mode)
    orc.paged_cache_write_np(kw, vw, kc, vc, bt, cu, start)
    assert np.array_equal(kcd.cpu().view(torch.int32).numpy().view(np.uint32), kc)      # untouched slots keep their fill
    assert np.array_equal(vcd.cpu().view(torch.int32).numpy().view(np.uint32), vc)


def test_prefill_then_decode_agree(dev, orc):
    """End to end: causal prefill over packed sequences, the same K/V written to a paged cache, and the
    decode kernel asked for the LAST token of every sequence give the same rows."""
    from feather_amd.routines.attention import flash_attention_fp8_varlen_acc_fp32_gpu
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu, paged_cache_write
    rng = np.random.default_rng(9)
    mode, n_heads, n_kv, d, bs = "E4M3", 8, 2, 64, 16
    lens = [300, 17, 1024]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    total, max_blocks = int(cu[-1]), 64
    q = orc.pack_fp8(rng.standard_normal((n_heads, total, d)).astype(np.float16), mode).reshape(n_heads, total, d // 4)
    k = orc.pack_fp8(rng.standard_normal((n_kv, total, d)).astype(np.float16), mode).reshape(n_kv, total, d // 4)
    v = orc.pack_fp8(rng.standard_normal((n_kv, total, d)).astype(np.float16), mode).reshape(n_kv, total, d // 4)
    qd, kd, vd = (_dev_words(a, dev, a.shape) for a in (q, k, v))
    cud = torch.from_numpy(cu).to(dev)
    pre = flash_attention_fp8_varlen_acc_fp32_gpu(qd, kd, vd, cud, max(lens), mode=mode, causal=True)
    n_blocks = 3 * max_blocks
    bt = torch.from_numpy(rng.permutation(n_blocks).reshape(3, max_blocks).astype(np.int32)).to(dev)
    kc = torch.zeros((n_blocks, n_kv, bs, d // 4), dtype=torch.int32, device=dev).view(torch.uint32)
    vc = torch.zeros_like(kc)
    paged_cache_write(kd, vd, kc, vc, bt, cud, mode=mode)
    last = torch.from_numpy(cu[1:] - 1).to(dev).long()
    q_last = qd.view(torch.int32)[:, last].permute(1, 0, 2).contiguous().view(torch.uint32)      # [n_seq, n_heads, d/4]
    dec = paged_attention_fp8_acc_fp32_gpu(q_last, kc, vc, bt, torch.tensor(lens, dtype=torch.int32, device=dev), mode=mode)
    want = pre[:, last].permute(1, 0, 2)
    assert ((dec - want).abs().max() / want.abs().max()).item() <= TOL
