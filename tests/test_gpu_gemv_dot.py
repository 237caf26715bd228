"""GPU parity: packed GEMV / dot kernels against the CPU oracle.

Tolerance for floating-point results: max |y - y_ref| / max |y_ref| <= 1e-3 against the
kernel-semantics decode followed by a float64 reduction (outputs cross zero, so the error
is normalised by the output scale).  Integer-valued inputs must match exactly."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _dev_words(a, dev):
    return torch.from_numpy(a.view(np.int32).copy()).to(dev).view(torch.uint32)


def _nerr(got, want):
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))



def _host_decode(words: torch.Tensor, mode: str, orc) -> torch.Tensor:
    """Packed words copied to the host and decoded there by the oracle's table (kernel semantics); float64 on the CPU."""
    return torch.from_numpy(orc.decode_np(words.reshape(-1).view(torch.int32).cpu().numpy().view(np.uint32), mode))


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_gemv_docstring_known_answer(dev, kats, mode):
    import feather_amd as feather
    k = kats["gemv"]
    a = torch.tensor(k["matrix"], dtype=torch.float16)
    b = torch.tensor(k["vector"], dtype=torch.float16)
    ap = feather.pack_fp8_tensor(a, mode=mode).to(dev)
    bp = feather.pack_fp8_tensor(b, mode=mode).to(dev)
    out = feather.gemv(ap, bp, original_shape=a.shape, mode=mode)
    assert out.dtype == torch.float32 and out.is_cuda and out.tolist() == k["expected"]
    from feather_amd.routines.gemv import gemv_fp8_e4m3_acc_fp32_gpu, gemv_fp8_e5m2_acc_fp32_gpu
    f = gemv_fp8_e5m2_acc_fp32_gpu if mode == "E5M2" else gemv_fp8_e4m3_acc_fp32_gpu
    assert f(ap, bp, a.shape).tolist() == k["expected"]


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("M,K", [(4096, 4096), (300, 8192), (7, 20), (129, 1040), (16, 36864), (1, 16)])
def test_gemv_integer_inputs_exact(dev, mode, M, K):
    """Reference harness inputs (bench_gemv.py:53-57): the result is the exact integer matvec."""
    import feather_amd as feather
    g = torch.Generator().manual_seed(M * 31 + K)
    a = torch.randint(-3, 3, (M, K), generator=g).to(torch.float16)
    b = torch.randint(-3, 3, (K,), generator=g).to(torch.float16)
    out = feather.gemv(feather.pack_fp8_tensor(a.to(dev), mode=mode), feather.pack_fp8_tensor(b.to(dev), mode=mode),
                       original_shape=(M, K), mode=mode)
    want = torch.mv(a.double(), b.double())
    assert torch.equal(out.cpu().double(), want)


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("M,K", [(512, 8192), (1000, 2048), (64, 16384), (33, 48), (8, 40000)])
def test_gemv_random_vs_oracle(dev, orc, mode, M, K):
    import feather_amd as feather
    rng = np.random.default_rng(M + K)
    a = rng.standard_normal((M, K)).astype(np.float32)
    a[rng.random((M, K)) < 0.01] *= 1e-3                      # E4M3 zero-exponent codes (flush semantics)
    b = rng.standard_normal(K).astype(np.float32)
    b[rng.random(K) < 0.01] *= 1e-3
    mp, vp = orc.pack_fp8(a.astype(np.float16), mode), orc.pack_fp8(b.astype(np.float16), mode)
    out = feather.gemv(_dev_words(mp, dev), _dev_words(vp, dev), original_shape=(M, K), mode=mode).cpu().numpy()
    want64 = orc.gemv_f64_np(mp, vp, M, K, mode)
    assert _nerr(out, want64) <= TOL
    if M * K <= 1 << 20:                                      # reference-structured fp32 oracle on small cases
        assert _nerr(out, orc.gemv(mp, vp, M, K, mode)) <= TOL
    assert _nerr(out, want64) <= 1e-4                         # fp32 accumulation is far inside the bar


def test_gemv_e4m3_uses_kernel_decode_not_ieee(dev, orc):
    """A matrix made only of zero-exponent codes separates the two decodes by 2^8."""
    import feather_amd as feather
    codes = np.tile(np.array([1, 2, 3, 4, 5, 6, 7, 0x87], np.uint8), 64 * 16 // 8).reshape(16, 64)
    v = np.full(64, 0x38, np.uint8)                           # 1.0 in E4M3
    out = feather.gemv(_dev_words(codes.reshape(-1).view(np.uint32), dev), _dev_words(v.view(np.uint32), dev),
                       original_shape=(16, 64), mode="E4M3").cpu().numpy()
    want = orc.gemv(codes.reshape(-1).view(np.uint32), v.view(np.uint32), 16, 64, "E4M3", acc64=True)
    assert np.allclose(out, want, rtol=1e-6) and np.allclose(out, 8 * (28 - 7) * 2.0 ** -17)
    nan_codes = np.full((16, 64), 0x7F, np.uint8)             # NaN code decodes to 480 in the kernels
    out = feather.gemv(_dev_words(nan_codes.reshape(-1).view(np.uint32), dev), _dev_words(v.view(np.uint32), dev),
                       original_shape=(16, 64), mode="E4M3").cpu().numpy()
    assert np.array_equal(out, np.full(16, 480.0 * 64, np.float32))
    # NaN codes mixed with ordinary and zero-exponent codes, in the matrix and in the vector
    rng = np.random.default_rng(99)
    M, K = 48, 2048
    mc = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    mc[rng.random((M, K)) < 0.02] = 0x7F
    mc[rng.random((M, K)) < 0.02] = 0xFF
    for vec_nan in (False, True):
        vc = rng.integers(0, 256, size=K).astype(np.uint8)
        vc[(vc & 0x7F) == 0x7F] = 0x30
        if vec_nan:
            vc[[5, 700, 2047]] = [0x7F, 0xFF, 0x7F]
        out = feather.gemv(_dev_words(mc.reshape(-1).view(np.uint32), dev), _dev_words(vc.view(np.uint32), dev),
                           original_shape=(M, K), mode="E4M3").cpu().numpy()
        want = orc.gemv(mc.reshape(-1).view(np.uint32), vc.view(np.uint32), M, K, "E4M3", acc64=True)
        assert _nerr(out, want) <= 1e-4


def test_gemv_config_sized_properties(dev, orc):
    """16384 x 16384 (too large for the scalar oracle): linearity in the vector and agreement
    with a torch float64 matvec of the operands decoded by the HIP unpack kernel, both on device.  That
    check leans on the unpack kernel (which test_gpu_pack.py holds bit-exact to the oracle's decode on
    all 256 codes of both modes in the same run), so 1 024 rows -- the first and last rows of the matrix, of
    eight-row groups and of random positions -- are also checked without it: their packed words are copied to
    the host, decoded by the oracle's table and summed in float64."""
    import feather_amd as feather
    g = torch.Generator().manual_seed(2)
    M = K = 16384
    x = torch.randn(M, K, generator=g)
    x[torch.rand(M, K, generator=g) < 0.01] *= 1e-3
    v = torch.randn(K, generator=g)
    for mode in ("E5M2", "E4M3"):
        mp = feather.pack_fp8_tensor(x.half().to(dev), mode=mode)
        vp = feather.pack_fp8_tensor(v.half().to(dev), mode=mode)
        out = feather.gemv(mp, vp, original_shape=(M, K), mode=mode)
        md = feather.unpack_fp8_tensor(mp, mode=mode, semantics="kernel").view(M, K)
        vd = feather.unpack_fp8_tensor(vp, mode=mode, semantics="kernel")
        want = torch.mv(md.double(), vd.double())
        assert ((out.double() - want).abs().max() / want.abs().max()).item() <= 1e-4
        rows = np.unique(np.concatenate([np.arange(16), M - 1 - np.arange(16), 8 * np.arange(0, M // 8, 37),
                                         8 * np.arange(0, M // 8, 41) + 7,
                                         np.random.default_rng(3).integers(0, M, 400)]))
        words = mp.view(torch.int32).view(M, K // 4)[torch.from_numpy(rows).to(dev)].cpu().numpy().view(np.uint32)
        m_host = orc.decode_np(words.reshape(-1), mode).reshape(len(rows), K).astype(np.float64)
        v_host = orc.decode_np(vp.view(torch.int32).cpu().numpy().view(np.uint32), mode)[:K].astype(np.float64)
        want_rows = m_host @ v_host
        got_rows = out.cpu().numpy().astype(np.float64)[rows]
        assert np.abs(got_rows - want_rows).max() / np.abs(want_rows).max() <= 1e-4
        # twice the vector (exact in FP8: exponent + 1) doubles the result exactly
        vp2 = feather.pack_fp8_tensor((2 * v.half()).to(dev), mode=mode)
        vd2 = feather.unpack_fp8_tensor(vp2, mode=mode, semantics="kernel")
        if torch.equal(vd2, 2 * vd):
            assert torch.equal(feather.gemv(mp, vp2, original_shape=(M, K), mode=mode), 2 * out)
        del mp, md
    torch.cuda.empty_cache()


def test_gemv_rejects_bad_shapes(dev):
    import feather_amd as feather
    w = torch.zeros(12, dtype=torch.int32, device=dev)
    with pytest.raises(ValueError):
        feather.gemv(w, w, original_shape=(4, 6))
    with pytest.raises(ValueError):
        feather.gemv(w, w, original_shape=(4, 16))            # m holds 12 words, needs 16
    assert feather.gemv(w[:0], w[:4], original_shape=(0, 16)).shape == (0,)


@pytest.mark.parametrize("mode", ["E4M3", "E5M2"])
@pytest.mark.parametrize("M,K,nvec", [(2048, 2048, 32), (256, 5632, 32), (50, 512, 5), (33, 1024, 64), (16, 100, 3), (130, 768, 17),
                                      (6, 256, 1), (4100, 2048, 48), (130, 4096, 17), (70, 1536, 9),
                                      # K walks of >= 32 chunks start at a rotated chunk per row tile (one and two K groups)
                                      (200, 8192, 32), (70, 8448, 5), (130, 16384, 17), (1100, 8192, 64)])
def test_gemv_batched_vs_oracle(dev, orc, mode, M, K, nvec):
    from feather_amd.routines.gemv import gemv_fp8_batched_acc_fp32_gpu
    rng = np.random.default_rng(M + K + nvec)
    w = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float16)
    x = rng.standard_normal((nvec, K)).astype(np.float16)
    wp, xp = orc.pack_fp8(w, mode), orc.pack_fp8(x, mode)
    out = gemv_fp8_batched_acc_fp32_gpu(_dev_words(wp, dev), _dev_words(xp, dev), (M, K), nvec, mode).cpu().numpy()
    want = orc.decode_np(xp, mode).reshape(nvec, K) @ orc.decode_np(wp, mode).reshape(M, K).T
    assert out.shape == (nvec, M) and _nerr(out, want) <= TOL
    if M * K * nvec <= 1 << 22:
        assert _nerr(out, orc.gemv_batched(wp, xp, M, K, nvec, mode)) <= TOL


@pytest.mark.parametrize("M,K", [(32000, 2048), (11264, 2048), (2048, 5632), (2560, 2048)])
def test_gemv_batched_decode_shapes_vs_fp64_math(dev, orc, M, K):
    """The weight shapes of the TinyLlama-shaped decode step at batch 32, E4M3: against a float64 matmul of the
    operands, whose packed words are copied to the host and decoded there by the oracle's table (the scalar
    oracle's own loop is too slow at these sizes)."""
    import feather_amd as feather
    from feather_amd.routines.gemv import gemv_fp8_batched_acc_fp32_gpu
    g = torch.Generator(device=dev).manual_seed(M + K)
    w16 = (torch.randn(M, K, generator=g, device=dev) / K ** 0.5).half()
    x16 = torch.randn(32, K, generator=g, device=dev).half()
    wp, xp = feather.pack_fp8_tensor(w16, mode="E4M3"), feather.pack_fp8_tensor(x16, mode="E4M3")
    out = gemv_fp8_batched_acc_fp32_gpu(wp, xp, (M, K), 32, "E4M3")
    wd = orc.decode_np(wp.view(torch.int32).cpu().numpy().view(np.uint32).reshape(-1), "E4M3").reshape(M, K)
    xd = orc.decode_np(xp.view(torch.int32).cpu().numpy().view(np.uint32).reshape(-1), "E4M3").reshape(32, K)
    want = xd @ wd.T
    assert out.shape == (32, M)
    assert np.abs(out.cpu().numpy().astype(np.float64) - want).max() / np.abs(want).max() <= TOL


@pytest.mark.parametrize("seed", range(10))
def test_gemv_batched_random_shapes(dev, orc, seed):
    """Seeded random (mode, M, K, nvec) draws against a float64 matmul of the decoded operands on
    the device: the launcher switches between one and two K groups per workgroup and the
    per-vector path on K, M and the vector count; codes are raw random bytes (every code occurs,
    NaN / inf codes of E5M2 masked out)."""
    import feather_amd as feather
    from feather_amd.routines.gemv import gemv_fp8_batched_acc_fp32_gpu
    rng = np.random.default_rng(500 + seed)
    mode = ("E4M3", "E5M2")[seed % 2]
    M = int(rng.integers(1, 700))
    K = int(rng.choice([4, 100, 256, 512, 768, 1024, 1280, 2048, 4096, 5632]))
    nvec = int(rng.integers(1, 65))
    def codes(n):
        b = rng.integers(0, 256, size=n, dtype=np.uint8)
        if mode == "E5M2":
            b = np.where((b & 0x7C) == 0x7C, b & 0x83, b).astype(np.uint8)   # no inf / NaN codes
        return torch.from_numpy(b.view(np.int32).copy()).to(dev).view(torch.uint32)
    wp, xp = codes(M * K), codes(nvec * K)
    out = gemv_fp8_batched_acc_fp32_gpu(wp, xp, (M, K), nvec, mode)
    wd, xd = _host_decode(wp, mode, orc).view(M, K), _host_decode(xp, mode, orc).view(nvec, K)
    want = xd @ wd.T
    scale = (xd.abs() @ wd.abs().T).max()               # cancellation-free error scale of the fp32 sums
    assert out.shape == (nvec, M)
    assert ((out.double().cpu() - want).abs().max() / scale).item() <= 1e-5


@pytest.mark.parametrize("seed", range(14))
def test_gemv_random_shapes(dev, orc, seed):
    """Seeded random (mode, M, K) draws for the single-vector GEMV against a float64 matvec of the
    decoded operands on the device: rows shorter and longer than four 1 KiB steps, ragged last steps,
    rows longer than one 32768-code vector chunk, row counts that are not a multiple of a workgroup's
    eight rows, rows that are not 16-byte aligned (generic path); raw random codes."""
    import feather_amd as feather
    rng = np.random.default_rng(900 + seed)
    mode = ("E4M3", "E5M2")[seed % 2]
    M = int(rng.integers(1, 300))
    K = int(rng.choice([16, 1024, 2064, 4096, 4112, 5008, 8192, 12304, 32768, 33808, 40000, 65536 + 48, 4 * 77, 4 * 1031]))
    def codes(n):
        b = rng.integers(0, 256, size=n, dtype=np.uint8)
        if mode == "E5M2":
            b = np.where((b & 0x7C) == 0x7C, b & 0x83, b).astype(np.uint8)   # no inf / NaN codes
        return torch.from_numpy(b.view(np.int32).copy()).to(dev).view(torch.uint32)
    wp, xp = codes(M * K), codes(K)
    print(f"seed {seed}: {mode} M {M} K {K}", flush=True)
    out = feather.gemv(wp, xp, original_shape=(M, K), mode=mode)
    wd, xd = _host_decode(wp, mode, orc).view(M, K), _host_decode(xp, mode, orc).view(K)
    want = wd @ xd
    scale = (wd.abs() @ xd.abs()).max()                 # cancellation-free error scale of the fp32 sums
    assert out.shape == (M,)
    assert ((out.double().cpu() - want).abs().max() / scale).item() <= 1e-5


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_gemv_vector_and_matrix_at_word_offsets(dev, mode):
    """Operands that are only 4-byte aligned (views one word into a buffer): the vector then takes the
    word-wise staging path, the matrix the generic kernel; results equal the aligned call bit for bit
    for the vector case (same summation order) and to fp32 rounding for the matrix case."""
    import feather_amd as feather
    g = torch.Generator(device=dev).manual_seed(7)
    M, K = 40, 16384
    w = feather.pack_fp8_tensor(torch.randn(M, K, generator=g, device=dev).half(), mode=mode)
    x = feather.pack_fp8_tensor(torch.randn(K, generator=g, device=dev).half(), mode=mode)
    want = feather.gemv(w, x, original_shape=(M, K), mode=mode)
    xbuf = torch.zeros(x.numel() + 1, dtype=x.dtype, device=dev)
    xbuf[1:].copy_(x)
    assert xbuf[1:].data_ptr() % 16 == 4
    assert torch.equal(feather.gemv(w, xbuf[1:], original_shape=(M, K), mode=mode), want)
    wbuf = torch.zeros(w.numel() + 1, dtype=w.dtype, device=dev)
    wbuf[1:].copy_(w)
    got = feather.gemv(wbuf[1:], x, original_shape=(M, K), mode=mode)
    assert ((got - want).abs().max() / want.abs().max()).item() <= 1e-5


# ---------------------------------------------------------------- dot

def test_dot_docstring_known_answers(dev, kats):
    import feather_amd as feather
    from feather_amd.packers import fp16
    from feather_amd.routines import dot
    k = kats["dot_fp8_e5m2"]
    x1, x2 = (torch.tensor(k[n], dtype=torch.float16, device=dev) for n in ("x1", "x2"))
    out = dot.dot_fp8_e5m2_acc_fp32_gpu(feather.pack_fp8_tensor(x1), feather.pack_fp8_tensor(x2))
    assert out.shape == () and out.dtype == torch.float32 and out.item() == k["expected"]
    assert feather.dot(feather.pack_fp8_tensor(x1, mode="E4M3"), feather.pack_fp8_tensor(x2, mode="E4M3"),
                       mode="E4M3").item() == k["expected"]
    k = kats["dot_fp16"]
    a, b = (np.array(k[n], dtype=np.float16) for n in ("x1", "x2"))
    assert dot.dot_fp16_acc_fp32_vec(fp16.pack_fp16_ndarray(a), fp16.pack_fp16_ndarray(b)) == k["expected"]
    assert dot.dot_fp16_acc_fp32_numba(fp16.pack_fp16_ndarray(a), fp16.pack_fp16_ndarray(b), None) == k["expected"]
    ta = torch.from_numpy(fp16.pack_fp16_ndarray(a)).view(torch.uint32).to(dev)
    tb = torch.from_numpy(fp16.pack_fp16_ndarray(b)).view(torch.uint32).to(dev)
    assert dot.dot_fp16_acc_fp32_gpu(ta, tb).item() == k["expected"]


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("n", [4, 10_000, 500_000, 1_500_000, 16384, (1 << 22) + 12])
def test_dot_fp8_vs_oracle(dev, orc, mode, n):
    """Sizes of the reference harness (bench_dot.py:15) plus ragged ones."""
    import feather_amd as feather
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    a[rng.random(n) < 0.01] *= 1e-3
    x1, x2 = orc.pack_fp8(a.astype(np.float16), mode), orc.pack_fp8(b.astype(np.float16), mode)
    got = feather.dot(_dev_words(x1, dev), _dev_words(x2, dev), mode=mode).item()
    want = float(orc.decode_np(x1, mode) @ orc.decode_np(x2, mode))
    norm = float(np.abs(orc.decode_np(x1, mode) * orc.decode_np(x2, mode)).sum())
    assert abs(got - want) <= TOL * max(abs(want), 1e-3 * norm)
    assert abs(got - orc.dot_fp8(x1, x2, mode, acc64=True)) <= 1e-5 * norm
    again = feather.dot(_dev_words(x1, dev), _dev_words(x2, dev), mode=mode).item()
    assert again == got                                        # deterministic reduction order


@pytest.mark.parametrize("mode", ["E4M3", "E5M2"])
def test_dot_config_size_2_pow_24_vs_oracle(dev, orc, mode):
    """n = 2^24 with 1 % of the entries scaled by 1e-3 (E4M3 subnormal codes): the launch of 1024
    workgroups plus the ordered finish over 1024 partials, against the C oracle's O(n) loop with a
    float64 accumulator (reference semantics: dot.py:145-192 decode and products, summation order
    free) and against the LUT decode + float64 BLAS reduction."""
    import feather_amd as feather
    n = 1 << 24
    rng = np.random.default_rng(24)
    a = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    a[rng.random(n) < 0.01] *= 1e-3
    b[rng.random(n) < 0.01] *= 1e-3
    x1, x2 = orc.pack_fp8(a.astype(np.float16), mode), orc.pack_fp8(b.astype(np.float16), mode)
    d1, d2 = orc.decode_np(x1, mode), orc.decode_np(x2, mode)
    norm = float(np.abs(d1 * d2).sum())
    want = float(orc.dot_fp8(x1, x2, mode, acc64=True))
    assert abs(want - float(d1 @ d2)) <= 1e-9 * norm              # the two oracles agree
    t1, t2 = _dev_words(x1, dev), _dev_words(x2, dev)
    got = feather.dot(t1, t2, mode=mode).item()
    assert abs(got - want) <= 1e-6 * norm                         # fp32 partial sums of 16384 terms each
    assert abs(got - want) <= TOL * max(abs(want), 1e-3 * norm)
    assert feather.dot(t1, t2, mode=mode).item() == got           # deterministic


def test_gemv_config_size_8192_vs_oracle(dev, orc):
    """BASELINE config 1 at its own size: E5M2, 8192 x 8192 N(0,1) from seed 1.  The scalar oracle
    checks a sample of rows (every 64th plus the last); all rows are checked against a float64 matvec
    of the operands decoded by the HIP unpack kernel, which the pack tests of the same run hold
    bit-exact to the oracle's decode on all 256 codes."""
    import feather_amd as feather
    g = torch.Generator().manual_seed(1)
    M = K = 8192
    m = torch.randn(M, K, generator=g).half()
    v = torch.randn(K, generator=g).half()
    mp = feather.pack_fp8_tensor(m.to(dev), mode="E5M2")
    vp = feather.pack_fp8_tensor(v.to(dev), mode="E5M2")
    out = feather.gemv(mp, vp, original_shape=(M, K), mode="E5M2")
    rows = np.r_[0:M:64, M - 1]
    mw = mp.view(torch.int32).cpu().numpy().view(np.uint32).reshape(M, K // 4)
    assert np.array_equal(mw[rows], orc.pack_fp8(m.numpy()[rows], "E5M2").reshape(len(rows), K // 4))   # packing bit-exact
    vw = vp.view(torch.int32).cpu().numpy().view(np.uint32)
    want = orc.gemv(np.ascontiguousarray(mw[rows]).reshape(-1), vw, len(rows), K, "E5M2", acc64=True)
    full = torch.mv(_host_decode(mp, "E5M2", orc).view(M, K), _host_decode(vp, "E5M2", orc)[:K])   # every row, float64 on the host
    scale = full.abs().max().item()
    assert np.abs(out.cpu().numpy()[rows] - want).max() / scale <= 1e-5
    assert ((out.double().cpu() - full).abs().max() / scale).item() <= 1e-5


@pytest.mark.parametrize("n", [2, 1001, 1 << 20])
def test_dot_fp16_vs_oracle(dev, orc, n):
    from feather_amd.routines import dot
    rng = np.random.default_rng(n)
    a = (rng.standard_normal(n) * 2).astype(np.float16)
    b = (rng.standard_normal(n) * 2).astype(np.float16)
    x1, x2 = orc.pack_fp16(a), orc.pack_fp16(b)
    norm = float(np.abs(a.astype(np.float64) * b.astype(np.float64)).sum())
    got = dot.dot_fp16_acc_fp32_gpu(_dev_words(x1, dev), _dev_words(x2, dev)).item()
    assert abs(got - float(orc.dot_fp16(x1, x2, acc64=True))) <= 1e-5 * norm     # same fp16 roundings, fp32 sums
    wide = float(dot.dot_fp16_acc_fp32_vec(x1.view(np.float32), x2.view(np.float32)))
    assert abs(wide - float(a.astype(np.float64) @ b.astype(np.float64))) <= 1e-5 * norm


def test_dot_empty_and_mismatch(dev):
    import feather_amd as feather
    z = torch.zeros(0, dtype=torch.int32, device=dev)
    assert feather.dot(z, z).item() == 0.0
    with pytest.raises(ValueError):
        feather.dot(torch.zeros(4, dtype=torch.int32, device=dev), torch.zeros(8, dtype=torch.int32, device=dev))
