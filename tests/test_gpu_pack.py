"""GPU parity: pack / unpack kernels against the CPU oracle and the golden tables (bit-exact)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    return torch.device("cuda:0")


def _words(t):
    return t.view(torch.int32).cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_pack_all_fp16_patterns_bit_exact(dev, orc, tables, mode):
    import feather_amd as feather
    h = np.arange(65536, dtype=np.uint16)
    x = torch.from_numpy(h.view(np.float16).copy()).to(dev)
    got = _words(feather.pack_fp8_tensor(x, mode=mode)).view(np.uint8)
    assert np.array_equal(got, tables["enc_e5m2" if mode == "E5M2" else "enc_e4m3"])
    assert np.array_equal(got, orc.enc_table(mode))


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 15, 16, 17, 63, 1000, 4099, 1 << 20])
def test_pack_sizes_tails_and_padding(dev, orc, mode, n):
    import feather_amd as feather
    rng = np.random.default_rng(n + 1)
    x = (rng.standard_normal(n) * rng.choice([1e-3, 1.0, 100.0], size=n)).astype(np.float16)
    got = feather.pack_fp8_tensor(torch.from_numpy(x).to(dev), mode=mode)
    assert got.dtype == torch.uint32 and got.is_cuda and got.shape == ((n + 3) // 4,)
    assert np.array_equal(_words(got), orc.pack_fp8(x, mode))


def test_pack_unaligned_view_and_2d_and_cpu_input(dev, orc):
    import feather_amd as feather
    rng = np.random.default_rng(3)
    x = rng.standard_normal((33, 70)).astype(np.float16)
    t = torch.from_numpy(x).to(dev)
    assert np.array_equal(_words(feather.pack_fp8_tensor(t, mode="E4M3")), orc.pack_fp8(x, "E4M3"))
    flat = t.reshape(-1)[1:]                                   # 2-byte aligned only
    assert np.array_equal(_words(feather.pack_fp8_tensor(flat, mode="E5M2")), orc.pack_fp8(x.reshape(-1)[1:], "E5M2"))
    cpu = feather.pack_fp8_tensor(torch.from_numpy(x), mode="E5M2")   # host tensor in -> host tensor out
    assert not cpu.is_cuda and np.array_equal(cpu.view(torch.int32).numpy().view(np.uint32), orc.pack_fp8(x, "E5M2"))


def test_legacy_truncating_pack(dev, orc):
    from feather_amd.packers import fp8
    h = np.arange(65536, dtype=np.uint16)
    x = torch.from_numpy(h.view(np.float16).copy()).to(dev)
    got = fp8.pack_fp8_tensor_legacy(x)
    assert got.dtype == torch.float32
    assert np.array_equal(got.view(torch.int32).cpu().numpy().view(np.uint8), (h >> 8).astype(np.uint8))
    with pytest.raises(NotImplementedError):
        fp8.pack_fp8_tensor_legacy(x, mode="E4M3")


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("semantics", ["ieee", "kernel"])
def test_unpack_all_codes(dev, orc, mode, semantics):
    import feather_amd as feather
    w = torch.from_numpy(np.arange(256, dtype=np.uint8).view(np.int32).copy()).to(dev)
    sem = orc.SEM_IEEE if semantics == "ieee" else orc.SEM_KERNEL
    want = orc.dec_table(mode, sem)
    for dt in (torch.float32, torch.float16):
        got = feather.unpack_fp8_tensor(w, mode=mode, semantics=semantics, dtype=dt).float().cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))   # bit-exact, signed zeros too


def test_numpy_api_matches_reference_shapes(dev, orc):
    from feather_amd.packers import fp8, fp16
    rng = np.random.default_rng(4)
    x = rng.standard_normal(10).astype(np.float16)
    p = fp8.pack_fp8_ndarray(x, mode="E4M3")
    assert p.dtype == np.float32 and p.shape == (3,)
    assert np.array_equal(p.view(np.uint32), orc.pack_fp8(x, "E4M3"))
    u = fp8.unpack_into_fp8_ndarray(p, mode="E4M3")
    assert u.dtype == np.float16 and u.shape == (12,)
    assert np.array_equal(u.astype(np.float32), orc.unpack_fp8(p, "E4M3", orc.SEM_IEEE))
    one = fp8.pack_fp8_into_fp32(x[0], x[1], x[2], x[3], mode="E5M2")
    assert np.float32(one).view(np.uint32) == orc.pack_fp8(x[:4], "E5M2")[0]
    cols = fp8.pack_fp8_into_fp32(x[0:2], x[2:4], x[4:6], x[6:8], mode="E5M2")
    inter = np.stack([x[0:2], x[2:4], x[4:6], x[6:8]], axis=-1).reshape(-1)
    assert np.array_equal(cols.view(np.uint32), orc.pack_fp8(inter, "E5M2"))
    four = fp8.unpack_fp8_from_fp32(p[0], mode="E4M3")
    assert four.shape == (4, 1) and np.array_equal(four[:, 0], orc.unpack_fp8(p[:1], "E4M3", orc.SEM_IEEE))
    leg = fp8.unpack_fp8_from_fp32_legacy(fp8.pack_fp8_into_fp32_legacy(x[0], x[1], x[2], x[3]))
    assert np.array_equal(leg, (x[:4].view(np.uint16) & 0xFF00).view(np.float16).astype(np.float32))
    with pytest.raises(NotImplementedError):
        fp8.pack_fp8_ndarray(x, mode="E1M6")
    # fp16 container
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    w = fp16.pack_fp16_ndarray(h[:1001])
    assert w.dtype == np.float32 and np.array_equal(w.view(np.uint32), orc.pack_fp16(h[:1001]))
    back = fp16.unpack_into_fp16_ndarray(w)
    assert np.array_equal(back.view(np.uint16)[:1001], h[:1001].view(np.uint16)) and back[1001] == 0
    full = fp16.unpack_fp16_tensor(fp16.pack_fp16_tensor(torch.from_numpy(h.copy()).to(dev)))
    assert np.array_equal(full.cpu().numpy().view(np.uint16), h.view(np.uint16))        # NaN payloads survive
    pair = fp16.pack_fp16_into_fp32(h[15360], h[49152])
    assert np.float32(pair).view(np.uint32) == (49152 << 16 | 15360)
    assert np.array_equal(fp16.unpack_fp32_into_fp16(pair).view(np.uint16), [15360, 49152])


def test_relu(dev, orc):
    from feather_amd.routines.activations import relu1d_fp8_ret_fp32_feather_gpu
    import feather_amd as feather
    rng = np.random.default_rng(5)
    x = rng.integers(-4, 5, size=10_001).astype(np.float16)      # bench_activations.py:28
    p = feather.pack_fp8_tensor(torch.from_numpy(x).to(dev), mode="E5M2")
    got = relu1d_fp8_ret_fp32_feather_gpu(p, x.size).cpu().numpy()
    assert np.array_equal(got, orc.relu_fp8_e5m2(orc.pack_fp8(x))[: x.size])
    assert np.array_equal(got, np.maximum(x.astype(np.float32), 0))


def test_pack_full_size_roundtrip_property(dev):
    """Config-sized input (16384 x 16384): encode -> decode -> encode is idempotent and the
    word count / padding are right; checked on device without the oracle."""
    import feather_amd as feather
    g = torch.Generator(device="cpu").manual_seed(2)
    x = torch.randn(4096, 16384, generator=g).half().to(dev)
    for mode in ("E5M2", "E4M3"):
        p = feather.pack_fp8_tensor(x, mode=mode)
        assert p.numel() == x.numel() // 4
        y = feather.unpack_fp8_tensor(p, mode=mode, semantics="ieee", dtype=torch.float16)
        p2 = feather.pack_fp8_tensor(y, mode=mode)
        assert torch.equal(p.view(torch.int32), p2.view(torch.int32))
        err = (y.float() - x.reshape(-1).float()).abs().max().item()
        assert err <= (0.5 if mode == "E5M2" else 0.26)          # half an ulp at |x| < 8


@pytest.mark.gpu
def test_saved_packed_matrix_feeds_gemv_unchanged(dev, tmp_path):
    import feather_amd as feather
    from feather_amd.packers.serial import PackedTensor, load_packed, save_packed
    g = torch.Generator(device=dev).manual_seed(11)
    m = torch.randn(96, 256, generator=g, device=dev).half()
    v = torch.randn(256, generator=g, device=dev).half()
    mp, vp = feather.pack_fp8_tensor(m, mode="E4M3"), feather.pack_fp8_tensor(v, mode="E4M3")
    save_packed(tmp_path / "m.fthr", PackedTensor(mp, m.shape, "E4M3"))
    back = load_packed(tmp_path / "m.fthr", device=dev)
    assert back.shape == (96, 256) and back.words.device == mp.device
    assert torch.equal(back.words.view(torch.int32), mp.view(torch.int32))
    assert torch.equal(feather.gemv(back.words, vp, original_shape=back.shape, mode=back.mode),
                       feather.gemv(mp, vp, original_shape=m.shape, mode="E4M3"))
