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


@pytest.mark.parametrize("L", [1, 5, 63, 65, 70, 130])
def test_flash_attention_ragged_tails(dev, orc, L):
    from feather_amd.routines.attention import flash_attention_fp8_acc_fp32_gpu
    rng = np.random.default_rng(L)
    d = 64
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


def test_flash_attention_config_sized_property(dev):
    """B4 H16 L4096 d64 E5M2: too big for the scalar oracle; compare with torch SDPA (fp32
    math) of the decoded operands on device and check determinism."""
    import feather_amd as feather
    g = torch.Generator().manual_seed(3)
    B, H, L, d = 4, 16, 4096, 64
    qkv = [torch.randn(B, H, L, d, generator=g).half().to(dev) for _ in range(3)]
    p = [feather.pack_fp8_tensor(t, mode="E5M2").view(B, H, L, d // 4) for t in qkv]
    out = feather.flash_attention_fp8_e5m2_acc_fp32_gpu(p[0], p[1], p[2], L, d // 4)
    assert out.shape == (B, H, L, d)
    dec = [feather.unpack_fp8_tensor(t, mode="E5M2", semantics="kernel").view(B, H, L, d) for t in p]
    with torch.backends.cuda.sdp_kernel(enable_flash=False, enable_mem_efficient=False, enable_math=True):
        want = torch.nn.functional.scaled_dot_product_attention(dec[0][:, :2], dec[1][:, :2], dec[2][:, :2])
    err = (out[:, :2] - want).abs().max() / want.abs().max()
    assert err.item() <= TOL
    again = feather.flash_attention_fp8_e5m2_acc_fp32_gpu(p[0], p[1], p[2], L, d // 4)
    assert torch.equal(out, again)


# ---------------------------------------------------------------- paged decode

@pytest.mark.parametrize("mode,n_seq,Hq,Hkv,d,bs,max_ctx", [
    ("E5M2", 3, 8, 2, 64, 16, 100), ("E4M3", 4, 32, 4, 64, 16, 700), ("E4M3", 2, 4, 4, 128, 16, 300),
    ("E5M2", 2, 16, 1, 64, 8, 90), ("E4M3", 1, 2, 1, 256, 32, 257),
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
