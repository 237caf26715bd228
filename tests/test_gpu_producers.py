"""GPU parity of the producers that emit packed FP8 operands (quantise + pack fused into the kernel
that computes the values), through the C ABI.

Integer work is held to exact equality: the packed words a producer writes must equal
``oracle.decode_ref.quant_codes`` (fp32 -> fp16 -> FP8, round to nearest even twice, i.e. the
oracle's ``pack_fp8`` of ``x.astype(float16)``) of the SAME fp32 values, which every fused producer
can also write out.  Those fp32 values are compared with the oracle's float arithmetic to a stated
floating-point tolerance."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _np_words(t):
    return t.view(torch.int32).cpu().numpy().view(np.uint32)


def _hard_fp32_values():
    """fp32 values on which a wrong rounding chain shows: E4M3 overflow edge (464 ties to 448, anything
    above goes to 0x7F), the subnormal tie 2^-10, +-inf, +-0, fp16 overflow (65504 / 65520), values that
    round differently when rounded to FP8 directly instead of through fp16 (just above an FP8 tie but
    rounded onto it by the fp16 step), fp16 subnormals, and every fp16 pattern nudged by +-1 fp32 ulp."""
    v = [0.0, -0.0, np.inf, -np.inf, 464.0, 465.0, 464.0001, 463.9999, 448.0, 472.0, 480.0, -464.0, -465.0,
         2.0 ** -10, -(2.0 ** -10), 2.0 ** -10 * 1.0001, 2.0 ** -10 * 0.9999, 3 * 2.0 ** -10, 2.0 ** -9, 2.0 ** -6,
         65504.0, 65519.9, 65520.0, 1e9, -1e9, 61440.0, 61439.9, 57344.0, 1e-8, -1e-8, 6e-8, 2.0 ** -24, 2.0 ** -25]
    # double rounding: 1 + 2^-4 is the E4M3 tie between 1.0 and 1.125 (ties to even: 1.0); 1 + 2^-4 + 2^-12 is
    # above the tie (direct rounding: 1.125) but the fp16 step (ulp 2^-10) rounds it onto the tie first -> 1.0
    for base, e in ((1.0, 0), (2.0, 1), (0.25, -2), (96.0, 6)):
        for m in (1, 3, 5, 7):                                   # E4M3 ties m/16, E5M2 ties at m/8
            for frac in (2.0 ** -12, -(2.0 ** -12), 2.0 ** -13, 2.0 ** -11 + 2.0 ** -20):
                v.append((1 + m / 16 + frac) * 2.0 ** e)
                v.append(-(1 + m / 8 + frac) * 2.0 ** e)
    v = np.array(v, dtype=np.float32)
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h)]
    up = np.nextafter(h, np.float32(np.inf)).astype(np.float32)
    dn = np.nextafter(h, np.float32(-np.inf)).astype(np.float32)
    mid = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)   # exact fp16 ties
    return np.concatenate([v, h, up, dn, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])


@pytest.mark.parametrize("mode", ["E4M3", "E5M2"])
def test_quant_pack_f32_bit_exact(dev, orc, mode):
    from feather_amd.routines.producers import quant_pack_f32
    from oracle import decode_ref
    rng = np.random.default_rng(1)
    x = np.concatenate([_hard_fp32_values(), rng.standard_normal(100_003).astype(np.float32),
                        (rng.standard_normal(50_000) * 1e-3).astype(np.float32),
                        (rng.standard_normal(50_000) * 300).astype(np.float32)])
    want = decode_ref.quant_codes(x, mode)
    got = _np_words(quant_pack_f32(torch.from_numpy(x).to(dev), mode))
    assert got.shape == want.shape and np.array_equal(got, want)
    # and it is pack_fp8_tensor of the fp16-rounded input (the reference packer's contract, fp8.py:260-281)
    import feather_amd as feather
    ref = _np_words(feather.pack_fp8_tensor(torch.from_numpy(x).to(dev).half(), mode=mode))
    assert np.array_equal(got, ref)
    for n in (0, 1, 3, 4, 5, 17, 63, 64, 65):                    # ragged sizes, zero padding of the last word
        g = _np_words(quant_pack_f32(torch.from_numpy(x[:n].copy()).to(dev), mode))
        assert np.array_equal(g, decode_ref.quant_codes(x[:n], mode))
    base = torch.from_numpy(x[:4099].copy()).to(dev)             # a source that is not 16-byte aligned
    assert np.array_equal(_np_words(quant_pack_f32(base[3:], mode)), decode_ref.quant_codes(x[3:4099], mode))


@pytest.mark.parametrize("mode,batch,hidden,n_part", [("E4M3", 32, 2048, 8), ("E5M2", 3, 256, 1), ("E4M3", 5, 320, 3),
                                                      ("E4M3", 2, 5632, 11), ("E5M2", 4, 20480, 2), ("E4M3", 7, 1024, 0)])
def test_add_rmsnorm_pack_bit_exact_codes(dev, orc, mode, batch, hidden, n_part):
    """Residual add of K-slice partials + RMSNorm + quantise + pack.  Codes: exactly quant_codes of the
    kernel's own fp32 result.  That result: the oracle's rmsnorm within 2e-6 relative (fp32 arithmetic,
    other summation order).  Residual stream: h + partials added in slice order, exact."""
    from feather_amd.routines.producers import add_rmsnorm_pack
    from oracle import decode_ref
    rng = np.random.default_rng(hidden + n_part)
    h = rng.standard_normal((batch, hidden)).astype(np.float32)
    h[0, :8] = [0.0, -0.0, 1e-6, 300.0, -300.0, 2.0 ** -10, 17.0, -1e-3]
    gain = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    delta = (0.3 * rng.standard_normal((n_part, batch, hidden))).astype(np.float32) if n_part else None
    ht = torch.from_numpy(h).to(dev)
    xq, y = add_rmsnorm_pack(ht, torch.from_numpy(gain).to(dev), torch.from_numpy(delta).to(dev) if n_part else None,
                             eps=1e-5, mode=mode, return_f32=True)
    h_new = h.copy()
    if n_part:
        d = delta[0].copy()
        for s in range(1, n_part):
            d = d + delta[s]
        h_new = h + d
    assert np.array_equal(ht.cpu().numpy(), h_new)
    y = y.cpu().numpy()
    assert np.array_equal(_np_words(xq).reshape(-1), decode_ref.quant_codes(y, mode))
    want = decode_ref.rmsnorm(h_new, gain, 1e-5)
    assert np.abs(y - want).max() <= 2e-6 * np.abs(want).max()
    # without the fp32 output the same words come out
    xq2 = add_rmsnorm_pack(torch.from_numpy(h_new).to(dev), torch.from_numpy(gain).to(dev), None, eps=1e-5, mode=mode)
    assert np.array_equal(_np_words(xq2), _np_words(xq))


@pytest.mark.parametrize("mode,inter,K,nvec", [("E4M3", 5632, 2048, 32),      # the TinyLlama gate/up shape at batch 32
                                               ("E5M2", 96, 256, 3), ("E4M3", 1000, 1024, 17), ("E4M3", 36, 512, 64)])
def test_gemv_swiglu_epilogue_bit_exact_codes(dev, orc, mode, inter, K, nvec):
    """The gate/up GEMV with the SwiGLU activation and the FP8 packing in its epilogue.  Codes: exactly
    quant_codes of the kernel's own fp32 activation.  Activation: silu(g) * u of the float64 GEMV of the
    decoded operands within 1e-3 of the output scale (fp32 sums; hardware exp2 / reciprocal in silu)."""
    import feather_amd as feather
    from feather_amd.routines.producers import gemv_fp8_batched_swiglu
    from oracle import decode_ref
    g = torch.Generator(device=dev).manual_seed(inter)
    w = (torch.randn(2 * inter, K, generator=g, device=dev) / K ** 0.5).half()
    x = torch.randn(nvec, K, generator=g, device=dev).half()
    wp, xp = feather.pack_fp8_tensor(w, mode=mode), feather.pack_fp8_tensor(x, mode=mode)
    act, f = gemv_fp8_batched_swiglu(wp, xp, inter, K, nvec, mode=mode, return_f32=True)
    f = f.cpu().numpy()
    assert np.array_equal(_np_words(act).reshape(-1), decode_ref.quant_codes(f, mode))
    wd = torch.from_numpy(orc.decode_np(_np_words(wp).reshape(-1), mode)).view(2 * inter, K)      # decoded on the host
    xd = torch.from_numpy(orc.decode_np(_np_words(xp).reshape(-1), mode)).view(nvec, K)
    gu = xd @ wd.T
    want = (torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]).numpy()
    assert np.abs(f - want).max() <= 1e-3 * np.abs(want).max()
    if (inter, K) == (96, 256):                                 # a shape the scalar oracle covers: its own GEMV, too
        gu_o = orc.gemv(_np_words(wp), _np_words(xp)[: K // 4], 2 * inter, K, mode, acc64=True)
        w0 = gu_o[:inter] / (1 + np.exp(-gu_o[:inter])) * gu_o[inter:]
        assert np.abs(f[0] - w0).max() <= 1e-3 * np.abs(w0).max()
    act2 = gemv_fp8_batched_swiglu(wp, xp, inter, K, nvec, mode=mode)
    assert np.array_equal(_np_words(act2), _np_words(act))


@pytest.mark.parametrize("mode,nq,nkv,d,bs,n_part", [("E4M3", 32, 4, 64, 16, 7), ("E5M2", 4, 2, 128, 8, 1),
                                                      ("E4M3", 5, 1, 64, 4, 3)])
def test_rope_append_bit_exact_codes_and_placement(dev, orc, mode, nq, nkv, d, bs, n_part):
    """Rotary embedding + pack of q + encode-and-append of k / v.  Codes (q words, appended cache rows):
    exactly quant_codes of the kernel's own rotated fp32 values.  Rotated values: the oracle's rope
    within 2e-5 of the row scale.  Placement: exactly the slots the block table names, every other
    cache word untouched.  Sequences without a valid slot are reported and not written."""
    from feather_amd.routines.producers import rope_append
    from oracle import decode_ref
    rng = np.random.default_rng(nq + d)
    B, max_blocks = 6, 5
    n_blocks = B * max_blocks + 2
    heads, cap = nq + 2 * nkv, max_blocks * bs
    parts = rng.standard_normal((n_part, B, heads * d)).astype(np.float32)
    ctx = np.array([0, 3, bs, cap - 1, cap, -2], dtype=np.int32)          # last two: full table, negative length
    bt = rng.permutation(n_blocks)[: B * max_blocks].reshape(B, max_blocks).astype(np.int32)
    bt[1, ctx[1] // bs] = n_blocks + 5                                      # a table entry outside the cache
    kc0 = rng.integers(0, 2 ** 32, (n_blocks, nkv, bs, d // 4), dtype=np.uint64).astype(np.uint32)
    vc0 = rng.integers(0, 2 ** 32, (n_blocks, nkv, bs, d // 4), dtype=np.uint64).astype(np.uint32)
    to_dev = lambda a: torch.from_numpy(a.view(np.int32).copy()).to(dev)
    kc, vc = to_dev(kc0), to_dev(vc0)
    qp, ctx_after, status, rot = rope_append(torch.from_numpy(parts).to(dev), torch.from_numpy(ctx).to(dev),
                                             torch.from_numpy(bt).to(dev), kc, vc, n_q_heads=nq, rope_theta=10000.0,
                                             mode=mode, return_f32=True)
    rot, qp = rot.cpu().numpy(), _np_words(qp)
    assert status.cpu().tolist() == [0, 2, 0, 0, 1, 1]
    assert ctx_after.cpu().tolist() == [1, 3, bs + 1, cap, cap, 0]
    qkv = parts[0].copy()
    for s in range(1, n_part):
        qkv = qkv + parts[s]
    qkv = qkv.reshape(B, heads, d)
    kc_want, vc_want = kc0.copy(), vc0.copy()
    for b in range(B):
        pos = int(ctx[b]) if 0 <= ctx[b] < cap else 0
        want = np.concatenate([decode_ref.rope(qkv[b, : nq + nkv], pos, 10000.0), qkv[b, nq + nkv:]])
        if status[b].item() != 1:                                           # a bad position has no defined angle
            assert np.abs(rot[b] - want).max() <= 2e-5 * np.abs(want).max()
            assert np.array_equal(rot[b, nq + nkv:], qkv[b, nq + nkv:])      # v is not rotated
        assert np.array_equal(qp[b].reshape(-1), decode_ref.quant_codes(rot[b, :nq], mode))
        if status[b].item() == 0:
            blk, slot = bt[b, ctx[b] // bs], ctx[b] % bs
            kc_want[blk, :, slot] = decode_ref.quant_codes(rot[b, nq:nq + nkv], mode).reshape(nkv, d // 4)
            vc_want[blk, :, slot] = decode_ref.quant_codes(rot[b, nq + nkv:], mode).reshape(nkv, d // 4)
    assert np.array_equal(_np_words(kc), kc_want) and np.array_equal(_np_words(vc), vc_want)


def test_paged_attention_packed_output_bit_exact(dev, orc):
    """The attention epilogue that emits the packed operand of the output projection: exactly
    quant_codes of the fp32 result the same call returns, with and without the split merge."""
    import feather_amd as feather
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
    from oracle import decode_ref
    g = torch.Generator().manual_seed(9)
    for mode, max_ctx in (("E4M3", 300), ("E4M3", 1500), ("E5M2", 700)):
        n_seq, Hq, Hkv, d, bs = 5, 8, 2, 64, 16
        max_blocks = (max_ctx + bs - 1) // bs
        n_blocks = n_seq * max_blocks
        ctx = torch.randint(1, max_ctx + 1, (n_seq,), generator=g, dtype=torch.int32)
        ctx[0], ctx[1] = max_ctx, 0
        bt = torch.randperm(n_blocks, generator=g).to(torch.int32).view(n_seq, max_blocks)
        pk = lambda *s: feather.pack_fp8_tensor(torch.randn(*s, generator=g).half().to(dev), mode=mode)
        out, packed = paged_attention_fp8_acc_fp32_gpu(pk(n_seq, Hq, d).view(n_seq, Hq, d // 4),
                                                       pk(n_blocks, Hkv, bs, d).view(n_blocks, Hkv, bs, d // 4),
                                                       pk(n_blocks, Hkv, bs, d).view(n_blocks, Hkv, bs, d // 4),
                                                       bt.to(dev), ctx.to(dev), mode=mode, max_context_len=max_ctx,
                                                       return_packed=True)
        assert np.array_equal(_np_words(packed).reshape(-1), decode_ref.quant_codes(out.cpu().numpy(), mode))
        assert not out[1].any() and not packed[1].view(torch.int32).any()
