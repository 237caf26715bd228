"""Every kernel gives the same bits from call to call on the same operands.  A race, a missing wait state or an
order of additions that depends on timing shows up here even when every single result is inside its tolerance (that
is how a missing wait state between the score MFMAs and the row maximum of the attention kernels was found).  The
reference adds its dot-product partials with fp32 atomics (feather/routines/dot.py:142, :189) and is not repeatable;
this library is, by construction, and this file holds it to that."""
import pytest
import torch

pytestmark = pytest.mark.gpu

CALLS = 6


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a HIP device")
    return torch.device("cuda:0")


def _pack(gen, dev, mode, *shape):
    import feather_amd as feather
    return feather.pack_fp8_tensor(torch.randn(*shape, generator=gen, device=dev).half(), mode=mode)


def _same(fn):
    first = fn()
    first = [t.clone() for t in first] if isinstance(first, (tuple, list)) else [first.clone()]
    for _ in range(CALLS - 1):
        again = fn()
        again = list(again) if isinstance(again, (tuple, list)) else [again]
        for a, b in zip(first, again):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32))


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("M,K", [(16384, 16384), (8192, 8192), (4096, 4096), (1000, 2052), (37, 8192)])
def test_gemv_repeats(dev, mode, M, K):
    import feather_amd as feather
    g = torch.Generator(device=dev).manual_seed(M + K)
    m, v = _pack(g, dev, mode, M, K), _pack(g, dev, mode, K)
    _same(lambda: feather.gemv(m, v, original_shape=(M, K), mode=mode))


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("M,K,nvec", [(16384, 16384, 32), (2560, 2048, 32), (2048, 5632, 32), (32000, 2048, 32),
                                        (8192, 8192, 64), (4096, 4096, 5)])
def test_gemv_batched_repeats(dev, mode, M, K, nvec):
    """The long walks run two K groups per workgroup that meet through LDS; the result has one order of additions."""
    from feather_amd.routines.gemv import gemv_fp8_batched_acc_fp32_gpu
    g = torch.Generator(device=dev).manual_seed(M + K + nvec)
    w, x = _pack(g, dev, mode, M, K), _pack(g, dev, mode, nvec, K)
    _same(lambda: gemv_fp8_batched_acc_fp32_gpu(w, x, (M, K), nvec, mode=mode))


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
def test_gemv_swiglu_repeats(dev, mode):
    from feather_amd.routines.producers import gemv_fp8_batched_swiglu
    inter, K, nvec = 5632, 2048, 32
    g = torch.Generator(device=dev).manual_seed(3)
    w, x = _pack(g, dev, mode, 2 * inter, K), _pack(g, dev, mode, nvec, K)
    _same(lambda: gemv_fp8_batched_swiglu(w, x, inter, K, nvec, mode=mode, return_f32=True))


@pytest.mark.parametrize("n", [1 << 24, 1_500_000, 16384, 1000])
def test_dot_repeats(dev, n):
    """Per-workgroup partials are added in a fixed order by a second kernel."""
    import feather_amd as feather
    g = torch.Generator(device=dev).manual_seed(n)
    for mode in ("E5M2", "E4M3"):
        a, b = _pack(g, dev, mode, n), _pack(g, dev, mode, n)
        _same(lambda: feather.dot(a, b, mode=mode))
    h1 = feather.pack_fp16_tensor(torch.randn(n, generator=g, device=dev).half())
    h2 = feather.pack_fp16_tensor(torch.randn(n, generator=g, device=dev).half())
    _same(lambda: feather.dot(h1, h2, mode="FP16"))


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("d,bs,max_ctx", [(64, 16, 4096), (64, 16, 512), (128, 16, 2000), (256, 8, 1500), (512, 16, 1100),
                                            (64, 12, 3000)])
def test_paged_attention_repeats(dev, mode, d, bs, max_ctx):
    """Split kernel (four waves merged through LDS) + merge kernel, fp32 and packed outputs."""
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
    n_seq, Hq, Hkv = 16, 16, 2
    g = torch.Generator(device=dev).manual_seed(d + bs + max_ctx)
    max_blocks = (max_ctx + bs - 1) // bs
    n_blocks = n_seq * max_blocks
    q = _pack(g, dev, mode, n_seq, Hq, d).view(n_seq, Hq, d // 4)
    kc = _pack(g, dev, mode, n_blocks, Hkv, bs, d).view(n_blocks, Hkv, bs, d // 4)
    vc = _pack(g, dev, mode, n_blocks, Hkv, bs, d).view(n_blocks, Hkv, bs, d // 4)
    ctx = torch.randint(1, max_ctx + 1, (n_seq,), generator=g, device=dev, dtype=torch.int32)
    bt = torch.randperm(n_blocks, generator=g, device=dev).to(torch.int32).view(n_seq, max_blocks)
    _same(lambda: paged_attention_fp8_acc_fp32_gpu(q, kc, vc, bt, ctx, mode=mode, max_context_len=max_ctx,
                                                   return_packed=True))


@pytest.mark.parametrize("mode", ["E5M2", "E4M3"])
@pytest.mark.parametrize("heads,L,d", [(8, 2048, 64), (16, 1024, 64), (4, 1500, 128), (2, 900, 256)])
def test_causal_varlen_attention_repeats(dev, mode, heads, L, d):
    from feather_amd.routines.attention import flash_attention_fp8_varlen_acc_fp32_gpu
    g = torch.Generator(device=dev).manual_seed(heads + L + d)
    q, k, v = (_pack(g, dev, mode, heads, L, d).view(heads, L, d // 4) for _ in range(3))
    cu = torch.tensor([0, L // 3, L // 3 + 7, L], dtype=torch.int32, device=dev)
    for causal in (False, True):
        _same(lambda: flash_attention_fp8_varlen_acc_fp32_gpu(q, k, v, cu, L - L // 3 - 7, mode=mode, causal=causal))


@pytest.mark.parametrize("hd,nq,nkv", [(64, 8, 2), (128, 4, 2)])
def test_decode_step_repeats(dev, hd, nq, nkv):
    """Both attention paths of the step (fused prologue at head dim 64, separate rotary kernel otherwise): logits and the
    appended cache rows of a step repeated from the same cache state."""
    from feather_amd.routines.decode import DecoderConfig, PackedDecoder, random_weights
    cfg = DecoderConfig(vocab=1000, hidden=nq * hd, n_layers=3, n_q_heads=nq, n_kv_heads=nkv, head_dim=hd, inter=1024)
    B, bs, max_blocks = 8, 16, 128
    n_blocks = B * max_blocks
    dec = PackedDecoder(cfg, random_weights(cfg, seed=1, device=dev), n_blocks=n_blocks, max_blocks=max_blocks, mode="E4M3",
                        device=dev)
    g = torch.Generator(device=dev).manual_seed(2)
    for lay in dec.layers:
        for name in ("k_cache", "v_cache"):
            lay[name].view(-1).copy_(_pack(g, dev, "E4M3", lay[name].numel() * 4).view(torch.int32))
    saved = [(lay["k_cache"].clone(), lay["v_cache"].clone()) for lay in dec.layers]
    ctx = torch.randint(1, 2000, (B,), generator=g, device=dev, dtype=torch.int32)
    bt = torch.randperm(n_blocks, generator=g, device=dev).to(torch.int32).view(B, max_blocks)
    tok = torch.randint(0, cfg.vocab, (B,), generator=g, device=dev, dtype=torch.int32)

    def step():
        for lay, (k0, v0) in zip(dec.layers, saved):
            lay["k_cache"].copy_(k0)
            lay["v_cache"].copy_(v0)
        logits = dec.step(tok, bt, ctx).clone()
        return [logits] + [lay[name].clone() for lay in dec.layers for name in ("k_cache", "v_cache")]

    _same(step)
