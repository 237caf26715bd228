"""GPU parity of the packed decode step (build-defined; the reference has no model code)
against its numpy restatement in oracle/decode_ref.py.

Tolerance: every activation is re-quantised to FP8 between kernels, so a last-bit difference
in an fp32 sum can flip one FP8 code (a 6-12 % change of that element) now and then; logits
are therefore compared with max |x - ref| / max |ref| <= 2e-2, and the KV codes appended by
the first layer (no upstream quantisation flips) must agree in >= 99.5 % of the bytes."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode,hidden,nq,nkv,inter", [("E4M3", 512, 8, 2, 1024), ("E5M2", 256, 4, 4, 512),
                                                      ("E4M3", 1024, 16, 1, 1536), ("E4M3", 320, 5, 1, 704)])
def test_decode_step_vs_oracle(orc, mode, hidden, nq, nkv, inter):
    from feather_amd.routines.decode import DecoderConfig, PackedDecoder, random_weights
    from oracle import decode_ref
    dev = torch.device("cuda:0")
    cfg = DecoderConfig(n_layers=2, hidden=hidden, n_q_heads=nq, n_kv_heads=nkv, head_dim=64, inter=inter, vocab=1000)
    B, max_blocks = 3, 6
    n_blocks = B * max_blocks + 2
    w = random_weights(cfg, seed=hidden)
    dec = PackedDecoder(cfg, w, n_blocks=n_blocks, max_blocks=max_blocks, mode=mode, device=dev)
    g = torch.Generator().manual_seed(1)
    bt = torch.randperm(n_blocks, generator=g)[: B * max_blocks].to(torch.int32).view(B, max_blocks)
    ctx = torch.tensor([5, 40, 0], dtype=torch.int32)
    # pre-fill the caches with random codes for the tokens already "seen"
    dw = cfg.head_dim // 4
    kc_np, vc_np = [], []
    for lay in dec.layers:
        for name, store in (("k_cache", kc_np), ("v_cache", vc_np)):
            vals = torch.randn(n_blocks, nkv, cfg.block_size, cfg.head_dim, generator=g).half()
            import feather_amd as feather
            packed = feather.pack_fp8_tensor(vals.to(dev), mode=mode).view(n_blocks, nkv, cfg.block_size, dw)
            lay[name].copy_(packed.view(torch.int32))
            store.append(packed.view(torch.int32).cpu().numpy().view(np.uint32).copy())
    wnp = {k: v.numpy() for k, v in w.items()}
    for step in range(2):
        tokens = torch.randint(0, cfg.vocab, (B,), generator=g, dtype=torch.int32)
        logits = dec.step(tokens.to(dev), bt.to(dev), ctx.to(dev)).cpu().numpy()
        want = decode_ref.decode_step_ref(cfg, wnp, kc_np, vc_np, tokens.numpy(), bt.numpy(), ctx.numpy(), mode)
        err = np.abs(logits - want).max() / np.abs(want).max()
        assert err <= 2e-2, f"step {step}: normalised logit error {err}"
        assert np.mean(np.abs(logits - want) <= 2e-3 * np.abs(want).max()) >= 0.97
        got_k = dec.layers[0]["k_cache"].cpu().numpy().view(np.uint32).view(np.uint8)
        got_v = dec.layers[0]["v_cache"].cpu().numpy().view(np.uint32).view(np.uint8)
        assert np.mean(got_k == kc_np[0].view(np.uint8)) >= 0.995 and np.mean(got_v == vc_np[0].view(np.uint8)) >= 0.995
        # continue from the oracle's cache state so that a flipped code does not accumulate across steps
        for l, lay in enumerate(dec.layers):
            lay["k_cache"].copy_(torch.from_numpy(kc_np[l].view(np.int32)))
            lay["v_cache"].copy_(torch.from_numpy(vc_np[l].view(np.int32)))
        ctx = ctx + 1


def test_decode_step_long_contexts_use_split_attention(orc):
    """Contexts longer than one 512-token split: the attention of the step runs as several splits
    plus the merge kernel that emits the packed operand of W_o."""
    import feather_amd as feather
    from feather_amd.routines.decode import DecoderConfig, PackedDecoder, random_weights
    from oracle import decode_ref
    dev = torch.device("cuda:0")
    mode = "E4M3"
    cfg = DecoderConfig(n_layers=1, hidden=256, n_q_heads=4, n_kv_heads=2, head_dim=64, inter=512, vocab=300)
    B, max_blocks = 4, 80                                     # up to 1280 tokens: three splits
    n_blocks = B * max_blocks
    w = random_weights(cfg, seed=3)
    dec = PackedDecoder(cfg, w, n_blocks=n_blocks, max_blocks=max_blocks, mode=mode, device=dev)
    g = torch.Generator().manual_seed(2)
    bt = torch.randperm(n_blocks, generator=g).to(torch.int32).view(B, max_blocks)
    ctx = torch.tensor([700, 1279, 512, 3], dtype=torch.int32)
    dw = cfg.head_dim // 4
    vals = [torch.randn(n_blocks, cfg.n_kv_heads, cfg.block_size, cfg.head_dim, generator=g).half() for _ in range(2)]
    packed = [feather.pack_fp8_tensor(v.to(dev), mode=mode).view(n_blocks, cfg.n_kv_heads, cfg.block_size, dw) for v in vals]
    dec.layers[0]["k_cache"].copy_(packed[0].view(torch.int32))
    dec.layers[0]["v_cache"].copy_(packed[1].view(torch.int32))
    kc_np = [packed[0].view(torch.int32).cpu().numpy().view(np.uint32).copy()]
    vc_np = [packed[1].view(torch.int32).cpu().numpy().view(np.uint32).copy()]
    tokens = torch.randint(0, cfg.vocab, (B,), generator=g, dtype=torch.int32)
    logits = dec.step(tokens.to(dev), bt.to(dev), ctx.to(dev)).cpu().numpy()
    want = decode_ref.decode_step_ref(cfg, {k: v.numpy() for k, v in w.items()}, kc_np, vc_np, tokens.numpy(), bt.numpy(),
                                      ctx.numpy(), mode)
    assert np.abs(logits - want).max() / np.abs(want).max() <= 2e-2
    got_k = dec.layers[0]["k_cache"].cpu().numpy().view(np.uint32)
    assert np.mean(got_k.view(np.uint8) == kc_np[0].view(np.uint8)) >= 0.9999


def test_decode_step_rejects_bad_arguments():
    from feather_amd.routines.decode import DecoderConfig, PackedDecoder, random_weights
    dev = torch.device("cuda:0")
    cfg = DecoderConfig(n_layers=1, hidden=256, n_q_heads=4, n_kv_heads=2, head_dim=64, inter=512, vocab=100)
    dec = PackedDecoder(cfg, random_weights(cfg), n_blocks=8, max_blocks=4, device=dev)
    bt = torch.zeros((2, 4), dtype=torch.int32, device=dev)
    tok = torch.zeros(2, dtype=torch.int32, device=dev)
    ctx = torch.zeros(2, dtype=torch.int32, device=dev)
    assert dec.step(tok, bt, ctx).shape == (2, 100)
    with pytest.raises(ValueError):
        dec.step(tok.long(), bt, ctx)
    with pytest.raises(ValueError):
        dec.step(tok, bt[:, :3].contiguous(), ctx)
    with pytest.raises(ValueError):
        dec.step(tok, bt, ctx, max_ctx=1000)
    with pytest.raises(NotImplementedError):
        PackedDecoder(cfg, random_weights(cfg), n_blocks=8, max_blocks=4, mode="E3M4", device=dev)


def test_entry_points_replay_in_a_graph():
    """Every entry point only enqueues kernels on the caller's stream (no allocation, memset or
    synchronisation), so a captured sequence of calls replays to the same bits as the eager run:
    GEMV, dot, flash attention, paged attention and a decode step, replayed three times with other
    work in between."""
    import feather_amd as feather
    from feather_amd.routines.decode import DecoderConfig, PackedDecoder, random_weights
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(4)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev)
    M, K = 512, 1024
    mp, vp = feather.pack_fp8_tensor(rn(M, K).half(), mode="E4M3"), feather.pack_fp8_tensor(rn(K).half(), mode="E4M3")
    qkv = [feather.pack_fp8_tensor(rn(2, 256, 64).half(), mode="E5M2").view(2, 256, 16) for _ in range(3)]
    cfg = DecoderConfig(n_layers=2, hidden=256, n_q_heads=4, n_kv_heads=2, head_dim=64, inter=512, vocab=200)
    B, max_blocks = 3, 48                                      # contexts up to 768: two attention splits
    dec = PackedDecoder(cfg, random_weights(cfg, seed=1), n_blocks=B * max_blocks, max_blocks=max_blocks, mode="E4M3", device=dev)
    for lay in dec.layers:
        for name in ("k_cache", "v_cache"):
            lay[name].view(-1).copy_(feather.pack_fp8_tensor(rn(lay[name].numel() * 4).half(), mode="E4M3").view(torch.int32))
    bt = torch.randperm(B * max_blocks, generator=g, device=dev).to(torch.int32).view(B, max_blocks)
    ctx = torch.tensor([700, 30, 513], dtype=torch.int32, device=dev)
    tok = torch.tensor([1, 2, 3], dtype=torch.int32, device=dev)
    q1 = feather.pack_fp8_tensor(rn(B, 4, 64).half(), mode="E4M3").view(B, 4, 16)

    def work():
        y = feather.gemv(mp, vp, original_shape=(M, K), mode="E4M3")
        d = feather.dot(mp, mp, mode="E4M3")
        a = feather.flash_attention_fp8_acc_fp32_gpu(qkv[0], qkv[1], qkv[2], 256, 16, mode="E5M2", causal=True)
        p = paged_attention_fp8_acc_fp32_gpu(q1, dec.layers[0]["k_cache"], dec.layers[0]["v_cache"], bt, ctx, mode="E4M3")
        lg = dec.step(tok, bt, ctx)
        return y, d, a, p, lg

    caches0 = [(lay["k_cache"].clone(), lay["v_cache"].clone()) for lay in dec.layers]
    def reset():
        for lay, (k0, v0) in zip(dec.layers, caches0):
            lay["k_cache"].copy_(k0); lay["v_cache"].copy_(v0)

    eager = [t.clone() for t in work()]
    reset()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()                                                 # warm-up on a side stream (allocations happen here)
    torch.cuda.current_stream().wait_stream(side)
    reset()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = work()
    for _ in range(3):
        reset()
        for t in outs:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want)
        feather.gemv(mp, vp, original_shape=(M, K), mode="E4M3")   # eager work between the replays
