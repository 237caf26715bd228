"""The allocation-free paged-attention entry point (`feather_paged_attn_fp8_static`) against the
entry point with a caller-owned scratch buffer, through the C ABI: bit-identical results on two
calls in a row, the second on a smaller problem (the built-in buffer keeps the first call's
partials), and a clear error for a problem whose partials do not fit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a HIP device")
    return torch.device("cuda:0")


def _problem(dev, seed, n_seq, Hq, Hkv, d, bs, max_ctx, mode):
    import feather_amd as feather
    g = torch.Generator().manual_seed(seed)
    max_blocks = (max_ctx + bs - 1) // bs
    n_blocks = n_seq * max_blocks
    ctx = torch.randint(1, max_ctx + 1, (n_seq,), generator=g, dtype=torch.int32)
    ctx[0] = max_ctx
    bt = torch.randperm(n_blocks, generator=g).to(torch.int32).view(n_seq, max_blocks)
    pk = lambda *shape: feather.pack_fp8_tensor(torch.randn(*shape, generator=g).half().to(dev), mode=mode)
    return dict(q=pk(n_seq, Hq, d), kc=pk(n_blocks, Hkv, bs, d), vc=pk(n_blocks, Hkv, bs, d), bt=bt.to(dev),
                ctx=ctx.to(dev), n_seq=n_seq, Hq=Hq, Hkv=Hkv, d=d, bs=bs, max_blocks=max_blocks, max_ctx=max_ctx,
                mode=mode)


def _run(P, static, dev):
    from feather_amd import _native as N
    L = N.lib()
    out = torch.full((P["n_seq"], P["Hq"], P["d"]), float("nan"), dtype=torch.float32, device=dev)
    code = N.mode_code(P["mode"])
    scale = float(P["d"]) ** -0.5
    stream = N.stream_ptr(dev)
    n_blocks = P["kc"].numel() * 4 // (P["Hkv"] * P["bs"] * P["d"])
    shape = (P["n_seq"], P["Hq"], P["Hkv"], P["d"], P["bs"], P["max_blocks"], n_blocks, P["max_ctx"], code, scale, stream)
    ptrs = [P[k].data_ptr() for k in ("q", "kc", "vc", "bt", "ctx")]
    if static:
        rc = L.feather_paged_attn_fp8_static(*ptrs, out.data_ptr(), None, *shape)
    else:
        nbytes = int(L.feather_paged_attn_scratch_bytes(P["n_seq"], P["Hq"], P["d"], P["max_ctx"]))
        scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
        rc = L.feather_paged_attn_fp8(*ptrs, out.data_ptr(), None, scratch.data_ptr(), *shape)
    N.check(rc)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_static_scratch_matches_caller_scratch_twice(dev):
    big = _problem(dev, 11, n_seq=32, Hq=32, Hkv=4, d=64, bs=16, max_ctx=4096, mode="E4M3")    # 8 splits, 2.1 MB of partials
    small = _problem(dev, 12, n_seq=3, Hq=8, Hkv=2, d=128, bs=16, max_ctx=1100, mode="E5M2")    # 3 splits
    for P in (big, small):
        print(f"static paged attention: {P['mode']} n_seq {P['n_seq']} Hq {P['Hq']} d {P['d']} max_ctx {P['max_ctx']}",
              flush=True)
        want = _run(P, False, dev)
        got = _run(P, True, dev)
        assert np.isfinite(want).all()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # one split (no partials at all) after the buffer has been used
    one = _problem(dev, 13, n_seq=2, Hq=4, Hkv=4, d=64, bs=16, max_ctx=300, mode="E4M3")
    assert np.array_equal(_run(one, True, dev).view(np.uint32), _run(one, False, dev).view(np.uint32))


def test_static_scratch_rejects_oversized_problem(dev):
    from feather_amd import _native as N
    L = N.lib()
    # 64 sequences x 64 heads x 16 splits x 130 floats = 34 MB of partials: more than the built-in 4 MiB
    rc = L.feather_paged_attn_fp8_static(None, None, None, None, None, None, None, 64, 64, 4, 128, 16, 512, 9, 8192,
                                         N.E4M3, 0.1, None)
    assert rc == N.ESHAPE
    assert b"built-in buffer" in L.feather_last_error()


def test_static_entry_allocates_nothing_and_replays_in_a_graph(dev):
    """Free device memory is the same before and after calls of the allocation-free entry point, and a captured
    call replays to the bits of the eager call (the first call on a device, which looks up the buffer's address,
    is made before the capture, as the header asks)."""
    from feather_amd import _native as N
    L = N.lib()
    P = _problem(dev, 21, n_seq=8, Hq=16, Hkv=2, d=64, bs=16, max_ctx=1500, mode="E4M3")       # 3 splits + merge
    want = _run(P, True, dev)                                   # first use on the device: outside any capture
    out = torch.full((P["n_seq"], P["Hq"], P["d"]), float("nan"), dtype=torch.float32, device=dev)
    code, scale = N.mode_code(P["mode"]), float(P["d"]) ** -0.5
    n_blocks = P["kc"].numel() * 4 // (P["Hkv"] * P["bs"] * P["d"])
    ptrs = [P[k].data_ptr() for k in ("q", "kc", "vc", "bt", "ctx")]

    def call():
        shape = (P["n_seq"], P["Hq"], P["Hkv"], P["d"], P["bs"], P["max_blocks"], n_blocks, P["max_ctx"], code, scale,
                 N.stream_ptr(dev))
        N.check(L.feather_paged_attn_fp8_static(*ptrs, out.data_ptr(), None, *shape))

    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(dev)
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(dev)
    assert free1 == free0, f"free device memory changed across the calls: {free0} -> {free1}"
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    other = _problem(dev, 22, n_seq=4, Hq=8, Hkv=2, d=64, bs=16, max_ctx=900, mode="E4M3")
    for _ in range(3):
        out.fill_(float("nan"))
        _run(other, True, dev)                                  # eager work on the same buffer between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
