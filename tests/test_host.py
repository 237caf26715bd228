"""Host-side checks that need no GPU: the C-ABI library loads and exports every
symbol the header declares, argument validation and error mapping follow the
reference's conventions, and nothing in the product falls back to the CPU."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "feather_hip.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(feather_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    from feather_amd import _native as N
    assert os.path.exists(N.LIB_PATH), "build with `python -m feather_amd.build`"
    lib = ctypes.CDLL(N.LIB_PATH)
    names = _declared()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/feather_hip.h but not exported"
    assert sorted(N.SIGNATURES) == names          # the ctypes table covers the header exactly


def test_version_and_error_string():
    from feather_amd import _native as N
    L = N.lib()
    assert L.feather_version() // 100 == N.ABI_VERSION // 100      # header, library and binding agree (major.minor)
    assert isinstance(L.feather_last_error(), bytes)
    assert L.feather_dot_scratch_bytes() >= 64 + 4
    assert L.feather_paged_attn_scratch_bytes(32, 32, 64, 4096) == 32 * 32 * 8 * 66 * 4


def test_c_abi_argument_checks_without_gpu():
    """Validation runs before any launch, so error codes can be exercised on the CPU."""
    from feather_amd import _native as N
    L = N.lib()
    assert L.feather_pack_fp8(None, None, 16, 7, 0, None) == N.EMODE
    assert b"mode 7" in L.feather_last_error()
    assert L.feather_pack_fp8(None, None, 16, N.E4M3, N.ROUND_TRUNC, None) == N.EMODE
    assert L.feather_pack_fp8(None, None, 16, N.E5M2, 0, None) == N.EINVAL          # null pointers
    assert L.feather_pack_fp8(None, None, -1, N.E5M2, 0, None) == N.EINVAL
    assert L.feather_pack_fp8(None, None, 0, N.E5M2, 0, None) == N.OK               # empty input: nothing to do
    assert L.feather_gemv_fp8(None, None, None, 4, 6, N.E5M2, None) == N.ESHAPE     # K % 4
    assert b"multiple of 4" in L.feather_last_error()
    assert L.feather_gemv_fp8(None, None, None, 4, 8, 3, None) == N.EMODE
    assert L.feather_gemv_fp8(None, None, None, 0, 8, N.E5M2, None) == N.OK
    assert L.feather_gemv_fp8_batched(None, None, None, 16, 512, 65, N.E4M3, None) == N.ESHAPE
    assert L.feather_flash_attn_fp8(None, None, None, None, 1, 64, 96, 1, N.E5M2, 0.1, 0, None) in (N.EINVAL, N.ESHAPE)
    assert L.feather_flash_attn_fp8(None, None, None, None, 3, 64, 64, 2, N.E5M2, 0.1, 0, None) == N.ESHAPE
    assert L.feather_flash_attn_fp8(None, None, None, None, 1, 64, 64, 1, N.E5M2, 0.1, 5, None) == N.EINVAL
    assert L.feather_unpack_fp8(None, None, 4, N.E5M2, 9, 0, 0, None) == N.EINVAL
    assert L.feather_dot_fp8(None, None, None, None, 4, 2, None) == N.EMODE
    assert L.feather_paged_attn_fp8(None, None, None, None, None, None, None, None, 1, 6, 4, 64, 16, 4, 8, 64, N.E5M2,
                                    0.1, None) == N.ESHAPE
    assert L.feather_paged_attn_fp8(None, None, None, None, None, None, None, None, 1, 8, 4, 64, 16, 4, 0, 64, N.E5M2,
                                    0.1, None) == N.EINVAL                           # a cache without blocks
    assert L.feather_paged_attn_fp8_static(None, None, None, None, None, None, None, 64, 64, 4, 128, 16, 512, 9, 8192,
                                           N.E4M3, 0.1, None) == N.ESHAPE            # partials beyond the built-in buffer
    assert b"built-in buffer" in L.feather_last_error()
    # a zero or negative softmax scale is rejected everywhere (the running maximum is kept on raw scores)
    assert L.feather_flash_attn_fp8(None, None, None, None, 1, 64, 64, 1, N.E5M2, 0.0, 0, None) == N.EINVAL
    assert L.feather_flash_attn_fp8(None, None, None, None, 1, 64, 64, 1, N.E5M2, -0.125, 0, None) == N.EINVAL
    assert b"scale" in L.feather_last_error()
    assert L.feather_flash_attn_fp8_varlen(None, None, None, None, None, 1, 64, 64, 1, 64, 1, N.E5M2, -1.0, 0,
                                           None) == N.EINVAL
    assert L.feather_paged_attn_fp8(None, None, None, None, None, None, None, None, 1, 8, 4, 64, 16, 4, 8, 64, N.E5M2,
                                    0.0, None) == N.EINVAL
    # the fused producers
    assert L.feather_quant_pack_f32(None, None, 8, 5, None) == N.EMODE
    assert L.feather_quant_pack_f32(None, None, 8, N.E4M3, None) == N.EINVAL
    assert L.feather_quant_pack_f32(None, None, 0, N.E4M3, None) == N.OK
    assert L.feather_add_rmsnorm_pack(None, None, 0, 0, None, None, None, 2, 30, 1e-5, N.E4M3, None) == N.ESHAPE
    assert L.feather_add_rmsnorm_pack(None, None, 0, 0, None, None, None, 2, 32, 1e-5, N.E4M3, None) == N.EINVAL
    assert L.feather_gemv_fp8_batched_swiglu(None, None, None, None, 64, 100, 4, N.E4M3, None) == N.ESHAPE
    assert L.feather_gemv_fp8_batched_swiglu(None, None, None, None, 64, 256, 65, N.E4M3, None) == N.ESHAPE
    assert L.feather_rope_append(None, 1, 0, None, None, None, None, None, None, None, None, 2, 4, 2, 60, 16, 4, 8,
                                 10000.0, N.E4M3, None) == N.ESHAPE
    assert L.feather_rope_append(None, 1, 0, None, None, None, None, None, None, None, None, 2, 4, 2, 64, 16, 4, 0,
                                 10000.0, N.E4M3, None) == N.EINVAL                  # n_blocks = 0
    assert L.feather_rope_append(None, 1, 0, None, None, None, None, None, None, None, None, 2, 1 << 20, 2, 1024, 16, 4, 8,
                                 10000.0, N.E4M3, None) == N.ESHAPE                  # more (head, 8-element) items than the grid holds
    assert b"exceeds the grid" in L.feather_last_error()
    assert L.feather_flash_attn_fp8_varlen(None, None, None, None, None, 1, 8, 8, 1, 16, 1, N.E5M2, 0.1, 0, None) == N.ESHAPE
    assert b"head dim 16" in L.feather_last_error()                                 # 32, 64, 128, 256, 512 only
    assert L.feather_paged_attn_fp8(None, None, None, None, None, None, None, None, 1, 8, 4, 32, 16, 4, 8, 64, N.E5M2,
                                    0.1, None) == N.ESHAPE                           # paged decode: 64, 128, 256, 512
    assert L.feather_paged_cache_write(None, None, 0, None, None, None, None, None, 1, 4, 2, 64, 16, 4, -1, N.E5M2,
                                       None) == N.EINVAL
    # attention with a workspace: how much the library asks for (pure host arithmetic) and its argument checks
    ws = L.feather_flash_attn_workspace_bytes
    assert ws(8, 1024, 512) == 2 * 8 * 1024 * 514 * 4      # 128 workgroups: two key ranges fill the 256 CUs
    assert ws(8, 1024, 128) == 4 * 8 * 1024 * 130 * 4      # 64 workgroups of 128 queries: four ranges
    assert ws(8, 4096, 512) == 0 and ws(64, 8192, 64) == 0 and ws(1, 100, 256) == 0 and ws(0, 64, 256) == 0
    assert L.feather_flash_attn_fp8_ws(None, None, None, None, 8, 64, 1, 64, 64, 1, N.E5M2, 0.1, 0, None) == N.EINVAL
    assert b"workspace" in L.feather_last_error()          # misaligned
    assert L.feather_flash_attn_fp8_ws(None, None, None, None, None, 64, 1, 64, 64, 1, N.E5M2, 0.1, 0, None) == N.EINVAL
    assert L.feather_flash_attn_fp8_ws(None, None, None, None, None, 0, 0, 64, 64, 1, N.E5M2, 0.1, 0, None) == N.OK


def test_error_mapping():
    from feather_amd import _native as N
    L = N.lib()
    with pytest.raises(NotImplementedError):
        N.check(L.feather_pack_fp8(None, None, 16, 9, 0, None))
    with pytest.raises(ValueError):
        N.check(L.feather_gemv_fp8(None, None, None, 4, 6, N.E5M2, None))
    with pytest.raises(NotImplementedError):
        N.mode_code("E3M4")
    assert N.mode_code("E5M2") == 0 and N.mode_code("E4M3") == 1


def test_python_validation_before_any_device_work():
    import feather_amd as feather
    from feather_amd.routines import attention, dot, gemv
    w = torch.zeros(8, dtype=torch.int32)
    with pytest.raises(NotImplementedError):                     # reference: fp8.py:114
        feather.pack_fp8_tensor(torch.zeros(4, dtype=torch.float16), mode="E3M4")
    with pytest.raises(ValueError):                              # K % 4 != 0
        gemv.gemv_fp8_e5m2_acc_fp32_gpu(w, w, (4, 6))
    with pytest.raises(ValueError):                              # CPU tensors are not silently computed on the host
        gemv.gemv_fp8_e5m2_acc_fp32_gpu(w, w, (4, 8))
    with pytest.raises(ValueError):
        dot.dot_fp8_e5m2_acc_fp32_gpu(w, w)
    with pytest.raises(ValueError):
        gemv.gemv_fp8_e4m3_acc_fp32_gpu(w.to(torch.float16), w, (4, 8))
    with pytest.raises(ValueError):
        attention.flash_attention_fp8_e5m2_acc_fp32_gpu(w, w, w, 4, 24)   # d = 96 unsupported
    with pytest.raises(NotImplementedError):
        feather.gemv(w, w, original_shape=(4, 8), mode="E2M5")
    with pytest.raises(ValueError):
        feather.gemv(w, w)


def test_wrappers_reject_host_tensors_before_any_launch():
    """A CPU tensor handed to a wrapper would reach the kernel as a host pointer (a GPU memory fault);
    every wrapper must raise ValueError before the C ABI is called.  Runs without a GPU: nothing is launched."""
    from feather_amd.routines import attention, producers
    from feather_amd.routines.paged_attention import paged_attention_fp8_acc_fp32_gpu, paged_cache_write
    w = lambda *s: torch.zeros(s, dtype=torch.int32)
    i32 = lambda *s: torch.zeros(s, dtype=torch.int32)
    kc = w(4, 2, 16, 16)
    h16 = torch.zeros((2, 8, 64), dtype=torch.float16)
    with pytest.raises(ValueError):                              # fp16 K/V on the host (the packed branch had this check already)
        paged_cache_write(h16, h16, kc, kc, i32(1, 2), i32(2), mode="E5M2")
    with pytest.raises(ValueError):
        paged_cache_write(w(2, 8, 16), w(2, 8, 16), kc, kc, i32(1, 2), i32(2), mode="E5M2")
    with pytest.raises(ValueError):
        paged_attention_fp8_acc_fp32_gpu(w(1, 4, 16), kc, kc, i32(1, 2), i32(1), mode="E4M3")
    with pytest.raises(ValueError):
        producers.quant_pack_f32(torch.zeros(8))
    with pytest.raises(ValueError):
        producers.add_rmsnorm_pack(torch.zeros(2, 64), torch.ones(64))
    with pytest.raises(ValueError):
        producers.rope_append(torch.zeros(1, 8 * 64), i32(1), i32(1, 2), kc, kc, n_q_heads=4)
    with pytest.raises(ValueError):
        producers.gemv_fp8_batched_swiglu(w(2 * 8 * 256 // 4), w(256 // 4), 8, 256, 1)
    with pytest.raises(ValueError):                              # non-positive softmax scale
        attention.flash_attention_fp8_acc_fp32_gpu(w(64 * 16), w(64 * 16), w(64 * 16), 64, 16, scale=0.0)


def test_decoder_step_validates_out_and_status_without_launching():
    """PackedDecoder.step checks a caller-supplied `out` / `status` (device, dtype, shape, contiguity)
    before the C call.  Exercised on an instance built without a device: validation comes first."""
    from feather_amd.routines.decode import DecoderConfig, PackedDecoder
    cfg = DecoderConfig(n_layers=1, hidden=256, n_q_heads=4, n_kv_heads=2, head_dim=64, inter=512, vocab=100)
    dec = PackedDecoder.__new__(PackedDecoder)
    dec.cfg, dec.device, dec.max_blocks, dec.n_blocks = cfg, torch.device("cuda", 0), 4, 8
    tok = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(ValueError, match="token_ids"):           # host tensors never reach the library
        dec.step(tok, torch.zeros((2, 4), dtype=torch.int32), tok)


def test_cache_index_arithmetic_stays_inside_the_cache():
    """CPU model of the device-side index arithmetic of the cache writers and readers
    (csrc/kv_cache.hip, rope_append_kernel, paged_attn_split_kernel): whatever the table entries and
    positions are -- negative, past the table, padding values -- every word offset that is written or
    read lies inside [0, n_blocks * n_kv * block_size * dw)."""
    rng = np.random.default_rng(3)
    n_blocks, n_kv, bs, dw, max_blocks = 5, 2, 4, 16, 3
    size = n_blocks * n_kv * bs * dw
    cap = max_blocks * bs

    def append_offset(pos_raw, blk):                             # rope_append_kernel / paged_cache_write_kernel
        pos_ok = 0 <= pos_raw < cap
        blk_ok = 0 <= blk < n_blocks
        if not (pos_ok and blk_ok):
            return None, (min(max(pos_raw, 0), cap), 1 if not pos_ok else 2)
        return [((blk * n_kv + h) * bs + pos_raw % bs) * dw for h in range(n_kv)], (pos_raw + 1, 0)

    def read_offset(blk, tok, kvh):                              # paged_attn_split_kernel: unsigned min with n_blocks - 1
        b = min(blk & 0xFFFFFFFF, n_blocks - 1)
        return ((b * n_kv + kvh) * bs + tok % bs) * dw

    for pos_raw in (-7, -1, 0, 1, cap - 1, cap, cap + 5, 2**31 - 1):
        for blk in (-2**31, -1, 0, n_blocks - 1, n_blocks, 10**6, 2**31 - 1):
            offs, (ctx_after, status) = append_offset(pos_raw, blk)
            if offs is None:
                assert status in (1, 2) and 0 <= ctx_after <= cap
            else:
                assert status == 0 and ctx_after == pos_raw + 1 <= cap
                assert all(0 <= o and o + dw <= size for o in offs)
            for tok in range(cap):
                for kvh in range(n_kv):
                    o = read_offset(blk, tok, kvh)
                    assert 0 <= o and o + dw <= size


def test_no_cpu_fallback_when_no_device():
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    import feather_amd as feather
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        feather.pack_fp8_tensor(torch.zeros(8, dtype=torch.float16))
    from feather_amd.packers import fp8
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fp8.pack_fp8_ndarray(np.zeros(8, np.float16))


def test_reference_api_surface_is_present():
    """Names a user of the reference imports (feather/packers/*.py, feather/routines/*.py,
    README.md:95-107) exist with the same spelling."""
    import feather_amd as feather
    from feather_amd.packers import fp8, fp16
    from feather_amd.routines import activations, attention, dot, gemv
    for n in ("pack_fp8_into_fp32_legacy", "pack_fp8_into_fp32", "pack_fp8_ndarray_legacy", "pack_fp8_ndarray",
              "pack_fp8_tensor_legacy", "pack_fp8_tensor", "unpack_fp8_from_fp32_legacy", "unpack_fp8_from_fp32",
              "unpack_into_fp8_ndarray"):
        assert callable(getattr(fp8, n))
    for n in ("pack_fp16_into_fp32", "unpack_fp32_into_fp16", "pack_fp16_ndarray", "unpack_into_fp16_ndarray"):
        assert callable(getattr(fp16, n))
    for n in ("gemv_fp8_e5m2_acc_fp32_gpu", "gemv_fp8_e4m3_acc_fp32_gpu"):
        assert callable(getattr(gemv, n))
    for n in ("dot_fp16_acc_fp32_vec", "dot_fp16_acc_fp32_numba", "dot_fp16_acc_fp32_gpu", "dot_fp8_e5m2_acc_fp32_gpu"):
        assert callable(getattr(dot, n))
    assert callable(attention.flash_attention_fp8_e5m2_acc_fp32_gpu)
    assert callable(activations.relu1d_fp8_ret_fp32_feather_gpu)
    for n in ("pack_fp8_tensor", "pack_fp16_tensor", "gemv", "dot"):
        assert callable(getattr(feather, n))
    import feather as shim                                         # drop-in package name
    assert shim.pack_fp8_tensor is feather.pack_fp8_tensor
    from feather.packers.fp8 import pack_fp8_tensor as p2
    from feather.routines.gemv import gemv_fp8_e5m2_acc_fp32_gpu as g2
    assert p2 is fp8.pack_fp8_tensor and g2 is gemv.gemv_fp8_e5m2_acc_fp32_gpu


def test_product_does_not_import_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "feather_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text and "feather_oracle" not in text, f


def test_bench_refuses_more_than_one_gpu():
    """Nothing in this build uses a second GPU: `bench.py --gpus N` with N above 1 exits with a message that says so
    (before it touches a device)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stderr + r.stdout)
    assert not any(line.startswith("{") for line in r.stdout.splitlines())     # no result line
