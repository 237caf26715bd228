"""ctypes binding of libfeather_hip.so (the C ABI declared in include/feather_hip.h).

PyTorch is used for device memory and streams only: tensors are passed as raw
device pointers plus the current HIP stream.  There is no CPU fallback: every
routine raises if the library or a GPU is missing.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfeather_hip.so")

OK, EINVAL, EMODE, ESHAPE, ELAUNCH = 0, -1, -2, -3, -4
ABI_VERSION = 10400   # FEATHER_HIP_VERSION of the include/feather_hip.h these signatures were written against
E5M2, E4M3 = 0, 1
ROUND_RNE, ROUND_TRUNC = 0, 1
SEM_KERNEL, SEM_IEEE = 0, 1
OUT_F32, OUT_F16 = 0, 1
TAIL_MASK, TAIL_REFERENCE = 0, 1

_MODES = {"E5M2": E5M2, "E4M3": E4M3}

# every exported symbol with (restype, argtypes); kept in step with include/feather_hip.h
_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
SIGNATURES = {
    "feather_version": (_i32, []),
    "feather_last_error": (ctypes.c_char_p, []),
    "feather_pack_fp8": (_i32, [_vp, _vp, _i64, _i32, _i32, _vp]),
    "feather_quant_pack_f32": (_i32, [_vp, _vp, _i64, _i32, _vp]),
    "feather_unpack_fp8": (_i32, [_vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp]),
    "feather_pack_fp16": (_i32, [_vp, _vp, _i64, _vp]),
    "feather_unpack_fp16": (_i32, [_vp, _vp, _i64, _vp]),
    "feather_gemv_fp8": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, _vp]),
    "feather_gemv_fp8_batched": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp]),
    "feather_gemv_fp8_batched_swiglu": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp]),
    "feather_dot_scratch_bytes": (_i64, []),
    "feather_dot_fp8": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _vp]),
    "feather_dot_fp16": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _vp]),
    "feather_flash_attn_fp8": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _f32, _i32, _vp]),
    "feather_flash_attn_fp8_ws": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i32, _f32, _i32, _vp]),
    "feather_flash_attn_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "feather_flash_attn_fp8_varlen": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _f32,
                                             _i32, _vp]),
    "feather_paged_cache_write": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                                         _i64, _i32, _vp]),
    "feather_paged_attn_scratch_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "feather_paged_attn_fp8": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                      _i64, _i32, _f32, _vp]),
    "feather_paged_attn_fp8_static": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                                             _i64, _i64, _i32, _f32, _vp]),
    "feather_decode_step_scratch_bytes": (_i64, [_vp, _i64, _i64]),
    "feather_decode_step_attention_path": (_i32, [_vp, _i64, _i64]),
    "feather_decode_step": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp]),
    "feather_add_rmsnorm_pack": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _f32, _i32, _vp]),
    "feather_rope_append": (_i32, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                   _i64, _i64, _f32, _i32, _vp]),
}


class DecoderLayer(ctypes.Structure):
    """feather_decoder_layer_t (include/feather_hip.h)."""
    _fields_ = [("w_qkv", _vp), ("w_o", _vp), ("w_gate_up", _vp), ("w_down", _vp), ("norm_attn", _vp),
                ("norm_mlp", _vp), ("k_cache", _vp), ("v_cache", _vp)]


class Decoder(ctypes.Structure):
    """feather_decoder_t (include/feather_hip.h)."""
    _fields_ = [("n_layers", ctypes.c_int32), ("hidden", ctypes.c_int32), ("n_q_heads", ctypes.c_int32),
                ("n_kv_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("inter", ctypes.c_int32),
                ("vocab", ctypes.c_int32), ("block_size", ctypes.c_int32), ("max_blocks", ctypes.c_int32),
                ("n_blocks", ctypes.c_int32), ("mode", ctypes.c_int32), ("rms_eps", _f32), ("rope_theta", _f32),
                ("layers", ctypes.POINTER(DecoderLayer)), ("embed_f16", _vp), ("norm_final", _vp),
                ("w_lm_head", _vp)]

_lib = None
_lock = threading.Lock()


def lib() -> ctypes.CDLL:
    """Load the HIP library once; fail loudly if it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f"{LIB_PATH} is missing: build it with `python -m feather_amd.build` "
                        "(hipcc, gfx950). There is no CPU fallback.")
                L = ctypes.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(L, name)  # AttributeError here = header and library out of step
                    fn.restype = res
                    fn.argtypes = args
                got = L.feather_version()
                if got // 100 != ABI_VERSION // 100:   # major.minor: any signature or struct change
                    raise RuntimeError(
                        f"{LIB_PATH} reports version {got}, this binding was written against {ABI_VERSION}: "
                        "rebuild the library with `python -m feather_amd.build`")
                _lib = L
    return _lib


def mode_code(mode) -> int:
    """"E5M2"/"E4M3" -> C enum; anything else raises like the reference packer
    (feather/packers/fp8.py:114)."""
    if isinstance(mode, str) and mode in _MODES:
        return _MODES[mode]
    raise NotImplementedError(f"Mode {mode} not supported")


def check(rc: int) -> None:
    if rc == OK:
        return
    msg = lib().feather_last_error().decode("utf-8", "replace")
    if rc == EMODE:
        raise NotImplementedError(msg)
    if rc in (EINVAL, ESHAPE):
        raise ValueError(msg)
    raise RuntimeError(f"feather_hip error {rc}: {msg}")


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("feather_amd needs a HIP device (torch.cuda.is_available() is False); "
                           "there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def stream_ptr(device: torch.device) -> int:
    """Raw hipStream_t of torch's current stream on `device`."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(idx)


def call(device: torch.device, name: str, *args) -> None:
    """Run one C-ABI entry point on torch's current stream of `device` (made current for
    the call if it is not) and raise on a non-zero return code."""
    fn = getattr(lib(), name)
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx == torch.cuda.current_device():
        rc = fn(*args, torch._C._cuda_getCurrentRawStream(idx))
    else:
        with torch.cuda.device(idx):
            rc = fn(*args, torch._C._cuda_getCurrentRawStream(idx))
    if rc != OK:
        check(rc)


def ptr(t: torch.Tensor) -> int:
    return t.data_ptr()


_WORD_DTYPES = (torch.uint32, torch.int32, torch.float32)


def as_words(t: torch.Tensor, name: str) -> torch.Tensor:
    """Packed operands are 4-byte containers: uint32 (reference callers use
    ``.view(torch.uint32)``), int32 or the float32 container the numpy packers
    return.  Must be a contiguous tensor on a HIP device."""
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name}: expected a torch.Tensor of packed words, got {type(t).__name__}")
    if t.dtype not in _WORD_DTYPES:
        raise ValueError(f"{name}: packed words must be uint32/int32/float32 containers, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name}: must live on a HIP device ('cuda'), got {t.device}")
    if not t.is_contiguous():
        t = t.contiguous()
    return t


_scratch: dict = {}


def scratch(device: torch.device, nbytes: int, tag: str) -> torch.Tensor:
    """Per (device, stream, tag) scratch buffer, allocated once and re-used."""
    key = (device.index, stream_ptr(device), tag)
    buf = _scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _scratch[key] = buf
    return buf
