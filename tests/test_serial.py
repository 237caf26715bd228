"""Container format for packed tensors (host logic, no GPU): round trips, the byte layout
pinned by a literal record, and rejection of damaged files."""
import io
import struct
import zlib

import numpy as np
import pytest
import torch

from feather_amd.packers import serial
from feather_amd.packers.serial import PackedTensor, load_packed, load_packed_dict, save_packed, save_packed_dict


def _words(vals):
    return torch.from_numpy(np.array(vals, dtype=np.uint32).view(np.int32)).view(torch.uint32)


def test_layout_is_pinned_byte_for_byte():
    t = PackedTensor(_words([0x44434241, 0x00000045]), (5,), "E4M3")
    got = serial.dumps(t)
    payload = struct.pack("<II", 0x44434241, 0x45)
    want = (b"FTHRPACK" + struct.pack("<IIII", 1, 1, 0, 1) + struct.pack("<QQ", 5, 2) +
            struct.pack("<8Q", 5, 0, 0, 0, 0, 0, 0, 0) + struct.pack("<II", 0, zlib.crc32(payload)) + b"\0" * 16 +
            payload + b"\0" * 56)
    assert len(want) == 128 + 64 and got == want
    assert got[128:133] == b"ABCDE"          # element i of the tensor is byte i of the payload


@pytest.mark.parametrize("mode,shape,nw", [("E5M2", (3, 7), 6), ("E4M3", (2, 2, 2), 2), ("FP16", (9,), 5), ("E5M2", (0, 4), 0),
                                           ("E4M3", (), 1)])
def test_round_trip(tmp_path, mode, shape, nw):
    rng = np.random.default_rng(nw)
    t = PackedTensor(_words(rng.integers(0, 2**32, nw, dtype=np.uint64)), shape, mode, "truncate" if mode == "E5M2" else "rne")
    p = tmp_path / "t.fthr"
    save_packed(p, t)
    u = load_packed(p)
    assert u.shape == tuple(shape) and u.mode == mode and u.rounding == t.rounding
    assert u.words.dtype == torch.uint32 and torch.equal(u.words.view(torch.int32), t.words.view(torch.int32))
    assert p.stat().st_size % 64 == 0


def test_dict_round_trip_keeps_order_and_names():
    a = PackedTensor(_words([1, 2, 3]), (3, 4), "E5M2")
    b = PackedTensor(_words([7]), (2,), "FP16")
    f = io.BytesIO()
    save_packed_dict(f, {"layers.0.w_qkv": a, "norm/ünïcode": b})
    f.seek(0)
    d = load_packed_dict(f)
    assert list(d) == ["layers.0.w_qkv", "norm/ünïcode"]
    assert d["layers.0.w_qkv"].shape == (3, 4) and d["norm/ünïcode"].mode == "FP16"
    assert torch.equal(d["layers.0.w_qkv"].words.view(torch.int32), a.words.view(torch.int32))
    with pytest.raises(ValueError):
        save_packed_dict(io.BytesIO(), [("x", a), ("x", b)])


def test_accepts_reference_containers():
    # the reference's packers hand out uint32 (fp8.py:280) or float32 views (fp8.py:257, fp16.py:43)
    w = _words([0x3C003C00])
    for view in (torch.uint32, torch.int32, torch.float32):
        t = PackedTensor(w.view(view), (2,), "FP16")
        assert torch.equal(load_packed(io.BytesIO(serial.dumps(t))).words.view(torch.int32), w.view(torch.int32))


def test_rejects_inconsistent_tensors():
    with pytest.raises(ValueError):
        PackedTensor(_words([1, 2]), (3,), "E5M2")            # 3 elements need 1 word
    with pytest.raises(NotImplementedError):
        PackedTensor(_words([1]), (4,), "E3M4")
    with pytest.raises(ValueError):
        PackedTensor(_words([1]), (4,), "E5M2", rounding="stochastic")
    with pytest.raises(ValueError):
        PackedTensor(torch.zeros(1, dtype=torch.float16), (4,), "E5M2")


def test_rejects_damaged_files():
    good = serial.dumps(PackedTensor(_words([1, 2, 3]), (12,), "E5M2"))
    for bad, msg in [(b"NOTAFILE" + good[8:], "magic"), (good[:100], "header"), (good[:130], "truncated"),
                     (good[:128] + b"\xff" + good[129:], "checksum"), (good[:8] + struct.pack("<I", 2) + good[12:], "version"),
                     (b"", "empty")]:
        with pytest.raises(ValueError, match=msg):
            load_packed(io.BytesIO(bad))
    wrong_count = bytearray(good)
    wrong_count[24:32] = struct.pack("<Q", 11)               # header says 11 elements, shape says 12
    with pytest.raises(ValueError, match="corrupt"):
        load_packed(io.BytesIO(bytes(wrong_count)))
