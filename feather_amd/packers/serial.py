"""On-disk container for packed tensors.

``pack_fp8_tensor`` returns a flat ``uint32`` tensor and drops the shape and the
mode (reference feather/packers/fp8.py:280-281), so a packed weight cannot be
stored and handed to ``gemv`` later without side information.  A record keeps
both next to the words:

    offset  size  field
    0       8     magic  b"FTHRPACK"
    8       4     version (1)
    12      4     mode: 0 = E5M2, 1 = E4M3, 2 = FP16 container (two fp16 per word)
    16      4     rounding: 0 = round to nearest even, 1 = truncation (legacy E5M2 packer)
    20      4     ndim (<= 8)
    24      8     n_elements (product of the shape)
    32      8     n_words (= ceil(n_elements / 4), or / 2 for the FP16 container)
    40      64    shape, 8 x uint64, unused entries 0
    104     4     name length in bytes (<= 65535; 0 in a single-tensor file)
    108     4     CRC-32 (zlib) of the payload
    112     16    zero
    128     ...   name (UTF-8), zero-padded to a multiple of 64 bytes
    ...     ...   payload: n_words little-endian uint32, zero-padded to a multiple of 64 bytes

All integers are little endian.  A file is one record or several back to back
(a dictionary of named tensors).  Loading places the words on the requested
device; the payload itself is never converted on the host.
"""
from __future__ import annotations

import dataclasses
import io
import math
import os
import struct
import zlib
from typing import BinaryIO, Dict, Iterable, Tuple, Union

import numpy as np
import torch

__all__ = ["PackedTensor", "save_packed", "load_packed", "save_packed_dict", "load_packed_dict"]

MAGIC = b"FTHRPACK"
VERSION = 1
_HEADER = struct.Struct("<8sIIIIQQ8QII16x")
assert _HEADER.size == 128
_MODES = {"E5M2": 0, "E4M3": 1, "FP16": 2}
_MODE_NAMES = {v: k for k, v in _MODES.items()}
_ROUNDINGS = {"rne": 0, "truncate": 1}
_ROUNDING_NAMES = {v: k for k, v in _ROUNDINGS.items()}
_PER_WORD = {"E5M2": 4, "E4M3": 4, "FP16": 2}


@dataclasses.dataclass
class PackedTensor:
    """Packed words together with what is needed to use them: the shape before packing, the mode
    and the rounding the packer used."""
    words: torch.Tensor
    shape: Tuple[int, ...]
    mode: str = "E5M2"
    rounding: str = "rne"

    def __post_init__(self):
        self.shape = tuple(int(s) for s in self.shape)
        if self.mode not in _MODES:
            raise NotImplementedError(f"mode {self.mode!r} not supported (E5M2, E4M3, FP16)")
        if self.rounding not in _ROUNDINGS:
            raise ValueError(f"rounding {self.rounding!r} not supported (rne, truncate)")
        if len(self.shape) > 8 or any(s < 0 for s in self.shape):
            raise ValueError(f"shape {self.shape} not supported (at most 8 non-negative dimensions)")
        if not isinstance(self.words, torch.Tensor) or self.words.dtype not in (torch.uint32, torch.int32, torch.float32):
            raise ValueError("words must be a torch tensor of 4-byte elements (uint32, int32 or float32 container)")
        per = _PER_WORD[self.mode]
        if self.words.numel() != (self.n_elements + per - 1) // per:
            raise ValueError(f"{self.words.numel()} words do not hold shape {self.shape} "
                             f"({self.n_elements} elements, {per} per word)")

    @property
    def n_elements(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n


def _pad64(n: int) -> int:
    return (-n) % 64


def _write_record(f: BinaryIO, t: PackedTensor, name: str) -> None:
    payload = t.words.detach().reshape(-1).contiguous().cpu().view(torch.int32).numpy().astype("<i4", copy=False).tobytes()
    nm = name.encode("utf-8")
    if len(nm) > 65535:
        raise ValueError("name too long")
    shape8 = list(t.shape) + [0] * (8 - len(t.shape))
    f.write(_HEADER.pack(MAGIC, VERSION, _MODES[t.mode], _ROUNDINGS[t.rounding], len(t.shape), t.n_elements,
                         len(payload) // 4, *shape8, len(nm), zlib.crc32(payload) & 0xFFFFFFFF))
    if nm:
        f.write(nm + b"\0" * _pad64(len(nm)))
    f.write(payload + b"\0" * _pad64(len(payload)))


def _read_exact(f: BinaryIO, n: int, what: str) -> bytes:
    b = f.read(n)
    if len(b) != n:
        raise ValueError(f"truncated file: expected {n} bytes of {what}, got {len(b)}")
    return b


def _read_record(f: BinaryIO, device) -> Union[None, Tuple[str, PackedTensor]]:
    head = f.read(_HEADER.size)
    if not head:
        return None
    if len(head) != _HEADER.size:
        raise ValueError("truncated file: incomplete record header")
    magic, version, mode, rounding, ndim, n_elem, n_words, *rest = _HEADER.unpack(head)
    shape8, name_len, crc = rest[:8], rest[8], rest[9]
    if magic != MAGIC:
        raise ValueError("not a packed-tensor file (bad magic)")
    if version != VERSION:
        raise ValueError(f"unsupported container version {version}")
    if mode not in _MODE_NAMES:
        raise NotImplementedError(f"mode code {mode} not supported")
    if rounding not in _ROUNDING_NAMES or ndim > 8 or name_len > 65535:
        raise ValueError("corrupt record header")
    # the header is not covered by the checksum: check the word count against the shape and against
    # what is left of the file before trusting it with a read
    per = _PER_WORD[_MODE_NAMES[mode]]
    if n_words != (n_elem + per - 1) // per or n_elem != math.prod(shape8[:ndim]):
        raise ValueError("corrupt record header: element and word counts do not match the shape")
    name = _read_exact(f, name_len + _pad64(name_len), "name")[:name_len].decode("utf-8") if name_len else ""
    if f.seekable():
        here = f.tell()
        left = f.seek(0, os.SEEK_END) - here
        f.seek(here)
        if 4 * n_words > left:
            raise ValueError(f"truncated file: record {name!r} claims {4 * n_words} payload bytes, {left} remain")
    payload = _read_exact(f, 4 * n_words + _pad64(4 * n_words), "payload")[:4 * n_words]
    if zlib.crc32(payload) & 0xFFFFFFFF != crc:
        raise ValueError(f"checksum mismatch in record {name!r}")
    words = torch.from_numpy(np.frombuffer(payload, dtype="<i4").astype(np.int32)).view(torch.uint32)
    if device is not None:
        words = words.view(torch.int32).to(device).view(torch.uint32)
    t = PackedTensor(words, tuple(shape8[:ndim]), _MODE_NAMES[mode], _ROUNDING_NAMES[rounding])
    if t.n_elements != n_elem:
        raise ValueError(f"corrupt record {name!r}: shape {t.shape} does not hold {n_elem} elements")
    return name, t


def _open(file, mode: str):
    if isinstance(file, (str, os.PathLike)):
        return open(file, mode), True
    return file, False


def save_packed(file, packed: PackedTensor) -> None:
    """Write one packed tensor to ``file`` (a path or a binary file object)."""
    f, close = _open(file, "wb")
    try:
        _write_record(f, packed, "")
    finally:
        if close:
            f.close()


def load_packed(file, device=None) -> PackedTensor:
    """Read the packed tensor written by ``save_packed``; the words go to ``device`` (default: CPU)."""
    f, close = _open(file, "rb")
    try:
        rec = _read_record(f, device)
        if rec is None:
            raise ValueError("empty file")
        return rec[1]
    finally:
        if close:
            f.close()


def save_packed_dict(file, tensors: Union[Dict[str, PackedTensor], Iterable[Tuple[str, PackedTensor]]]) -> None:
    """Write named packed tensors back to back (for example every weight of a model)."""
    items = list(tensors.items()) if isinstance(tensors, dict) else list(tensors)
    names = [n for n, _ in items]
    if len(set(names)) != len(names) or any(not n for n in names):
        raise ValueError("names must be unique and non-empty")
    f, close = _open(file, "wb")
    try:
        for name, t in items:
            _write_record(f, t, name)
    finally:
        if close:
            f.close()


def load_packed_dict(file, device=None) -> Dict[str, PackedTensor]:
    """Read every record of a file written by ``save_packed_dict``."""
    f, close = _open(file, "rb")
    out: Dict[str, PackedTensor] = {}
    try:
        while True:
            rec = _read_record(f, device)
            if rec is None:
                return out
            if rec[0] in out:
                raise ValueError(f"duplicate record {rec[0]!r}")
            out[rec[0]] = rec[1]
    finally:
        if close:
            f.close()


def dumps(packed: PackedTensor) -> bytes:
    """The bytes ``save_packed`` would write."""
    b = io.BytesIO()
    save_packed(b, packed)
    return b.getvalue()
