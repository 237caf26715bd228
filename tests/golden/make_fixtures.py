"""Writes the golden fixtures of this directory.  Run from the repository root:

    python tests/golden/make_fixtures.py

Nothing here imports the reference (it needs ml_dtypes, numba and Python 3.11,
none of which this image has).  The vectors come from sources independent of
both the oracle and the HIP kernels:

* ``fp8_tables.npz``
    - ``enc_e5m2`` / ``enc_e4m3``: uint8[65536], torch-CPU casts
      ``x.to(torch.float8_e5m2 / float8_e4m3fn)`` of every fp16 bit pattern
      (the same round-to-nearest-even, overflow-to-inf / overflow-to-NaN rules
      as the ml_dtypes casts the reference packer calls, fp8.py:109-120);
    - ``dec_e5m2_ieee`` / ``dec_e4m3_ieee``: float32[256], torch-CPU widening of
      every code (what the reference's CPU unpack returns, fp8.py:381-391);
    - ``dec_e4m3_kernel_bits``: uint16[256], the reference kernel's formula
      (gemv.py:83-88) evaluated with plain Python integers.
* ``kats.json``: the known answers printed in the reference's docstrings.
"""
import json
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def main() -> None:
    h = np.arange(65536, dtype=np.uint16)
    x = torch.from_numpy(h.view(np.float16).copy())
    enc5 = x.to(torch.float8_e5m2).view(torch.uint8).numpy()
    enc4 = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    c = torch.arange(256, dtype=torch.uint8)
    dec5 = c.view(torch.float8_e5m2).to(torch.float32).numpy()
    dec4 = c.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    kern = []
    for code in range(256):
        e = (code & 0x78) >> 3
        kern.append(((code & 0x80) << 8) | (((e + 8) * (1 if e > 0 else 0)) << 10) | ((code & 0x07) << 7))
    np.savez_compressed(os.path.join(HERE, "fp8_tables.npz"), enc_e5m2=enc5, enc_e4m3=enc4, dec_e5m2_ieee=dec5,
                        dec_e4m3_ieee=dec4, dec_e4m3_kernel_bits=np.array(kern, dtype=np.uint16))

    kats = {
        "gemv": {  # feather/routines/gemv.py:163-174 (E5M2) and :214-225 (same numbers through the E4M3 kernel)
            "source": "feather/routines/gemv.py:163-174,214-225",
            "matrix": [[1, 1, -2, 0], [-3, -3, -2, -3], [0, 1, 1, -2], [2, 0, -1, 2]],
            "vector": [2, 2, -1, 2],
            "expected": [6, -16, -3, 9],
        },
        "dot_fp8_e5m2": {  # feather/routines/dot.py:244-251
            "source": "feather/routines/dot.py:244-251",
            "x1": [2, 0, -3, 1], "x2": [-1, 0, -3, 1], "expected": 8,
        },
        "dot_fp16": {  # feather/routines/dot.py:35-42 and :83-92
            "source": "feather/routines/dot.py:35-42,83-92",
            "x1": [-3, -3, -3, 1], "x2": [-3, 1, 2, -1], "expected": -1,
        },
        # the 16 E4M3 codes on which the kernel decode (gemv.py:83-88) and the CPU unpack
        # (fp8.py:381-391) disagree: zero exponent field with a non-zero mantissa, and the NaN code
        "e4m3_decode_exceptions": [1, 2, 3, 4, 5, 6, 7, 127, 129, 130, 131, 132, 133, 134, 135, 255],
    }
    with open(os.path.join(HERE, "kats.json"), "w") as f:
        json.dump(kats, f, indent=1)
    print("wrote fp8_tables.npz, kats.json")


if __name__ == "__main__":
    main()
