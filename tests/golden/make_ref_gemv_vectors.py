#!/usr/bin/env python3
"""Writes tests/golden/ref_int4_gemv.json: outputs of the reference's own C kernel
(sources/ShrikeKernelsC/int4_affine_gemv.c, compiled in place into oracle/_ref by oracle/Makefile) on
seeded inputs. Run in the build container, where the reference checkout exists; the GPU box and
the CPU suite only read the JSON. Inputs are regenerated from the seed by the test; outputs are kept
as fp32 bit patterns (a CRC per case plus the first 16 words)."""
import json
import os
import sys
import zlib

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402
from shrike_amd import synth as S  # noqa: E402

CASES = [(2048, 512), (512, 2048), (128, 64), (2880, 2880), (1024, 2304), (64, 64)]


def inputs(rows, n):
    rng = S.SeedTree(0x5EED0001).key(f"golden.gemv.{rows}.{n}")
    w, s, b = S.affine_matrix(rng, rows, n, 4, S.META_BF16)
    return w, s, b, rng.normal(n).astype(np.float32)


def main():
    if O.ref_lib() is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle` where /root/reference exists")
    out = []
    for rows, n in CASES:
        w, s, b, x = inputs(rows, n)
        y = O.ref_int4_affine_gemv(w, s, b, x, rows, n).view(np.uint32)
        out.append({"rows": rows, "n": n, "crc32": zlib.crc32(y.tobytes()), "head": [int(v) for v in y[:16]]})
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_int4_gemv.json"), "w") as f:
        json.dump({"seed": "0x5EED0001", "label": "golden.gemv.<rows>.<n>", "cases": out}, f, indent=1)
    print("wrote", len(out), "cases")


if __name__ == "__main__":
    main()
