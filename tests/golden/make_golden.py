#!/usr/bin/env python3
"""Writes tests/golden/dequant_golden.npz from the reference's own CPU dequantizer.

Runs only in the build container: it needs oracle/_ref/libref_dequant.so, which `make -C oracle ref` compiles from
/root/reference/tests/ref/dequant.cpp where it lies. The fixture holds DATA only: block bytes (inputs) and the float
bit patterns / matvec results the reference produced for them (expected outputs).

Per type T (name as in type_name()):
  sane_blocks_T / sane_bits_T   blocks from the oracle's seeded generator (sane fp16 scales), 1024 elements
  raw_blocks_T  / raw_bits_T    uniformly random bytes (scales may be NaN/Inf/denormal), 1024 elements
  mv_W_T, mv_x, mv_y_T          ref::matvec_ref on an 8 x 512 matrix of sane blocks (float32 result of a double dot)
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as O  # noqa: E402


def main():
    R = O.load_ref()
    if R is None:
        raise SystemExit("oracle/_ref/libref_dequant.so is missing: run `make -C oracle ref` in the build container")
    out = {}
    rng = np.random.default_rng(20240607)
    n = 1024
    x = O.randn(512, 4242)
    out["mv_x"] = x
    for t in O.ALL_TYPES:
        name = O.TYPE_NAMES[t]
        sane = O.random_blocks(t, n, 1000 + t, 0.01)
        raw = rng.integers(0, 256, O.row_bytes(t, n), dtype=np.uint8)
        out["sane_blocks_" + name] = sane
        out["sane_bits_" + name] = O.ref_dequant(t, sane, n).view(np.uint32)
        out["raw_blocks_" + name] = raw
        out["raw_bits_" + name] = O.ref_dequant(t, raw, n).view(np.uint32)
        W = O.random_blocks(t, 8 * 512, 2000 + t, 0.01)
        y = np.empty(8, dtype=np.float32)
        R.refshim_matvec(t, W.ctypes.data, 8, 512, x.ctypes.data, y.ctypes.data)
        out["mv_W_" + name] = W
        out["mv_y_" + name] = y
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dequant_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
