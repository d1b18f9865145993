#!/usr/bin/env python3
"""Writes tests/golden/router_golden.npz from the reference's own CPU router twin.

Runs only in the build container: it needs oracle/_ref/libref_arch.so, which `make -C oracle ref` compiles from
/root/reference/tests/ref/arch_ref.cpp where it lies. The fixture holds DATA only: seeded logits / bias (inputs, built
like the reference's test does, tests/test_arch_router.mm:62-66: N(0, 3) logits with some pushed through the
softplus-threshold branch and some to -25) and what ref_arch::router / ref_arch::route_lists returned for them.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as O  # noqa: E402


def main():
    if O.load_ref_arch() is None:
        raise SystemExit("oracle/_ref/libref_arch.so is missing: run `make -C oracle ref` in the build container")
    n = 96
    logits = O.randn(n * 384, 777, 3.0)
    logits[::97] = 30.0 + O.randn(len(logits[::97]), 778)
    logits[5::89] = -25.0
    logits = logits.reshape(n, 384)
    logits[7, :] = 0.25      # all keys tie apart from the bias
    logits[8, 10:20] = 4.0   # ten-way tie at the top
    bias = O.randn(384, 779, 0.3)
    bias[100:104] = bias[100]  # equal biases inside the tie rows
    ids, w = O.ref_router(logits, bias)
    counts, offsets, entry, tok, lw, slot_of = O.ref_route_lists(ids, w)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "router_golden.npz")
    np.savez_compressed(path, logits=logits, bias=bias, ids=ids, w_bits=w.view(np.uint32), counts=counts, offsets=offsets,
                        entry=entry, tok=tok, lw_bits=lw.view(np.uint32), slot_of=slot_of)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
