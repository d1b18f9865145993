"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

import oracle as O
from macseek_amd import quant as q

# north-star tolerance: max |gpu - ref| <= 1e-3 * ||w_row||_2 * ||x||_2
TOL_NORTH_STAR = 1e-3
# reference-style tolerance (|gpu - ref| / sum_c |w_c x_c|): the reference allows 2e-5 for its F32-activation n = 1 kernels
# (tests/test_quant_matvec.mm:42) and 2e-4 against an F32 reference when activations are staged as fp16
# (tests/test_quant_matvec_n.mm:45). At n = 1 the block formats here multiply integer payloads with activations rounded
# at 2^-16 of the largest value of their run of columns, and Q8_0 / F32 / F16 / BF16 keep fp32 activations: the
# reference's 2e-5 is asserted for every type and width.
TOL_REF_F32_X = 2e-5
TOL_REF_F16_X = 2e-4


def tol_ref(t, cols):
    return TOL_REF_F32_X


def up(a, dev="cuda:0"):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def place_in_arena(mats, first=4, gap=12, dev="cuda:0"):
    """Copies byte arrays into one device arena at 4-byte-aligned, not 16-byte-aligned, offsets (the reference tests
    do the same: tests/test_quant_moe.mm:50-56). Returns (arena tensor, [Buffer])."""
    total = first + sum(m.size + gap for m in mats) + 64
    host = np.zeros(total, dtype=np.uint8)
    offs, off = [], first
    for m in mats:
        host[off:off + m.size] = m
        offs.append(off)
        off += m.size + gap
    arena = up(host, dev)
    base = q.Buffer.of(arena)
    return arena, [base.sub(o, m.size) for o, m in zip(offs, mats)]


def matvec_errors(got, ry, mag, wn2, x, rows, cols, groups):
    xn = np.sqrt((x.astype(np.float64) ** 2).reshape(groups, cols).sum(1))
    xnr = np.repeat(xn, rows // groups)
    d = np.abs(got.astype(np.float64) - ry)
    if not np.all(np.isfinite(got)):
        return np.inf, np.inf
    return float(np.max(d / (mag + 1e-12))), float(np.max(d / (np.sqrt(wn2) * xnr + 1e-30)))


def same_floats(got, ref_bits):
    """Bit equality of float32 arrays, with any NaN equal to any NaN: the reference's own bit-exactness test treats
    NaN == NaN (tests/test_quant_ref.mm:40-53); hardware conversions quiet a signalling NaN, software ones do not."""
    g = np.ascontiguousarray(got, dtype=np.float32)
    r = np.ascontiguousarray(ref_bits).view(np.float32)
    both_nan = np.isnan(g) & np.isnan(r)
    return bool(np.all((g.view(np.uint32) == r.view(np.uint32)) | both_nan))
