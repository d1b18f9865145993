"""ctypes binding of the CPU oracle (oracle.c). TEST INFRASTRUCTURE ONLY: the product never imports this.

`load()` returns the built liboracle.so (building it with `make` when it is missing); `load_ref()` returns the
reference's own dequant.cpp compiled under oracle/_ref, or None where that does not exist (e.g. on the GPU box).
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

F32, F16, Q8_0, Q5_K, Q6_K, IQ2_XXS, IQ1_S, IQ4_NL, BF16 = 0, 1, 8, 13, 14, 16, 19, 20, 30
TYPE_NAMES = {F32: "F32", F16: "F16", Q8_0: "Q8_0", Q5_K: "Q5_K", Q6_K: "Q6_K", IQ2_XXS: "IQ2_XXS", IQ1_S: "IQ1_S",
              IQ4_NL: "IQ4_NL", BF16: "BF16"}
ALL_TYPES = (Q8_0, Q5_K, Q6_K, IQ2_XXS, IQ1_S, IQ4_NL, BF16, F16, F32)

_lib = None
_ref = None


def build(force=False):
    so = os.path.join(HERE, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", HERE, "liboracle.so"] + (["-B"] if force else []))
    return so


def load():
    global _lib
    if _lib is not None:
        return _lib
    L = C.CDLL(build())
    vp, i32, i64, u64, f32 = C.c_void_p, C.c_int, C.c_int64, C.c_uint64, C.c_float
    L.orc_block_elems.argtypes = [i32]; L.orc_block_elems.restype = i32
    L.orc_block_bytes.argtypes = [i32]; L.orc_block_bytes.restype = C.c_size_t
    L.orc_row_bytes.argtypes = [i32, i64]; L.orc_row_bytes.restype = C.c_size_t
    L.orc_fp16_to_f32.argtypes = [C.c_uint16]; L.orc_fp16_to_f32.restype = f32
    L.orc_f32_to_fp16.argtypes = [f32]; L.orc_f32_to_fp16.restype = C.c_uint16
    L.orc_bf16_to_f32.argtypes = [C.c_uint16]; L.orc_bf16_to_f32.restype = f32
    L.orc_f32_to_bf16.argtypes = [f32]; L.orc_f32_to_bf16.restype = C.c_uint16
    L.orc_iq1s_entry.argtypes = [i32, vp]; L.orc_iq2xxs_entry.argtypes = [i32, vp]
    L.orc_ksign.argtypes = [i32]; L.orc_ksign.restype = C.c_uint8
    L.orc_dequant_row.argtypes = [i32, vp, vp, i64]; L.orc_dequant_row.restype = i32
    L.orc_matvec.argtypes = [i32, vp, i32, i32, vp, i32, vp, vp, vp, i32]; L.orc_matvec.restype = i32
    L.orc_swiglu.argtypes = [C.c_double] * 3; L.orc_swiglu.restype = C.c_double
    L.orc_moe_decode.argtypes = [i32] * 7 + [vp] * 9 + [i32]; L.orc_moe_decode.restype = i32
    L.orc_moe_prefill.argtypes = [i32] * 8 + [vp] * 8 + [i32, i32, vp, vp, i32]; L.orc_moe_prefill.restype = i32
    L.orc_randn.argtypes = [vp, i64, u64, f32]
    L.orc_random_blocks.argtypes = [i32, i64, u64, f32, vp]; L.orc_random_blocks.restype = i32
    L.orc_router.argtypes = [vp, vp, i32, i32, f32, vp, vp]; L.orc_router.restype = None
    L.orc_rmsnorm.argtypes = [vp, vp, vp, i32, C.c_double]; L.orc_rmsnorm.restype = None
    L.orc_route_lists.argtypes = [vp, vp, i32, i32, i32] + [vp] * 6; L.orc_route_lists.restype = None
    _lib = L
    return L


def load_ref():
    """The reference's tests/ref/dequant.cpp as a shared object, or None when it was not built here."""
    global _ref
    if _ref is None:
        so = os.path.join(HERE, "_ref", "libref_dequant.so")
        if not os.path.exists(so):
            return None
        R = C.CDLL(so)
        R.refshim_dequant_row.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_longlong]
        R.refshim_matvec.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        R.refshim_f32_to_fp16.argtypes = [C.c_float]; R.refshim_f32_to_fp16.restype = C.c_ushort
        R.refshim_fp16_to_f32.argtypes = [C.c_ushort]; R.refshim_fp16_to_f32.restype = C.c_float
        _ref = R
    return _ref


_ref_arch = None


def load_ref_arch():
    """The reference's tests/ref/arch_ref.cpp (router, route lists) as a shared object, or None when not built here."""
    global _ref_arch
    if _ref_arch is None:
        so = os.path.join(HERE, "_ref", "libref_arch.so")
        if not os.path.exists(so):
            return None
        R = C.CDLL(so)
        R.refshim_router.argtypes = [C.c_void_p] * 4 + [C.c_float]; R.refshim_router.restype = None
        R.refshim_route_lists.argtypes = [C.c_void_p, C.c_void_p, C.c_int] + [C.c_void_p] * 6
        R.refshim_route_lists.restype = None
        R.refshim_rmsnorm.argtypes = [C.c_void_p] * 3 + [C.c_int, C.c_double]; R.refshim_rmsnorm.restype = None
        _ref_arch = R
    return _ref_arch


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def block_elems(t):
    return load().orc_block_elems(t)


def block_bytes(t):
    return load().orc_block_bytes(t)


def row_bytes(t, cols):
    return load().orc_row_bytes(t, cols)


def random_blocks(t, n_elems, seed, scale=0.01):
    """uint8 array of n_elems/block_elems blocks: random bytes with sane fp16 scales."""
    out = np.empty(row_bytes(t, n_elems), dtype=np.uint8)
    if load().orc_random_blocks(t, n_elems, seed, scale, _p(out)) != 0:
        raise ValueError("random_blocks: bad type/size")
    return out


def randn(n, seed, scale=1.0):
    out = np.empty(int(n), dtype=np.float32)
    load().orc_randn(_p(out), int(n), seed, scale)
    return out


def dequant(t, blocks, n_elems):
    """float32[n_elems] from raw block bytes."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    assert blocks.size >= row_bytes(t, n_elems)
    out = np.empty(int(n_elems), dtype=np.float32)
    if load().orc_dequant_row(t, _p(blocks), _p(out), int(n_elems)) != 0:
        raise ValueError("dequant: unknown type %d" % t)
    return out


def ref_dequant(t, blocks, n_elems):
    R = load_ref()
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    out = np.empty(int(n_elems), dtype=np.float32)
    R.refshim_dequant_row(t, _p(blocks), _p(out), int(n_elems))
    return out


def matvec(t, W, rows, cols, x, groups=1, nthreads=8):
    """Returns (y, mag, wn2): float64 dot, sum|w x| and sum w^2 per row."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.size >= cols * groups and W.size >= row_bytes(t, cols) * rows
    y = np.empty(rows); mag = np.empty(rows); wn2 = np.empty(rows)
    if load().orc_matvec(t, _p(W), rows, cols, _p(x), groups, _p(y), _p(mag), _p(wn2), nthreads) != 0:
        raise ValueError("matvec: unsupported arguments")
    return y, mag, wn2


def swiglu(g, u, w):
    return load().orc_swiglu(float(g), float(u), float(w))


def _ptr_array(mats):
    arr = (C.c_void_p * len(mats))()
    for i, m in enumerate(mats):
        arr[i] = m.ctypes.data
    return arr


def moe_decode(t_gu, t_down, t_shared, n_routed, has_shared, dim, inter, gate, up, down, wts, x, y0, nthreads=8):
    """gate/up/down: lists of uint8 arrays, length n_routed (+1 with the shared expert last).
    Returns (y, ymag, h, hscale)."""
    ne = n_routed + (1 if has_shared else 0)
    assert len(gate) == len(up) == len(down) == ne
    y = np.array(y0, dtype=np.float64)
    ymag = np.empty(dim)
    h = np.zeros((n_routed + 1) * inter, dtype=np.float32)
    hs = np.zeros((n_routed + 1) * inter)
    wts = np.ascontiguousarray(wts, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    rc = load().orc_moe_decode(t_gu, t_down, t_shared, n_routed, int(has_shared), dim, inter,
                               C.cast(_ptr_array(gate), C.c_void_p), C.cast(_ptr_array(up), C.c_void_p),
                               C.cast(_ptr_array(down), C.c_void_p), _p(wts), _p(x), _p(y), _p(ymag), _p(h), _p(hs),
                               nthreads)
    if rc != 0:
        raise ValueError("moe_decode: unsupported arguments")
    return y, ymag, h, hs


def moe_prefill(t_gu, t_down, t_shared, n_tokens, n_exp, has_shared, dim, inter, gate, up, down, offs, tok, wt, X,
                chk, x_round, Y0, nthreads=8):
    """Reference Y (float64 [len(chk), dim]) and error scale for the checked tokens. Y0: float32 [n_tokens, dim]."""
    offs = np.ascontiguousarray(offs, dtype=np.int32); tok = np.ascontiguousarray(tok, dtype=np.int32)
    wt = np.ascontiguousarray(wt, dtype=np.float32); X = np.ascontiguousarray(X, dtype=np.float32)
    chk = np.ascontiguousarray(chk, dtype=np.int32)
    Y = np.ascontiguousarray(np.asarray(Y0, dtype=np.float64).reshape(n_tokens, dim)[chk])
    Ymag = np.abs(Y)
    rc = load().orc_moe_prefill(t_gu, t_down, t_shared, n_tokens, n_exp, int(has_shared), dim, inter,
                                C.cast(_ptr_array(gate), C.c_void_p), C.cast(_ptr_array(up), C.c_void_p),
                                C.cast(_ptr_array(down), C.c_void_p), _p(offs), _p(tok), _p(wt), _p(X), _p(chk),
                                len(chk), x_round, _p(Y), _p(Ymag), nthreads)
    if rc != 0:
        raise ValueError("moe_prefill: unsupported arguments")
    return Y, Ymag


N_EXPERTS, TOP_K, ROUTE_SCALE = 384, 6, 1.5  # the reference's router constants (src/kernels/arch_router.metal:5-6,53)


def router(logits, bias, top_k=TOP_K, route_scale=ROUTE_SCALE):
    """logits float32 [n, n_exp], bias float32 [n_exp] -> ids int32 [n, top_k], w float32 [n, top_k]."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    n, n_exp = logits.shape
    ids = np.empty((n, top_k), dtype=np.int32)
    w = np.empty((n, top_k), dtype=np.float32)
    L = load()
    for t in range(n):
        L.orc_router(_p(logits[t]), _p(bias), n_exp, top_k, route_scale, _p(ids[t]), _p(w[t]))
    return ids, w


def ref_router(logits, bias, route_scale=ROUTE_SCALE):
    R = load_ref_arch()
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    n = logits.shape[0]
    ids = np.empty((n, 6), dtype=np.int32)
    w = np.empty((n, 6), dtype=np.float32)
    for t in range(n):
        R.refshim_router(_p(logits[t]), _p(bias), _p(ids[t]), _p(w[t]), route_scale)
    return ids, w


def _route_outputs(n_entries, n_exp):
    return (np.empty(n_exp, np.uint32), np.empty(n_exp + 1, np.uint32), np.empty(n_entries, np.uint32),
            np.empty(n_entries, np.uint32), np.empty(n_entries, np.float32), np.empty(n_entries, np.uint32))


def route_lists(ids, w, n_exp=N_EXPERTS, top_k=TOP_K):
    """ids int32 / w float32 [n_tokens * top_k] -> (counts, offsets, entry, tok, lw, slot_of)."""
    ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    out = _route_outputs(ids.size, n_exp)
    load().orc_route_lists(_p(ids), _p(w), ids.size, n_exp, top_k, *[_p(o) for o in out])
    return out


def ref_route_lists(ids, w):
    ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    out = _route_outputs(ids.size, 384)
    load_ref_arch().refshim_route_lists(_p(ids), _p(w), ids.size // 6, *[_p(o) for o in out])
    return out


def rmsnorm(x, w, eps):
    """float32[dim]: x * rsqrt(mean(x^2) + eps) * w in double, rounded once (w may be None)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = None if w is None else np.ascontiguousarray(w, dtype=np.float32)
    y = np.empty_like(x)
    load().orc_rmsnorm(_p(x), _p(w) if w is not None else None, _p(y), x.size, float(eps))
    return y


def ref_rmsnorm(x, w, eps):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = None if w is None else np.ascontiguousarray(w, dtype=np.float32)
    y = np.empty_like(x)
    load_ref_arch().refshim_rmsnorm(_p(x), _p(w) if w is not None else None, _p(y), x.size, float(eps))
    return y
