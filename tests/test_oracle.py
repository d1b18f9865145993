"""Pins the CPU oracle (oracle/oracle.c): golden vectors written from the reference's own dequant.cpp, closed-form
known answers per block format, codebook invariants, numpy float64 dots and brute-force MoE compositions."""
import os

import numpy as np
import pytest

import oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "dequant_golden.npz"))
BLOCK_TYPES = (O.Q8_0, O.Q5_K, O.Q6_K, O.IQ2_XXS, O.IQ1_S, O.IQ4_NL)


def f16(v):
    return np.float16(v).view(np.uint16).item()


def put16(buf, off, h):
    buf[off] = h & 0xFF
    buf[off + 1] = h >> 8


# ---------------------------------------------------------------- golden vectors (reference dequant.cpp outputs)
@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("kind", ["sane", "raw"])
def test_dequant_matches_reference_golden(t, kind):
    name = O.TYPE_NAMES[t]
    got = O.dequant(t, GOLD[f"{kind}_blocks_{name}"], 1024).view(np.uint32)
    assert np.array_equal(got, GOLD[f"{kind}_bits_{name}"])


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_matvec_matches_reference_golden(t):
    name = O.TYPE_NAMES[t]
    y, _, _ = O.matvec(t, GOLD["mv_W_" + name], 8, 512, GOLD["mv_x"])
    assert np.array_equal(y.astype(np.float32), GOLD["mv_y_" + name])  # same double dot, same final rounding


@pytest.mark.skipif(O.load_ref() is None, reason="reference checker not built here (oracle/_ref)")
@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_dequant_differential_vs_compiled_reference(t):
    rng = np.random.default_rng(t)
    n = 256 * 256
    for blocks in (O.random_blocks(t, n, 77 + t), rng.integers(0, 256, O.row_bytes(t, n), dtype=np.uint8)):
        assert np.array_equal(O.dequant(t, blocks, n).view(np.uint32), O.ref_dequant(t, blocks, n).view(np.uint32))


# ---------------------------------------------------------------- geometry (quant_types.hpp:13-34)
def test_geometry():
    expect = {O.F32: (1, 4), O.F16: (1, 2), O.BF16: (1, 2), O.Q8_0: (32, 34), O.Q5_K: (256, 176), O.Q6_K: (256, 210),
              O.IQ2_XXS: (256, 66), O.IQ1_S: (256, 50), O.IQ4_NL: (32, 18)}
    for t, (be, bb) in expect.items():
        assert O.block_elems(t) == be and O.block_bytes(t) == bb
    assert O.row_bytes(O.IQ1_S, 7168) == 1400 and O.row_bytes(O.IQ2_XXS, 7168) == 1848
    assert O.row_bytes(O.Q6_K, 7168) == 5880 and O.row_bytes(O.Q8_0, 4096) == 4352
    assert O.row_bytes(O.IQ1_S, 7168) * 4096 == 5734400 and O.row_bytes(O.IQ2_XXS, 7168) * 4096 == 7569408


# ---------------------------------------------------------------- scalar conversions
def test_fp16_conversions_match_numpy():
    L = O.load()
    allh = np.arange(65536, dtype=np.uint16)
    mine = np.array([L.orc_fp16_to_f32(int(h)) for h in allh], dtype=np.float32)
    ref = allh.view(np.float16).astype(np.float32)
    assert np.array_equal(mine.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.all(np.isnan(mine[np.isnan(ref)]))
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(3000).astype(np.float32) * s for s in (1e-8, 1e-6, 1e-4, 1, 300, 70000)])
    xs = np.concatenate([xs, np.array([65504, 65519.9, 65520, 1e-7, 5.96e-8, 2.9802322e-8, 2.98e-8, 0, -0.0, np.inf,
                                       -np.inf, 6.1035156e-05, 6.0975552e-05], dtype=np.float32)])
    with np.errstate(over="ignore"):
        ref16 = xs.astype(np.float16).view(np.uint16)
    assert np.array_equal(np.array([L.orc_f32_to_fp16(float(v)) for v in xs], dtype=np.uint16), ref16)
    # bf16: truncation-with-RNE closed form
    bits = xs.view(np.uint32).astype(np.uint64)
    rne = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    fin = np.isfinite(xs)
    assert np.array_equal(np.array([L.orc_f32_to_bf16(float(v)) for v in xs[fin]], dtype=np.uint16), rne[fin])


# ---------------------------------------------------------------- codebook invariants
def test_codebook_invariants():
    L = O.load()
    e1 = np.zeros((2048, 8), dtype=np.int8)
    for i in range(2048):
        L.orc_iq1s_entry(i, e1[i].ctypes.data)
    assert set(np.unique(e1)) == {-1, 0, 1}
    assert len({tuple(r) for r in e1}) == 2048
    # entries are sorted when element 0 is the least significant base-3 digit
    key = ((e1.astype(np.int64) + 1) * (3 ** np.arange(8))).sum(1)
    assert np.all(np.diff(key) > 0)
    assert tuple(e1[0]) == (-1,) * 8 and tuple(e1[2047]) == (1,) * 8
    e2 = np.zeros((256, 8), dtype=np.uint8)
    for i in range(256):
        L.orc_iq2xxs_entry(i, e2[i].ctypes.data)
    assert set(np.unique(e2)) == {8, 25, 43}
    assert len({tuple(r) for r in e2}) == 256
    assert tuple(e2[0]) == (8,) * 8
    # the grid is a subset of an E8-like lattice: the ranks {0,1,2} of the 8 elements sum to an even number
    rank = np.searchsorted(np.array([8, 25, 43]), e2)
    assert np.all(rank.sum(1) % 2 == 0)
    for i in range(128):
        assert L.orc_ksign(i) == (i | ((bin(i).count("1") & 1) << 7))
        assert bin(L.orc_ksign(i)).count("1") % 2 == 0  # sign bytes always flip an even number of elements


# ---------------------------------------------------------------- closed-form known answers per format
def test_q8_0_known_answer():
    b = np.zeros(34, dtype=np.uint8)
    put16(b, 0, f16(1.0))
    b[2:34] = (np.arange(32) - 16).astype(np.int8).view(np.uint8)
    assert np.array_equal(O.dequant(O.Q8_0, b, 32), (np.arange(32) - 16).astype(np.float32))
    put16(b, 0, f16(0.5))
    assert np.array_equal(O.dequant(O.Q8_0, b, 32), 0.5 * (np.arange(32) - 16).astype(np.float32))


def test_iq4_nl_known_answer():
    kv = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)
    b = np.zeros(18, dtype=np.uint8)
    put16(b, 0, f16(2.0))
    b[2:18] = np.arange(16) | ((15 - np.arange(16)) << 4)  # low nibble j, high nibble 15-j
    y = O.dequant(O.IQ4_NL, b, 32)
    assert np.array_equal(y[:16], 2 * kv) and np.array_equal(y[16:], 2 * kv[::-1])


def test_iq1_s_known_answers():
    b = np.zeros(50, dtype=np.uint8)
    put16(b, 0, f16(1.0))
    # all-zero qs/qh: grid[0] = all -1, scale 2*0+1, delta +0.125 -> -0.875
    assert np.array_equal(O.dequant(O.IQ1_S, b, 256), np.full(256, -0.875, np.float32))
    # qh = 0xF000 in sub-block 3: scale 2*7+1 = 15, delta -0.125 -> 15 * (-1.125)
    put16(b, 34 + 2 * 3, 0xF000)
    y = O.dequant(O.IQ1_S, b, 256)
    assert np.all(y[96:128] == np.float32(15 * -1.125)) and np.all(y[:96] == np.float32(-0.875))
    # index 2047 (qs = 0xFF, high bits 7) = all +1 for group l = 2 of sub-block 0
    b[2 + 2] = 0xFF
    put16(b, 34, 7 << 6)
    y = O.dequant(O.IQ1_S, b, 256)
    assert np.all(y[16:24] == np.float32(1.125)) and np.all(y[:16] == np.float32(-0.875))


def test_iq2_xxs_known_answers():
    b = np.zeros(66, dtype=np.uint8)
    put16(b, 0, f16(1.0))
    # all-zero qs: grid[0] = all 8, db = (0.5 + 0) * 0.25 = 1/8, no signs -> 1.0
    assert np.array_equal(O.dequant(O.IQ2_XXS, b, 256), np.ones(256, np.float32))
    # sub-block 1: scale nibble 15, sign index 1 for group 0 -> element 0 and 7 (parity) negative
    a1 = (15 << 28) | 1
    b[2 + 8 + 4:2 + 8 + 8] = np.frombuffer(np.uint32(a1).tobytes(), dtype=np.uint8)
    y = O.dequant(O.IQ2_XXS, b, 256)
    v = np.float32(15.5 * 0.25 * 8)
    assert np.array_equal(y[32:40], np.array([-v, v, v, v, v, v, v, -v], np.float32))
    assert np.all(y[40:64] == v) and np.all(y[:32] == 1)


def test_q6_k_known_answers():
    b = np.zeros(210, dtype=np.uint8)
    put16(b, 208, f16(0.5))
    b[192:208] = (np.arange(16) - 8).astype(np.int8).view(np.uint8)  # scales -8..7
    # all-zero ql/qh: q = -32, y = d * sc * -32; scale of element e: half h = e // 128, run k, 16-group is
    y = O.dequant(O.Q6_K, b, 256)
    e = np.arange(256)
    h, rem = e // 128, e % 128
    sc = (8 * h + (rem % 32) // 16 + 2 * (rem // 32)) - 8
    assert np.array_equal(y, (0.5 * sc * -32).astype(np.float32))
    # element 5: low nibble of ql[5] = 9, qh[5] bits 0-1 = 2 -> q = (9 | 2 << 4) - 32 = 9
    b[5] = 0x09
    b[128 + 5] = 0x02
    y = O.dequant(O.Q6_K, b, 256)
    assert y[5] == np.float32(0.5 * -8 * 9)
    # element 128 + 96 + 3: high nibble of ql[64 + 32 + 3], qh[32 + 3] bits 6-7
    b[64 + 32 + 3] = 0xF0
    b[128 + 32 + 3] = 0xC0
    y = O.dequant(O.Q6_K, b, 256)
    assert y[128 + 96 + 3] == np.float32(0.5 * (8 + 6 - 8) * (63 - 32))


def test_q5_k_known_answers():
    b = np.zeros(176, dtype=np.uint8)
    put16(b, 0, f16(2.0))
    put16(b, 2, f16(0.5))
    # 6-bit scales sc[is] = is + 1, mins m[is] = 10 + is, packed as scale_min_k4 expects
    sc = np.arange(8) + 1
    mn = np.arange(8) + 10
    q = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        q[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        q[j + 4] = mn[j] | ((mn[j + 4] >> 4) << 6)
        q[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    b[4:16] = q
    y = O.dequant(O.Q5_K, b, 256)  # all quants zero: y = -dmin * m
    assert np.array_equal(y, np.repeat(-0.5 * mn, 32).astype(np.float32))
    # element 70 (group 1, first half, l = 6): low nibble 11, high bit set (qh bit 2) -> q = 27, scale index 2
    b[48 + 32 + 6] = 0x0B
    b[16 + 6] = 1 << 2
    y = O.dequant(O.Q5_K, b, 256)
    assert y[70] == np.float32(np.float32(2.0 * 3) * 27 - np.float32(0.5 * 12))
    # element 64*3 + 32 + 1 (group 3, second half): high nibble 5, qh bit 7 -> q = 21, scale index 7
    b[48 + 96 + 1] = 0x50
    b[16 + 1] = 1 << 7
    y = O.dequant(O.Q5_K, b, 256)
    assert y[64 * 3 + 32 + 1] == np.float32(np.float32(2.0 * 8) * 21 - np.float32(0.5 * 17))


def test_dense_known_answers():
    v = np.array([1.5, -2.25, 0.0, 65504, 1e-3, -7, 3, 0.333], dtype=np.float32)
    assert np.array_equal(O.dequant(O.F32, v.view(np.uint8), 8), v)
    assert np.array_equal(O.dequant(O.F16, v.astype(np.float16).view(np.uint8), 8), v.astype(np.float16).astype(np.float32))
    bf = (v.view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(O.dequant(O.BF16, bf.view(np.uint8), 8), (bf.astype(np.uint32) << 16).view(np.float32))


# ---------------------------------------------------------------- matvec against numpy float64
@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_matvec_is_a_float64_dot(t):
    rows, cols, groups = 12, 512, 3
    W = O.random_blocks(t, rows * cols, 5 + t)
    x = O.randn(cols * groups, 6)
    y, mag, wn2 = O.matvec(t, W, rows, cols, x, groups, nthreads=3)
    w = O.dequant(t, W, rows * cols).reshape(rows, cols).astype(np.float64)
    xs = x.astype(np.float64).reshape(groups, cols)[np.arange(rows) // (rows // groups)]
    assert np.allclose(y, (w * xs).sum(1), rtol=1e-12, atol=1e-300)
    assert np.allclose(mag, np.abs(w * xs).sum(1), rtol=1e-12)
    assert np.allclose(wn2, (w * w).sum(1), rtol=1e-12)
    y1, _, _ = O.matvec(t, W, rows, cols, x, groups, nthreads=1)
    assert np.array_equal(y, y1)  # threading only splits rows


def test_matvec_rejects_bad_shapes():
    W = np.zeros(4096, dtype=np.uint8)
    x = np.zeros(512, dtype=np.float32)
    with pytest.raises(ValueError):
        O.matvec(O.Q6_K, W, 4, 128, x)  # cols not a multiple of the block
    with pytest.raises(ValueError):
        O.matvec(O.Q8_0, W, 5, 64, x, groups=2)  # rows % groups


# ---------------------------------------------------------------- SwiGLU closed form and clamps
def test_swiglu():
    assert O.swiglu(0.0, 5.0, 1.0) == 0.0
    assert O.swiglu(2.0, 3.0, 0.5) == pytest.approx(2.0 / (1 + np.exp(-2.0)) * 3.0 * 0.5, rel=1e-15)
    assert O.swiglu(50.0, 50.0, 1.0) == pytest.approx(10.0 / (1 + np.exp(-10.0)) * 10.0, rel=1e-15)  # both clamps
    assert O.swiglu(1.0, -50.0, 2.0) == pytest.approx(1.0 / (1 + np.exp(-1.0)) * -10.0 * 2.0, rel=1e-15)
    assert O.swiglu(-30.0, 1.0, 1.0) == pytest.approx(-30.0 / (1 + np.exp(30.0)), rel=1e-12)  # gate has no lower clamp


# ---------------------------------------------------------------- MoE decode = composition of the pieces
def _np_swiglu(g, u, w):
    g = np.minimum(g, 10.0)
    u = np.clip(u, -10.0, 10.0)
    return g / (1 + np.exp(-g)) * u * w


@pytest.mark.parametrize("n_routed,has_shared", [(3, True), (2, False), (0, True)])
def test_moe_decode_composition(n_routed, has_shared):
    dim, inter = 512, 256
    tgu, td, ts = O.IQ1_S, O.IQ2_XXS, O.Q6_K
    ne = n_routed + int(has_shared)
    types = [(tgu, td)] * n_routed + ([(ts, ts)] if has_shared else [])
    G = [O.random_blocks(types[e][0], inter * dim, 10 + 3 * e, 0.05) for e in range(ne)]
    U = [O.random_blocks(types[e][0], inter * dim, 11 + 3 * e, 0.05) for e in range(ne)]
    D = [O.random_blocks(types[e][1], inter * dim, 12 + 3 * e, 0.05) for e in range(ne)]
    wts = np.array([0.4, 0.35, 0.25], dtype=np.float32)
    x = O.randn(dim, 1, 3.0)
    y0 = O.randn(dim, 2)
    y, ymag, h, hs = O.moe_decode(tgu, td, ts, n_routed, has_shared, dim, inter, G, U, D, wts, x, y0, nthreads=2)
    ref = y0.astype(np.float64)
    for e in range(ne):
        wg = O.dequant(types[e][0], G[e], inter * dim).reshape(inter, dim).astype(np.float64)
        wu = O.dequant(types[e][0], U[e], inter * dim).reshape(inter, dim).astype(np.float64)
        wd = O.dequant(types[e][1], D[e], inter * dim).reshape(dim, inter).astype(np.float64)
        we = 1.0 if e == n_routed else float(wts[e])
        he = _np_swiglu(wg @ x.astype(np.float64), wu @ x.astype(np.float64), we).astype(np.float32)
        assert np.allclose(h[e * inter:(e + 1) * inter], he, rtol=1e-6, atol=1e-30)
        ref += wd @ he.astype(np.float64)
    assert np.allclose(y, ref, rtol=1e-10, atol=1e-12)
    assert np.all(ymag >= np.abs(y) - 1e-9)


def test_moe_prefill_composition():
    dim, inter, n, k, ne = 256, 256, 7, 2, 3
    tgu, td, ts = O.IQ2_XXS, O.IQ1_S, O.Q8_0
    types = [(tgu, td)] * ne + [(ts, ts)]
    G = [O.random_blocks(types[e][0], inter * dim, 20 + 3 * e, 0.05) for e in range(ne + 1)]
    U = [O.random_blocks(types[e][0], inter * dim, 21 + 3 * e, 0.05) for e in range(ne + 1)]
    D = [O.random_blocks(types[e][1], inter * dim, 22 + 3 * e, 0.05) for e in range(ne + 1)]
    # token t routes to experts (t % 3, (t + 1) % 3); expert-sorted lists
    rt = [[t % 3, (t + 1) % 3] for t in range(n)]
    rw = [[0.6, 0.4] for _ in range(n)]
    offs, tok, wt = [0], [], []
    for j in range(ne):
        for t in range(n):
            for kk in range(k):
                if rt[t][kk] == j:
                    tok.append(t); wt.append(rw[t][kk])
        offs.append(len(tok))
    X = O.randn(n * dim, 3).reshape(n, dim)
    Y0 = O.randn(n * dim, 4).reshape(n, dim)
    chk = [0, 3, 6]
    Y, Ymag = O.moe_prefill(tgu, td, ts, n, ne, True, dim, inter, G, U, D, offs, tok, wt, X, chk, 0, Y0, nthreads=2)
    deq = lambda t, b, r, c: O.dequant(t, b, r * c).reshape(r, c).astype(np.float64)
    for qi, t in enumerate(chk):
        ref = Y0[t].astype(np.float64)
        xt = X[t].astype(np.float64)
        for j, w in list(zip(rt[t], rw[t])) + [(ne, 1.0)]:
            hj = _np_swiglu(deq(types[j][0], G[j], inter, dim) @ xt, deq(types[j][0], U[j], inter, dim) @ xt,
                            np.float64(np.float32(w))).astype(np.float32)
            ref += deq(types[j][1], D[j], dim, inter) @ hj.astype(np.float64)
        assert np.allclose(Y[qi], ref, rtol=1e-10, atol=1e-12)
    # rounding modes only perturb: fp16-staged activations stay within 1e-2 of the exact result's scale
    Yh, _ = O.moe_prefill(tgu, td, ts, n, ne, True, dim, inter, G, U, D, offs, tok, wt, X, chk, 1, Y0, nthreads=2)
    assert np.max(np.abs(Yh - Y) / (Ymag + 1e-9)) < 2e-3 and not np.array_equal(Yh, Y)


# ---------------------------------------------------------------- seeded generators are reproducible and sane
def test_generators():
    a = O.randn(100000, 7)
    assert np.array_equal(a, O.randn(100000, 7)) and not np.array_equal(a, O.randn(100000, 8))
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1) < 0.02
    for t in BLOCK_TYPES:
        b = O.random_blocks(t, 256 * 40, 3)
        assert np.array_equal(b, O.random_blocks(t, 256 * 40, 3))
        w = O.dequant(t, b, 256 * 40)
        assert np.all(np.isfinite(w)) and np.max(np.abs(w)) < 100


# ------------------------------------------------------------------------------------------------ router, route lists
def _router_golden():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "router_golden.npz"))


def test_router_matches_reference_golden():
    g = _router_golden()
    ids, w = O.router(g["logits"], g["bias"])
    assert np.array_equal(ids, g["ids"]) and np.array_equal(w.view(np.uint32), g["w_bits"])
    lists = O.route_lists(ids, w)
    for got, name in zip(lists, ("counts", "offsets", "entry", "tok", "lw_bits", "slot_of")):
        assert np.array_equal(got.view(np.uint32), g[name]), name


@pytest.mark.skipif(O.load_ref_arch() is None, reason="reference checkout not compiled here (oracle/_ref)")
def test_router_differential_vs_compiled_reference():
    logits = O.randn(200 * 384, 5, 3.0).reshape(200, 384)
    logits[:, ::7] += 25.0
    bias = O.randn(384, 6, 0.3)
    ids, w = O.router(logits, bias)
    rid, rw = O.ref_router(logits, bias)
    assert np.array_equal(ids, rid) and np.array_equal(w.view(np.uint32), rw.view(np.uint32))
    for a, b in zip(O.route_lists(ids, w), O.ref_route_lists(ids, w)):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_router_known_answers():
    # equal logits, zero bias: every key ties, the six lowest ids win and share the scale equally
    ids, w = O.router(np.zeros((1, 384), np.float32), np.zeros(384, np.float32))
    assert ids.tolist() == [[0, 1, 2, 3, 4, 5]] and np.allclose(w, 0.25, rtol=1e-7)
    # score = sqrt(softplus(x)): ln 2 at 0, x itself above the threshold 20; weights are score ratios times 1.5
    lg = np.full((1, 384), -30.0, np.float32)
    lg[0, [300, 200, 100, 50, 20, 10]] = [30.0, 25.0, 0.0, 0.0, -1.0, -2.0]
    ids, w = O.router(lg, np.zeros(384, np.float32))
    sc = np.sqrt([30.0, 25.0, np.log(2.0), np.log(2.0), np.log1p(np.exp(-1.0)), np.log1p(np.exp(-2.0))])
    assert ids.tolist() == [[300, 200, 50, 100, 20, 10]]  # the tie between 50 and 100 goes to the lower id
    assert np.allclose(w[0], sc / sc.sum() * 1.5, rtol=1e-6) and abs(float(w.sum()) - 1.5) < 1e-6
    # the bias picks, the score weighs: a large bias brings in an expert with a tiny score, first in the order
    b = np.zeros(384, np.float32)
    b[7] = 100.0
    ids2, w2 = O.router(lg, b)
    assert ids2[0, 0] == 7 and ids2[0, 1:].tolist() == [300, 200, 50, 100, 20]
    s7 = np.sqrt(np.log1p(np.exp(-30.0)))
    assert np.isclose(w2[0, 0], s7 / (s7 + sc[:5].sum()) * 1.5, rtol=1e-5)
    # other sizes and scales
    ids3, w3 = O.router(O.randn(4 * 128, 3).reshape(4, 128), np.zeros(128, np.float32), top_k=6, route_scale=2.5)
    assert np.allclose(w3.sum(1), 2.5, rtol=1e-6) and all(len(set(r)) == 6 for r in ids3.tolist())


def test_route_lists_are_a_stable_sort():
    rng = np.random.default_rng(3)
    for n, n_exp in ((1, 384), (17, 384), (300, 64), (0, 384)):
        ids = rng.integers(0, n_exp, n * 6).astype(np.int32)
        if n > 1:
            ids[: 6 * (n // 2)] = ids[0]  # one crowded expert
        w = rng.random(n * 6).astype(np.float32)
        counts, offsets, entry, tok, lw, slot_of = O.route_lists(ids, w, n_exp=n_exp)
        order = np.argsort(ids, kind="stable")
        assert np.array_equal(entry, order) and np.array_equal(tok, order // 6) and np.array_equal(lw, w[order])
        assert np.array_equal(slot_of[order], np.arange(n * 6)) and np.array_equal(counts, np.bincount(ids, minlength=n_exp))
        assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]))


def test_rmsnorm_known_answers_and_reference():
    x = np.full(512, 2.0, np.float32)
    assert np.allclose(O.rmsnorm(x, None, 0.0), 1.0, rtol=1e-7)                 # x / sqrt(mean(x^2)) = 1
    w = np.arange(512, dtype=np.float32)
    assert np.allclose(O.rmsnorm(x, w, 0.0), w, rtol=1e-7)                      # ... times the weight
    assert np.allclose(O.rmsnorm(x, None, 12.0), 2.0 / 4.0, rtol=1e-7)          # sqrt(4 + 12) = 4
    xr, wr = O.randn(1280, 3, 3.0), 1.0 + 0.2 * O.randn(1280, 4)
    y = O.rmsnorm(xr, wr, 1e-20)
    want = xr.astype(np.float64) / np.sqrt(np.mean(xr.astype(np.float64) ** 2) + 1e-20) * wr
    assert np.allclose(y, want, rtol=2e-7, atol=0)
    if O.load_ref_arch() is not None:
        assert np.array_equal(y.view(np.uint32), O.ref_rmsnorm(xr, wr, 1e-20).view(np.uint32))
        assert np.array_equal(O.rmsnorm(xr, None, 1e-6).view(np.uint32), O.ref_rmsnorm(xr, None, 1e-6).view(np.uint32))
