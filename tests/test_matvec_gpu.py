"""GPU parity of msq_dequant and msq_matvec against the CPU oracle, through the C ABI.

Mirrors the reference's tests/test_quant_ref.mm (bit-exact dequantization) and tests/test_quant_matvec.mm (every real
shape x type, block-diagonal groups, accumulate, odd/tiny rows), plus the BASELINE shapes (7168 / 4096 / 2048)."""
import os

import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import quant as q
from util import TOL_NORTH_STAR, matvec_errors, place_in_arena, same_floats, tol_ref, up

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "dequant_golden.npz"))
ids = lambda t: O.TYPE_NAMES[t]


def gpu_dequant(blocks, t, n, dev):
    arena, (W,) = place_in_arena([blocks])
    out = torch.empty(n, dtype=torch.float32, device=dev)
    e = q.Enc()
    q.encode_dequant(e, t, W, n, q.Buffer.of(out))
    e.wait()
    return out.cpu().numpy()


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=ids)
@pytest.mark.parametrize("kind", ["sane", "raw"])
def test_dequant_golden_bit_exact(dev, t, kind):
    name = O.TYPE_NAMES[t]
    got = gpu_dequant(GOLD[f"{kind}_blocks_{name}"], t, 1024, dev)
    assert same_floats(got, GOLD[f"{kind}_bits_{name}"])


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=ids)
def test_dequant_1m_elements_bit_exact(dev, t):
    # the reference checks 1 M random elements per type with memcmp (tests/test_quant_ref.mm:40-53)
    n = 1 << 20
    rng = np.random.default_rng(100 + t)
    for blocks in (O.random_blocks(t, n, 31 + t), rng.integers(0, 256, O.row_bytes(t, n), dtype=np.uint8)):
        ref = O.dequant(t, blocks, n)
        got = gpu_dequant(blocks, t, n, dev)
        assert same_floats(got, ref.view(np.uint32))


# (type, rows, cols, groups, accumulate, what): reference list (tests/test_quant_matvec.mm:13-29) + BASELINE shapes
CASES = [
    (O.Q8_0, 4096, 4096, 1, False, "baseline cfg1"),
    (O.IQ2_XXS, 4096, 7168, 1, False, "baseline cfg2 gate/up"), (O.IQ2_XXS, 7168, 4096, 1, False, "baseline cfg2 down"),
    (O.IQ1_S, 4096, 7168, 1, False, "baseline cfg2 gate/up"), (O.IQ1_S, 7168, 4096, 1, True, "baseline cfg2 down acc"),
    (O.IQ1_S, 2048, 7168, 1, False, "baseline cfg3 gate"), (O.IQ1_S, 7168, 2048, 1, False, "baseline cfg3 down"),
    (O.Q6_K, 1536, 7168, 1, False, "baseline cfg5 q"), (O.Q5_K, 512, 7168, 1, False, "baseline cfg5 kv"),
    (O.IQ4_NL, 7168, 4096, 1, False, "baseline cfg5 out"), (O.BF16, 384, 7168, 1, False, "baseline cfg5 router"),
    (O.Q6_K, 1280, 5120, 1, False, "attn_q_a"), (O.Q5_K, 1280, 5120, 1, False, "attn_q_a"),
    (O.Q6_K, 32768, 1280, 1, False, "attn_q_b"), (O.Q5_K, 32768, 1280, 1, False, "attn_q_b"),
    (O.Q6_K, 512, 5120, 1, False, "attn_kv"), (O.Q5_K, 512, 5120, 1, True, "attn_kv acc"),
    (O.Q6_K, 8192, 4096, 8, False, "attn_output_a"), (O.Q5_K, 8192, 4096, 8, True, "attn_output_a acc"),
    (O.Q6_K, 5120, 8192, 1, False, "attn_output_b"), (O.Q5_K, 5120, 8192, 1, False, "attn_output_b"),
    (O.IQ1_S, 2304, 5120, 1, False, "exp gate"), (O.IQ1_S, 5120, 2304, 1, True, "exp down acc"),
    (O.IQ2_XXS, 2304, 5120, 1, False, "exp gate"), (O.IQ2_XXS, 5120, 2304, 1, False, "exp down"),
    (O.Q6_K, 2304, 5120, 1, False, "shexp gate"), (O.Q6_K, 5120, 2304, 1, False, "shexp down"),
    (O.Q8_0, 2304, 5120, 1, False, "shexp gate"), (O.Q8_0, 5120, 2304, 1, True, "shexp down acc"),
    (O.Q6_K, 25600, 6144, 1, False, "engram_kv"), (O.IQ4_NL, 4096, 1024, 1, True, "iq4_nl acc"),
    (O.F32, 384, 5120, 1, False, "router"), (O.F32, 24, 20480, 1, False, "hc_fn"),
    (O.BF16, 512, 5120, 1, False, "compressor_kv"), (O.BF16, 4096, 1280, 1, False, "indexer q_b"),
    (O.BF16, 32, 5120, 1, False, "indexer proj"), (O.BF16, 128, 512, 1, False, "indexer k"),
    (O.F16, 1280, 5120, 1, False, "f16 synthetic"), (O.F16, 7, 768, 1, True, "f16 odd rows"),
    (O.Q6_K, 3, 256, 1, False, "tiny"), (O.IQ1_S, 1, 256, 1, False, "one row one block"),
    (O.IQ2_XXS, 5, 512, 1, True, "tiny acc"), (O.Q8_0, 9, 32, 1, False, "one q8 block per row"),
    # activation rows staged through LDS: block-diagonal groups (one staged row per group), rows too long to stage
    (O.IQ4_NL, 4096, 1024, 4, False, "staged x, groups"), (O.IQ1_S, 2048, 2048, 2, True, "staged x, groups acc"),
    (O.Q8_0, 1024, 2048, 2, False, "staged x, groups"), (O.IQ2_XXS, 2048, 1024, 8, False, "staged x, groups"),
    (O.IQ2_XXS, 16, 36864, 1, False, "row too long for LDS"), (O.Q8_0, 8, 16384, 1, True, "row too long for LDS acc"),
    (O.IQ1_S, 600, 12288, 1, False, "long staged row"),
    # weight rows through LDS (large Q6_K / Q8_0 matrices): ragged row counts, a row that ends in a short wave slice
    (O.Q6_K, 4099, 4096, 1, False, "large q6_k, ragged rows"), (O.Q6_K, 3001, 5376, 1, True, "large q6_k, 21 blocks per row acc"),
    (O.Q8_0, 8201, 5120, 1, True, "large q8_0 acc"), (O.Q8_0, 16400, 2592, 1, False, "large q8_0, 81 blocks per row"),
    # ... and with rows of two and a half / three and a half waves of units, which go two rows at a time when the row
    # count is even (the last pair ragged against the tile; an odd count keeps the one-row form)
    (O.Q6_K, 3002, 5120, 1, True, "large q6_k, row pairs acc"), (O.Q6_K, 2100, 7168, 1, False, "large q6_k, row pairs of 7 waves"),
    (O.Q8_0, 7990, 5120, 1, False, "large q8_0, row pairs"), (O.Q6_K, 3003, 5120, 1, False, "large q6_k, odd rows"),
]


@pytest.mark.parametrize("t,rows,cols,groups,acc,what", CASES, ids=lambda v: str(v).replace(" ", "_") if isinstance(v, str) else None)
def test_matvec_vs_oracle(dev, t, rows, cols, groups, acc, what):
    Wb = O.random_blocks(t, rows * cols, 7 + rows + cols)
    x = O.randn(cols * groups, 99 + cols)
    y0 = O.randn(rows, 5)
    ry, mag, wn2 = O.matvec(t, Wb, rows, cols, x, groups)
    if acc:
        ry, mag = ry + y0, mag + np.abs(y0)
    arena, (W,) = place_in_arena([Wb])  # weight base 4-byte aligned only
    xd, yd = up(x), up(y0.copy())
    e = q.Enc()
    q.encode_matvec(e, t, W, rows, cols, q.Buffer.of(xd), q.Buffer.of(yd), acc, groups)
    e.wait()
    got = yd.cpu().numpy()
    err_ref, err_ns = matvec_errors(got, ry, mag, wn2 + (y0.astype(np.float64) ** 2 if acc else 0), x, rows, cols, groups)
    print(f"  {O.TYPE_NAMES[t]:8s} {what:24s} [{cols:5d} -> {rows:6d}] g{groups} err/sum|wx| {err_ref:.2e} err/(|w||x|) {err_ns:.2e}")
    assert err_ns <= TOL_NORTH_STAR
    assert err_ref <= tol_ref(t, cols)


@pytest.mark.parametrize("t,rows,cols", [(O.IQ1_S, 4096, 7168), (O.IQ4_NL, 520, 4096), (O.Q8_0, 300, 2048), (O.Q6_K, 1536, 7168)])
def test_activation_offset_four_bytes(dev, t, rows, cols):
    # x and y start 4 bytes into their buffers (not 16-byte aligned): the staging copies and the 128-bit slice loads
    # must not assume more than the 4-byte alignment the operator interface gives
    Wb = O.random_blocks(t, rows * cols, 17 + rows)
    x = O.randn(cols, 23)
    ry, mag, wn2 = O.matvec(t, Wb, rows, cols, x, 1)
    arena, (W,) = place_in_arena([Wb])
    xd = up(np.concatenate([np.zeros(1, np.float32), x]))
    yd = up(np.zeros(rows + 1, np.float32))
    e = q.Enc()
    q.encode_matvec(e, t, W, rows, cols, q.Buffer.of(xd).sub(4, cols * 4), q.Buffer.of(yd).sub(4, rows * 4), False, 1)
    e.wait()
    got = yd.cpu().numpy()
    assert got[0] == 0.0
    err_ref, err_ns = matvec_errors(got[1:], ry, mag, wn2, x, rows, cols, 1)
    assert err_ns <= TOL_NORTH_STAR
    assert err_ref <= tol_ref(t, cols)


def test_output_head_shape(dev):
    # Q6_K 129280 x 5120 (543 MB), the largest matrix the reference test covers (tests/test_quant_matvec.mm:23)
    t, rows, cols = O.Q6_K, 129280, 5120
    Wb = O.random_blocks(t, rows * cols, 3)
    x = O.randn(cols, 4)
    ry, mag, wn2 = O.matvec(t, Wb, rows, cols, x)
    Wd, xd = up(Wb), up(x)
    yd = torch.empty(rows, dtype=torch.float32, device=dev)
    e = q.Enc()
    q.encode_matvec(e, t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(xd), q.Buffer.of(yd))
    e.wait()
    err_ref, err_ns = matvec_errors(yd.cpu().numpy(), ry, mag, wn2, x, rows, cols, 1)
    assert err_ns <= TOL_NORTH_STAR and err_ref <= tol_ref(t, cols)


@pytest.mark.parametrize("t", [O.IQ1_S, O.Q6_K, O.Q8_0], ids=ids)
def test_row_chunks_are_bit_identical(dev, t):
    # "splitting a matrix into row chunks that all use matvec_cfg's shape gives bit-identical rows" (quant.hpp:16-18)
    rows, cols = 4096, 2048
    Wb = O.random_blocks(t, rows * cols, 17)
    x = O.randn(cols, 18)
    Wd, xd = up(Wb), up(x)
    W = q.Buffer.of(Wd)
    rb = q.row_bytes(t, cols)
    full = torch.empty(rows, dtype=torch.float32, device=dev)
    parts = torch.empty(rows, dtype=torch.float32, device=dev)
    cfg = q.matvec_cfg(t, rows, cols)
    e = q.Enc()
    q.encode_matvec(e, t, W, rows, cols, q.Buffer.of(xd), q.Buffer.of(full))
    chunk = cfg.nr * cfg.rsg * 37
    for r0 in range(0, rows, chunk):
        n = min(chunk, rows - r0)
        q.encode_matvec(e, t, W.sub(r0 * rb, n * rb), n, cols, q.Buffer.of(xd), q.Buffer.of(parts).sub(r0 * 4, n * 4), False, 1, cfg)
    # rows per wave / row-waves per workgroup never change a row's bits either
    other = torch.empty(rows, dtype=torch.float32, device=dev)
    q.encode_matvec(e, t, W, rows, cols, q.Buffer.of(xd), q.Buffer.of(other), False, 1, q.MvCfg(nr=3, rsg=1, ks=cfg.ks))
    e.wait()
    assert torch.equal(full, parts) and torch.equal(full, other)


def test_environment_imposes_the_launch_shape(dev, tmp_path):
    # MSQ_MV_NR / _RSG / _KS (reference: MACSEEK_MV_*, quant.mm:78-83) are read once per process: a child process runs with
    # them set; its matvec_cfg reports the imposed shape and its result has the bits of the same shape passed as MvCfg
    import os, subprocess, sys
    t, rows, cols = O.Q6_K, 1024, 2048
    child = (
        "import sys, numpy as np, torch\n"
        "sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
        "import oracle as O\nfrom macseek_amd import quant as q\nfrom util import up\n"
        "t, rows, cols = O.Q6_K, 1024, 2048\n"
        "c = q.matvec_cfg(t, rows, cols)\nassert (c.nr, c.rsg, c.ks) == (3, 2, 1), (c.nr, c.rsg, c.ks)\n"
        "Wd, xd = up(O.random_blocks(t, rows * cols, 5)), up(O.randn(cols, 6))\n"
        "y = torch.empty(rows, dtype=torch.float32, device='cuda:0')\ne = q.Enc()\n"
        "q.encode_matvec(e, t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(xd), q.Buffer.of(y))\ne.wait()\n"
        "np.save(%r, y.cpu().numpy())\n"
    ) % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.dirname(os.path.abspath(__file__)), str(tmp_path / "y.npy"))
    env = dict(os.environ, MSQ_MV_NR="3", MSQ_MV_RSG="2", MSQ_MV_KS="1")
    subprocess.run([sys.executable, "-c", child], env=env, check=True, timeout=100)
    Wd, xd = up(O.random_blocks(t, rows * cols, 5)), up(O.randn(cols, 6))
    y = torch.empty(rows, dtype=torch.float32, device=dev)
    e = q.Enc()
    q.encode_matvec(e, t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(xd), q.Buffer.of(y), False, 1, q.MvCfg(nr=3, rsg=2, ks=1))
    e.wait()
    assert np.array_equal(np.load(tmp_path / "y.npy").view(np.uint32), y.cpu().numpy().view(np.uint32))


def test_repeat_is_bit_identical_and_unwritten_rows_untouched(dev):
    t, rows, cols = O.IQ2_XXS, 1000, 7168
    Wb = O.random_blocks(t, rows * cols, 1)
    Wd, xd = up(Wb), up(O.randn(cols, 2))
    y = torch.full((rows + 64,), 7.0, dtype=torch.float32, device=dev)
    e = q.Enc()
    q.encode_matvec(e, t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(xd), q.Buffer.of(y).sub(0, rows * 4))
    e.wait()
    first = y.clone()
    q.encode_matvec(e, t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(xd), q.Buffer.of(y).sub(0, rows * 4))
    e.wait()
    assert torch.equal(first, y) and bool((y[rows:] == 7.0).all())


def test_matvec_errors_raise_like_the_reference_aborts(dev):
    W = q.Buffer.of(torch.zeros(1 << 16, dtype=torch.uint8, device=dev))
    v = q.Buffer.of(torch.zeros(4096, dtype=torch.float32, device=dev))
    e = q.Enc()
    with pytest.raises(q.QuantError, match=r"macseek quant: matvec unsupported \(type IQ1_S rows 8 cols 300\)"):
        q.encode_matvec(e, q.QType.IQ1_S, W, 8, 300, v, v)
    with pytest.raises(q.QuantError):
        q.encode_matvec(e, q.QType.Q6_K, W, 9, 256, v, v, False, 2)
    with pytest.raises(q.QuantError):
        q.encode_matvec(e, 39, W, 8, 256, v, v)
