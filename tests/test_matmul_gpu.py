"""GPU parity of msq_matmul / msq_matmul_h / msq_f32_to_f16 against the CPU oracle, through the C ABI.

Mirrors the reference's tests/test_quant_matmul.mm: its eleven cases (types, shapes, accumulate) and its two
references per case -- "half-exact" (weights and activations rounded to fp16, the kernel's defined numerics, double
accumulation; bound 1e-5 of sum|w x|) and the pure F32 dequant reference (bound 2e-3) -- plus the north-star bound
1e-3 * ||w_row|| * ||x||, a strided fp16 input, and the error contract.
"""
import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import quant as q
from util import TOL_NORTH_STAR, place_in_arena, up

pytestmark = pytest.mark.gpu

CASES = [  # (type, rows, cols, n, accumulate): tests/test_quant_matmul.mm:18-25
    (O.Q6_K, 1280, 5120, 77, False), (O.Q5_K, 1024, 1280, 160, True), (O.Q6_K, 512, 5120, 64, False),
    (O.Q8_0, 2304, 5120, 33, False), (O.Q6_K, 640, 8192, 40, False), (O.IQ1_S, 2304, 5120, 50, False),
    (O.IQ2_XXS, 5120, 2304, 37, True), (O.IQ1_S, 300, 2304, 129, False), (O.BF16, 512, 5120, 48, False),
    (O.F16, 256, 1280, 70, False), (O.F32, 384, 5120, 36, False),
    (O.IQ4_NL, 1024, 4096, 32, False), (O.Q6_K, 48, 256, 1, True),
    # both sides of the switches from the fused kernel to dequantize-then-GEMM (the reference's sits at 512 tokens,
    # quant.mm:204): 128 tokens for matrices of more than 2048 rows, 256 tokens below
    (O.IQ4_NL, 2304, 512, 128, False), (O.IQ4_NL, 2304, 512, 129, True), (O.Q6_K, 384, 1024, 256, False),
    (O.Q5_K, 272, 1024, 257, True), (O.Q6_K, 384, 1024, 512, False), (O.IQ4_NL, 96, 512, 700, False),
    # the fused kernel with one K slice per tile (two stages of K: nothing to cut) and with many (the cases above)
    (O.Q8_0, 16384, 256, 100, True),
    (O.IQ4_NL, 200, 640, 90, False), (O.Q8_0, 130, 384, 70, True), (O.IQ2_XXS, 144, 1024, 100, False),
    (O.Q5_K, 130, 2304, 66, True), (O.Q6_K, 1536, 7168, 128, False),
    # the tile kernel (IQ1_S, IQ2_XXS, IQ4_NL, Q8_0 matrices of 12 M weights and more, 65 to 256 tokens; 128-token tiles
    # below 192 tokens, 256-token tiles from there): ragged row and token counts, an odd number of 128-column stages
    # (half a weight stage at the end of a row), accumulate, both sides of its upper token bound
    (O.IQ2_XXS, 4096, 4096, 100, False), (O.Q8_0, 3200, 3968, 70, True), (O.IQ4_NL, 4104, 3072, 129, False),
    (O.IQ1_S, 2048, 6144, 256, True), (O.IQ4_NL, 3104, 4224, 200, True), (O.IQ2_XXS, 3000, 4096, 257, False),
]


def reference(t, Wb, rows, cols, X, n):
    """(half-exact product, F32 product, sum|w x|, ||w_row||) in float64."""
    Wd = O.dequant(t, Wb, rows * cols).reshape(rows, cols).astype(np.float64)
    Wh = Wd.astype(np.float16).astype(np.float64)  # every type, F32 included, is multiplied as fp16 here
    Xf = X.reshape(n, cols).astype(np.float64)
    Xh = X.reshape(n, cols).astype(np.float16).astype(np.float64)
    return Xh @ Wh.T, Xf @ Wd.T, np.abs(Xf) @ np.abs(Wd).T, np.sqrt((Wd ** 2).sum(1))


@pytest.mark.parametrize("t,rows,cols,n,acc", CASES, ids=lambda v: None)
def test_matmul_vs_oracle(dev, t, rows, cols, n, acc):
    Wb = O.random_blocks(t, rows * cols, 3 + rows)
    X = O.randn(n * cols, 11 + n)
    Y0 = O.randn(n * rows, 12)
    arena, (W,) = place_in_arena([Wb], first=16, gap=16)
    Xd, Yd = up(X), up(Y0.copy())
    e = q.Enc()
    q.encode_matmul(e, t, W, rows, cols, q.Buffer.of(Xd), q.Buffer.of(Yd), n, acc)
    e.wait()
    got = Yd.cpu().numpy().astype(np.float64).reshape(n, rows)
    sh, sf, mag, wn = reference(t, Wb, rows, cols, X, n)
    base = Y0.reshape(n, rows).astype(np.float64) if acc else 0.0
    mag = mag + np.abs(base)
    err_h = float(np.max(np.abs(got - (sh + base)) / (mag + 1e-12)))
    err_f = float(np.max(np.abs(got - (sf + base)) / (mag + 1e-12)))
    xn = np.sqrt((X.reshape(n, cols).astype(np.float64) ** 2).sum(1))
    err_ns = float(np.max(np.abs(got - (sf + base)) / (np.sqrt(wn[None, :] ** 2 + (base ** 2 if acc else 0)) * xn[:, None] + 1e-30)))
    print(f"  {O.TYPE_NAMES[t]:8s} [{cols:5d} -> {rows:5d}] n={n:<4d} {'acc' if acc else '   '} err(half-exact) {err_h:.2e}  "
          f"err(vs F32) {err_f:.2e}  north-star {err_ns:.2e}")
    assert err_h <= 1e-5 and err_f <= 2e-3 and err_ns <= TOL_NORTH_STAR  # tests/test_quant_matmul.mm:60


def test_f32_to_f16_and_strided_matmul_h(dev):
    t, rows, cols, n, xs = O.Q8_0, 96, 256, 5, 384
    Wb = O.random_blocks(t, rows * cols, 1)
    X = O.randn(n * xs, 2)
    Xd = up(X)
    X16 = torch.zeros(n * xs + 8, dtype=torch.float16, device=dev)
    e = q.Enc()
    q.encode_f32_to_f16(e, q.Buffer.of(Xd), q.Buffer.of(X16), n * xs)
    Y = torch.full((n * rows + 4,), 3.0, dtype=torch.float32, device=dev)
    q.encode_matmul_h(e, t, q.Buffer.of(up(Wb)), rows, cols, q.Buffer.of(X16), q.Buffer.of(Y), n, False, xs)
    e.wait()
    assert np.array_equal(X16.cpu().numpy()[: n * xs], X.astype(np.float16)) and not X16[n * xs:].any()
    Xs = X.reshape(n, xs)[:, :cols].copy()
    sh, _, mag, _ = reference(t, Wb, rows, cols, Xs, n)
    got = Y.cpu().numpy()
    assert (got[n * rows:] == 3.0).all()
    assert float(np.max(np.abs(got[: n * rows].reshape(n, rows) - sh) / (mag + 1e-12))) <= 1e-5


@pytest.mark.parametrize("xs", [3976, 3970])
def test_tile_matmul_h_strided(dev, xs):
    """fp16 activations with a row stride, a large Q8_0 matrix at 96 tokens: rows on 16-byte boundaries go to the tile
    kernel as they are, any other stride to the kernel that fetches lane by lane; both give the half-exact product."""
    t, rows, cols, n = O.Q8_0, 3200, 3968, 96
    Wb = O.random_blocks(t, rows * cols, 5)
    X = O.randn(n * xs, 6)
    X16 = up(X.astype(np.float16))
    Y = torch.full((n * rows + 4,), 3.0, dtype=torch.float32, device=dev)
    e = q.Enc()
    q.encode_matmul_h(e, t, q.Buffer.of(up(Wb)), rows, cols, q.Buffer.of(X16), q.Buffer.of(Y), n, False, xs)
    e.wait()
    Xs = X.reshape(n, xs)[:, :cols].copy()
    sh, _, mag, _ = reference(t, Wb, rows, cols, Xs, n)
    got = Y.cpu().numpy()
    assert (got[n * rows:] == 3.0).all()
    assert float(np.max(np.abs(got[: n * rows].reshape(n, rows) - sh) / (mag + 1e-12))) <= 1e-5


def test_tile_matmul_in_a_captured_graph(dev):
    """The tile route allocates nothing either (the fp16 copy of the activations and the partial sums live in
    file-scope device arrays): captured, every replay repeats the eager result bit for bit."""
    t, rows, cols, n = O.IQ2_XXS, 3072, 4096, 130
    Wb = O.random_blocks(t, rows * cols, 31)
    X = O.randn(n * cols, 32)
    sh, _, mag, _ = reference(t, Wb, rows, cols, X, n)
    Wd, Xd = up(Wb), up(X)
    Yd = torch.zeros(n * rows, dtype=torch.float32, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        q.encode_matmul(q.Enc(side), t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(Xd), q.Buffer.of(Yd), n)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = Yd.clone()
    got = eager.cpu().numpy().astype(np.float64).reshape(n, rows)
    assert float(np.max(np.abs(got - sh) / (mag + 1e-12))) <= 1e-5
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        q.encode_matmul(q.Enc(torch.cuda.current_stream()), t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(Xd), q.Buffer.of(Yd), n)
    for rep in range(3):
        Yd.fill_(7.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(Yd, eager), f"replay {rep} differs from the eager result"
        _ = (Xd * 2).sum().item()


def test_fused_matmul_in_a_captured_graph(dev):
    """Up to 128 tokens the call allocates nothing and only enqueues: captured into a HIP graph (the K-sliced kernel and
    the ordered sum of its slices), every replay repeats the eager result bit for bit, with eager work between the
    replays."""
    t, rows, cols, n = O.Q6_K, 640, 2048, 40
    Wb = O.random_blocks(t, rows * cols, 21)
    X = O.randn(n * cols, 22)
    sh, _, mag, _ = reference(t, Wb, rows, cols, X, n)
    Wd, Xd = up(Wb), up(X)
    Yd = torch.zeros(n * rows, dtype=torch.float32, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        q.encode_matmul(q.Enc(side), t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(Xd), q.Buffer.of(Yd), n)  # warm-up
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = Yd.clone()
    got = eager.cpu().numpy().astype(np.float64).reshape(n, rows)
    assert float(np.max(np.abs(got - sh) / (mag + 1e-12))) <= 1e-5
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        q.encode_matmul(q.Enc(torch.cuda.current_stream()), t, q.Buffer.of(Wd), rows, cols, q.Buffer.of(Xd), q.Buffer.of(Yd), n)
    for rep in range(4):
        Yd.fill_(7.0)  # the replay itself must overwrite Y
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(Yd, eager), f"replay {rep} differs from the eager result"
        _ = (Xd * 2).sum().item()  # eager work between the replays


def test_matmul_misuse(dev):
    W = q.Buffer.of(torch.zeros(1 << 20, dtype=torch.uint8, device=dev))
    v = q.Buffer.of(torch.zeros(1 << 18, dtype=torch.float32, device=dev))
    e = q.Enc()
    with pytest.raises(q.QuantError, match=r"macseek quant: matmul unsupported \(type Q6_K rows 16 cols 192\)"):
        q.encode_matmul(e, q.QType.Q6_K, W, 16, 192, v, v, 4)  # cols % 128 (quant.mm:196)
    with pytest.raises(q.QuantError, match="matmul unsupported"):
        q.encode_matmul(e, q.QType.Q6_K, W, 16, 256, v, v, 0)
    # a multiple of 128 columns that is not whole 256-weight blocks: refused on the host, on both routes and entry points
    # (nothing is launched: the output keeps its bytes)
    out = torch.full((2048 * 16,), 7.0, dtype=torch.float32, device=dev)
    for t in (q.QType.Q6_K, q.QType.Q5_K, q.QType.IQ1_S, q.QType.IQ2_XXS):
        for n in (4, 512):  # the fused kernel's range and the materialising route's
            with pytest.raises(q.QuantError, match=r"matmul unsupported \(type \S+ rows 16 cols 384\)"):
                q.encode_matmul(e, t, W, 16, 384, v, q.Buffer.of(out), n)
            with pytest.raises(q.QuantError, match=r"matmul unsupported \(type \S+ rows 16 cols 384\)"):
                q.encode_matmul_h(e, t, W, 16, 384, v, q.Buffer.of(out), n)
    e.wait()
    assert bool((out == 7.0).all())
    with pytest.raises(q.QuantError, match="f32_to_f16 unsupported"):
        q.encode_f32_to_f16(e, v, v, 6)
