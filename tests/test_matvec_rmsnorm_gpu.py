"""GPU tests of msq_rmsnorm and msq_matvec_rmsnorm (the decode matvec with the input RMSNorm fused in).

Mirrors the reference's tests/test_dec_fuse.mm:27-53: the fused call must equal rmsnorm -> matvec bit for bit, on its
six cases plus the BASELINE shapes; and, since that identity alone would also hold for two wrong kernels, both are
compared with the CPU oracle (norm in double; double dot of the normalized row).
"""
import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import arch, quant as q
from util import TOL_NORTH_STAR, matvec_errors, place_in_arena, tol_ref, up

pytestmark = pytest.mark.gpu

CASES = [  # tests/test_dec_fuse.mm:30-31, then the attention-projection shapes of BASELINE configs[4] and edge shapes
    (O.Q6_K, 32768, 1280), (O.Q5_K, 32768, 1280), (O.BF16, 4096, 1280), (O.Q8_0, 1000, 2048), (O.F32, 77, 1536),
    (O.Q6_K, 300, 5120),
    (O.Q6_K, 1536, 7168), (O.Q5_K, 512, 7168), (O.IQ4_NL, 7168, 4096), (O.BF16, 384, 7168), (O.F16, 40, 256),
    (O.Q8_0, 5000, 1024), (O.Q6_K, 64, 14336),
]


@pytest.mark.parametrize("t,rows,cols", CASES, ids=lambda v: None)
def test_fused_equals_norm_then_matvec_and_oracle(dev, t, rows, cols):
    eps = 1e-20 if rows % 2 else 1e-6
    Wb = O.random_blocks(t, rows * cols, 11 + cols, 0.03)
    x = (O.randn(cols, 5) * 3.0).astype(np.float32)
    nw = (1.0 + 0.2 * O.randn(cols, 6)).astype(np.float32)
    arena, (W,) = place_in_arena([Wb])
    xd, nwd = up(x), up(nw)
    xn = torch.zeros(cols, dtype=torch.float32, device=dev)
    y0 = torch.zeros(rows, dtype=torch.float32, device=dev)
    y1 = torch.full((rows + 8,), 4.0, dtype=torch.float32, device=dev)
    e = q.Enc()
    arch.encode_rmsnorm(e, q.Buffer.of(xd), q.Buffer.of(nwd), q.Buffer.of(xn), 1, cols, eps)
    e.barrier()
    q.encode_matvec(e, t, W, rows, cols, q.Buffer.of(xn), q.Buffer.of(y0))
    q.encode_matvec_rmsnorm(e, t, W, rows, cols, q.Buffer.of(xd), q.Buffer.of(nwd), eps, q.Buffer.of(y1))
    e.wait()
    assert torch.equal(y0, y1[:rows]) and bool((y1[rows:] == 4.0).all())        # bit for bit; nothing past the rows
    # the norm against the oracle (float reduction against double: a few ulp)
    xn_ref = O.rmsnorm(x, nw, eps)
    assert np.allclose(xn.cpu().numpy(), xn_ref, rtol=2e-6, atol=0)
    # the fused result against the double dot of the oracle's normalized row
    ry, mag, wn2 = O.matvec(t, Wb, rows, cols, xn_ref)
    err_ref, err_ns = matvec_errors(y1[:rows].cpu().numpy(), ry, mag, wn2, xn_ref, rows, cols, 1)
    print(f"  matvec_rmsnorm {O.TYPE_NAMES[t]:7s} {rows:5d} x {cols:5d}: bit-identical; err {err_ref:.2e} north-star {err_ns:.2e}")
    assert err_ns <= TOL_NORTH_STAR and err_ref <= tol_ref(t, cols)


def test_rmsnorm_rows_strides_no_weight_and_alias(dev):
    rows, dim, ins, outs = 5, 1000, 1024, 1100
    X = O.randn(rows * ins, 9, 2.0)
    Xd = up(X)
    Y = torch.full((rows * outs,), 7.0, dtype=torch.float32, device=dev)
    e = q.Enc()
    arch.encode_rmsnorm(e, q.Buffer.of(Xd), None, q.Buffer.of(Y), rows, dim, 1e-6, ins, outs)
    e.wait()
    got = Y.cpu().numpy().reshape(rows, outs)
    for r in range(rows):
        assert np.allclose(got[r, :dim], O.rmsnorm(X[r * ins:r * ins + dim], None, 1e-6), rtol=2e-6, atol=0)
        assert (got[r, dim:] == 7.0).all()
    w = up(O.randn(dim, 10))
    arch.encode_rmsnorm(e, q.Buffer.of(Xd), q.Buffer.of(w), q.Buffer.of(Xd), rows, dim, 1e-6, ins, ins)  # in place
    e.wait()
    got = Xd.cpu().numpy().reshape(rows, ins)
    for r in range(rows):
        assert np.allclose(got[r, :dim], O.rmsnorm(X[r * ins:r * ins + dim], w.cpu().numpy(), 1e-6), rtol=2e-6, atol=1e-30)
        assert np.array_equal(got[r, dim:], X.reshape(rows, ins)[r, dim:])


def test_matvec_rmsnorm_misuse(dev):
    W = q.Buffer.of(torch.zeros(1 << 22, dtype=torch.uint8, device=dev))
    v = q.Buffer.of(torch.zeros(1 << 16, dtype=torch.float32, device=dev))
    e = q.Enc()
    # codebook formats have no fused norm (src/kernels/quant.mm:110)
    with pytest.raises(q.QuantError, match=r"macseek quant: matvec_rmsnorm unsupported \(type IQ1_S rows 64 cols 2048\)"):
        q.encode_matvec_rmsnorm(e, q.QType.IQ1_S, W, 64, 2048, v, v, 1e-6, v)
    with pytest.raises(q.QuantError, match="matvec_rmsnorm unsupported"):
        q.encode_matvec_rmsnorm(e, q.QType.Q6_K, W, 64, 1000, v, v, 1e-6, v)
    with pytest.raises(q.QuantError, match="matvec_rmsnorm unsupported"):  # wider than the LDS row
        q.encode_matvec_rmsnorm(e, q.QType.Q8_0, W, 16, 16384, v, v, 1e-6, v)
