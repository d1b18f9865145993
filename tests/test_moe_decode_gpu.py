"""GPU parity of the fused one-token MoE layer against the CPU oracle, through the C ABI.

Mirrors the reference's tests/test_quant_moe.mm (type combinations, 0/3/6 routed experts, with and without the shared
expert, clamp-heavy activations, matrices at 4-byte offsets in one arena in shuffled order) and part (A) of
tests/test_dec_sync.mm (pointer-table variant and the MoePart identities), at the reference shape 5120/2304 and the
BASELINE shape 7168/2048 with an IQ2_XXS shared expert."""
import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import quant as q
from util import place_in_arena, up

pytestmark = pytest.mark.gpu
W6 = np.array([0.31, 0.22, 0.17, 0.12, 0.1, 0.08], dtype=np.float32)  # tests/test_quant_moe.mm:60


class Layer:
    """Random expert weights placed like the reference test does, plus the oracle's answer."""

    def __init__(self, gu, dn, sh, n_routed, shared, dim, inter, xscale=1.0, seed=100):
        self.dim, self.inter, self.n_routed, self.shared = dim, inter, n_routed, shared
        self.types = (gu, dn, sh)
        ne = n_routed + int(shared)
        tg = [sh if e == n_routed else gu for e in range(ne)]
        td = [sh if e == n_routed else dn for e in range(ne)]
        self.G = [O.random_blocks(tg[e], inter * dim, seed + 3 * e) for e in range(ne)]
        self.U = [O.random_blocks(tg[e], inter * dim, seed + 1 + 3 * e) for e in range(ne)]
        self.D = [O.random_blocks(td[e], inter * dim, seed + 2 + 3 * e) for e in range(ne)]
        mats = []
        for e in range(ne - 1, -1, -1):  # shuffled: last expert first, down / gate / up
            mats += [self.D[e], self.G[e], self.U[e]]
        self.arena, bufs = place_in_arena(mats)
        self.slots = [None] * ne
        for i, e in enumerate(range(ne - 1, -1, -1)):
            d, g, u = bufs[3 * i:3 * i + 3]
            self.slots[e] = q.ExpertSlot(g, u, d)
        self.x = O.randn(dim, 77, xscale)
        self.y0 = O.randn(dim, 78)
        self.w = W6[:max(n_routed, 1)].copy()
        self.xd, self.wd = up(self.x), up(W6.copy())
        self.scratch = torch.zeros(q.moe_decode_scratch_bytes(inter) // 4, dtype=torch.float32, device="cuda:0")

    def args(self, y):
        a = q.MoeDecodeArgs()
        a.t_gate_up, a.t_down, a.t_shared = self.types
        a.n_routed, a.has_shared = self.n_routed, self.shared
        for e in range(self.n_routed):
            a.slot[e] = self.slots[e]
        if self.shared:
            a.shared = self.slots[self.n_routed]
        a.weights, a.x, a.y, a.scratch = q.Buffer.of(self.wd), q.Buffer.of(self.xd), q.Buffer.of(y), q.Buffer.of(self.scratch)
        a.dim, a.inter = self.dim, self.inter
        return a

    def table(self):
        t = np.zeros(18, dtype=np.uint64)
        for e in range(self.n_routed):
            s = self.slots[e]
            t[3 * e:3 * e + 3] = [s.gate.dev + s.gate.off, s.up.dev + s.up.off, s.down.dev + s.down.off]
        return up(t.view(np.int64))

    def oracle(self):
        return O.moe_decode(*self.types, self.n_routed, self.shared, self.dim, self.inter, self.G, self.U, self.D,
                            W6, self.x, self.y0)

    def check(self, y, h=None, what="", h_tol=2e-5, y_tol=5e-5, chain_tol=5e-5):
        """Stage-wise parity (the reference test checks h, then y: tests/test_quant_moe.mm:82-92):
        h against the oracle's h; y against the float64 down projection of the h the GPU produced (so stage 2 is
        judged on its own inputs), both in the reference's metric and in the north-star metric
        max |dy| <= 1e-3 * (sum_e ||Wd_e[r]||_2 ||h_e||_2 + |y0[r]|); finally the whole chain -- y against the down
        projection of the ORACLE's h, which is the reference test's y check (tests/test_quant_moe.mm:88-93, 5e-5) --
        to chain_tol (the reference's 5e-5 unless CHAIN_TOL below names the case)."""
        ry, ymag, rh, hs = self.oracle()
        got = y.cpu().numpy().astype(np.float64)
        assert np.all(np.isfinite(got))
        ne = self.n_routed + int(self.shared)
        experts = list(range(self.n_routed)) + ([self.n_routed] if self.shared else [])
        chain_err = float(np.max(np.abs(got - ry) / (ymag + 1e-12)))
        h_err = y_err = ns_err = 0.0
        if h is not None:
            hg = h.cpu().numpy()[:(self.n_routed + 1) * self.inter]
            y2 = self.y0.astype(np.float64)
            mag2 = np.abs(y2)
            scale = np.abs(y2)
            for i, e in enumerate(experts):
                sl = slice(e * self.inter, (e + 1) * self.inter)
                h_err = max(h_err, float(np.max(np.abs(hg[sl].astype(np.float64) - rh[sl]) / (hs[sl] * 12 + 1e-6))))
                td = self.types[2] if e == self.n_routed else self.types[1]
                yd, ydm, wn2 = O.matvec(td, self.D[i], self.dim, self.inter, hg[sl])
                y2, mag2 = y2 + yd, mag2 + ydm
                scale = scale + np.sqrt(wn2) * np.linalg.norm(hg[sl].astype(np.float64))
            y_err = float(np.max(np.abs(got - y2) / (mag2 + 1e-12)))
            ns_err = float(np.max(np.abs(got - y2) / (scale + 1e-30)))
        print(f"  {what} h_err {h_err:.2e} y_err {y_err:.2e} north-star {ns_err:.2e} chain {chain_err:.2e}")
        # the reference's own bounds for its F32-activation kernels: h 2e-5, y 5e-5 (tests/test_quant_moe.mm:82-93)
        assert h_err <= h_tol and y_err <= y_tol and ns_err <= 1e-3 and chain_err <= chain_tol
        return ry


T = O
CASES = [  # (gu, down, shared type, n_routed, shared, xscale, dim, inter)
    (T.IQ1_S, T.IQ1_S, T.Q6_K, 6, True, 1.0, 5120, 2304),
    (T.IQ1_S, T.IQ2_XXS, T.Q8_0, 6, True, 1.0, 5120, 2304),
    (T.IQ1_S, T.IQ2_XXS, T.Q6_K, 6, True, 1.0, 5120, 2304),
    (T.IQ2_XXS, T.IQ2_XXS, T.Q6_K, 6, True, 1.0, 5120, 2304),
    (T.IQ2_XXS, T.IQ2_XXS, T.Q8_0, 3, False, 1.0, 5120, 2304),
    (T.IQ1_S, T.IQ1_S, T.Q6_K, 0, True, 1.0, 5120, 2304),
    (T.IQ1_S, T.IQ1_S, T.Q6_K, 6, True, 40.0, 5120, 2304),   # drives gate/up past the +-10 clamps
    (T.IQ1_S, T.IQ1_S, T.IQ2_XXS, 6, True, 1.0, 7168, 2048),  # BASELINE batch-1 MoE layer
    (T.IQ2_XXS, T.IQ1_S, T.IQ1_S, 5, True, 1.0, 7168, 2048),
    (T.IQ1_S, T.IQ1_S, T.IQ2_XXS, 1, True, 40.0, 512, 256),   # smallest shapes the kernels accept
    (T.IQ1_S, T.IQ1_S, T.Q8_0, 2, True, 1.0, 32768, 256),     # x too long to stage in LDS: gate/up reads it directly
    (T.IQ2_XXS, T.IQ1_S, T.IQ2_XXS, 1, True, 1.0, 256, 16384),  # h rows too long to stage: down reads them directly
    (T.IQ1_S, T.IQ1_S, T.IQ2_XXS, 6, True, 1500.0, 7168, 2048),  # activations near the top of the fp16 range (max |x| about 6e3)
    (T.IQ1_S, T.IQ1_S, T.IQ2_XXS, 6, True, 0.02, 7168, 2048),    # small activations: h of the order of 1e-6 .. 1e-4
]
# The reference's kernels take x as F32 and its test holds h 2e-5, y 5e-5 and, for the whole chain (y against the down
# projection of the reference's own h), 5e-5 (tests/test_quant_moe.mm:82-93). Here gate/up rounds x at 2^-16 of the
# largest value of its 32 columns (IQ1_S, IQ2_XXS, Q6_K: integer decoders) or not at all (Q8_0), and down multiplies h
# rounded to fp16. All three reference bounds are asserted, with these exceptions (measured value in brackets):
#   down over h = products of two small Gaussians (heavy-tailed, xs = 0.02): y 6e-5 [4.8e-5], chain 6e-5 [4.9e-5]
#   inputs on which SwiGLU saturates (xs = 40: h stops growing with x, its rounding error does not): chain 1e-4 [6.8e-5];
#   on the smallest shape (512-column rows, 256-column h rows: few terms to average the roundings over) 1.5e-4 [1.0e-4]
H_TOL = {}
Y_TOL = {(T.IQ1_S, T.IQ1_S, T.IQ2_XXS, 6, True, 0.02, 7168, 2048): 6e-5}
CHAIN_TOL = {(T.IQ1_S, T.IQ1_S, T.IQ2_XXS, 6, True, 0.02, 7168, 2048): 6e-5,
             (T.IQ1_S, T.IQ1_S, T.Q6_K, 6, True, 40.0, 5120, 2304): 1e-4,
             (T.IQ1_S, T.IQ1_S, T.IQ2_XXS, 1, True, 40.0, 512, 256): 1.5e-4}
SMALL_SHAPE_CHAIN_TOL = 1.5e-4  # other tests' layers with 512-column rows and 256-column h rows [6.2e-5, 8.7e-5]


def chain_tol_of(case):
    return CHAIN_TOL.get(case, 5e-5)


@pytest.mark.parametrize("gu,dn,sh,nr,shared,xs,dim,inter", CASES)
def test_moe_decode_vs_oracle(dev, gu, dn, sh, nr, shared, xs, dim, inter):
    L = Layer(gu, dn, sh, nr, shared, dim, inter, xs)
    y = up(L.y0.copy())
    e = q.Enc()
    q.encode_moe_decode(e, L.args(y))
    e.wait()
    L.check(y, L.scratch, f"gu={O.TYPE_NAMES[gu]} down={O.TYPE_NAMES[dn]} shared={O.TYPE_NAMES[sh] if shared else '-'} routed={nr} xs={xs}",
            h_tol=H_TOL.get((gu, dn, sh, nr, shared, xs, dim, inter), 2e-5), y_tol=Y_TOL.get((gu, dn, sh, nr, shared, xs, dim, inter), 5e-5),
            chain_tol=chain_tol_of((gu, dn, sh, nr, shared, xs, dim, inter)))


@pytest.mark.parametrize("dim,inter,sh", [(5120, 2304, O.Q6_K), (7168, 2048, O.IQ2_XXS)])
def test_table_variant_and_parts(dev, dim, inter, sh):
    L = Layer(O.IQ1_S, O.IQ2_XXS, sh, 6, True, dim, inter)
    tbl = q.Buffer.of(L.table())
    e = q.Enc()

    def run(parts, bound=False):
        y = up(L.y0.copy())
        L.scratch.zero_()
        a = L.args(y)
        if bound:
            q.encode_moe_decode(e, a)
        else:
            for p in parts:
                q.encode_moe_decode_table_part(e, a, tbl, p)
        e.wait()
        return y, L.scratch.clone()

    y_all, h_all = run([q.MoePart.All])
    L.check(y_all, h_all, "table All")
    y_bound, h_bound = run(None, bound=True)
    assert torch.equal(y_all, y_bound) and torch.equal(h_all, h_bound)  # same kernels, pointers by value or by table
    y2, h2 = run([q.MoePart.SharedGu, q.MoePart.AfterSharedGu])
    assert torch.equal(y_all, y2) and torch.equal(h_all, h2)            # bit-identical (quant.hpp:80)
    y3, _ = run([q.MoePart.Shared, q.MoePart.Routed])
    ry = L.check(y3, None, "Shared + Routed")
    assert float((y3 - y_all).abs().max()) <= 1e-5 * float(np.max(np.abs(ry)))  # tests/test_dec_sync.mm: 1e-5 max|y|
    y4, h4 = run([q.MoePart.Shared])
    y5, h5 = run([q.MoePart.SharedGu, q.MoePart.SharedDown])
    assert torch.equal(y4, y5) and torch.equal(h4, h5)                  # bit-identical (quant.hpp:82)
    y7, h7 = run([q.MoePart.Gu, q.MoePart.Down])
    assert torch.equal(y_all, y7) and torch.equal(h_all, h7)
    # launch-shape overrides do not change any row's summation order (quant.hpp:67-69)
    y6 = up(L.y0.copy())
    a = L.args(y6)
    a.gu_nr, a.gu_rsg, a.d_nr, a.d_rsg = 3, 1, 5, 2
    q.encode_moe_decode_table(e, a, tbl)
    e.wait()
    assert torch.equal(y_all, y6)


def test_moe_decode_misuse(dev):
    L = Layer(O.IQ1_S, O.IQ1_S, O.IQ2_XXS, 2, True, 512, 256)
    y = up(L.y0.copy())
    e = q.Enc()
    a = L.args(y)
    a.n_routed = 7
    with pytest.raises(q.QuantError, match="moe_decode n_routed unsupported"):
        q.encode_moe_decode(e, a)
    a = L.args(y)
    a.t_gate_up = q.QType.Q8_0
    with pytest.raises(q.QuantError, match="moe_decode type combo unsupported"):
        q.encode_moe_decode(e, a)
    a = L.args(y)
    a.scratch = a.scratch.sub(0, 64)
    with pytest.raises(q.QuantError, match="scratch too small"):
        q.encode_moe_decode(e, a)
    # an expert address table that is not 8-byte aligned is refused on the host (the kernels read it with scalar loads)
    tbl = torch.zeros(20, dtype=torch.int64, device=dev)
    with pytest.raises(q.QuantError, match="table not 8-byte aligned"):
        q.encode_moe_decode_table(e, L.args(y), q.Buffer.of(tbl).sub(4, 152))
    a = L.args(y)
    a.n_routed, a.has_shared = 0, False   # nothing to do: silent return, y untouched (quant.mm:269)
    q.encode_moe_decode(e, a)
    e.wait()
    assert np.array_equal(y.cpu().numpy(), L.y0)
