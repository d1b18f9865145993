"""GPU parity of the router and routing-list kernels against the CPU oracle, through the C ABI.

Mirrors the reference's tests/test_arch_router.mm: top-6 from logits for n in {1, 5, 2048} with the softplus branches
exercised, routing lists compared bit-exactly, the fused decode router (matvec + selection) over several inputs and a
repeat-dispatch identity check. The kernels compute scores in double precision like the reference's CPU twin, so
expert ids and weight bits are compared exactly; a differing pick would be accepted only for a near-tie of the keys
(key gap below 1e-5, the reference's own rule) and the test prints how many it saw.
"""
import os

import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import arch, quant as q
from util import up

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "router_golden.npz")


def check_tokens(logits, bias, gid, gw, rid, rw, rtol=1e-6, atol=0.0):
    """Equal ids and close weights, or a near-tie (tests/test_arch_router.mm:21-44). Returns the number of near-ties."""
    ties = 0
    for t in range(logits.shape[0]):
        if np.array_equal(gid[t], rid[t]):
            assert np.allclose(gw[t], rw[t], rtol=rtol, atol=atol), (t, gw[t], rw[t])
            continue
        key = np.sqrt(np.log1p(np.exp(logits[t].astype(np.float64)))) + bias
        for k in range(6):
            assert gid[t, k] == rid[t, k] or abs(key[gid[t, k]] - key[rid[t, k]]) < 1e-5, (t, k, gid[t], rid[t])
        ties += 1
    return ties


def make_logits(n, n_exp, seed):
    lg = O.randn(n * n_exp, seed, 3.0)
    lg[::97] = 30.0 + O.randn(len(lg[::97]), seed + 1)  # softplus threshold branch
    lg[5::89] = -25.0                                    # tiny-softplus branch
    return lg.reshape(n, n_exp)


def test_router_topk_matches_reference_golden(dev):
    g = np.load(GOLD)
    n = g["logits"].shape[0]
    ids = torch.full((n, 6), -1, dtype=torch.int32, device=dev)
    w = torch.zeros((n, 6), dtype=torch.float32, device=dev)
    e = q.Enc()
    arch.encode_router_topk(e, q.Buffer.of(up(g["logits"])), q.Buffer.of(up(g["bias"])), q.Buffer.of(ids), q.Buffer.of(w), n)
    L = arch.RouteLists.create(n)
    arch.encode_route_lists(e, q.Buffer.of(ids), q.Buffer.of(w), n, L)
    e.wait()
    assert np.array_equal(ids.cpu().numpy(), g["ids"])
    assert np.array_equal(w.cpu().numpy().view(np.uint32), g["w_bits"])
    for t, name in ((L.t_counts, "counts"), (L.t_offsets, "offsets"), (L.t_entry, "entry"), (L.t_tok, "tok"),
                    (L.t_w, "lw_bits"), (L.t_slot_of, "slot_of")):
        assert np.array_equal(t.cpu().numpy().view(np.uint32)[: len(g[name])], g[name]), name


@pytest.mark.parametrize("n,n_exp", [(1, 384), (5, 384), (2048, 384), (33, 64), (7, 512)])
def test_router_topk_and_route_lists_vs_oracle(dev, n, n_exp):
    logits = make_logits(n, n_exp, 11 + n)
    bias = O.randn(n_exp, 12 + n, 0.3)
    ids = torch.full((n + 1, 6), -7, dtype=torch.int32, device=dev)
    w = torch.full((n + 1, 6), 9.0, dtype=torch.float32, device=dev)
    e = q.Enc()
    arch.encode_router_topk(e, q.Buffer.of(up(logits)), q.Buffer.of(up(bias)), q.Buffer.of(ids), q.Buffer.of(w), n, n_exp)
    L = arch.RouteLists.create(n, n_exp)
    arch.encode_route_lists(e, q.Buffer.of(ids), q.Buffer.of(w), n, L)
    e.wait()
    gid, gw = ids.cpu().numpy(), w.cpu().numpy()
    assert (gid[n] == -7).all() and (gw[n] == 9.0).all()  # nothing past the last token is written
    rid, rw = O.router(logits, bias)
    ties = check_tokens(logits, bias, gid[:n], gw[:n], rid, rw)
    exact = int(np.sum(gw[:n].view(np.uint32) == rw.view(np.uint32)))
    print(f"  router_topk n={n} experts={n_exp}: near-ties {ties}, weight bits equal {exact}/{6 * n}")
    assert ties == 0 and exact == 6 * n
    # lists from the GPU's own ids, as the reference's test does
    ref = O.route_lists(gid[:n], gw[:n], n_exp=n_exp)
    got = (L.t_counts, L.t_offsets, L.t_entry, L.t_tok, L.t_w, L.t_slot_of)
    for a, b in zip(got, ref):
        assert np.array_equal(a.cpu().numpy().view(np.uint32)[: len(b)], b.view(np.uint32))
    assert int(L.t_offsets[n_exp]) == 6 * n


def test_route_lists_crowded_invalid_and_empty(dev):
    n, n_exp = 700, 384
    rng = np.random.default_rng(5)
    ids_h = rng.integers(0, n_exp, (n, 6)).astype(np.int32)
    ids_h[:400, 0] = 17          # one expert holds 400+ entries
    ids_h[5, 3] = -1             # "none" and out-of-range ids are left out
    ids_h[6, 0] = n_exp
    w_h = rng.random((n, 6)).astype(np.float32)
    L = arch.RouteLists.create(n, n_exp)
    L.t_slot_of.fill_(-5)
    e = q.Enc()
    arch.encode_route_lists(e, q.Buffer.of(up(ids_h)), q.Buffer.of(up(w_h)), n, L)
    e.wait()
    flat = ids_h.reshape(-1)
    valid = np.flatnonzero((flat >= 0) & (flat < n_exp))
    order = valid[np.argsort(flat[valid], kind="stable")]
    m = len(order)
    assert np.array_equal(L.t_entry.cpu().numpy()[:m], order) and np.array_equal(L.t_tok.cpu().numpy()[:m], order // 6)
    assert np.array_equal(L.t_w.cpu().numpy()[:m], w_h.reshape(-1)[order])
    slot = L.t_slot_of.cpu().numpy()
    assert np.array_equal(slot[order], np.arange(m)) and slot[5 * 6 + 3] == -5 and slot[6 * 6] == -5
    assert np.array_equal(L.t_counts.cpu().numpy(), np.bincount(flat[valid], minlength=n_exp))
    assert int(L.t_offsets[n_exp]) == m
    # no tokens: counts and offsets are all zero, nothing else is touched
    arch.encode_route_lists(e, None, None, 0, L)
    e.wait()
    assert not L.t_counts.any() and not L.t_offsets.any() and np.array_equal(L.t_entry.cpu().numpy()[:m], order)
    with pytest.raises(q.QuantError, match="exceed the lists' capacity"):
        arch.encode_route_lists(e, q.Buffer.of(up(ids_h)), q.Buffer.of(up(w_h)), n + 1, L)


@pytest.mark.parametrize("wtype,dim", [(q.QType.F32, 5120), (q.QType.BF16, 7168), (q.QType.F32, 7168)])
def test_router_fused_vs_oracle(dev, wtype, dim):
    n_exp = 384
    W = O.randn(n_exp * dim, 21, 0.02)
    if wtype == q.QType.BF16:
        Wd = up(W).to(torch.bfloat16)
        W = Wd.float().cpu().numpy()
    else:
        Wd = up(W)
    bias = O.randn(n_exp, 22, 0.1)
    bd = up(bias)
    s = arch.Scratch.create(n_exp)
    ids = torch.zeros(6, dtype=torch.int32, device=dev)
    w = torch.zeros(6, dtype=torch.float32, device=dev)
    e = q.Enc()
    ties = 0
    for it in range(20):
        x = O.randn(dim, 100 + it)
        arch.encode_router_fused(e, q.Buffer.of(up(x)), q.Buffer.of(Wd), q.Buffer.of(bd), q.Buffer.of(ids), q.Buffer.of(w), s,
                                 dim, wtype)
        e.wait()
        logits = (W.reshape(n_exp, dim).astype(np.float64) @ x.astype(np.float64)).astype(np.float32)
        got_logits = s.mem[: n_exp * 4].view(torch.float32).cpu().numpy()
        assert np.allclose(got_logits, logits, rtol=1e-4, atol=1e-5)  # tests/test_arch_router.mm:112
        # selection checked on the kernel's own logits (exact), and against the double-precision logits (near-ties)
        rid, rw = O.router(got_logits[None], bias)
        assert np.array_equal(ids.cpu().numpy()[None], rid) and np.array_equal(w.cpu().numpy()[None].view(np.uint32), rw.view(np.uint32))
        rid2, rw2 = O.router(logits[None], bias)
        ties += check_tokens(logits[None], bias, ids.cpu().numpy()[None], w.cpu().numpy()[None], rid2, rw2, 1e-5, 1e-5)
    print(f"  router_fused {wtype.name} dim={dim}: near-ties against fp64 logits {ties}")


@pytest.mark.parametrize("n_exp", [64, 128, 384, 512])
def test_router_fused_ties_expert_counts_and_nan(dev, n_exp):
    """The fused router selects in two levels (each wave of the last workgroup from its quarter of the experts, then one
    wave from the 24 survivors): exact ties inside a lane's pair of experts, across lanes and across quarters must go to
    the lower expert id, fewer than six comparable keys give expert 0 with weight 0, for every supported expert count."""
    dim = 256
    rng = np.random.default_rng(n_exp)
    W = (rng.standard_normal((n_exp, dim)) * 0.05).astype(np.float32)
    q4 = n_exp // 4
    # identical rows: same logit, same bias -> same key. Pairs (e, e + 64) share a lane when the quarter has 128
    # experts; (e, e + q4) sit in different quarters; runs of equal rows sit in neighbouring lanes
    W[3 + q4] = W[3]
    W[7 + 2 * q4] = W[7]
    W[10:14] = W[10]
    if q4 > 64:
        W[5 + 64] = W[5]
    big = np.array([3, 7, 10, 5], dtype=np.int64)
    W[big] *= 6.0  # make the tied rows the likely winners
    W[3 + q4], W[7 + 2 * q4], W[10:14] = W[3], W[7], W[10]
    if q4 > 64:
        W[5 + 64] = W[5]
    bias = np.zeros(n_exp, dtype=np.float32)
    Wd, bd = up(W.reshape(-1)), up(bias)
    s = arch.Scratch.create(n_exp)
    ids = torch.zeros(6, dtype=torch.int32, device=dev)
    w = torch.zeros(6, dtype=torch.float32, device=dev)
    e = q.Enc()
    for it in range(6):
        x = O.randn(dim, 300 + it)
        x = np.abs(x) * np.sign(W[10] + 1e-9) if it % 2 else x  # odd rounds: row 10 (and its copies) gets a large logit
        arch.encode_router_fused(e, q.Buffer.of(up(x.astype(np.float32))), q.Buffer.of(Wd), q.Buffer.of(bd), q.Buffer.of(ids), q.Buffer.of(w), s, dim)
        e.wait()
        got_logits = s.mem[: n_exp * 4].view(torch.float32).cpu().numpy()
        assert np.array_equal(got_logits[3], got_logits[3 + q4]) and np.array_equal(got_logits[10], got_logits[13])
        rid, rw = O.router(got_logits[None], bias)
        assert np.array_equal(ids.cpu().numpy()[None], rid), (it, ids.cpu().numpy(), rid)
        assert np.array_equal(w.cpu().numpy()[None].view(np.uint32), rw.view(np.uint32))
    # NaN activations: every logit is NaN, nothing is comparable
    x = np.full(dim, np.nan, dtype=np.float32)
    arch.encode_router_fused(e, q.Buffer.of(up(x)), q.Buffer.of(Wd), q.Buffer.of(bd), q.Buffer.of(ids), q.Buffer.of(w), s, dim)
    e.wait()
    assert not ids.any() and not w.any()
    # and the scratch is left re-armed: the next call works
    x = O.randn(dim, 999)
    arch.encode_router_fused(e, q.Buffer.of(up(x)), q.Buffer.of(Wd), q.Buffer.of(bd), q.Buffer.of(ids), q.Buffer.of(w), s, dim)
    e.wait()
    rid, rw = O.router(s.mem[: n_exp * 4].view(torch.float32).cpu().numpy()[None], bias)
    assert np.array_equal(ids.cpu().numpy()[None], rid)


def test_router_fused_repeats_bit_identically_and_checks_arguments(dev):
    n_exp, dim, R = 384, 7168, 300
    Wd, bd, xd = up(O.randn(n_exp * dim, 1, 0.02)), up(O.randn(n_exp, 2, 0.1)), up(O.randn(dim, 3))
    s = arch.Scratch.create(n_exp)
    ids = torch.zeros((R, 6), dtype=torch.int32, device=dev)
    w = torch.zeros((R, 6), dtype=torch.float32, device=dev)
    e = q.Enc()
    for i in range(R):  # tests/test_arch_router.mm:121-128: 300 dispatches in a row, identical results
        arch.encode_router_fused(e, q.Buffer.of(xd), q.Buffer.of(Wd), q.Buffer.of(bd), q.Buffer.of(ids).sub(i * 24, 24),
                                 q.Buffer.of(w).sub(i * 24, 24), s, dim)
    e.wait()
    assert bool((ids == ids[0]).all()) and bool((w == w[0]).all()) and len(set(ids[0].tolist())) == 6
    with pytest.raises(q.QuantError, match=r"macseek quant: router_fused unsupported \(type Q8_0 rows 384 cols 7168\)"):
        arch.encode_router_fused(e, q.Buffer.of(xd), q.Buffer.of(Wd), q.Buffer.of(bd), q.Buffer.of(ids), q.Buffer.of(w), s, dim,
                                 q.QType.Q8_0)
    with pytest.raises(q.QuantError, match="router_topk unsupported"):
        arch.encode_router_topk(e, q.Buffer.of(xd), q.Buffer.of(bd), q.Buffer.of(ids), q.Buffer.of(w), 1, 100)
