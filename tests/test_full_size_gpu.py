"""GPU parity at the full BASELINE sizes: all 384 experts resident in one device arena (3.3 GB of IQ1_S for the
batch-1 layer of configs[2], 4.3 GB of IQ2_XXS for the prefill GEMM of configs[3], so expert addresses lie beyond
4 GiB from the arena's base), weights generated on the device, and the oracle run on what a few sampled steps / tokens
touch (the experts they route to are copied back to the host). The smaller cases of test_moe_decode_gpu.py and
test_moe_prefill_gpu.py cover the shapes and edge cases; these two cover the resident layout and the real routing."""
import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import quant as q
from test_moe_decode_gpu import W6, Layer
from util import up

pytestmark = pytest.mark.gpu
DIM, INTER, NE, TOPK = 7168, 2048, 384, 6


def device_blocks(t, n_blocks, d_sigma, seed):
    """Random GGUF blocks on the device: uniform random bytes, fp16 d = |N(0, d_sigma)|."""
    bb = q.block_bytes(t)
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    W = torch.randint(0, 256, (n_blocks, bb), dtype=torch.uint8, device="cuda:0", generator=g)
    d = (torch.randn(n_blocks, device="cuda:0", generator=g) * d_sigma).abs()
    W[:, 0:2] = d.to(torch.float16).view(torch.uint8).view(n_blocks, 2)
    return W.view(-1)


def host(t):
    return t.cpu().numpy()


def test_decode_layer_with_384_resident_experts(dev):
    tr, ts = q.QType.IQ1_S, q.QType.IQ2_XXS
    gu_b, dn_b = q.row_bytes(tr, DIM) * INTER, q.row_bytes(tr, INTER) * DIM
    sgu_b, sdn_b = q.row_bytes(ts, DIM) * INTER, q.row_bytes(ts, INTER) * DIM
    per_exp = 2 * gu_b + dn_b
    arena = device_blocks(tr, NE * per_exp // 50, 0.01, 1)
    shared = device_blocks(ts, (2 * sgu_b + sdn_b) // 66, 0.01, 2)
    A, S = q.Buffer.of(arena), q.Buffer.of(shared)
    rng = np.random.default_rng(5)
    for ids in ([0, 1, 2, 3, 4, 5], [383, 200, 17, 101, 350, 64], list(rng.permutation(NE)[:TOPK])):
        L = Layer.__new__(Layer)  # the checks of the small cases, on experts that live in the resident arena
        L.dim, L.inter, L.n_routed, L.shared, L.types = DIM, INTER, TOPK, True, (int(tr), int(tr), int(ts))
        L.slots, L.G, L.U, L.D = [], [], [], []
        for e in ids:
            o = int(e) * per_exp
            L.slots.append(q.ExpertSlot(A.sub(o, gu_b), A.sub(o + gu_b, gu_b), A.sub(o + 2 * gu_b, dn_b)))
            L.G.append(host(arena[o:o + gu_b])); L.U.append(host(arena[o + gu_b:o + 2 * gu_b])); L.D.append(host(arena[o + 2 * gu_b:o + per_exp]))
        L.slots.append(q.ExpertSlot(S.sub(0, sgu_b), S.sub(sgu_b, sgu_b), S.sub(2 * sgu_b, sdn_b)))
        L.G.append(host(shared[:sgu_b])); L.U.append(host(shared[sgu_b:2 * sgu_b])); L.D.append(host(shared[2 * sgu_b:]))
        L.x, L.y0 = O.randn(DIM, 77 + int(ids[0])), O.randn(DIM, 78)
        L.xd, L.wd = up(L.x), up(W6.copy())
        L.scratch = torch.zeros(q.moe_decode_scratch_bytes(INTER) // 4, dtype=torch.float32, device="cuda:0")
        y = up(L.y0.copy())
        e = q.Enc()
        tbl = L.table()
        q.encode_moe_decode_table(e, L.args(y), q.Buffer.of(tbl))
        e.wait()
        L.check(y, L.scratch, f"resident experts {[int(i) for i in ids]}")


def test_prefill_gemm_2048_tokens_over_384_resident_experts(dev):
    t = q.QType.IQ2_XXS
    N = 2048
    gu_b, dn_b = q.row_bytes(t, DIM) * INTER, q.row_bytes(t, INTER) * DIM
    per_exp = 2 * gu_b + dn_b
    arena = device_blocks(t, NE * per_exp // 66, 0.01, 7)
    # top-6 distinct experts per token, popularity ~ rank^-1.1 over a seeded expert permutation (Gumbel top-k)
    rng = np.random.default_rng(4321)
    pw = np.zeros(NE)
    pw[rng.permutation(NE)] = 1.0 / np.arange(1, NE + 1) ** 1.1
    ids = np.argsort(-(np.log(pw)[None, :] + rng.gumbel(size=(N, NE))), axis=1)[:, :TOPK]
    w = rng.random((N, TOPK)).astype(np.float32) + 0.1
    w = w / w.sum(1, keepdims=True)
    counts = np.bincount(ids.ravel(), minlength=NE)
    used = np.nonzero(counts)[0]
    order = np.lexsort((np.repeat(np.arange(N), TOPK), ids.ravel()))  # expert-sorted, token order inside an expert
    tok = (order // TOPK).astype(np.int32)
    wt = w.ravel()[order].astype(np.float32)
    slot_of = np.empty(N * TOPK, dtype=np.int32)
    slot_of[order] = np.arange(N * TOPK, dtype=np.int32)
    offs = np.concatenate([[0], np.cumsum(counts[used])]).astype(np.int32)
    total = int(offs[-1])
    A = q.Buffer.of(arena)
    a = q.MoePrefillArgs()
    a.t_gate_up = a.t_down = t
    a.has_shared = False
    a.n_tokens, a.n_exp, a.k_per_token, a.dim, a.inter, a.x_is_bf16 = N, len(used), TOPK, DIM, INTER, True
    a.slots = [q.ExpertSlot(A.sub(int(e) * per_exp, gu_b), A.sub(int(e) * per_exp + gu_b, gu_b), A.sub(int(e) * per_exp + 2 * gu_b, dn_b))
               for e in used]
    a.offs = [int(v) for v in offs]
    X = torch.randn(N, DIM, device="cuda:0").to(torch.bfloat16)
    Y0 = O.randn(N * DIM, 9).reshape(N, DIM)
    Y = up(Y0.copy())
    keep = [up(tok), up(wt), up(slot_of)]
    scratch = torch.empty(q.moe_prefill_scratch_bytes(total, N, len(used), DIM, INTER), dtype=torch.uint8, device="cuda:0")
    a.tok, a.wt, a.slot_of, a.X, a.Y, a.scratch = (q.Buffer.of(v) for v in (keep[0], keep[1], keep[2], X, Y, scratch))
    e = q.Enc()
    q.encode_moe_prefill(e, a)
    e.wait()
    y1 = Y.clone()
    Y.copy_(up(Y0))
    q.encode_moe_prefill(e, a)  # same inputs again: bit-identical Y
    e.wait()
    assert torch.equal(y1, Y)

    # tokens to check (the reference checks up to 40 plus the tile-boundary ones, tests/test_quant_moe_prefill.mm:165-177):
    # the first two and the last; in the most popular expert (its 1545 entries are cut into blocks of 112 entries = seven
    # 16-entry tiles) the entries around tile and block boundaries and its last ones; one token of a least popular expert
    popular, rare = int(np.argmax(counts)), int(used[np.argmin(counts[used])])
    pe = int(np.nonzero(used == popular)[0][0])
    m = int(counts[popular])
    inside = [0, 1, 15, 16, 17, 47, 48, 49, 79, 80, 81, 95, 96, 111, 112, 113, 223, 224, 225, 335, 336, 337,
              112 * (m // 112) - 1, 112 * (m // 112), 112 * (m // 112) + 1, m - 17, m - 16, m - 2, m - 1]
    chk = {0, 1, N - 1, int(np.nonzero((ids == rare).any(1))[0][0])}
    chk |= {int(tok[offs[pe] + i]) for i in inside if 0 <= i < m}
    # and the first entry of ten mid-sized experts (two- and three-tile items)
    mid = [j for j in range(len(used)) if 17 <= counts[used[j]] <= 48][:10]
    chk |= {int(tok[offs[j]]) for j in mid}
    chk = sorted(chk)
    assert len(chk) >= 40
    need = sorted(set(int(x) for x in ids[chk].ravel()))
    mats = {x: (host(arena[x * per_exp:x * per_exp + gu_b]), host(arena[x * per_exp + gu_b:x * per_exp + 2 * gu_b]),
                host(arena[x * per_exp + 2 * gu_b:(x + 1) * per_exp])) for x in need}
    dummy = mats[need[0]]  # experts no checked token routes to are never read by the oracle
    G = [mats.get(int(x), dummy)[0] for x in used]; U = [mats.get(int(x), dummy)[1] for x in used]; D = [mats.get(int(x), dummy)[2] for x in used]
    Xh = X.float().cpu().numpy()
    chk = np.asarray(chk, dtype=np.int32)
    got = y1.cpu().numpy().astype(np.float64)[chk]
    assert np.all(np.isfinite(got))
    args = (int(t), int(t), int(t), N, len(used), False, DIM, INTER, G, U, D, offs, tok, wt, Xh, chk)
    Yh, Ym = O.moe_prefill(*args, 1, Y0)
    Yf, _ = O.moe_prefill(*args, 0, Y0)
    err_h = float(np.max(np.abs(got - Yh) / (Ym + 1e-9)))
    err_f = float(np.max(np.abs(got - Yf) / (Ym + 1e-9)))
    print(f"  2048 tokens, {len(used)} experts used, entries {total} (max {counts.max()} per expert), {len(chk)} tokens checked: "
          f"err(fp16-staged ref) {err_h:.2e} err(vs F32) {err_f:.2e}")
    assert err_h <= 1e-3 and err_f <= 5e-3  # the bounds of the small cases (tests/test_quant_moe_prefill.mm:223)
