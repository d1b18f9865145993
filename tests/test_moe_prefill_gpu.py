"""GPU parity of msq_moe_prefill (grouped MoE GEMM) against the CPU oracle, through the C ABI.

Mirrors the reference's tests/test_quant_moe_prefill.mm: expert-sorted routing with experts in one arena at 4-byte
offsets, shared expert, a popular multi-tile expert, explicit expert sizes that hit every token-tile boundary
(1, 15..17, 31..33, 47..49, 63..65, ...), a skewed Zipf top-k routing; the reference emulating the fp16 staging of X
and H (tight bound) and the pure F32 one; every case runs twice and must give bit-identical Y."""
import numpy as np
import pytest
import torch

import oracle as O
from macseek_amd import quant as q
from util import place_in_arena, up

pytestmark = pytest.mark.gpu
SIZES = [1, 1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 100, 129, 200, 300]  # test_quant_moe_prefill.mm:65


def make_routing(kind, n, k, n_exp, rng):
    rt = [[] for _ in range(n)]
    if kind == "popular":  # slot 0 -> expert 0 for every token, other slots random distinct
        for t in range(n):
            rt[t] = [0] + list(1 + rng.permutation(n_exp - 1)[:k - 1])
    elif kind == "sizes":  # expert 0 takes every token, the rest straddle the tile boundaries
        for t in range(n):
            rt[t].append(0)
        nxt = 0
        for j in range(1, n_exp):
            for _ in range(SIZES[j - 1]):
                t = nxt
                while len(rt[t]) >= k:
                    t = (t + 1) % n
                rt[t].append(j)
                nxt = (t + 7) % n
    else:  # Zipf popularity over a random expert permutation, k distinct experts per token
        s = float(kind.split(":")[1])
        pw = np.zeros(n_exp)
        pw[rng.permutation(n_exp)] = 1.0 / np.arange(1, n_exp + 1) ** s
        for t in range(n):
            rt[t] = list(rng.choice(n_exp, size=k, replace=False, p=pw / pw.sum()))
    return rt


def build(gu, dn, sh, n, k, n_exp, shared, kind, dim, inter, seed=0):
    rng = np.random.default_rng(42 + n + seed)
    rt = make_routing(kind, n, k, n_exp, rng)
    rw = [[0.1 + 0.2 * ((t * 7 + kk * 3) % 5) / 5 for kk in range(len(rt[t]))] for t in range(n)]
    offs, tok, wt = [0], [], []
    slot_of = -np.ones(n * k, dtype=np.int32)
    for j in range(n_exp):
        for t in range(n):
            for kk, e in enumerate(rt[t]):
                if e == j:
                    slot_of[t * k + kk] = len(tok)
                    tok.append(t); wt.append(rw[t][kk])
        offs.append(len(tok))
    ne_all = n_exp + int(shared)
    tg = [sh if j == n_exp else gu for j in range(ne_all)]
    td = [sh if j == n_exp else dn for j in range(ne_all)]
    G = [O.random_blocks(tg[j], inter * dim, 500 + 3 * j) for j in range(ne_all)]
    U = [O.random_blocks(tg[j], inter * dim, 501 + 3 * j) for j in range(ne_all)]
    D = [O.random_blocks(td[j], inter * dim, 502 + 3 * j) for j in range(ne_all)]
    mats = []
    for j in range(ne_all - 1, -1, -1):
        mats += [U[j], D[j], G[j]]
    arena, bufs = place_in_arena(mats, first=4, gap=8)
    slots = [None] * ne_all
    for i, j in enumerate(range(ne_all - 1, -1, -1)):
        u, d, g = bufs[3 * i:3 * i + 3]
        slots[j] = q.ExpertSlot(g, u, d)
    X = O.randn(n * dim, 9).reshape(n, dim)
    Y0 = O.randn(n * dim, 10).reshape(n, dim)
    return dict(rt=rt, offs=offs, tok=np.array(tok, np.int32), wt=np.array(wt, np.float32), slot_of=slot_of, G=G, U=U, D=D,
                arena=arena, slots=slots, X=X, Y0=Y0, types=(gu, dn, sh), n=n, k=k, n_exp=n_exp, shared=shared, dim=dim, inter=inter)


def run_gpu(c, x_bf16=False):
    total = len(c["tok"])
    Xd = up(c["X"]).to(torch.bfloat16) if x_bf16 else up(c["X"])
    Yd = up(c["Y0"].copy())
    keep = [up(c["tok"] if total else np.zeros(1, np.int32)), up(c["wt"] if total else np.zeros(1, np.float32)), up(c["slot_of"])]
    scratch = torch.empty(q.moe_prefill_scratch_bytes(total, c["n"], c["n_exp"], c["dim"], c["inter"]), dtype=torch.uint8, device="cuda:0")
    a = q.MoePrefillArgs()
    a.t_gate_up, a.t_down, a.t_shared = c["types"]
    a.n_tokens, a.n_exp, a.slots, a.offs = c["n"], c["n_exp"], c["slots"][:c["n_exp"]], c["offs"]
    a.tok, a.wt, a.slot_of = q.Buffer.of(keep[0]), q.Buffer.of(keep[1]), q.Buffer.of(keep[2])
    a.k_per_token, a.has_shared = c["k"], c["shared"]
    if c["shared"]:
        a.shared = c["slots"][c["n_exp"]]
    a.X, a.Y, a.scratch = q.Buffer.of(Xd), q.Buffer.of(Yd), q.Buffer.of(scratch)
    a.dim, a.inter, a.x_is_bf16 = c["dim"], c["inter"], x_bf16
    e = q.Enc()
    q.encode_moe_prefill(e, a)
    e.wait()
    y1 = Yd.clone()
    Yd.copy_(up(c["Y0"]))
    q.encode_moe_prefill(e, a)  # run-to-run determinism: same inputs again -> bit-identical Y
    e.wait()
    return y1, torch.equal(y1, Yd)


def test_moe_prefill_in_a_captured_graph(dev):
    """The call only enqueues (quant.hpp:3,91-92): captured into a HIP graph -- nothing may be read from host memory at
    replay time -- every replay repeats the eager result bit for bit, with eager work and synchronizations between the
    replays and the host-side argument structures destroyed after the capture."""
    c = build(O.IQ2_XXS, O.IQ1_S, O.Q8_0, 600, 6, 20, True, "sizes", 512, 256)
    y_eager, same = run_gpu(c)
    assert same
    total = len(c["tok"])
    Xd, Yd = up(c["X"]), up(c["Y0"].copy())
    keep = [up(c["tok"]), up(c["wt"]), up(c["slot_of"])]
    scratch = torch.empty(q.moe_prefill_scratch_bytes(total, c["n"], c["n_exp"], c["dim"], c["inter"]), dtype=torch.uint8, device="cuda:0")

    def args():
        a = q.MoePrefillArgs()
        a.t_gate_up, a.t_down, a.t_shared = c["types"]
        a.n_tokens, a.n_exp, a.slots, a.offs = c["n"], c["n_exp"], c["slots"][:c["n_exp"]], list(c["offs"])
        a.tok, a.wt, a.slot_of = q.Buffer.of(keep[0]), q.Buffer.of(keep[1]), q.Buffer.of(keep[2])
        a.k_per_token, a.has_shared, a.shared = c["k"], True, c["slots"][c["n_exp"]]
        a.X, a.Y, a.scratch = q.Buffer.of(Xd), q.Buffer.of(Yd), q.Buffer.of(scratch)
        a.dim, a.inter, a.x_is_bf16 = c["dim"], c["inter"], False
        return a

    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        q.encode_moe_prefill(q.Enc(side), args())  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        q.encode_moe_prefill(q.Enc(torch.cuda.current_stream()), args())
    import gc
    gc.collect()
    for rep in range(4):
        Yd.copy_(up(c["Y0"]))
        scratch.random_(0, 255)  # the header must be rewritten by the replay itself
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(Yd, y_eager), f"replay {rep} differs from the eager result"
        _ = (Xd * 2).sum().item()  # eager work between the replays


def check(c, y, n_check, x_bf16=False):
    n = c["n"]
    if n_check <= 0 or n_check >= n:
        chk = np.arange(n)
    else:
        on = np.zeros(n, bool)
        for j in range(c["n_exp"]):
            if c["offs"][j + 1] - c["offs"][j] <= 2:
                on[c["tok"][c["offs"][j]:c["offs"][j + 1]]] = True
        for t in (0, 15, 16, 31, 32, 47, 48, 63, 64, 65, 127, 128, 511, 512, 513, n - 1):
            if t < n:
                on[t] = True
        on[np.random.default_rng(1).integers(0, n, n_check)] = True
        chk = np.nonzero(on)[0]
    X = c["X"]
    if x_bf16:
        X = (X.view(np.uint32) & 0xFFFF0000).view(np.float32)  # what torch's bf16 cast keeps, up to rounding: use torch
        X = up(c["X"]).to(torch.bfloat16).float().cpu().numpy()
    got = y.cpu().numpy().astype(np.float64)[chk]
    assert np.all(np.isfinite(got))
    gu, dn, sh = c["types"]
    args = (gu, dn, sh, n, c["n_exp"], c["shared"], c["dim"], c["inter"], c["G"], c["U"], c["D"], c["offs"], c["tok"], c["wt"], X, chk)
    Yh, Ym = O.moe_prefill(*args, 1, c["Y0"])
    Yf, _ = O.moe_prefill(*args, 0, c["Y0"])
    err_h = float(np.max(np.abs(got - Yh) / (Ym + 1e-9)))
    err_f = float(np.max(np.abs(got - Yf) / (Ym + 1e-9)))
    return err_h, err_f, len(chk)


T = O
CASES = [  # (gu, down, shared type, n, k, n_exp, shared, routing, dim, inter, n_check)
    (T.IQ1_S, T.IQ1_S, T.Q6_K, 80, 2, 5, True, "popular", 1024, 512, 0),
    (T.IQ2_XXS, T.IQ2_XXS, T.Q8_0, 70, 2, 4, True, "popular", 1024, 512, 0),
    (T.IQ1_S, T.IQ2_XXS, T.Q6_K, 40, 3, 4, False, "popular", 1024, 512, 0),
    (T.IQ1_S, T.IQ1_S, T.Q6_K, 600, 6, 20, True, "sizes", 1024, 512, 40),
    (T.IQ2_XXS, T.IQ1_S, T.Q8_0, 600, 6, 20, True, "sizes", 512, 256, 40),
    (T.IQ1_S, T.IQ2_XXS, T.Q6_K, 256, 6, 64, True, "zipf:0.8", 512, 512, 40),
    (T.IQ2_XXS, T.IQ2_XXS, T.IQ2_XXS, 300, 6, 48, True, "zipf:1.1", 768, 256, 40),
    (T.IQ1_S, T.IQ1_S, T.Q6_K, 48, 2, 5, True, "popular", 5120, 2304, 6),     # reference expert shape
    (T.IQ2_XXS, T.IQ2_XXS, T.IQ2_XXS, 64, 6, 24, False, "zipf:1.1", 7168, 2048, 6),  # BASELINE shape, no shared expert
]


@pytest.mark.parametrize("gu,dn,sh,n,k,n_exp,shared,kind,dim,inter,n_check", CASES)
def test_moe_prefill_vs_oracle(dev, gu, dn, sh, n, k, n_exp, shared, kind, dim, inter, n_check):
    c = build(gu, dn, sh, n, k, n_exp, shared, kind, dim, inter)
    y, same = run_gpu(c)
    err_h, err_f, nc = check(c, y, n_check)
    sizes = np.diff(c["offs"])
    print(f"  gu={O.TYPE_NAMES[gu]} down={O.TYPE_NAMES[dn]} shared={O.TYPE_NAMES[sh] if shared else '-'} {kind} n={n} k={k} "
          f"experts={n_exp} entries={len(c['tok'])} (m {sizes.min()}..{sizes.max()}) {dim}x{inter} checked={nc} "
          f"err(fp16-staged ref) {err_h:.2e} err(vs F32) {err_f:.2e} {'repeat bit-identical' if same else 'REPEAT DIFFERS'}")
    # reference bounds (tests/test_quant_moe_prefill.mm:223): 1e-3 against the half-emulating reference (which also
    # rounds weights, this kernel does not), 5e-3 against F32
    assert same and err_h <= 1e-3 and err_f <= 5e-3


def test_bf16_activations_and_edge_cases(dev):
    c = build(O.IQ2_XXS, O.IQ2_XXS, O.IQ2_XXS, 50, 3, 6, False, "zipf:1.1", 512, 256)
    y, same = run_gpu(c, x_bf16=True)
    err_h, err_f, _ = check(c, y, 0, x_bf16=True)
    assert same and err_h <= 1e-3 and err_f <= 5e-3
    # tokens routed to no expert keep their Y; n_exp = 0 with a shared expert; n_tokens = 0 is a silent no-op
    c = build(O.IQ1_S, O.IQ1_S, O.Q8_0, 20, 2, 3, False, "popular", 512, 256)
    c["slot_of"][:] = -1          # reduction sees no entries at all
    y, same = run_gpu(c)
    assert same and np.array_equal(y.cpu().numpy(), c["Y0"])
    c = build(O.IQ1_S, O.IQ1_S, O.Q8_0, 33, 2, 3, True, "popular", 512, 256)
    c2 = dict(c, n_exp=0, offs=[0], tok=np.zeros(0, np.int32), wt=np.zeros(0, np.float32), slot_of=-np.ones(33 * 2, np.int32),
              G=c["G"][3:], U=c["U"][3:], D=c["D"][3:], slots=c["slots"][3:])
    y, same = run_gpu(c2)
    err_h, err_f, _ = check(c2, y, 0)
    assert same and err_h <= 1e-3
    a = q.MoePrefillArgs()
    a.n_tokens = 0
    q.encode_moe_prefill(q.Enc(), a)


def test_moe_prefill_misuse(dev):
    c = build(O.IQ1_S, O.IQ1_S, O.Q8_0, 8, 2, 3, True, "popular", 512, 256)
    dev_buf = q.Buffer.of(torch.zeros(1 << 16, dtype=torch.uint8, device=dev))
    a = q.MoePrefillArgs()
    a.n_tokens, a.n_exp, a.slots, a.offs = 8, 3, c["slots"][:3], c["offs"]
    a.shared, a.t_shared, a.dim, a.inter, a.k_per_token = c["slots"][3], q.QType.Q8_0, 512, 256, 2
    a.tok = a.wt = a.slot_of = a.X = a.Y = dev_buf
    a.scratch = dev_buf.sub(0, 1024)
    with pytest.raises(q.QuantError, match="moe_prefill scratch too small"):
        q.encode_moe_prefill(q.Enc(), a)
    a.t_gate_up = q.QType.Q5_K
    with pytest.raises(q.QuantError, match="moe_prefill types unsupported"):
        q.encode_moe_prefill(q.Enc(), a)


def test_moe_prefill_eager_call_while_another_stream_captures(dev):
    """The library forks part of a call onto a stream of its own. While a caller's capture is open that stream belongs
    to the capture; a second call from another stream in that window -- eager, with its own scratch -- must neither be
    swallowed by the capture nor fail: it stays on its caller's stream, runs at once and gives the eager result, and
    the captured graph still replays the eager result afterwards."""
    c = build(O.IQ2_XXS, O.IQ1_S, O.Q8_0, 600, 6, 20, True, "sizes", 512, 256)
    y_eager, same = run_gpu(c)
    assert same
    total = len(c["tok"])
    keep = [up(c["tok"]), up(c["wt"]), up(c["slot_of"])]
    nbytes = q.moe_prefill_scratch_bytes(total, c["n"], c["n_exp"], c["dim"], c["inter"])
    Xd = up(c["X"])
    Y = [up(c["Y0"].copy()) for _ in range(2)]
    scr = [torch.empty(nbytes, dtype=torch.uint8, device="cuda:0") for _ in range(2)]

    def args(i):
        a = q.MoePrefillArgs()
        a.t_gate_up, a.t_down, a.t_shared = c["types"]
        a.n_tokens, a.n_exp, a.slots, a.offs = c["n"], c["n_exp"], c["slots"][:c["n_exp"]], list(c["offs"])
        a.tok, a.wt, a.slot_of = q.Buffer.of(keep[0]), q.Buffer.of(keep[1]), q.Buffer.of(keep[2])
        a.k_per_token, a.has_shared, a.shared = c["k"], True, c["slots"][c["n_exp"]]
        a.X, a.Y, a.scratch = q.Buffer.of(Xd), q.Buffer.of(Y[i]), q.Buffer.of(scr[i])
        a.dim, a.inter, a.x_is_bf16 = c["dim"], c["inter"], False
        return a

    other = torch.cuda.Stream()
    host = torch.empty_like(Y[1], device="cpu").pin_memory()
    want = y_eager.cpu()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, capture_error_mode="relaxed"):
        q.encode_moe_prefill(q.Enc(torch.cuda.current_stream()), args(0))
        # the capture is still open: an eager call on another stream
        q.encode_moe_prefill(q.Enc(other), args(1))
        with torch.cuda.stream(other):
            host.copy_(Y[1], non_blocking=True)
        other.synchronize()
        ran_eagerly = bool(torch.equal(host, want))
    assert ran_eagerly, "the eager call did not run (or ran wrongly) while the other stream was capturing"
    assert torch.equal(Y[0].cpu(), torch.from_numpy(c["Y0"])), "the captured call ran during the capture"
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(Y[0], y_eager)

