#!/usr/bin/env python3
"""Benchmark of the MI355X quantized matvec / MoE hot path. Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload moe_decode|matvec|q8_0]

A "step" is one pass of the hot path over one batch of synthetic input, inputs resident in HBM:
  moe_decode (default; BASELINE configs[2])  one token through a 384-expert MoE layer: 6 routed IQ1_S experts
             (gate/up 2048x7168, down 7168x2048) + 1 shared IQ2_XXS expert, SwiGLU; every step routes to a fresh
             seeded top-6 set and takes the next of 24 copies of the shared expert, so all weights stream from HBM
             (3.3 GB + 0.27 GB resident, far above the last-level cache)
  matvec     (BASELINE configs[1])  one single-expert decode matvec, IQ1_S or IQ2_XXS, 4096x7168, weights rotated
             over >= 2 GiB of distinct copies
  q8_0       (BASELINE configs[0])  Q8_0 4096x4096 matvec, same rotation
`value` is algorithmic bytes / time in GB/s. `roofline` prices the dominant kernel against 8 TB/s HBM from per-launch
HIP-event timings; `cpu_baseline` times the CPU oracle (a port of the reference's CPU path) on this host's cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "MoE decode matvec GB/s (% of HBM peak) + prefill MoE GEMM TFLOP/s (% MFMA)"
HBM_PEAK_GBPS = 8000.0


def profile_traffic(name, line_start):
    """HBM bytes that profiles/<name> records for the line that starts with `line_start`: the summaries of the
    FETCH_SIZE / WRITE_SIZE counter runs give such a line's total as "= <MB> MB per launch" or ": <MB> MB per step" (KiB per
    dispatch scaled by what the same counters read for a 1 GiB copy; the file says how). None when the file or the
    line is missing, so a stale constant can never stand in for a measurement."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", name)) as f:
            for l in f:
                if l.startswith(line_start):
                    m = re.search(r"[=:]\s*([0-9.]+) MB per (?:launch|step)", l)
                    if m:
                        return int(round(float(m.group(1)) * 1e6))
    except OSError:
        pass
    return None


def cores():
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    return max(1, min(n, 16))


def gen_blocks(torch, t, n_blocks, d_sigma, seed, dev):
    """Random GGUF blocks on the device: uniform random bytes, fp16 d = |N(0, d_sigma)| (BASELINE configs[1..2])."""
    from macseek_amd import quant as q
    bb = q.block_bytes(t)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W = torch.randint(0, 256, (n_blocks, bb), dtype=torch.uint8, device=dev, generator=g)
    d = (torch.randn(n_blocks, device=dev, generator=g) * d_sigma).abs()
    if t == q.QType.Q8_0:  # BASELINE configs[0]: d = |N(0, 0.02)| / 127, quants uniform in [-127, 127]
        d = d / 127.0
        qs = torch.randint(-127, 128, (n_blocks, 32), dtype=torch.int8, device=dev, generator=g)
        W[:, 2:34] = qs.view(torch.uint8)
    W[:, 0:2] = d.to(torch.float16).view(torch.uint8).view(n_blocks, 2)
    return W.view(-1)


def event_ms_per_launch(torch, launch, n):
    """Average GPU duration of one launch, from a HIP event pair around each of n launches on the current stream."""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i, (a, b) in enumerate(evs):
        a.record()
        launch(i)
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return float(np.mean(ts)), float(ts[len(ts) // 2]), float(ts[0])


def graph_ms_per_launch(torch, launch, n):
    """Average duration of one launch when launches of the same kernel run back to back: n launches are captured in one
    HIP graph (no host in the loop); after 20 ms of untimed replays, three regions of back-to-back replays, each inside
    one HIP event pair on the replay's stream and at least 10 ms long, are timed; the median region counts."""
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        for i in range(n):
            launch(i)

    def region(replays):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(replays):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b)

    done, spent = 0, 0.0
    while spent < 20.0:
        spent += region(2)
        done += 2
    R = int(min(20000, max(1, -(-10.0 // max(spent / done, 1e-4)))))
    return float(np.median([region(R) / (R * n) for _ in range(3)]))


def timed_graph(torch, enqueue_steps, steps, warmup):
    """Captures `steps` back-to-back steps in one HIP graph (from Python the loop is launch-bound otherwise) and times
    replays of it with HIP events on the replay's stream: after at least `warmup` steps and 50 ms of untimed replays,
    five regions of R back-to-back replays each, every region inside ONE event pair and at least 10 ms long, so that
    neither the host's graph-launch latency nor the clock ramp of an idle device sits in a region. Returns (median
    region in ms per step, all five, R)."""
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue_steps(min(steps, 8))  # library / module bring-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        enqueue_steps(steps)

    def region(replays):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(replays):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b)

    done, spent, reps = 0, 0.0, max(1, -(-warmup // steps))
    while done * steps < warmup or spent < 50.0:
        spent += region(reps)
        done += reps
    per_replay = max(spent / done, 1e-4)
    R = int(min(20000, max(1, -(-10.0 // per_replay))))
    regions = [region(R) / (R * steps) for _ in range(5)]
    return float(np.median(regions)), regions, R


# ------------------------------------------------------------------------------------------------ MoE decode layer
def bench_moe_decode(torch, args):
    from macseek_amd import _lib
    from macseek_amd import quant as q
    import oracle as O
    dev = torch.device("cuda:0")
    L = _lib.load()
    DIM, INTER, NE, TOPK = 7168, 2048, 384, 6
    tr, ts = q.QType.IQ1_S, q.QType.IQ2_XXS
    gu_b, dn_b = q.row_bytes(tr, DIM) * INTER, q.row_bytes(tr, INTER) * DIM
    sgu_b, sdn_b = q.row_bytes(ts, DIM) * INTER, q.row_bytes(ts, INTER) * DIM
    per_exp = 2 * gu_b + dn_b
    arena = gen_blocks(torch, tr, NE * per_exp // 50, 0.01, 1, dev)
    # the shared expert in N_SHARED distinct copies, one per step in turn: like the routed experts it then streams from
    # HBM (a 40-layer token loop never finds a layer's shared expert in the 256 MB last-level cache either)
    N_SHARED = 24
    sh_b = 2 * sgu_b + sdn_b
    shared = gen_blocks(torch, ts, N_SHARED * sh_b // 66, 0.01, 2, dev)
    base = arena.data_ptr()
    n_sets = max(args.steps, 64)
    # seeded fp32 router: logits ~ N(0,1) over 384 experts, top-6, weights = softmax over the selected logits
    rng = np.random.default_rng(1234)
    logits = rng.standard_normal((n_sets, NE)).astype(np.float32)
    ids = np.argsort(-logits, axis=1)[:, :TOPK]
    sel = np.take_along_axis(logits, ids, axis=1)
    wts = np.exp(sel - sel.max(1, keepdims=True))
    wts = (wts / wts.sum(1, keepdims=True)).astype(np.float32)
    tables = np.zeros((n_sets, 18), dtype=np.uint64)
    for k in range(TOPK):
        e0 = base + ids[:, k].astype(np.uint64) * np.uint64(per_exp)
        tables[:, 3 * k] = e0
        tables[:, 3 * k + 1] = e0 + np.uint64(gu_b)
        tables[:, 3 * k + 2] = e0 + np.uint64(2 * gu_b)
    tables_d = torch.from_numpy(tables.view(np.int64)).to(dev)
    wts_d = torch.from_numpy(wts).to(dev)
    x = torch.randn(DIM, device=dev)
    y = torch.zeros(DIM, device=dev)
    scratch = torch.zeros(q.moe_decode_scratch_bytes(INTER) // 4, device=dev)

    sh = q.Buffer.of(shared)
    calls = []
    for i in range(n_sets):
        a = q.MoeDecodeArgs()
        a.t_gate_up = a.t_down = tr
        a.t_shared, a.n_routed, a.has_shared, a.dim, a.inter = ts, TOPK, True, DIM, INTER
        so = (i % N_SHARED) * sh_b
        a.shared = q.ExpertSlot(sh.sub(so, sgu_b), sh.sub(so + sgu_b, sgu_b), sh.sub(so + 2 * sgu_b, sdn_b))
        a.weights = q.Buffer.of(wts_d).sub(i * 24, 24)
        a.x, a.y, a.scratch = q.Buffer.of(x), q.Buffer.of(y), q.Buffer.of(scratch)
        calls.append((a.c(), q.Buffer.of(tables_d).sub(i * 144, 144).c()))

    def run_part(i, part):
        ca, tb = calls[i % n_sets]
        rc = L.msq_moe_decode_table_part(C.c_void_p(torch.cuda.current_stream().cuda_stream), C.byref(ca), C.byref(tb), part)
        if rc != 0:
            raise RuntimeError(L.msq_last_error().decode())

    def enqueue(n):
        for i in range(n):
            run_part(i, q.MoePart.All)

    ms_step, ms_reps, replays = timed_graph(torch, enqueue, args.steps, args.warmup)
    w_bytes = TOPK * per_exp + 2 * sgu_b + sdn_b
    h_bytes = (TOPK + 1) * INTER * 4
    step_bytes = w_bytes + DIM * 4 + 2 * h_bytes + 2 * DIM * 4
    value = step_bytes / (ms_step * 1e-3) / 1e9

    # dominant kernel = gate/up (two thirds of the bytes): per-launch HIP-event timing of that kernel alone
    n_ev = min(max(args.steps, 50), 400)
    gu_mean, gu_med, gu_min = event_ms_per_launch(torch, lambda i: run_part(i, q.MoePart.Gu), n_ev)
    dn_mean, dn_med, dn_min = event_ms_per_launch(torch, lambda i: run_part(i, q.MoePart.Down), n_ev)
    # eager event pairs also bracket the host's launch latency whenever the queue runs dry; the graph figure does not
    gu_graph = graph_ms_per_launch(torch, lambda i: run_part(i, q.MoePart.Gu), n_ev)
    dn_graph = graph_ms_per_launch(torch, lambda i: run_part(i, q.MoePart.Down), n_ev)
    # h leaves gate/up as fp32 and as fp16 (6 bytes a value); down reads the fp16 copy (2 bytes a value)
    gu_bytes = TOPK * 2 * gu_b + 2 * sgu_b + DIM * 4 + h_bytes * 3 // 2
    dn_bytes = TOPK * dn_b + sdn_b + h_bytes // 2 + 2 * DIM * 4
    achieved = gu_bytes / (gu_graph * 1e-3) / 1e9

    # parity spot check of the last state against the oracle is the tests' job; here only the CPU baseline leg
    nth = cores()
    i0 = 0
    host = lambda t_: t_.cpu().numpy()
    G, U, D = [], [], []
    for k in range(TOPK):
        o = int(ids[i0, k]) * per_exp
        G.append(host(arena[o:o + gu_b])); U.append(host(arena[o + gu_b:o + 2 * gu_b])); D.append(host(arena[o + 2 * gu_b:o + per_exp]))
    G.append(host(shared[:sgu_b])); U.append(host(shared[sgu_b:2 * sgu_b])); D.append(host(shared[2 * sgu_b:sh_b]))
    xh = host(x)
    t0 = time.perf_counter()
    n_cpu = 0
    while not args.gpu_only:
        O.moe_decode(int(tr), int(tr), int(ts), TOPK, True, DIM, INTER, G, U, D, wts[i0], xh, np.zeros(DIM, np.float32), nthreads=nth)
        n_cpu += 1
        el = time.perf_counter() - t0
        if el > 10.0 or n_cpu >= 200:
            break
    el = time.perf_counter() - t0
    cpu_value = step_bytes * n_cpu / el / 1e9 if n_cpu else None
    # the reference's own form of the CPU path is single-threaded (tests/ref/dequant.cpp:122-131): same port, one thread
    t1 = time.perf_counter()
    n_cpu1 = 0
    while not args.gpu_only:
        O.moe_decode(int(tr), int(tr), int(ts), TOPK, True, DIM, INTER, G, U, D, wts[i0], xh, np.zeros(DIM, np.float32), nthreads=1)
        n_cpu1 += 1
        if time.perf_counter() - t1 > 8.0 or n_cpu1 >= 50:
            break
    el1 = time.perf_counter() - t1
    cpu_value1 = step_bytes * n_cpu1 / el1 / 1e9 if n_cpu1 else None
    # what this device gives a kernel that only reads, at the layer's and the dominant kernel's size and at 1 GiB
    stream = None
    if not args.gpu_only:
        del G, U, D
        s_layer, s_gu, s_big = (stream_read_GBps(torch, b, arena) for b in (step_bytes, gu_bytes, 1 << 30))
        stream = {"read_GBps_at_layer_bytes": s_layer, "read_GBps_at_kernel_bytes": s_gu, "read_GBps_at_1GiB": s_big,
                  "layer_pct_of_stream_read": 100 * value / s_layer, "kernel_pct_of_stream_read": 100 * achieved / s_gu,
                  "layer_pct_of_1GiB_stream_read": 100 * value / s_big}

    return {
        "value": value, "ms_per_step": ms_step, "ms_per_step_of_each_region": ms_reps, "replays_timed": replays,
        "timing": "median of five regions, each %d back-to-back replays of a %d-step HIP graph inside one HIP event pair" % (replays, args.steps),
        "dtype": "int8 IQ1_S codebook x 16-bit block-fixed-point activations (i32, gate/up), f16 x f16 (IQ2_XXS shared expert, down); f32 accumulate",
        "config": {"workload": "BASELINE configs[2]: batch-1 MoE decode layer, 384 experts IQ1_S 7168x2048 (3.3 GB resident), "
                               "top-6 of a seeded softmax router + 1 shared IQ2_XXS expert, SwiGLU; fresh top-6 per step",
                   "bytes_per_step": step_bytes, "experts": NE, "top_k": TOPK, "dim": DIM, "inter": INTER},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": profile_traffic("moe_hbm_traffic_fetch_write.txt", "moe_gu_kernel<"), "traffic_source": "profiles/moe_hbm_traffic_fetch_write.txt", "kernel": "moe_gu_kernel<DecIQ1SQ,DecIQ2XXSQ>", "bytes_per_launch": gu_bytes,
                     "avg_launch_us": gu_graph * 1e3,
                     "timing": "HIP event pair around one graph replay of %d back-to-back launches of this kernel" % n_ev,
                     "eager_event_pair_us": {"mean": gu_mean * 1e3, "median": gu_med * 1e3, "min": gu_min * 1e3},
                     "second_kernel": {"kernel": "moe_down_kernel<DecIQ1S,DecIQ2XXS>", "bytes_per_launch": dn_bytes,
                                       "avg_launch_us": dn_graph * 1e3, "achieved": dn_bytes / (dn_graph * 1e-3) / 1e9,
                                       "eager_event_pair_us": {"mean": dn_mean * 1e3, "median": dn_med * 1e3, "min": dn_min * 1e3}}},
        "cpu_baseline": {"value": cpu_value, "unit": "GB/s", "cores": nth, "kind": "port",
                         "sample": "%d tokens of the same layer (token 0's experts) through oracle.c moe_decode, %.1f s" % (n_cpu, el),
                         "one_thread": {"value": cpu_value1, "cores": 1,
                                        "sample": "%d tokens, %.1f s (the form of the reference's own CPU path)" % (n_cpu1, el1)}},
        "pct_of_hbm_peak": 100 * value / HBM_PEAK_GBPS,
        "stream_read_reference": stream,
    }


# ------------------------------------------------------------------------------------------------ single matvec
def bench_matvec(torch, args, t, rows, cols, d_sigma, label):
    from macseek_amd import _lib
    from macseek_amd import quant as q
    import oracle as O
    dev = torch.device("cuda:0")
    L = _lib.load()
    mat_b = q.row_bytes(t, cols) * rows
    copies = max(2, -(-(2 << 30) // mat_b))
    arena = gen_blocks(torch, t, copies * mat_b // q.block_bytes(t), d_sigma, 3, dev)
    x = torch.randn(cols, device=dev)
    y = torch.zeros(rows, device=dev)
    Wb = [q.Buffer.of(arena).sub(i * mat_b, mat_b).c() for i in range(copies)]
    xb, yb = q.Buffer.of(x).c(), q.Buffer.of(y).c()

    def launch(i):
        rc = L.msq_matvec(C.c_void_p(torch.cuda.current_stream().cuda_stream), int(t), C.byref(Wb[i % copies]), rows, cols,
                          C.byref(xb), C.byref(yb), 0, 1, None)
        if rc != 0:
            raise RuntimeError(L.msq_last_error().decode())

    ms_step, ms_reps, replays = timed_graph(torch, lambda n: [launch(i) for i in range(n)], args.steps, args.warmup)
    step_bytes = mat_b + 4 * cols + 4 * rows
    value = step_bytes / (ms_step * 1e-3) / 1e9
    e_mean, e_med, e_min = event_ms_per_launch(torch, launch, min(max(args.steps, 50), 400))
    k_mean = graph_ms_per_launch(torch, launch, 400)  # an eager event pair brackets the host's launch latency as well
    achieved = step_bytes / (k_mean * 1e-3) / 1e9
    nth = cores()
    Wh, xh = arena[:mat_b].cpu().numpy(), x.cpu().numpy()
    t0 = time.perf_counter()
    n_cpu = 0
    while True:
        O.matvec(int(t), Wh, rows, cols, xh, 1, nthreads=nth)
        n_cpu += 1
        el = time.perf_counter() - t0
        if el > (0.2 if args.gpu_only else 10.0) or n_cpu >= 2000:  # profiling runs: a token CPU leg
            break
    t1 = time.perf_counter()
    n_cpu1 = 0
    while True:  # the reference's own CPU path is single-threaded (tests/ref/dequant.cpp:122-131)
        O.matvec(int(t), Wh, rows, cols, xh, 1, nthreads=1)
        n_cpu1 += 1
        el1 = time.perf_counter() - t1
        if el1 > (0.2 if args.gpu_only else 5.0) or n_cpu1 >= 500:
            break
    s_read = stream_read_GBps(torch, step_bytes, arena)
    return {
        "value": value, "ms_per_step": ms_step, "ms_per_step_of_each_region": ms_reps, "replays_timed": replays,
        "dtype": "f32" if t == q.QType.Q8_0 else "f16 activations, f32 accumulate",
        "config": {"workload": label, "bytes_per_step": step_bytes, "rows": rows, "cols": cols, "weight_copies": copies},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": None, "kernel": "decode matvec <%s> (mv_tok_kernel, mv_kernel or mv_ring_kernel by shape)" % q.type_name(t),
                     "bytes_per_launch": step_bytes, "avg_launch_us": k_mean * 1e3,
                     "timing": "HIP event pair around one graph replay of 400 back-to-back launches",
                     "eager_event_pair_us": {"mean": e_mean * 1e3, "median": e_med * 1e3, "min": e_min * 1e3}},
        "cpu_baseline": {"value": step_bytes * n_cpu / el / 1e9, "unit": "GB/s", "cores": nth, "kind": "port",
                         "sample": "%d matvecs of the same matrix through oracle.c (dequant row + double dot), %.1f s" % (n_cpu, el),
                         "one_thread": {"value": step_bytes * n_cpu1 / el1 / 1e9, "cores": 1, "sample": "%d matvecs, %.1f s" % (n_cpu1, el1)}},
        "pct_of_hbm_peak": 100 * value / HBM_PEAK_GBPS,
        "stream_read_reference": {"read_GBps_at_step_bytes": s_read, "pct_of_stream_read": 100 * achieved / s_read},
    }


# ------------------------------------------------------------------------------------------------ prefill grouped GEMM
MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 / bf16 matrix-core peak


def zipf_routing(n, n_exp, k, s, seed):
    """top-k distinct experts per token, popularity ~ rank^-s over a seeded expert permutation (bench/qmatmul.mm:135-152)."""
    rng = np.random.default_rng(seed)
    pw = np.zeros(n_exp)
    pw[rng.permutation(n_exp)] = 1.0 / np.arange(1, n_exp + 1) ** s
    # Gumbel top-k = sampling without replacement proportional to pw
    g = np.log(pw)[None, :] + rng.gumbel(size=(n, n_exp))
    ids = np.argsort(-g, axis=1)[:, :k]
    w = rng.random((n, k)).astype(np.float32) + 0.1
    w = w / w.sum(1, keepdims=True)  # renormalised routing weights
    return ids, w


def bench_moe_prefill(torch, steps, warmup, with_cpu=True):
    from macseek_amd import _lib
    from macseek_amd import quant as q
    import oracle as O
    dev = torch.device("cuda:0")
    L = _lib.load()
    N, DIM, INTER, NE, TOPK = 2048, 7168, 2048, 384, 6
    t = q.QType.IQ2_XXS
    gu_b, dn_b = q.row_bytes(t, DIM) * INTER, q.row_bytes(t, INTER) * DIM
    per_exp = 2 * gu_b + dn_b
    arena = gen_blocks(torch, t, NE * per_exp // 66, 0.01, 7, dev)
    ids, w = zipf_routing(N, NE, TOPK, 1.1, 4321)
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
    a.slots = [q.ExpertSlot(A.sub(int(e) * per_exp, gu_b), A.sub(int(e) * per_exp + gu_b, gu_b), A.sub(int(e) * per_exp + 2 * gu_b, dn_b)) for e in used]
    a.offs = [int(v) for v in offs]
    X = torch.randn(N, DIM, device=dev).to(torch.bfloat16)
    Y = torch.zeros(N, DIM, device=dev)
    tok_d, wt_d, slot_d = torch.from_numpy(tok).to(dev), torch.from_numpy(wt).to(dev), torch.from_numpy(slot_of).to(dev)
    scratch = torch.empty(q.moe_prefill_scratch_bytes(total, N, len(used), DIM, INTER), dtype=torch.uint8, device=dev)
    a.tok, a.wt, a.slot_of, a.X, a.Y, a.scratch = (q.Buffer.of(v) for v in (tok_d, wt_d, slot_d, X, Y, scratch))
    ca = a.c()

    def call():
        rc = L.msq_moe_prefill(C.c_void_p(torch.cuda.current_stream().cuda_stream), C.byref(ca))
        if rc != 0:
            raise RuntimeError(L.msq_last_error().decode())

    for _ in range(max(3, warmup)):
        call()
    torch.cuda.synchronize()
    steps = max(steps, 4)  # a timed region of at least 10 ms
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(steps):
        call()
    ev1.record()
    torch.cuda.synchronize()
    ms_step = ev0.elapsed_time(ev1) / steps
    flops = 2.0 * 3 * DIM * INTER * total
    value = flops / (ms_step * 1e-3) / 1e12
    # dominant kernel: the routed gate/up GEMM (two thirds of the FLOPs), timed alone through the phase skip mask
    os.environ["MSQ_MOEP_SKIP"] = str(1 | 4 | 8 | 16 | 32)
    gu_mean, gu_med, gu_min = event_ms_per_launch(torch, lambda i: call(), max(3, min(steps, 10)))
    os.environ["MSQ_MOEP_SKIP"] = str(1 | 2 | 4 | 16 | 32)
    dn_mean, _, _ = event_ms_per_launch(torch, lambda i: call(), max(3, min(steps, 10)))
    # the item classes of the gate/up GEMM on their own: one-tile items, two- and three-tile items (one launch together
    # otherwise), popular experts' blocks
    split = {}
    for name, keep in (("one_tile_items", 64), ("two_three_tile_items", 128), ("blocks_of_popular_experts", 256)):
        os.environ["MSQ_MOEP_SKIP"] = str((1 | 4 | 8 | 16 | 32) | ((64 | 128 | 256) & ~keep))
        split[name + "_us"] = event_ms_per_launch(torch, lambda i: call(), 3)[0] * 1e3
    os.environ["MSQ_MOEP_SKIP"] = "0"
    n_one = int(np.sum((counts[used] <= 16)))
    n_mid = int(np.sum((counts[used] > 16) & (counts[used] <= 48)))
    split["experts_by_class"] = {"one_tile": n_one, "two_three_tiles": n_mid, "more": int(len(used)) - n_one - n_mid}
    split["entries_by_class"] = {"one_tile": int(counts[used][counts[used] <= 16].sum()),
                                 "two_three_tiles": int(counts[used][(counts[used] > 16) & (counts[used] <= 48)].sum()),
                                 "more": int(counts[used][counts[used] > 48].sum())}
    gu_flops = 2.0 * 2 * DIM * INTER * total
    achieved = gu_flops / (gu_mean * 1e-3) / 1e12
    out = {
        "value": value, "unit": "TFLOP/s", "ms_per_step": ms_step, "dtype": "f16 MFMA (bf16 activations staged as f16, IQ2_XXS weights dequantized to f16 tiles), f32 accumulate",
        "config": {"workload": "BASELINE configs[3]: prefill grouped MoE GEMM, 2048 tokens x 7168 bf16, top-6 of 384 experts, "
                               "Zipf(1.1) popularity, IQ2_XXS gate/up 2048x7168 + down 7168x2048, outputs combined with routing weights",
                   "entries": total, "experts_used": int(len(used)), "tokens_per_expert_max": int(counts.max()),
                   "tokens_per_expert_median": float(np.median(counts[used])), "flops_per_step": flops,
                   "weight_bytes_touched": int(len(used)) * per_exp},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS,
                     "traffic": profile_traffic("moe_prefill_hbm_traffic_fetch_write.txt", "gate/up ("), "traffic_source": "profiles/moe_prefill_hbm_traffic_fetch_write.txt",
                     "kernel": "moe_pf_block_kernel<BlkIQ2XXS, gate/up> (two launches: blocks of 49..112 entries of the popular experts; items of one to three token tiles)",
                     "gate_up_time_split": split,
                     "flops_per_launch": gu_flops,
                     "avg_launch_us": gu_mean * 1e3, "min_launch_us": gu_min * 1e3,
                     "weight_GBps": int(len(used)) * 2 * gu_b / (gu_mean * 1e-3) / 1e9,
                     "second_kernel": {"kernel": "moe_pf_block_kernel<BlkIQ2XXS, down> (two launches)", "avg_launch_us": dn_mean * 1e3,
                                       "achieved": 2.0 * DIM * INTER * total / (dn_mean * 1e-3) / 1e12}},
        "pct_of_mfma_peak": 100 * value / MFMA_PEAK_TFLOPS,
    }
    if with_cpu:
        nth = cores()
        n_chk = 4
        chk = np.arange(n_chk, dtype=np.int32)
        need = sorted(set(int(e) for e in ids[:n_chk].ravel()))
        host = {e: (arena[e * per_exp:e * per_exp + gu_b].cpu().numpy(), arena[e * per_exp + gu_b:e * per_exp + 2 * gu_b].cpu().numpy(),
                    arena[e * per_exp + 2 * gu_b:(e + 1) * per_exp].cpu().numpy()) for e in need}
        dummy = host[need[0]]
        G = [host.get(int(e), dummy)[0] for e in used]; U = [host.get(int(e), dummy)[1] for e in used]; D = [host.get(int(e), dummy)[2] for e in used]
        Xh = X.float().cpu().numpy()
        t0 = time.perf_counter()
        O.moe_prefill(int(t), int(t), int(t), N, len(used), False, DIM, INTER, G, U, D, offs, tok, wt, Xh, chk, 1,
                      np.zeros((N, DIM), np.float32), nthreads=nth)
        el = time.perf_counter() - t0
        cpu_flops = 2.0 * 3 * DIM * INTER * n_chk * TOPK
        t1 = time.perf_counter()
        O.moe_prefill(int(t), int(t), int(t), N, len(used), False, DIM, INTER, G, U, D, offs, tok, wt, Xh, chk[:1], 1,
                      np.zeros((N, DIM), np.float32), nthreads=1)
        el1 = time.perf_counter() - t1
        out["cpu_baseline"] = {"value": cpu_flops / el / 1e12, "unit": "TFLOP/s", "cores": nth, "kind": "port",
                               "sample": "%d tokens x top-6 of the same routing through oracle.c moe_prefill (dequant each needed "
                                         "expert row, double dots), %.1f s; whole job = x%d" % (n_chk, el, N // n_chk),
                               "one_thread": {"value": cpu_flops / n_chk / el1 / 1e12, "cores": 1, "sample": "1 token x top-6, %.1f s" % el1}}
    return out


# ------------------------------------------------------------------------------------------------ stream / copy references
def stream_read_GBps(torch, nbytes, arena=None):
    """What a kernel that only reads (msq_bw_probe) gets for `nbytes` per launch, launches back to back over distinct memory."""
    from macseek_amd import _lib
    from macseek_amd import quant as q
    L = _lib.load()
    dev = torch.device("cuda:0")
    if arena is None:
        arena = torch.randint(0, 256, (2 << 30,), dtype=torch.uint8, device=dev)
    sink = torch.zeros(4096, dtype=torch.uint8, device=dev)
    sb = q.Buffer.of(sink).c()
    nbytes = int(nbytes) // 4096 * 4096
    ncopies = max(1, arena.numel() // nbytes)
    bufs = [q.Buffer.of(arena).sub(i * nbytes, nbytes).c() for i in range(ncopies)]

    def launch(i):
        rc = L.msq_bw_probe(C.c_void_p(torch.cuda.current_stream().cuda_stream), C.byref(bufs[i % ncopies]), nbytes, C.byref(sb))
        if rc != 0:
            raise RuntimeError(L.msq_last_error().decode())
    ms = graph_ms_per_launch(torch, launch, min(200, max(20, 3 * ncopies)))
    return nbytes / (ms * 1e-3) / 1e9


def bench_stream(torch, args):
    """Plain streaming reads (msq_bw_probe: every lane sums 128-bit loads) at a few sizes: what this device delivers to
    a kernel that does nothing but read, next to the 8 TB/s the rooflines are priced against."""
    from macseek_amd import _lib
    from macseek_amd import quant as q
    L = _lib.load()
    dev = torch.device("cuda:0")
    arena = torch.randint(0, 256, (3 << 30,), dtype=torch.uint8, device=dev)
    sink = torch.zeros(4096, dtype=torch.uint8, device=dev)
    sb = q.Buffer.of(sink).c()
    rows = []
    for mb in (21, 42, 63, 256, 1024):
        nbytes = mb << 20
        ncopies = (3 << 30) // nbytes  # successive launches read different memory: nothing is served from a cache
        bufs = [q.Buffer.of(arena).sub(i * nbytes, nbytes).c() for i in range(ncopies)]

        def launch(i):
            rc = L.msq_bw_probe(C.c_void_p(torch.cuda.current_stream().cuda_stream), C.byref(bufs[i % ncopies]), nbytes, C.byref(sb))
            if rc != 0:
                raise RuntimeError(L.msq_last_error().decode())
        ms = graph_ms_per_launch(torch, launch, min(200, max(20, 3 * ncopies)))
        rows.append({"MiB": mb, "us_per_launch": ms * 1e3, "GBps": nbytes / (ms * 1e-3) / 1e9})
    best = max(r["GBps"] for r in rows)
    return {"value": best, "ms_per_step": rows[-1]["us_per_launch"] * 1e-3, "dtype": "u8",
            "config": {"workload": "streaming read probe (bw_probe_kernel), sizes in MiB, launches back to back in a graph", "sizes": rows},
            "roofline": {"bound": "hbm", "achieved": best, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": best / HBM_PEAK_GBPS,
                         "traffic": None, "kernel": "bw_probe_kernel"},
            "cpu_baseline": None, "pct_of_hbm_peak": 100 * best / HBM_PEAK_GBPS}


def bench_issue_probe(torch, args):
    """Instruction-issue probes (libmsq_probe.so, a measurement tool outside the library): ns per instruction group and SIMD for vector ops, matrix-core ops and
    LDS reads, alone and interleaved, at 1, 2 and 4 waves per SIMD (one workgroup per CU) and 8 (two workgroups)."""
    from macseek_amd import build as B
    if not os.path.exists(B.PROBE_OUT):
        raise RuntimeError("bench.py: %s is missing; build it with `python -m macseek_amd.build`" % B.PROBE_OUT)
    P = C.CDLL(B.PROBE_OUT)  # the probe is no part of libmsq.so
    P.msq_probe_issue.restype = C.c_int
    P.msq_probe_issue.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t]
    dev = torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.zeros(4 * cus * 4, dtype=torch.uint8, device=dev)
    VALU, MFMA16, MFMA4, MFMA8, LDS, VINT, VPK, VFMA = 1, 2, 4, 8, 16, 32, 64, 128
    mixes = [("valu32", VALU), ("mfma16_f16_x8", MFMA16), ("mfma_fp4_fp6_x8", MFMA4), ("mfma_fp8_x8", MFMA8), ("lds_b32_x16", LDS),
             ("valu32+mfma16_f16_x8", VALU | MFMA16), ("valu32+mfma_fp4_fp6_x8", VALU | MFMA4), ("valu32+lds_b32_x16", VALU | LDS),
             ("valu32+lds_b32_x16+mfma_fp4_fp6_x8", VALU | LDS | MFMA4), ("vint32", VINT), ("vint32+mfma16_f16_x8", VINT | MFMA16),
             ("vpk32", VPK), ("vpk32+mfma16_f16_x8", VPK | MFMA16), ("vfma32", VFMA), ("vfma32+mfma16_f16_x8", VFMA | MFMA16)]
    iters = 4096
    rows = []
    for wps, grid, block in ((1, cus, 256), (2, cus, 512), (4, cus, 1024), (8, 2 * cus, 1024)):
        row = {"waves_per_simd": wps}
        for name, mask in mixes:
            def launch(i):
                rc = P.msq_probe_issue(C.c_void_p(torch.cuda.current_stream().cuda_stream), mask, grid, block, iters,
                                       C.c_void_p(sink.data_ptr()), sink.numel())
                if rc != 0:
                    raise RuntimeError("msq_probe_issue failed: %d" % rc)
            ms = graph_ms_per_launch(torch, launch, 3)
            # one iteration of one wave = one group set; a SIMD runs wps waves: ns per group set and SIMD
            row[name] = round(ms * 1e6 / iters / wps, 2)
        rows.append(row)
    v = rows[2]["valu32"] / 32.0
    return {"value": 0.0, "ms_per_step": 0.0, "dtype": "instruction issue",
            "config": {"workload": "issue probes: ns per SIMD for one group set of a wave (valu32 = 32 vector ops, mfma*_x8 = 8 matrix ops, "
                                   "lds_b32_x16 = 16 random ds_read_b32 + 16 v_xor), by waves per SIMD", "rows": rows,
                       "ns_per_valu_issue_at_4_waves": round(v, 3)},
            "roofline": None, "cpu_baseline": None, "pct_of_hbm_peak": None}


def bench_lds_bank_probe(torch, args):
    """Which lanes of a wave the LDS serves in the same pass (libmsq_probe.so: lds_bank_probe_kernel). Lane l reads at
    256 l + 16 slot(l): two lanes collide exactly when their slots are equal, so a slot pattern that runs at the rate of
    distinct slots names lanes that never share a pass. The last rows check the resulting model for 16-byte reads --
    groups {0-7, 24-31}, {8-15, 16-23}, {32-39, 56-63}, {40-47, 48-55} -- against the activation layouts of the prefill
    kernels before and after they were changed to it."""
    from macseek_amd import build as B
    if not os.path.exists(B.PROBE_OUT):
        raise RuntimeError("bench.py: %s is missing; build it with `python -m macseek_amd.build`" % B.PROBE_OUT)
    P = C.CDLL(B.PROBE_OUT)
    P.msq_probe_lds_bank.restype = C.c_int
    P.msq_probe_lds_bank.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int]
    dev = torch.device("cuda:0")
    out = torch.zeros(2, dtype=torch.int64, device=dev)
    lane = lambda f: [256 * l + 16 * f(l) for l in range(64)]
    frag = lambda f: [f(l & 15, l >> 4) for l in range(64)]  # lane = 16 chunk + token, as the matrix fragments are read
    pats = [("distinct slots in every 16 lanes (l % 16)", lane(lambda l: l % 16)),
            ("all lanes one slot", lane(lambda l: 0)),
            ("aligned quads share (l / 4)", lane(lambda l: l // 4)),
            ("l, l+8 share and l, l+32 share (l % 8 + 8 (l / 16 % 2))", lane(lambda l: l % 8 + 8 * (l // 16 % 2))),
            ("l, l+8, l+16, l+24 share (l % 8 + 8 (l / 32 % 2))", lane(lambda l: l % 8 + 8 * (l // 32 % 2))),
            ("l, l+4, l+8, l+12 share (l % 4 + 4 (l / 16))", lane(lambda l: l % 4 + 4 * (l // 16))),
            ("neighbours share (l % 32 / 2)", lane(lambda l: l % 32 // 2)),
            ("fragment rows 528 B apart, chunks 128 B apart (prefill GEMM, old)", frag(lambda n, q: n * 528 + 128 * q)),
            ("fragment rows 528 B apart, chunks at 0, 256, 128, 384 (prefill GEMM, now)", frag(lambda n, q: n * 528 + 256 * (q & 1) + 128 * (q >> 1))),
            ("fragment rows 272 B apart, chunks 16 B apart (fused matmul)", frag(lambda n, q: n * 272 + 16 * q)),
            ("fragment rows 256 B apart, slot = chunk ^ token (tile matmul)", frag(lambda n, q: n * 256 + 16 * (q ^ n)))]
    iters, rows = 400, []
    for width in (16, 8, 4):
        for name, addr in pats:
            a = torch.tensor(addr, dtype=torch.int32, device=dev)
            for _ in range(2):
                rc = P.msq_probe_lds_bank(C.c_void_p(torch.cuda.current_stream().cuda_stream), width, C.c_void_p(a.data_ptr()),
                                          C.c_void_p(out.data_ptr()), iters)
                if rc != 0:
                    raise RuntimeError("msq_probe_lds_bank failed: %d" % rc)
                torch.cuda.synchronize()
            rows.append({"bytes_per_lane": width, "pattern": name, "cycles_per_wave_read": round(float(out[0].item()) / (iters * 16 * 8), 2)})
    for r in rows:
        sys.stderr.write("%2d B  %-78s %6.2f\n" % (r["bytes_per_lane"], r["pattern"], r["cycles_per_wave_read"]))
    return {"value": 0.0, "ms_per_step": 0.0, "dtype": "LDS reads",
            "config": {"workload": "LDS bank probe: cycles per wave-wide read with the LDS saturated by eight waves, by lane -> address pattern", "rows": rows},
            "roofline": None, "cpu_baseline": None, "pct_of_hbm_peak": None}


def bench_handover_probe(torch, args):
    """What a device-wide hand-over inside one launch costs (libmsq_probe.so: handover_probe_kernel), the step a
    single-launch MoE layer needs between gate/up and down: per workgroup, microseconds from its start until its h
    stores are acknowledged, its arrival is counted, all 256 arrivals are seen, and all of h (28 KB) has been read back
    with device-scope loads; flat counter and two-level (per-XCD) counter, median and slowest workgroup over 50 launches."""
    from macseek_amd import build as B
    P = C.CDLL(B.PROBE_OUT)
    P.msq_probe_handover.restype = C.c_int
    P.msq_probe_handover.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_uint32, C.c_int, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
    dev = torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    h_words = 7 * 2048 // 2  # seven h rows of 2048 values as fp16
    h = torch.zeros(h_words, dtype=torch.int32, device=dev)
    out = torch.zeros(5 * cus, dtype=torch.int64, device=dev)
    sink = torch.zeros(cus, dtype=torch.int32, device=dev)
    res = {}
    for mode, name in ((0, "flat_counter"), (1, "two_level_counter")):
        rows = []
        for epoch in range(60):
            rc = P.msq_probe_handover(C.c_void_p(torch.cuda.current_stream().cuda_stream), cus, C.c_void_p(h.data_ptr()), h_words, mode, epoch,
                                      20000, C.c_void_p(out.data_ptr()), C.c_void_p(sink.data_ptr()))
            if rc != 0:
                raise RuntimeError("msq_probe_handover failed: %d" % rc)
            torch.cuda.synchronize()
            o = out.cpu().numpy().reshape(cus, 5)
            if not o[:, 4].all():
                raise RuntimeError("hand-over probe: a workgroup gave up waiting (mode %s, launch %d)" % (name, epoch))
            if epoch >= 10:
                rows.append(o[:, :4].astype(np.float64) / 100.0)  # 100 MHz ticks -> us
        a = np.stack(rows)  # [launch][workgroup][stamp]
        med, worst = np.median(np.median(a, axis=1), axis=0), np.median(np.max(a, axis=1), axis=0)
        res[name] = {"median_wg_us": {"stores_acknowledged": med[0], "arrival_counted": med[1], "all_arrived": med[2], "h_read_back": med[3]},
                     "slowest_wg_us": {"stores_acknowledged": worst[0], "arrival_counted": worst[1], "all_arrived": worst[2], "h_read_back": worst[3]}}
    v = res["two_level_counter"]["slowest_wg_us"]["h_read_back"]
    return {"value": v, "unit": "us", "ms_per_step": v * 1e-3, "dtype": "device-scope stores, atomics and loads",
            "config": {"workload": "in-kernel device-wide hand-over of h (28 KB) among %d workgroups, one per CU; stamps per workgroup from its own start" % cus,
                       "results": res},
            "roofline": None, "cpu_baseline": None, "pct_of_hbm_peak": None}


def bench_copy_calibration(torch, args):
    """A device-to-device copy of known size (1 GiB read, 1 GiB written per launch): the reference that the FETCH_SIZE /
    WRITE_SIZE counters of a profiling run are scaled by."""
    dev = torch.device("cuda:0")
    n = 1 << 30
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reps = 10
    for _ in range(reps):
        dst.copy_(src)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / reps
    gbps = 2 * n / (ms * 1e-3) / 1e9
    return {"value": gbps, "ms_per_step": ms, "dtype": "u8",
            "config": {"workload": "device-to-device copy, 1 GiB read + 1 GiB written per launch (counter calibration)", "bytes_read": n, "bytes_written": n},
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": 2 * n,
                         "kernel": "torch elementwise copy"},
            "cpu_baseline": None, "pct_of_hbm_peak": 100 * gbps / HBM_PEAK_GBPS}


def bench_matvec_n(torch, args):
    """BASELINE configs[4]: small-N matvec on the attention-projection shapes, N in {1, 2, 4, 8, 16}. value = algorithmic
    bytes (W + 4 N (cols + rows)) per second of the Q6_K 1536 x 7168 case at N = 8; every case is listed in config."""
    import oracle as O
    from macseek_amd import _lib, quant as q
    L = _lib.load()
    dev = torch.device("cuda:0")
    cases = []
    head = None
    for t, name, rows, cols in ((q.QType.Q6_K, "Q6_K", 1536, 7168), (q.QType.Q5_K, "Q5_K", 512, 7168),
                                (q.QType.IQ4_NL, "IQ4_NL", 7168, 4096), (q.QType.BF16, "BF16", 384, 7168)):
        nb = q.row_bytes(t, cols) * rows
        copies = 32  # successive launches read different copies of the matrix
        if int(t) == 30:
            arena = (torch.randn(copies * rows * cols, device=dev) * 0.02).to(torch.bfloat16).view(torch.uint8)
        else:
            arena = gen_blocks(torch, t, copies * nb // q.block_bytes(t), 0.01, 1, dev)
        Ws = [q.Buffer.of(arena).sub(i * nb, nb).c() for i in range(copies)]
        for n in (1, 2, 4, 8, 16):
            x = torch.randn(n * cols, device=dev)
            y = torch.zeros(n * rows, device=dev)
            xb, yb = q.Buffer.of(x).c(), q.Buffer.of(y).c()

            def launch(i):
                rc = L.msq_matvec_n(C.c_void_p(torch.cuda.current_stream().cuda_stream), int(t), C.byref(Ws[i % copies]), rows, cols,
                                    C.byref(xb), C.byref(yb), n, 0, 1)
                if rc != 0:
                    raise RuntimeError(L.msq_last_error().decode())
            ms = graph_ms_per_launch(torch, launch, 200)
            byt = nb + 4 * n * (cols + rows)
            row = {"type": name, "rows": rows, "cols": cols, "n": n, "us_per_launch": ms * 1e3, "bytes": byt, "GBps": byt / (ms * 1e-3) / 1e9}
            cases.append(row)
            if name == "Q6_K" and n == 8:
                head = row
    cpu = None
    if not args.gpu_only:
        rows, cols, nt = 1536, 7168, 8
        Wh = O.random_blocks(O.Q6_K, rows * cols, 1)
        xh = O.randn(nt * cols, 2)
        nth = cores()
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 5.0:
            for i in range(nt):
                O.matvec(O.Q6_K, Wh, rows, cols, xh[i * cols:(i + 1) * cols], 1, nth)
            reps += 1
        el = time.perf_counter() - t0
        cpu = {"value": head["bytes"] * reps / el / 1e9, "unit": "GB/s", "cores": nth, "kind": "port",
               "sample": "%d x 8 tokens of the Q6_K 1536x7168 case through oracle.c (dequant row + double dot per token), %.1f s" % (reps, el)}
    return {"value": head["GBps"], "ms_per_step": head["us_per_launch"] * 1e-3, "dtype": "f16 activations (f32 for BF16 weights), f32 accumulate",
            "config": {"workload": "BASELINE configs[4]: small-N matvec (speculative verify), attention projections, N in {1,2,4,8,16}; "
                                   "one step = one msq_matvec_n launch of Q6_K 1536x7168 at N=8", "cases": cases},
            "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": head["GBps"] / HBM_PEAK_GBPS,
                         "traffic": None, "kernel": "mv_tok_kernel<DecQ6K, 1, 8>", "bytes_per_launch": head["bytes"],
                         "avg_launch_us": head["us_per_launch"], "timing": "HIP event pair around one graph replay of 200 back-to-back launches"},
            "cpu_baseline": cpu, "pct_of_hbm_peak": 100 * head["GBps"] / HBM_PEAK_GBPS}


def bench_table(torch, args):
    """The reference's per-matrix table (bench/qmatvec.mm:93-157, docs/modules/quant.md:160-187) in one run: every real
    projection shape of the reference plus BASELINE's configs[0], [1] and [4] shapes, one msq_matvec per step, weights
    rotated over >= 512 MiB of distinct copies so every launch streams from HBM. Per row: weight MB, us per launch,
    GB/s of algorithmic bytes (W + 4 cols + 4 rows), the fraction of the 8 TB/s roofline and of what a kernel that only
    reads (msq_bw_probe, 1 GiB, same run) gets on this device. value = the first row (Q8_0 4096x4096, configs[0], unless --only narrows the table)."""
    from macseek_amd import _lib, quant as q
    L = _lib.load()
    dev = torch.device("cuda:0")
    T = q.QType
    shapes = [
        (T.Q8_0, 4096, 4096, 1, "BASELINE configs[0]"),
        (T.IQ1_S, 4096, 7168, 1, "configs[1] gate/up"), (T.IQ1_S, 7168, 4096, 1, "configs[1] down"),
        (T.IQ2_XXS, 4096, 7168, 1, "configs[1] gate/up"), (T.IQ2_XXS, 7168, 4096, 1, "configs[1] down"),
        (T.Q6_K, 1536, 7168, 1, "configs[4] Q"), (T.Q5_K, 512, 7168, 1, "configs[4] KV"),
        (T.IQ4_NL, 7168, 4096, 1, "configs[4] output"), (T.BF16, 384, 7168, 1, "configs[4] router"),
        # the reference's own table (bench/qmatvec.mm:93-110)
        (T.Q6_K, 1280, 5120, 1, "attn_q_a"), (T.Q5_K, 1280, 5120, 1, "attn_q_a"),
        (T.Q6_K, 32768, 1280, 1, "attn_q_b"), (T.Q5_K, 32768, 1280, 1, "attn_q_b"),
        (T.Q6_K, 512, 5120, 1, "attn_kv"), (T.Q6_K, 8192, 4096, 8, "attn_output_a"),
        (T.Q6_K, 5120, 8192, 1, "attn_output_b"), (T.Q5_K, 5120, 8192, 1, "attn_output_b"),
        (T.IQ1_S, 2304, 5120, 1, "exp gate/up"), (T.IQ1_S, 5120, 2304, 1, "exp down"),
        (T.IQ2_XXS, 2304, 5120, 1, "exp gate/up"), (T.IQ2_XXS, 5120, 2304, 1, "exp down"),
        (T.Q6_K, 2304, 5120, 1, "shexp gate/up"), (T.Q6_K, 5120, 2304, 1, "shexp down"),
        (T.Q8_0, 2304, 5120, 1, "shexp gate/up"), (T.Q8_0, 5120, 2304, 1, "shexp down"),
        (T.Q6_K, 129280, 5120, 1, "output head"), (T.Q6_K, 25600, 6144, 1, "engram_kv"),
        (T.F32, 384, 5120, 1, "router"), (T.F32, 24, 20480, 1, "hc_fn"),
        (T.BF16, 512, 5120, 1, "compressor_kv"), (T.BF16, 4096, 1280, 1, "indexer q_b"),
        (T.F16, 5120, 5120, 1, "f16 synthetic"),
        (T.IQ1_S, 32768, 5120, 1, "big synthetic"), (T.IQ2_XXS, 32768, 5120, 1, "big synthetic"),
    ]
    if args.only:
        shapes = [r for r in shapes if args.only in "%s %s" % (q.type_name(r[0]), r[4])]
        if not shapes:
            raise SystemExit("bench.py: --only %r matches no row of the table" % args.only)
    pool = torch.randint(0, 256, (1 << 30,), dtype=torch.uint8, device=dev)  # raw bytes: timing only (as the reference's table)
    bw = stream_read_GBps(torch, 1 << 30, pool)
    rows_out = []
    for t, rows, cols, groups, what in shapes:
        nb = q.row_bytes(t, cols) * rows
        pitch = (nb + 255) // 256 * 256
        copies = int(min(max(2, -(-(512 << 20) // pitch)), (1 << 30) // pitch, 256))
        x = torch.randn(cols * groups, device=dev)
        y = torch.zeros(rows, device=dev)
        Wb = [q.Buffer.of(pool).sub(i * pitch, nb).c() for i in range(copies)]
        xb, yb = q.Buffer.of(x).c(), q.Buffer.of(y).c()

        def launch(i):
            rc = L.msq_matvec(C.c_void_p(torch.cuda.current_stream().cuda_stream), int(t), C.byref(Wb[i % copies]), rows, cols,
                              C.byref(xb), C.byref(yb), 0, groups, None)
            if rc != 0:
                raise RuntimeError(L.msq_last_error().decode())
        ms = graph_ms_per_launch(torch, launch, max(copies, 16))
        byt = nb + 4 * cols * groups + 4 * rows
        gbps = byt / (ms * 1e-3) / 1e9
        rows_out.append({"type": q.type_name(t), "tensor": what, "shape": "%d->%d%s" % (cols, rows, " g%d" % groups if groups > 1 else ""),
                         "MB": round(nb / 1e6, 2), "us": round(ms * 1e3, 2), "GBps": round(gbps, 1),
                         "frac_of_8TBps": round(gbps / HBM_PEAK_GBPS, 4), "pct_of_stream_read": round(100 * gbps / bw, 1)})
    head = rows_out[0]
    print("%-8s %-20s %-16s %9s %8s %8s %7s %9s" % ("type", "tensor", "shape", "MB", "us", "GB/s", "%8TB/s", "%stream"), file=sys.stderr)
    for r in rows_out:
        print("%-8s %-20s %-16s %9.2f %8.2f %8.1f %7.1f %9.1f" % (r["type"], r["tensor"], r["shape"], r["MB"], r["us"], r["GBps"],
                                                                   100 * r["frac_of_8TBps"], r["pct_of_stream_read"]), file=sys.stderr)
    return {"value": head["GBps"], "ms_per_step": head["us"] * 1e-3, "dtype": "f32 activations (Q8_0, dense) / 16-bit block-fixed-point activations and exact integer sums (block formats), f32 accumulate",
            "config": {"workload": "decode matvec table: the reference's projection shapes + BASELINE configs[0], [1], [4]; one step = one msq_matvec of "
                                   "the first row", "stream_read_GBps_1GiB": bw, "rows": rows_out},
            "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": head["GBps"] / HBM_PEAK_GBPS,
                         "traffic": None, "kernel": "decode matvec (mv_tok_kernel, mv_kernel or mv_ring_kernel by shape)", "avg_launch_us": head["us"],
                         "timing": "HIP event pair around back-to-back replays of a graph of >= 16 launches, >= 10 ms per region"},
            "cpu_baseline": None, "pct_of_hbm_peak": 100 * head["GBps"] / HBM_PEAK_GBPS}


def bench_router(torch, args):
    """The MoE router ahead of the two MoE paths: the fused decode router (BF16 384 x 7168 logits matvec + top-6 in one
    launch, BASELINE configs[4]'s router shape) and, for a 2048-token prefill, top-6 from logits + the expert-sorted
    routing lists. value = the fused router's algorithmic bytes (W + x + bias + ids + weights) per second."""
    import oracle as O
    from macseek_amd import arch, quant as q
    dev = torch.device("cuda:0")
    n_exp, dim, n = 384, 7168, 2048
    copies = 64  # 64 x 5.5 MB of router weights: successive launches do not find theirs in the caches
    W = (torch.randn(copies, n_exp, dim, device=dev) * 0.02).to(torch.bfloat16)
    bias = torch.randn(n_exp, device=dev) * 0.1
    x = torch.randn(dim, device=dev)
    s = arch.Scratch.create(n_exp)
    ids1 = torch.zeros(6, dtype=torch.int32, device=dev)
    w1 = torch.zeros(6, dtype=torch.float32, device=dev)
    e = q.Enc()
    Wb = [q.Buffer.of(W).sub(i * n_exp * dim * 2, n_exp * dim * 2) for i in range(copies)]

    def fused(i):
        arch.encode_router_fused(q.Enc(torch.cuda.current_stream()), q.Buffer.of(x), Wb[i % copies], q.Buffer.of(bias), q.Buffer.of(ids1),
                                 q.Buffer.of(w1), s, dim, q.QType.BF16)
    fused_ms = graph_ms_per_launch(torch, fused, 256)
    fused_bytes = n_exp * dim * 2 + dim * 4 + n_exp * 4 + 48
    logits_h = O.randn(n * n_exp, 1, 3.0).reshape(n, n_exp)
    logits = torch.from_numpy(logits_h).to(dev)
    ids = torch.zeros((n, 6), dtype=torch.int32, device=dev)
    w = torch.zeros((n, 6), dtype=torch.float32, device=dev)
    L = arch.RouteLists.create(n, n_exp)

    def topk(i):
        arch.encode_router_topk(q.Enc(torch.cuda.current_stream()), q.Buffer.of(logits), q.Buffer.of(bias), q.Buffer.of(ids), q.Buffer.of(w), n)

    def lists(i):
        arch.encode_route_lists(q.Enc(torch.cuda.current_stream()), q.Buffer.of(ids), q.Buffer.of(w), n, L)
    topk(0)
    torch.cuda.synchronize()
    topk_ms = graph_ms_per_launch(torch, topk, 100)
    lists_ms = graph_ms_per_launch(torch, lists, 100)
    cpu = None
    if not args.gpu_only:
        bias_h = bias.cpu().numpy()
        t0 = time.perf_counter()
        rid, rw = O.router(logits_h, bias_h)
        O.route_lists(rid, rw)
        el = time.perf_counter() - t0
        cpu = {"value": n / el, "unit": "tokens/s", "cores": 1, "kind": "port",
               "sample": "oracle.c router + route_lists over the same 2048 x 384 logits, %.3f s; the GPU pair takes %.1f us" % (el, (topk_ms + lists_ms) * 1e3)}
    gbps = fused_bytes / (fused_ms * 1e-3) / 1e9
    return {"value": gbps, "ms_per_step": fused_ms, "dtype": "bf16 weights x f32 activations, f32 accumulate; f64 scores",
            "config": {"workload": "MoE router: fused decode router BF16 384x7168 (one launch per token); prefill: top-6 of 2048x384 logits + routing lists",
                       "fused_bytes_per_launch": fused_bytes, "fused_us": fused_ms * 1e3, "topk_2048_tokens_us": topk_ms * 1e3,
                       "route_lists_2048_tokens_us": lists_ms * 1e3},
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": None,
                         "kernel": "router_fused_kernel<BF16>", "bytes_per_launch": fused_bytes, "avg_launch_us": fused_ms * 1e3},
            "cpu_baseline": cpu, "pct_of_hbm_peak": 100 * gbps / HBM_PEAK_GBPS}


def bench_matmul(torch, args):
    """Prefill matmul Y[n x rows] = X[n x cols] . W^T (msq_matmul) at n = 2048 on the attention-projection shapes of
    BASELINE configs[4]; value = algorithmic FLOPs (2 n rows cols) per second of the Q6_K 1536x7168 case, the whole call
    (activation conversion, weight dequantization to fp16, GEMM) timed with a HIP event pair over back-to-back calls."""
    import oracle as O
    from macseek_amd import quant as q
    dev = torch.device("cuda:0")
    rows_out = []
    # n = 2048 and 512: dequantize-then-GEMM; n <= 128 (<= 256 on matrices of at most 2048 rows and on K-quants): the fused
    # kernel (mm_fused_kernel); 65..256 tokens on large IQ4_NL / Q8_0 / codebook matrices: mm_tile_kernel; "route" names
    # which one served the case
    cases = [(2048, q.QType.Q6_K, "Q6_K", 1536, 7168), (2048, q.QType.Q5_K, "Q5_K", 512, 7168),
             (2048, q.QType.IQ4_NL, "IQ4_NL", 7168, 4096), (2048, q.QType.BF16, "BF16", 384, 7168)]
    for n in (512, 256, 128, 64, 16):
        cases += [(n, q.QType.Q6_K, "Q6_K", 1536, 7168), (n, q.QType.IQ4_NL, "IQ4_NL", 7168, 4096)]
    for n, t, name, rows, cols in cases:
        if int(t) == 30:
            W = (torch.randn(rows * cols, device=dev) * 0.02).to(torch.bfloat16).view(torch.uint8)
        else:
            W = gen_blocks(torch, t, rows * cols // q.block_elems(t), 0.01, 1, dev)
        X = torch.randn(n * cols, device=dev)
        Y = torch.zeros(n * rows, device=dev)
        e = q.Enc()
        Wb, Xb, Yb = q.Buffer.of(W), q.Buffer.of(X), q.Buffer.of(Y)
        for _ in range(3):
            q.encode_matmul(e, t, Wb, rows, cols, Xb, Yb, n)
        torch.cuda.synchronize()
        reps = 20
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            q.encode_matmul(e, t, Wb, rows, cols, Xb, Yb, n)
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / reps
        flops = 2.0 * n * rows * cols
        tile = name in ("IQ4_NL", "Q8_0", "IQ1_S", "IQ2_XXS") and 65 <= n <= 256 and rows * cols >= 12000000
        fused = n <= 128 or (n <= 256 and (rows <= 2048 or name in ("Q6_K", "Q5_K")))
        rows_out.append({"type": name, "rows": rows, "cols": cols, "n": n, "us_per_call": ms * 1e3, "TFLOPs": flops / (ms * 1e-3) / 1e12,
                         "route": "mm_tile_kernel" if tile else "mm_fused_kernel" if fused else "dequant + rocBLAS"})
    head = rows_out[0]
    n = 2048
    cpu = None
    if not args.gpu_only:
        rows, cols, nt = 1536, 7168, 64
        Wh = O.random_blocks(O.Q6_K, rows * cols, 1)
        xh = O.randn(nt * cols, 2)
        nth = min(16, os.cpu_count() or 1)
        t0 = time.perf_counter()
        for i in range(nt):
            O.matvec(O.Q6_K, Wh, rows, cols, xh[i * cols:(i + 1) * cols], 1, nth)
        el = time.perf_counter() - t0
        cpu = {"value": 2.0 * nt * rows * cols / el / 1e12, "unit": "TFLOP/s", "cores": nth, "kind": "port",
               "sample": "%d tokens of the Q6_K 1536x7168 case through oracle.c (dequant each row, double dot), %.2f s; whole job = x%d" % (nt, el, n // nt)}
    return {"value": head["TFLOPs"], "ms_per_step": head["us_per_call"] * 1e-3, "dtype": "f16 x f16 MFMA (weights and activations rounded to fp16), f32 accumulate",
            "config": {"workload": "prefill matmul, 2048 tokens, BASELINE configs[4] shapes; one step = one msq_matmul call of the Q6_K 1536x7168 case", "cases": rows_out},
            "roofline": {"bound": "mfma", "achieved": head["TFLOPs"], "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": head["TFLOPs"] / MFMA_PEAK_TFLOPS,
                         "traffic": None, "kernel": "f32_to_f16_kernel + dequant_kernel<Q6_K, fp16> + rocBLAS fp16 GEMM (whole call; few tokens: mm_fused_kernel, see cases)", "flops_per_launch": 2.0 * n * 1536 * 7168,
                         "avg_launch_us": head["us_per_call"]},
            "cpu_baseline": cpu}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="moe_decode",
                    choices=["moe_decode", "moe_prefill", "matvec_iq1s", "matvec_iq2xxs", "q8_0", "matvec_n", "router", "matmul", "stream", "copy_calibration", "issue_probe", "handover_probe", "lds_bank_probe", "table"])
    ap.add_argument("--one-stream", action="store_true",
                    help="profiling runs: msq_moe_prefill keeps its launches on one stream (MSQ_MOEP_ONE_STREAM=1), so that "
                         "per-kernel durations and counters are not those of two kernels sharing the device")
    ap.add_argument("--only", default="",
                    help="table workload: keep the rows whose 'type tensor' contains this text (profiling one matrix)")
    ap.add_argument("--gpu-only", action="store_true",
                    help="profiling runs: skip the CPU baseline leg and the prefill appendix of the default workload")
    args = ap.parse_args()
    if args.one_stream:
        os.environ["MSQ_MOEP_ONE_STREAM"] = "1"
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (one MI355X per box); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from macseek_amd import _lib
    from macseek_amd import quant as q
    L = _lib.load()
    if L.msq_init() != 0:
        print("bench.py: " + L.msq_last_error().decode(), file=sys.stderr)
        sys.exit(1)
    if args.workload == "moe_prefill":
        r = bench_moe_prefill(torch, max(1, min(args.steps, 20)), max(1, min(args.warmup, 3)), with_cpu=not args.gpu_only)
        out = {"metric": METRIC, "value": r["value"], "unit": "TFLOP/s", "n_gpus": 1, "steps": max(1, min(args.steps, 20)),
               "warmup": max(1, min(args.warmup, 3)), "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak",
               "vs_baseline": None, "dtype": r["dtype"], "data": "synthetic", "config": r["config"], "roofline": r["roofline"],
               "cpu_baseline": r.get("cpu_baseline"), "pct_of_mfma_peak": r["pct_of_mfma_peak"]}
        print(json.dumps(out))
        return
    if args.workload == "matmul":
        r = bench_matmul(torch, args)
        print(json.dumps({"metric": METRIC, "value": r["value"], "unit": "TFLOP/s", "n_gpus": 1, "steps": 20, "warmup": 3,
                          "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                          "dtype": r["dtype"], "data": "synthetic", "config": r["config"], "roofline": r["roofline"],
                          "cpu_baseline": r["cpu_baseline"], "pct_of_mfma_peak": 100 * r["value"] / MFMA_PEAK_TFLOPS}))
        return
    if args.workload == "moe_decode":
        r = bench_moe_decode(torch, args)
    elif args.workload == "stream":
        r = bench_stream(torch, args)
    elif args.workload == "copy_calibration":
        r = bench_copy_calibration(torch, args)
    elif args.workload == "issue_probe":
        r = bench_issue_probe(torch, args)
    elif args.workload == "handover_probe":
        r = bench_handover_probe(torch, args)
    elif args.workload == "lds_bank_probe":
        r = bench_lds_bank_probe(torch, args)
    elif args.workload == "router":
        r = bench_router(torch, args)
    elif args.workload == "table":
        r = bench_table(torch, args)
    elif args.workload == "matvec_n":
        r = bench_matvec_n(torch, args)
    elif args.workload == "matvec_iq1s":
        r = bench_matvec(torch, args, q.QType.IQ1_S, 4096, 7168, 0.01, "BASELINE configs[1]: single-expert decode matvec IQ1_S 4096x7168, batch 1")
    elif args.workload == "matvec_iq2xxs":
        r = bench_matvec(torch, args, q.QType.IQ2_XXS, 4096, 7168, 0.01, "BASELINE configs[1]: single-expert decode matvec IQ2_XXS 4096x7168, batch 1")
    else:
        r = bench_matvec(torch, args, q.QType.Q8_0, 4096, 4096, 0.02, "BASELINE configs[0]: Q8_0 4096x4096 matvec")
    out = {"metric": METRIC, "value": r["value"], "unit": r.get("unit", "GB/s"), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": r["dtype"], "data": "synthetic", "config": r["config"], "roofline": r["roofline"],
           "cpu_baseline": r["cpu_baseline"], "pct_of_hbm_peak": r["pct_of_hbm_peak"]}
    for k in ("ms_per_step_of_each_region", "replays_timed", "timing", "stream_read_reference"):
        if k in r:
            out[k] = r[k]
    if args.workload == "moe_decode" and not args.gpu_only:
        # the metric's second half, measured in the same run on the same device (BASELINE configs[3])
        torch.cuda.empty_cache()
        p = bench_moe_prefill(torch, 5, 2, with_cpu=True)
        out["prefill_moe_gemm"] = {"value": p["value"], "unit": "TFLOP/s", "ms_per_step": p["ms_per_step"],
                                   "pct_of_mfma_peak": p["pct_of_mfma_peak"], "config": p["config"], "roofline": p["roofline"],
                                   "cpu_baseline": p["cpu_baseline"]}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
