#!/usr/bin/env python3
"""Benchmark of the quantized-weight hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras]

Headline (the JSON line's `value`): the q8_0 lm_head GEMV of benchmark configuration 1 -- 163840 x 7168 int8 weights
with one f16 scale per 32, batch 1 -- as algorithmic HBM GB/s.  A step is one Q8Head::matvec: quantize the hidden row
to q8, then the GEMV over the whole head; inputs are resident in HBM before the timed region.

`roofline` is the GEMV kernel alone (HIP events around each launch, on the stream it runs on) against the 8 TB/s HBM
peak; `cpu_baseline` is the CPU oracle (a port of the reference's Rust kernels) on a bounded row sample of the same
head, on this host's cores.  `extras` holds the other configurations (MXFP4 GEMV stream, MoE decode layer tok/s,
q8 MLA decode, grouped expert GEMM), each with its own algorithmic-bytes roofline fraction.

Prints exactly one JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
FP4_PEAK_TFLOPS = 10100.0   # dense FP4/FP6 MFMA
FP8_PEAK_TFLOPS = 5000.0
INT8_PEAK_TOPS = 5000.0
F16_PEAK_TFLOPS = 2500.0
# The committed counter summary of the headline kernel: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per launch, each scaled by
# the reading of a plain 1 GiB copy.  Its line "traffic_bytes_per_launch = N" is what `roofline.traffic` reports.
LM_HEAD_B1_PROFILE = os.path.join(ROOT, "profiles", "q8_gemv_b1_lm_head_163840x7168.md")


def profile_traffic(path):
    """HBM bytes per launch as the committed counter summary states them, or None when the file or the line is absent."""
    import re
    try:
        m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", open(path).read())
    except OSError:
        return None
    return int(m.group(1)) if m else None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_events(torch, fn, iters, warmup=3):
    """Average milliseconds per call of fn(), each call bracketed by its own pair of events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return sum(ts) / len(ts), ts[len(ts) // 2]


def time_events_region(torch, fn, iters, warmup=3, rounds=5):
    """Median over `rounds` of the milliseconds per call of `iters` back-to-back calls between one pair of events:
    the stream's throughput, without the per-launch event cost that time_events carries (a few us per launch)."""
    for _ in range(warmup):
        fn()
    ts = []
    for _ in range(rounds):
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b) / iters)
    ts.sort()
    return ts[len(ts) // 2]


def time_region(torch, fn, iters, warmup=3):
    """Milliseconds per call over one timed region of `iters` back-to-back calls."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / iters


def time_graph(torch, calls, replays=10):
    """Milliseconds per call with the launch cost of the Python wrapper taken out: the calls are captured once
    into a HIP graph (the library only enqueues kernels on the stream it is given) and the graph is replayed.
    Each replay is separated from the next by a synchronisation; returns None if the capture is refused."""
    try:
        for c in calls:
            c()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                for c in calls:
                    c()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        ts = []
        for _ in range(replays):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            g.replay()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b))
        ts.sort()
        return ts[len(ts) // 2] / len(calls)
    except Exception as e:  # noqa: BLE001 - the eager figure is still reported
        log("graph timing unavailable:", repr(e))
        torch.cuda.synchronize()
        return None


def bench_lm_head(torch, steps, warmup):
    from microkimi_amd import model, q8, workloads as W
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    rows, cols = W.VOCAB, W.D_MODEL
    g = torch.Generator(device="cuda").manual_seed(1)
    q = torch.randint(-127, 128, (rows, cols), dtype=torch.int8, device="cuda", generator=g)
    s = (torch.randn((rows, cols // 32), device="cuda", generator=g).abs() * (0.02 / 127.0)).to(torch.float16)
    x = torch.randn((8, cols), device="cuda", generator=g)
    head = model.Q8Head.from_q8(q, s, rows, cols)
    out1 = torch.empty((1, rows), device="cuda")
    out8 = torch.empty((8, rows), device="cuda")
    x1 = x[:1].contiguous()

    def step():
        head.matvec(x1, out1)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps

    alg1 = rows * cols + rows * (cols // 32) * 2 + cols * 4 + rows * 4           # 1 248 489 472 B
    alg8 = rows * cols + rows * (cols // 32) * 2 + 8 * cols * 4 + 8 * rows * 4   # 1 253 277 696 B
    xq1 = q8.quantize_q8(x1)
    xq8 = q8.quantize_q8(x)

    def k1():
        check(lib.mk_dev_q8_matvec(ptr(head.q), ptr(head.scales), 1, rows, cols, ptr(xq1.q), ptr(xq1.scales), 1, ptr(out1), cur_stream()))

    def k8():
        check(lib.mk_dev_q8_matvec(ptr(head.q), ptr(head.scales), 1, rows, cols, ptr(xq8.q), ptr(xq8.scales), 8, ptr(out8), cur_stream()))

    k1_ms, k1_med = time_events(torch, k1, max(20, min(steps, 200)))
    k8_ms, k8_med = time_events(torch, k8, max(20, min(steps, 100)))
    am = head.argmax(out8)
    torch.cuda.synchronize()
    res = {
        "ms_per_step": ms_step,
        "value_gbs": alg1 / (ms_step * 1e-3) / 1e9,
        "kernel_ms": k1_ms,
        "kernel_gbs": alg1 / (k1_ms * 1e-3) / 1e9,
        "alg_bytes": alg1,
        "batch8": {"kernel_ms": k8_ms, "gbs": alg8 / (k8_ms * 1e-3) / 1e9, "frac": alg8 / (k8_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                   "alg_bytes": alg8, "tok_s": 8 / (k8_ms * 1e-3)},
    }
    return res, (q, s, x, out8, am)


def host_workers():
    """Threads for the CPU baseline: std::thread::hardware_concurrency as the reference's pool takes it, bounded by this
    process's CPU affinity and by OMP_NUM_THREADS where the host sets one (a shared machine's CPU share)."""
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    try:
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    except ValueError:
        pass
    return max(1, cores)


def cpu_baseline_lm_head(torch, tensors, sample_rows=163840, budget_s=12.0):
    """The CPU oracle's Q8Head::matvec on the same head, all rows (same pool split rule as the reference)."""
    import numpy as np
    import oracle
    q, s, x, out8, am = tensors
    cols = q.shape[1]
    qh = q[:sample_rows].cpu().numpy()
    sh = s[:sample_rows].float().cpu().numpy()
    xh = x[0].cpu().numpy()
    workers = host_workers()
    oracle.q8head_matvec(qh, sh, sample_rows, cols, xh, workers=workers)  # warm-up
    ts = []
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end and len(ts) < 200:
        t0 = time.perf_counter()
        want = oracle.q8head_matvec(qh, sh, sample_rows, cols, xh, workers=workers)
        ts.append(time.perf_counter() - t0)
    ts.sort()
    med = ts[len(ts) // 2]
    bytes_sample = sample_rows * cols + sample_rows * (cols // 32) * 4 + cols * 4 + sample_rows * 4  # f32 scales, as the reference keeps them
    # parity of the GPU logits on the sample, and of the greedy token over the whole head for row 0
    got = out8[0, :sample_rows].cpu().numpy()
    rel = float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want))
    # batch 8 on the CPU is eight matvecs, as the reference's decode loop runs them (one token at a time)
    x8 = x.cpu().numpy()
    t8 = []
    for _ in range(3):
        t0 = time.perf_counter()
        for b in range(8):
            oracle.q8head_matvec(qh, sh, sample_rows, cols, x8[b], workers=workers)
        t8.append(time.perf_counter() - t0)
    t8.sort()
    batch8 = {"ms": t8[1] * 1e3, "tok_s": 8 / t8[1], "cores": workers, "kind": "port",
              "sample": "the same head, 8 hidden rows as 8 matvecs, median of 3 passes"}
    return {"value": bytes_sample / med / 1e9, "unit": "GB/s", "cores": workers, "kind": "port", "batch8": batch8,
            "sample": f"{sample_rows} of 163840 rows x 7168, batch 1, median of {len(ts)} calls, {med * 1e3:.2f} ms/call, "
                      f"{workers} threads (hardware concurrency within this process's CPU share)",
            "gpu_vs_cpu_rel_l2_on_sample": rel}


def time_cpu(fn, budget_s=4.0, max_calls=50):
    """Median seconds per call of a CPU function over a bounded sample (one untimed call first)."""
    fn()
    ts = []
    t_end = time.perf_counter() + budget_s
    while (time.perf_counter() < t_end and len(ts) < max_calls) or not ts:
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], len(ts)


def rand_mxfp4(torch, g, rows, cols):
    p = torch.randint(0, 256, (rows, cols // 2), dtype=torch.uint8, device="cuda", generator=g)
    s = torch.randint(118, 131, (rows, cols // 32), dtype=torch.uint8, device="cuda", generator=g)
    return p, s


def bench_mxfp4_gemv(torch, cpu=True):
    """Configuration 0 as a stream over 64 distinct matrices (7.8 MB each, 500 MB in all: more than the 256 MB
    Infinity Cache), as one grouped launch and as 64 back-to-back launches."""
    from microkimi_amd import mxfp4, q8, workloads as W
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    rows, cols, nmat = 2048, W.D_MODEL, 64
    g = torch.Generator(device="cuda").manual_seed(2)
    mats = [rand_mxfp4(torch, g, rows, cols) for _ in range(nmat)]
    x = torch.randn(cols, device="cuda", generator=g)
    xq = q8.quantize_q8(x)
    outs = [torch.empty(rows, device="cuda") for _ in range(nmat)]
    mk = lambda ts: torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device="cuda")
    pp, sp, op = mk([m[0] for m in mats]), mk([m[1] for m in mats]), mk(outs)
    per = rows * cols // 2 + rows * cols // 32 + cols * 4 + rows * 4  # 7 835 648 B

    def grouped():
        check(lib.mk_dev_mxfp4_matvec_q8_grouped(ptr(pp), ptr(sp), nmat, rows, cols, ptr(xq.q), ptr(xq.scales), None, ptr(op), cur_stream()))

    def singles():
        for i in range(nmat):
            check(lib.mk_dev_mxfp4_matvec_q8(ptr(mats[i][0]), ptr(mats[i][1]), rows, cols, ptr(xq.q), ptr(xq.scales), ptr(outs[i]), cur_stream()))

    g_ms, _ = time_events(torch, grouped, 30, warmup=300)  # the GPU idles during the CPU baseline before this: 25 ms of launches let the clocks come back
    r_ms = time_events_region(torch, grouped, 30, warmup=100, rounds=9)
    s_ms = time_region(torch, singles, 10)
    xf = x.contiguous()

    def singles_f32():
        for i in range(nmat):
            check(lib.mk_dev_mxfp4_matvec_f32(ptr(mats[i][0]), ptr(mats[i][1]), rows, cols, ptr(xf), ptr(outs[i]), cur_stream()))

    f_ms = time_region(torch, singles_f32, 5)
    gbs = lambda ms: per * nmat / (ms * 1e-3) / 1e9
    cpu_port = None
    if cpu:
        # the CPU oracle's matvec_packed (q8 mode, one thread: what an expert job of the reference runs) on the first matrix
        import oracle
        ph, sh, xh = mats[0][0].cpu().numpy(), mats[0][1].cpu().numpy(), x.cpu().numpy()
        sec, n = time_cpu(lambda: oracle.matvec_packed(ph, sh, rows, cols, xh, mode=1))
        cpu_port = {"gbs": per / sec / 1e9, "us_per_gemv": sec * 1e6, "cores": 1, "kind": "port", "sample": f"one 2048x7168 matrix, median of {n} calls"}
    return {"workload": "64 distinct 2048x7168 MXFP4 matrices, batch 1", "alg_bytes_per_matrix": per, "cpu_port": cpu_port,
            "q8_grouped_launch": {"ms": r_ms, "gbs": gbs(r_ms), "frac": gbs(r_ms) / HBM_PEAK_GBS,
                                  "frac_stream": gbs(r_ms) / HBM_PEAK_GBS, "frac_per_launch": gbs(g_ms) / HBM_PEAK_GBS,
                                  "timing": "frac_stream: 30 launches back to back between one pair of events, median of 9 (the kernel plus the gap to the "
                                            "next launch); frac_per_launch: an event pair around each launch, mean of 30 (carries the events' own cost); "
                                            "the kernel trace under profiles/ gives the kernel alone",
                                  "ms_with_events_around_each_launch": g_ms},
            "q8_back_to_back": {"ms": s_ms, "gbs": gbs(s_ms), "frac": gbs(s_ms) / HBM_PEAK_GBS, "us_per_gemv": s_ms * 1e3 / nmat},
            "f32_back_to_back": {"ms": f_ms, "gbs": gbs(f_ms), "frac": gbs(f_ms) / HBM_PEAK_GBS}}


def bench_vq1(torch):
    """VQ1 / LUT GEMV (quant::matvec_vq) on an expert-sized matrix: 2048 x 7168 = 917 504 index bytes + the 16 KiB
    codebook; 16 distinct matrices per timed pass.  Far too small to be HBM-bound: the line reports time per matvec."""
    from microkimi_amd import workloads as W
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    rows, cols, nmat = 2048, W.D_MODEL, 16
    g = torch.Generator(device="cuda").manual_seed(6)
    cb = torch.randn((256, 16), device="cuda", generator=g) * 0.05
    idx = [torch.randint(0, 256, (rows, cols // 16), dtype=torch.uint8, device="cuda", generator=g) for _ in range(nmat)]
    x = torch.randn(cols, device="cuda", generator=g)
    out = torch.empty(rows, device="cuda")
    ws = torch.empty(lib.mk_vq1_workspace_bytes(cols), dtype=torch.uint8, device="cuda")
    res = {"workload": "VQ1 2048x7168 (one index byte per 16 weights, 256x16 f32 codebook), batch 1", "index_bytes": rows * cols // 16}
    for name, exact in (("fast", 0), ("exact", 1)):
        calls = [(lambda i=i, exact=exact: check(lib.mk_dev_vq1_matvec(ptr(cb), ptr(idx[i]), rows, cols, ptr(x), exact, ptr(ws), ptr(out),
                                                                        cur_stream()))) for i in range(nmat)]
        ms = time_graph(torch, calls)
        loop_ms = time_region(torch, lambda: [c() for c in calls], 5) / nmat
        res[name] = {"us_per_matvec": (ms if ms is not None else loop_ms) * 1e3, "us_python_loop": loop_ms * 1e3,
                     "timing": "graph replay (table + sweep kernels)" if ms is not None else "python loop"}
    return res


def bench_moe(torch, cpu=True):
    """Configuration 2: 256 routed + 1 shared MXFP4 experts (6.0 GB resident), softmax top-8 router, B in {1, 4, 16}."""
    from microkimi_amd import model, workloads as W
    d, inter, ne = W.D_MODEL, W.D_INTER, W.N_EXPERTS
    g = torch.Generator(device="cuda").manual_seed(3)
    w1 = [rand_mxfp4(torch, g, inter, d) for _ in range(ne + 1)]
    w3 = [rand_mxfp4(torch, g, inter, d) for _ in range(ne + 1)]
    w2 = [rand_mxfp4(torch, g, d, inter) for _ in range(ne + 1)]
    experts = model.PackedExperts(w1, w3, w2, d, inter)
    per_expert = 3 * (inter * d // 2 + inter * d // 32)  # 23 396 352 B
    res = {"workload": "256 routed + 1 shared MXFP4 experts (2048x7168 gate/up, 7168x2048 down), top-8, q8 mode",
           "bytes_per_expert": per_expert}
    for B in (1, 4, 16):
        logits_h, hidden_h = W.config2_tokens(B)
        logits = torch.from_numpy(logits_h).cuda()
        x = torch.from_numpy(hidden_h).cuda()  # hidden state ~ N(0, 1)
        ids, wts = model.router_softmax_topk(logits, W.TOP_K)
        out = torch.empty((B, d), device="cuda")
        n_distinct = len(set(ids.cpu().numpy().reshape(-1).tolist())) + 1
        alg = n_distinct * per_expert + B * 2 * d * 4
        # A decode step meets different experts in every layer: the timed calls rotate through 16 routings (the seeded
        # one and 15 shifted copies of it, each with another expert in the shared role), 3.4 GB at B = 1, so that
        # repeats are not served by the 256 MB Infinity Cache.
        routes = []
        for k in range(16):
            ids_k = ((ids + 16 * k) % ne).to(torch.int32).contiguous()
            used = set(ids_k.cpu().numpy().reshape(-1).tolist())
            shared_k = ne if k == 0 else next(e for e in range((7 * k) % ne, ne) if e not in used)
            routes.append((ids_k, shared_k))
        calls = [(lambda r=r: model.moe_decode(experts, r[0], wts, x, shared=r[1], out=out)) for r in routes]

        def step():
            for c in calls:
                c()

        ms_eager = time_region(torch, step, 4, warmup=1) / len(calls)
        ms_graph = time_graph(torch, calls)
        ms = ms_graph if ms_graph is not None else ms_eager
        res[f"B{B}"] = {"ms": ms, "ms_python_loop": ms_eager, "timing": "graph replay" if ms_graph is not None else "python loop",
                        "tok_s": B / (ms * 1e-3), "distinct_experts": n_distinct, "pairs": B * (W.TOP_K + 1), "alg_bytes": alg,
                        "gbs": alg / (ms * 1e-3) / 1e9, "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        "finite": bool(torch.isfinite(out).all().item())}
        # The layer as a decode step runs it: rmsnorm, router gate matvec (256 x 7168 f32), softmax top-8 (one call:
        # mk_dev_norm_gate_route), expert section.  16 gate matrices stand for 16 layers, so the routing is computed on the device and
        # differs from call to call; the shared expert rotates as above (it may coincide with a routed one: 3 % of calls).
        if B == 1:
            gates = [torch.randn((ne, d), device="cuda", generator=g) * (d ** -0.5) for _ in range(16)]
            norm_w = torch.rand(d, device="cuda", generator=g) + 0.5
        picked = []

        def layer(k, record=False):
            xn, _, ids_k, wts_k = model.norm_gate_route(x, norm_w, 1e-6, gates[k], W.TOP_K)
            model.moe_decode(experts, ids_k, wts_k, xn, shared=(37 * k) % ne, out=out)
            if record:
                picked.append(len(set(ids_k.cpu().numpy().reshape(-1).tolist()) | {(37 * k) % ne}))

        for k in range(16):
            layer(k, record=True)
        ms_chain = time_graph(torch, [(lambda k=k: layer(k)) for k in range(16)])
        if ms_chain is None:
            ms_chain = time_region(torch, lambda: [layer(k) for k in range(16)], 4, warmup=1) / 16
        alg_chain = sum(picked) / len(picked) * per_expert + ne * d * 4 + B * 4 * d * 4
        res[f"B{B}"]["layer_chain"] = {"ms": ms_chain, "tok_s": B / (ms_chain * 1e-3), "calls": "rmsnorm + gate matvec 256 x 7168 f32 + softmax top-8 (mk_dev_norm_gate_route), expert section "
                                       "(mk_dev_moe_decode); 16 such layers captured in one graph, routing computed on the device",
                                       "distinct_experts_mean": sum(picked) / len(picked), "alg_bytes_mean": alg_chain,
                                       "frac": alg_chain / (ms_chain * 1e-3) / 1e9 / HBM_PEAK_GBS, "finite": bool(torch.isfinite(out).all().item())}
        if cpu:
            # the CPU oracle on the same tokens: the distinct experts copied to the host, ids renumbered into that table;
            # one thread per expert job up to the host's share, as the reference's pool runs them
            import numpy as np
            import oracle
            ids_h = ids.cpu().numpy()
            used = sorted(set(ids_h.reshape(-1).tolist())) + [ne]
            local = {e: i for i, e in enumerate(used)}
            host = lambda pr: (pr[0].cpu().numpy(), pr[1].cpu().numpy())
            table = oracle.ExpertTable([host(w1[e]) for e in used], [host(w3[e]) for e in used], [host(w2[e]) for e in used], d, inter)
            wts_h, x_h = wts.cpu().numpy(), x.cpu().numpy()
            lid = np.vectorize(local.get)(ids_h).astype(np.uint32)
            threads = min(host_workers(), W.TOP_K + 1)  # token by token, the 9 expert jobs of a token side by side
            sec, n = time_cpu(lambda: oracle.moe_decode(table, lid, wts_h, x_h, shared=local[ne], mode=1, threads=threads),
                              budget_s=4.0 if B == 1 else 6.0, max_calls=50 if B == 1 else 5)
            res[f"B{B}"]["cpu_port"] = {"ms": sec * 1e3, "tok_s": B / sec, "cores": threads, "kind": "port",
                                        "sample": f"the same {B} token(s) and their {len(used)} experts, token by token with {threads} threads over a token's expert jobs, median of {n} calls"}
            del table
    return res


def bench_mla(torch, cpu=True):
    """Configuration 3: 128 heads over a shared q8_0 latent cache; 32 distinct caches are rotated at every context
    length (a model has 24 MLA layers) so repeats are not served by the Infinity Cache."""
    from microkimi_amd import model, workloads as W
    L, R, nh = W.MLA_LATENT, W.MLA_ROPE, W.MLA_HEADS
    g = torch.Generator(device="cuda").manual_seed(4)
    res = {"workload": "128 heads, latent 512 + rope 64 q8_0 (612 B/position), 32 rotating caches"}
    q = torch.randn((nh, L + R), device="cuda", generator=g)
    out = torch.empty((nh, L), device="cuda")
    from microkimi_amd._lib import lib
    ws = torch.empty(lib.mk_mla_decode_workspace_bytes(nh, L, 16384), dtype=torch.uint8, device="cuda")  # one scratch for all caches
    for ctx in (1024, 4096, 16384):
        caches = []
        for _ in range(32):
            c = model.MlaCache(L, R, ctx)
            c.lat_q.copy_(torch.randint(-127, 128, (ctx, L), dtype=torch.int8, device="cuda", generator=g))
            c.lat_s.copy_((torch.rand((ctx, L // 32), device="cuda", generator=g) * 0.03 + 0.005).to(torch.float16))
            c.rope_q.copy_(torch.randint(-127, 128, (ctx, R), dtype=torch.int8, device="cuda", generator=g))
            c.rope_s.copy_((torch.rand((ctx, R // 32), device="cuda", generator=g) * 0.03 + 0.005).to(torch.float16))
            c.n = ctx
            c._ws = ws
            caches.append(c)
        it = [0]

        def step():
            c = caches[it[0] % 32]
            it[0] += 1
            model.mla_attn_flash_q8_mqa(c, q, ctx - 1, W.MLA_SCALE, out)

        ms_eager = time_region(torch, step, 64, warmup=4)
        it[0] = 0
        ms_graph = time_graph(torch, [step] * 32)  # one pass over the 32 caches per replay
        ms = ms_graph if ms_graph is not None else ms_eager
        alg = ctx * 612 + nh * (L + R) * 4 + nh * L * 4
        flops = 2.0 * nh * (L + R + L) * ctx
        # matrix-core floor of this arithmetic: the scores as one int8 pass over latent + rope, P V as three f16 passes
        # (the exact split of an int8 x f16-scale product and of p into f16 halves)
        floor_us = (2.0 * nh * (L + R) * ctx / (INT8_PEAK_TOPS * 1e12) + 3 * 2.0 * nh * L * ctx / (F16_PEAK_TFLOPS * 1e12)) * 1e6
        res[f"ctx{ctx}"] = {"us": ms * 1e3, "us_python_loop": ms_eager * 1e3, "timing": "graph replay" if ms_graph is not None else "python loop",
                            "alg_bytes": alg, "gbs": alg / (ms * 1e-3) / 1e9, "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                            "hbm_frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "tflops": flops / (ms * 1e-3) / 1e12,
                            "mfma_floor_us": floor_us, "frac_of_mfma_floor": floor_us / (ms * 1e3)}
        if cpu and ctx == 1024:
            # the CPU oracle's mla_attn_flash_q8_mqa (one thread, as the reference runs it) on the first cache
            import oracle
            c0 = caches[0]
            lq, ls = c0.lat_q.cpu().numpy(), c0.lat_s.float().cpu().numpy()
            rq, rs = c0.rope_q.cpu().numpy(), c0.rope_s.float().cpu().numpy()
            qh = q.cpu().numpy()
            sec, n = time_cpu(lambda: oracle.mla_absorbed_decode(lq, ls, rq, rs, qh, nh, W.MLA_SCALE), budget_s=4.0, max_calls=10)
            res[f"ctx{ctx}"]["cpu_port"] = {"ms": sec * 1e3, "cores": 1, "kind": "port", "sample": f"the first cache, median of {n} calls"}
        if cpu and ctx == 16384:
            # 16 of the 128 heads over the whole 16k cache (one thread; the full call is 8 times this)
            import oracle
            c0 = caches[0]
            lq, ls = c0.lat_q.cpu().numpy(), c0.lat_s.float().cpu().numpy()
            rq, rs = c0.rope_q.cpu().numpy(), c0.rope_s.float().cpu().numpy()
            qh = q[:16].contiguous().cpu().numpy()
            sec, n = time_cpu(lambda: oracle.mla_absorbed_decode(lq, ls, rq, rs, qh, 16, W.MLA_SCALE), budget_s=4.0, max_calls=5)
            res[f"ctx{ctx}"]["cpu_port"] = {"ms": sec * 8 * 1e3, "cores": 1, "kind": "port",
                                            "sample": f"16 of the 128 heads over the first 16k cache ({sec * 1e3:.1f} ms, median of {n} calls), times 8"}
        del caches
    return res


def bench_lm_head_published(torch):
    """The q8 lm_head at the shape the reference publishes (KIMI.md:100: 65536 x 7168, int8 + f32 scale per 32 as
    Q8Head::from_f32 builds it, 5.1 ms per call on 10 CPU threads).  Two heads alternate (528 MB each)."""
    from microkimi_amd import model
    rows, cols = 65536, 7168
    g = torch.Generator(device="cuda").manual_seed(7)
    heads = []
    for _ in range(2):
        q = torch.randint(-127, 128, (rows, cols), dtype=torch.int8, device="cuda", generator=g)
        sc = torch.rand((rows, cols // 32), device="cuda", generator=g) * 0.01 + 0.001
        heads.append(model.Q8Head.from_q8(q, sc, rows, cols))
    x = torch.randn((1, cols), device="cuda", generator=g)
    out = torch.empty((1, rows), device="cuda")
    it = [0]

    def step():
        h = heads[it[0] % 2]
        it[0] += 1
        h.matvec(x, out)

    ms_eager = time_region(torch, step, 40, warmup=6)
    it[0] = 0
    ms_graph = time_graph(torch, [step] * 8)
    ms = ms_graph if ms_graph is not None else ms_eager
    alg = rows * cols + rows * (cols // 32) * 4 + cols * 4 + rows * 4
    return {"workload": "q8 lm_head 65536 x 7168, f32 scales, batch 1 (quantize + GEMV); the reference publishes 5.1 ms on 10 CPU threads",
            "us": ms * 1e3, "us_python_loop": ms_eager * 1e3, "timing": "graph replay" if ms_graph is not None else "python loop",
            "alg_bytes": alg, "gbs": alg / (ms * 1e-3) / 1e9, "hbm_frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "published_cpu_ms": 5.1, "published_cpu_ms_over_this": 5.1 / ms}


def bench_mla_heads(torch):
    """The attention over the reference's own cache layout (per head a q8 K-nope row and a q8 V row, one f32 rope row per
    position) on the case the reference publishes: 96 heads, nope 128 + rope 64, v 128 (KIMI.md:96, bench code
    src/main.rs:389-479: 16k positions 79.7 ms with the all-heads q8 kernel on one CPU thread).  Every cache byte is
    used once: HBM-bound.  Two caches alternate (each is larger than the Infinity Cache at 16k)."""
    from microkimi_amd import model
    nh, nope, rope, vd = 96, 128, 64, 128
    g = torch.Generator(device="cuda").manual_seed(6)
    res = {"workload": "96 heads, nope 128 + rope 64 (f32, shared), v 128, q8_0 with f32 scales: 27 904 B/position",
           "published_cpu_ms_16k": 79.7}
    q = torch.randn((1, nh * (nope + rope)), device="cuda", generator=g)
    scale = float((nope + rope) ** -0.5)
    for ctx in (1024, 4096, 16384):
        caches = []
        for _ in range(2):
            c = model.MlaHeadsCache(nh, nope, rope, vd, ctx)
            c.kq.copy_(torch.randint(-127, 128, c.kq.shape, dtype=torch.int8, device="cuda", generator=g))
            c.vq.copy_(torch.randint(-127, 128, c.vq.shape, dtype=torch.int8, device="cuda", generator=g))
            c.ks.copy_(torch.rand(c.ks.shape, device="cuda", generator=g) * 0.03 + 0.005)
            c.vs.copy_(torch.rand(c.vs.shape, device="cuda", generator=g) * 0.03 + 0.005)
            c.kr.copy_(torch.randn(c.kr.shape, device="cuda", generator=g))
            c.n = ctx
            caches.append(c)
        caches[0].attn(q, ctx - 1, scale)  # workspaces allocated before the capture
        caches[1].attn(q, ctx - 1, scale)
        it = [0]

        def step():
            c = caches[it[0] % 2]
            it[0] += 1
            c.attn(q, ctx - 1, scale)

        ms_eager = time_region(torch, step, 32, warmup=4)
        it[0] = 0
        ms_graph = time_graph(torch, [step] * 8)
        ms = ms_graph if ms_graph is not None else ms_eager
        alg = ctx * (nh * (nope + vd) * 9 // 8 + rope * 4) + nh * (nope + rope) * 4 + nh * vd * 4
        res[f"ctx{ctx}"] = {"us": ms * 1e3, "us_python_loop": ms_eager * 1e3, "timing": "graph replay" if ms_graph is not None else "python loop",
                            "alg_bytes": alg, "gbs": alg / (ms * 1e-3) / 1e9, "hbm_frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        if ctx == 16384:
            res[f"ctx{ctx}"]["published_cpu_ms_over_this"] = 79.7 / ms
        del caches
    # the attention loop of mla_prefill over the same cache: a 512-token chunk at the start of a prompt and behind 3584
    # cached positions (query i attends 0 ..= pos0 + i); 16 queries of a head share the K / V tiles on the matrix cores
    m = 512
    qs = torch.randn((m, nh * (nope + rope)), device="cuda", generator=g)
    for pos0 in (0, 3584):
        c = model.MlaHeadsCache(nh, nope, rope, vd, pos0 + m)
        c.kq.copy_(torch.randint(-127, 128, c.kq.shape, dtype=torch.int8, device="cuda", generator=g))
        c.vq.copy_(torch.randint(-127, 128, c.vq.shape, dtype=torch.int8, device="cuda", generator=g))
        c.ks.copy_(torch.rand(c.ks.shape, device="cuda", generator=g) * 0.03 + 0.005)
        c.vs.copy_(torch.rand(c.vs.shape, device="cuda", generator=g) * 0.03 + 0.005)
        c.kr.copy_(torch.randn(c.kr.shape, device="cuda", generator=g))
        c.n = pos0 + m
        ms = time_region(torch, lambda: c.attn(qs, pos0, scale), 10, warmup=2)
        pairs = sum(pos0 + i + 1 for i in range(m))
        flops = 2.0 * pairs * nh * (nope + rope + vd)
        res[f"prefill_{m}_at_{pos0}"] = {"ms": ms, "query_position_pairs": pairs, "tflops": flops / (ms * 1e-3) / 1e12,
                                         "cache_bytes": (pos0 + m) * (nh * (nope + vd) * 9 // 8 + rope * 4)}
        del c
    return res


def bench_gemm(torch):
    """Configuration 4: 512 tokens routed top-8 over 256 experts (about 16 rows per expert), gate GEMM 2048 x 7168 per
    expert on the block-scaled MFMA; and a large-M variant (512 rows on each of 8 experts)."""
    import numpy as np
    from microkimi_amd import dequant, model, workloads as W
    d, inter, ne = W.D_MODEL, W.D_INTER, W.N_EXPERTS
    g = torch.Generator(device="cuda").manual_seed(5)
    logits_h, x_h = W.config4_tokens()
    ids, _ = model.router_softmax_topk(torch.from_numpy(logits_h).cuda(), W.TOP_K)
    flat = ids.cpu().numpy().reshape(-1)
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=ne)
    offsets = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).cuda()
    xg = torch.from_numpy(x_h[order // W.TOP_K]).cuda()
    codes, exps = dequant.quantize_mxfp8(xg)
    mats = [rand_mxfp4(torch, g, inter, d) for _ in range(ne)]
    pl, sl = [m[0] for m in mats], [m[1] for m in mats]
    m = int(xg.shape[0])

    # the expert pointer tables and the result buffer are built once (a resident expert table, as mk_bin_load_experts
    # gives): the timed step is the C-ABI call alone
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    mkp = lambda ts: torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device="cuda")
    pp, sp = mkp(pl), mkp(sl)
    out_g = torch.empty((m, inter), dtype=torch.float32, device="cuda")

    def step():
        check(lib.mk_dev_mxfp4_grouped_gemm(ptr(pp), ptr(sp), ne, inter, d, ptr(codes), ptr(exps), ptr(offsets), m, ptr(out_g), cur_stream()))

    ms = time_region(torch, step, 10, warmup=2)
    used = int((counts > 0).sum())
    wbytes = used * (inter * d // 2 + inter * d // 32)
    alg = wbytes + m * d + m * d // 32 + m * inter * 4
    flops = 2.0 * m * inter * d
    res = {"workload": "gate GEMM of 512 tokens x top-8 over 256 experts (4096 rows, 2048 x 7168 per expert), MXFP8 activations",
           "prefill": {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "mfma_frac_fp8_peak": flops / (ms * 1e-3) / 1e12 / FP8_PEAK_TFLOPS,
                       "mfma_frac_fp4_peak": flops / (ms * 1e-3) / 1e12 / FP4_PEAK_TFLOPS, "alg_bytes": alg, "gbs": alg / (ms * 1e-3) / 1e9, "hbm_frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                       "rows_per_expert_max": int(counts.max()), "experts_used": used}}
    # the CPU oracle's matvec_packed_nt (the reference's prefill product, f32, one thread) on the busiest expert's rows
    import oracle
    e_max = int(np.argmax(counts))
    r0, r1 = int(offsets[e_max].item()), int(offsets[e_max + 1].item())
    xe = xg[r0:r1].cpu().numpy()
    m8 = (r1 - r0 + 7) // 8 * 8
    xt = np.zeros((d, m8), np.float32)
    xt[:, :r1 - r0] = xe.T
    ph, sh = pl[e_max].cpu().numpy(), sl[e_max].cpu().numpy()
    sec, ncalls = time_cpu(lambda: oracle.matvec_packed_nt(ph, sh, inter, d, xt, m8), budget_s=6.0, max_calls=10)
    res["prefill"]["cpu_port"] = {"tflops": 2.0 * (r1 - r0) * inter * d / sec / 1e12, "ms": sec * 1e3, "cores": 1, "kind": "port",
                                  "sample": f"expert {e_max}'s {r1 - r0} rows against its 2048 x 7168 gate matrix (1 of {used} experts), "
                                            f"matvec_packed_nt in f32, median of {ncalls} calls"}
    # large-M variant: the kernel's own ceiling
    M = 512
    xl = torch.randn((8 * M, d), device="cuda", generator=g)
    cl, el = dequant.quantize_mxfp8(xl)
    off2 = torch.arange(0, 9, dtype=torch.int32, device="cuda") * M

    out_l = torch.empty((8 * M, inter), dtype=torch.float32, device="cuda")

    def step2():
        check(lib.mk_dev_mxfp4_grouped_gemm(ptr(pp), ptr(sp), 8, inter, d, ptr(cl), ptr(el), ptr(off2), 8 * M, ptr(out_l), cur_stream()))

    ms2 = time_region(torch, step2, 20, warmup=3)
    fl2 = 2.0 * 8 * M * inter * d
    res["large_m"] = {"rows_per_expert": M, "experts": 8, "ms": ms2, "tflops": fl2 / (ms2 * 1e-3) / 1e12,
                      "mfma_frac_fp8_peak": fl2 / (ms2 * 1e-3) / 1e12 / FP8_PEAK_TFLOPS,
                      "mfma_frac_fp4_peak": fl2 / (ms2 * 1e-3) / 1e12 / FP4_PEAK_TFLOPS}
    del cl, el, xl, out_l
    # the whole expert section of the prefill layer on the device (grouping, gather + MXFP8, gate, up, activation,
    # down, combine): mk_dev_moe_prefill.  The gate matrices above are reused as W1; W3 and W2 are drawn here.
    w3 = [rand_mxfp4(torch, g, inter, d) for _ in range(ne)]
    w2 = [rand_mxfp4(torch, g, d, inter) for _ in range(ne)]
    experts = model.PackedExperts(mats, w3, w2, d, inter)
    ids_d, wts_d = model.router_softmax_topk(torch.from_numpy(logits_h).cuda(), W.TOP_K)
    x_d = torch.from_numpy(x_h).cuda()
    T = int(x_d.shape[0])
    out = torch.empty((T, d), device="cuda")

    def step3():
        model.moe_prefill(experts, ids_d, wts_d, x_d, out=out, mxfp8=True)

    ms3 = time_region(torch, step3, 5, warmup=2)
    y_mxfp8 = out.clone()
    per_expert = 3 * (inter * d // 2 + inter * d // 32)
    fl3 = 3 * 2.0 * m * inter * d
    # weights once per used expert; token rows in, MXFP8 gathered rows and MXFP8 activation rows written and read, f32 down
    # rows written and read (gate and up go from the accumulators to the activation's MXFP8 form: no f32 round trip)
    alg3 = used * per_expert + T * d * 4 + 2 * (m * d + m * d // 32) + 2 * (m * inter + m * inter // 32) + 2 * m * d * 4 + T * d * 4
    res["expert_section"] = {"workload": "512 tokens x top-8 over 256 experts: group, gather + MXFP8, gate + up + SwiGLU + MXFP8 (one launch), down, combine",
                             "ms": ms3, "tok_s": T / (ms3 * 1e-3), "tflops": fl3 / (ms3 * 1e-3) / 1e12,
                             "mfma_frac_fp8_peak": fl3 / (ms3 * 1e-3) / 1e12 / FP8_PEAK_TFLOPS,
                             "mfma_frac_fp4_peak": fl3 / (ms3 * 1e-3) / 1e12 / FP4_PEAK_TFLOPS, "weight_bytes": used * per_expert,
                             "alg_bytes": alg3, "gbs": alg3 / (ms3 * 1e-3) / 1e9, "hbm_frac": alg3 / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                             "finite": bool(torch.isfinite(out).all().item())}
    # the same section in the reference's own arithmetic (f32 rows against the dequantized weights, f32 matrix instruction)

    def step4():
        model.moe_prefill(experts, ids_d, wts_d, x_d, out=out, exact=True)

    ms4 = time_region(torch, step4, 3, warmup=1)
    y_f32 = out.clone()
    dist = lambda y: float((torch.linalg.vector_norm((y - y_f32).double()) / torch.linalg.vector_norm(y_f32.double())).item())
    res["expert_section"]["rel_l2_to_f32_section"] = dist(y_mxfp8)
    res["expert_section_f32"] = {"workload": "the same section, mk_dev_moe_prefill_f32: group, gate + up (one launch), activation, down, combine in f32",
                                 "ms": ms4, "tok_s": T / (ms4 * 1e-3), "tflops": fl3 / (ms4 * 1e-3) / 1e12,
                                 "mfma_frac_fp32_peak": fl3 / (ms4 * 1e-3) / 1e12 / 157.3,
                                 "finite": bool(torch.isfinite(out).all().item())}
    # and with bfloat16 activations (exact weights; every bfloat16 value as two e4m3 terms on the block-scaled matrix
    # instruction, or the bf16 matrix instruction with MK_PREFILL_BF16_MFMA=1)

    def step5():
        model.moe_prefill(experts, ids_d, wts_d, x_d, out=out, bf16=True)

    ms5 = time_region(torch, step5, 5, warmup=2)
    bf16_mfma = os.environ.get("MK_PREFILL_BF16_MFMA", "0") not in ("", "0")
    res["expert_section_bf16"] = {"workload": "the same section, mk_dev_moe_prefill_bf16: group, gather + bf16 "
                                              + ("(bf16 matrix instruction), gate + up (one launch), activation + bf16, down, combine" if bf16_mfma else
                                                 "as two e4m3 terms, gate + up + SwiGLU + bf16 as two terms (one launch, block-scaled matrix "
                                                 "instruction, two instructions a step), down, combine"),
                                  "ms": ms5, "tok_s": T / (ms5 * 1e-3), "tflops": fl3 / (ms5 * 1e-3) / 1e12,
                                  # useful flops (one product per bfloat16 value) against the peak of the instruction that runs
                                  ("mfma_frac_bf16_peak" if bf16_mfma else "mfma_frac_fp8_peak"): fl3 / (ms5 * 1e-3) / 1e12 / (2500.0 if bf16_mfma else 5000.0),
                                  "weight_bytes": used * per_expert, "weight_gbs": used * per_expert / (ms5 * 1e-3) / 1e9,
                                  "hbm_frac": used * per_expert / (ms5 * 1e-3) / 1e9 / 8000.0,
                                  "finite": bool(torch.isfinite(out).all().item()), "rel_l2_to_f32_section": dist(out)}
    # BASELINE states this configuration in bf16: the bf16 section leads, the other two arithmetics stand beside it with
    # their distance to the f32 section's result (which the parity tests hold within 1e-5 of the CPU oracle)
    res["lead"] = {"section": "expert_section_bf16", "ms": ms5, "tok_s": T / (ms5 * 1e-3), "dtype": "bf16 activations, exact MXFP4 weights, f32 sums",
                   "beside": {"expert_section_f32": {"ms": ms4, "rel_l2_to_f32_section": 0.0},
                              "expert_section (MXFP8 activations, explicit opt-in)": {"ms": ms3, "rel_l2_to_f32_section": res["expert_section"]["rel_l2_to_f32_section"]}}}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--only", default="",
                    help="comma-separated names of extras (mxfp4_gemv, moe_decode, mla_decode, mla_heads_decode, lm_head_published_shape, grouped_gemm, vq1_gemv): run only "
                         "those and print their figures as one JSON object (a development aid; the contract line needs a full run)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run five plain 1 GiB device copies (a kernel of known traffic to scale rocprofv3 --pmc byte counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (no CPU fallback exists for the measured path)", file=sys.stderr)
        sys.exit(3)
    from microkimi_amd import _lib
    _lib.require_device()
    torch.cuda.set_device(0)

    if args.copy_calibration:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    if args.only:
        table = {"mxfp4_gemv": bench_mxfp4_gemv, "moe_decode": bench_moe, "mla_decode": bench_mla, "mla_heads_decode": bench_mla_heads, "lm_head_published_shape": bench_lm_head_published,
                 "grouped_gemm": bench_gemm, "vq1_gemv": bench_vq1}
        res = {}
        for name in args.only.split(","):
            log(name, "...")
            fn = table[name]
            res[name] = fn(torch, not args.no_cpu) if name in ("mxfp4_gemv", "moe_decode", "mla_decode") else fn(torch)
            torch.cuda.empty_cache()
        print(json.dumps(res))
        return
    log("lm_head ...")
    head, tensors = bench_lm_head(torch, args.steps, args.warmup)
    cpu = None
    if not args.no_cpu:
        log("cpu baseline ...")
        cpu = cpu_baseline_lm_head(torch, tensors)
    del tensors
    torch.cuda.empty_cache()
    extras = {"lm_head_batch8": head.pop("batch8")}
    if cpu is not None:
        extras["lm_head_batch8"]["cpu_port"] = cpu.pop("batch8")
    if not args.no_extras:
        for name, fn in (("mxfp4_gemv", bench_mxfp4_gemv), ("moe_decode", bench_moe), ("mla_decode", bench_mla), ("mla_heads_decode", bench_mla_heads), ("lm_head_published_shape", bench_lm_head_published),
                         ("grouped_gemm", bench_gemm), ("vq1_gemv", bench_vq1)):
            log(name, "...")
            try:
                extras[name] = fn(torch, not args.no_cpu) if name in ("mxfp4_gemv", "moe_decode", "mla_decode") else fn(torch)
            except Exception as e:  # an extra must not hide the headline
                extras[name] = {"error": repr(e)}
            torch.cuda.empty_cache()

    line = {
        "metric": "q8_0 lm_head GEMV HBM GB/s",
        "value": head["value_gbs"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "config 1: q8_0 lm_head 163840x7168 (int8 + f16 scale per 32), batch 1; step = quantize_q8(x) + GEMV",
                   "rows": 163840, "cols": 7168, "batch": 1, "algorithmic_bytes": head["alg_bytes"]},
        "roofline": {"bound": "hbm", "achieved": head["kernel_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["kernel_gbs"] / HBM_PEAK_GBS, "traffic": profile_traffic(LM_HEAD_B1_PROFILE),
                     "kernel": "q8_gemv_b1_kernel<224, f16 scales>", "kernel_ms": head["kernel_ms"]},
        "cpu_baseline": cpu,
        "extras": extras,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
