"""Benchmark of the quantized MoE expert-matmul hot path on one MI355X.

A step is one decode pass of a Qwen3-30B-A3B-shaped MoE layer over one token: hidden 2048, 128 experts of
moe_intermediate 768, Q4_K gate/up and Q6_K down, softmax top-8 renormalised (the second configuration of
BASELINE.json). Per step the library runs, from inputs resident in HBM: the Q8_2_X4 quantizer on the token,
gate . up . SwiGLU with the down activation quantized in the same launch, and the route-weighted down
projection with the slot sum folded in. Steps are captured into one HIP graph (the decode mode of the reference)
and replayed; consecutive steps use different tokens, routings and layer copies so the expert rows come from HBM,
not from L2 or the memory-side cache.

Prints one JSON line: whole-job value (microseconds per token), the dominant kernel's roofline (HBM), and the
CPU baseline (the oracle's AVX2 restatement of the reference's qdot path on the box's host cores, a bounded
sample of the same workload).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

HIDDEN, FF, N_EXPERTS, TOP_K = 2048, 768, 128, 8
HBM_PEAK_GBS = 8000.0
# HBM bytes a launch of the headline configuration's dominant kernel moves (read + written), from the rocprofv3
# FETCH_SIZE / WRITE_SIZE summary under profiles/ (counter x the copy-kernel calibration measured in the same run).
GATE_UP_X_TRAFFIC_BYTES = 14425174


def host_threads():
    """Threads of the CPU baseline: the CPUs this process may run on, held to the worker-pool size the GPU box's harness
    sets for a one-GPU job (OMP_NUM_THREADS, 16 there), whatever the machine's core count."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    cap = os.environ.get("OMP_NUM_THREADS", "")
    return max(1, min(n, int(cap)) if cap.isdigit() and int(cap) > 0 else n)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_layer(ora, seed, threads, gate_type=None, down_type=None):
    """The layer's expert stacks: fp32 N(0, 0.02) quantized by the repo's K-quant rules (Q4_K, Q5_K, Q6_K `_ref`);
    the other types as random legal blocks with small scales."""
    rng = np.random.default_rng(seed)
    gate_type = ora.Q4_K if gate_type is None else gate_type
    down_type = ora.Q6_K if down_type is None else down_type
    out = []
    for wtype, rows, k in ((gate_type, N_EXPERTS * FF, HIDDEN), (gate_type, N_EXPERTS * FF, HIDDEN),
                           (down_type, N_EXPERTS * HIDDEN, FF)):
        rb = ora.row_bytes(wtype, k)
        raw = {ora.IQ4_XS: (136, 0, 2e-6, 8e-6),   # values d * (ls - 32) * level ~ 0.01
               ora.Q3_K: (110, 108, 1e-4, 4e-4),   # d * (scale - 32) * (code - 4)
               ora.IQ2_XXS: (66, 0, 1e-3, 4e-3),   # d * (0.5 + s) / 4 * magnitude
               ora.IQ3_XXS: (98, 0, 2e-4, 8e-4)}   # d * (0.5 + s) / 2 * magnitude
        if wtype in raw:  # types the oracle has no (fast) quantizer for: random legal blocks with small scales
            bb, d_off, lo, hi = raw[wtype]
            nb = rows * (k // 256)
            w = rng.integers(0, 256, nb * bb, dtype=np.uint8).reshape(nb, bb)
            d = rng.uniform(lo, hi, nb).astype(np.float16).view(np.uint16)
            w[:, d_off], w[:, d_off + 1] = d & 0xFF, d >> 8
            out.append(w.reshape(-1))
            continue
        q = np.empty(rows * rb, np.uint8)
        chunk = 8192
        for r0 in range(0, rows, chunk):
            n = min(chunk, rows - r0)
            x = (rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
            q[r0 * rb:(r0 + n) * rb] = ora.quantize_rows(wtype, x, n, k, n_threads=threads)
        out.append(q)
    return out


def make_tokens(ora, n_tokens, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n_tokens, HIDDEN), dtype=np.float32)
    ids = np.empty((n_tokens, TOP_K), np.uint32)
    wts = np.empty((n_tokens, TOP_K), np.float32)
    for t in range(n_tokens):
        ids[t], wts[t] = ora.route_softmax_topk(rng.standard_normal(N_EXPERTS, dtype=np.float32), TOP_K)
    return x, ids, wts


def load_probe():
    """The calibration launches: a library of their own beside the product's, built by the same Makefile."""
    import ctypes as C
    path = os.path.join(ROOT, "bloomery_amd", "libbm_bench_probe.so")
    if not os.path.exists(path):
        sys.exit(f"bench.py: {path} is not built (make -C bloomery_amd/csrc)")
    lib = C.CDLL(path)
    lib.bm_bench_probe_read.restype = C.c_int
    lib.bm_bench_probe_read.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
    return lib


def timed_graph(gpu, enqueue, unit, steps, warmup):
    """Capture `unit` steps into one graph, replay it for about `steps` timed steps; ms per step by wall clock
    (bracketed by synchronisation) and by events on the launch stream."""
    gpu.capture_begin()
    for i in range(unit):
        enqueue(i)
    graph = gpu.capture_end()
    reps_w, reps = max(1, -(-warmup // unit)), max(1, -(-steps // unit))
    for _ in range(reps_w):
        gpu.graph_launch(graph)
    gpu.sync()
    e0, e1 = gpu.event(), gpu.event()
    t0 = time.perf_counter()
    gpu.event_record(e0)
    for _ in range(reps):
        gpu.graph_launch(graph)
    gpu.event_record(e1)
    gpu.sync()
    wall = (time.perf_counter() - t0) * 1e3 / (reps * unit)
    ev = gpu.event_elapsed_ms(e0, e1) / (reps * unit)
    gpu.graph_destroy(graph)
    gpu.event_destroy(e0)
    gpu.event_destroy(e1)
    return wall, ev, reps * unit, reps_w * unit


def emit(metric, value, unit, steps, warmup, ms_per_step, workload, extra, roofline, cpu, higher=False):
    out = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
           "ms_per_step": ms_per_step, "higher_is_better": higher, "scaling": "weak", "vs_baseline": None,
           "dtype": "i8", "data": "synthetic", "config": {"workload": workload, "mode": "hipGraph replay"}}
    out.update(extra)
    out["roofline"] = roofline
    out["cpu_baseline"] = cpu
    print(json.dumps(out), flush=True)


def cpu_layer_baseline(ora, args, threads, types, shape, stacks, x, ids, wts, top_k, per_call_tokens, bytes_per_call):
    """The AVX2 restatement of the reference's qdot path on the host cores, a bounded sample of the same workload."""
    if args.no_cpu:
        return None
    hidden, ff, n_experts = shape
    pool = ora.lib.ora_pool_create(threads)
    try:
        n, t0 = 0, time.perf_counter()
        while True:
            lo = (n * per_call_tokens) % max(1, x.shape[0] - per_call_tokens + 1)
            ora.moe_forward(hidden, ff, n_experts, types, *stacks, x[lo:lo + per_call_tokens], ids[lo:lo + per_call_tokens],
                            wts[lo:lo + per_call_tokens], top_k, avx2_pool=pool)
            n += 1
            el = time.perf_counter() - t0
            if el >= args.cpu_seconds and n >= 3:
                break
    finally:
        ora.lib.ora_pool_destroy(pool)
    return {"value": el / (n * per_call_tokens) * 1e6, "unit": "us/token", "cores": threads, "kind": "port",
            "sample": f"{n} passes of {per_call_tokens} tokens of the same layer and routings, AVX2 restatement of qdot on "
                      f"{threads} threads, {el:.1f}s"}


def biased_routes(ora, n_tokens, n_experts, top_k, seed, bias_sigma=0.0, zipf=0.0):
    """Router draws: logits N(0, 1) (+ a fixed expert bias N(0, sigma), or + log of a Zipf popularity over a random
    expert permutation), softmax, top-k renormalised."""
    rng = np.random.default_rng(seed)
    bias = np.zeros(n_experts, np.float32)
    if bias_sigma:
        bias = (rng.standard_normal(n_experts) * bias_sigma).astype(np.float32)
    if zipf:
        pop = 1.0 / np.arange(1, n_experts + 1) ** zipf
        bias = np.log(pop / pop.sum())[rng.permutation(n_experts)].astype(np.float32)
    ids = np.empty((n_tokens, top_k), np.uint32)
    wts = np.empty((n_tokens, top_k), np.float32)
    for t in range(n_tokens):
        logits = (rng.standard_normal(n_experts, dtype=np.float32) + bias).astype(np.float32)
        ids[t], wts[t] = ora.route_softmax_topk(logits, top_k)
    return ids, wts


def parity_of(got, want):
    err = float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))
    p = {"max_abs_normalised_err": err, "bit_identical": bool(np.array_equal(got, want))}
    log(f"[bench] parity {p}")
    assert err <= 1e-4, p
    return p


def bench_gemv(args, bm, ora, threads):
    """Config 1: one Q4_K gemv, 768 x 2048, one column."""
    rng = np.random.default_rng(0xB1000001)
    w = ora.quantize_rows(ora.Q4_K, rng.standard_normal((FF, HIDDEN), dtype=np.float32) * np.float32(0.02), FF, HIDDEN,
                          n_threads=threads)
    x = np.random.default_rng(0xAC70001).standard_normal((64, HIDDEN), dtype=np.float32)
    gpu = bm.Gpu(0)
    copies = [gpu.weights(bm.Q4_K, FF, HIDDEN, w) for _ in range(64)]
    xd, y = gpu.upload(x, np.float32), gpu.buffer(np.float32, 64 * FF)
    acts = [gpu.act(bm.Q4_K, HIDDEN, 1) for _ in range(4)]

    def step(i):  # the quantizer folded into the gemv: one launch
        gpu.enqueue_gemv_x(copies[i % 64], xd.ptr + 4 * (i % 64) * HIDDEN, 1, y.ptr + 4 * (i % 64) * FF)

    def chain(i):  # the reference's two launches
        gpu.enqueue_quantize(xd.ptr + 4 * (i % 64) * HIDDEN, 1, acts[i % 4])
        gpu.enqueue_gemv(copies[i % 64], acts[i % 4], 1, y.ptr + 4 * (i % 64) * FF)

    for i in range(4):
        step(i)
    got = y.download()[:4 * FF].reshape(4, FF)
    want = np.stack([ora.gemv(ora.Q4_K, w, FF, HIDDEN, ora.quantize_col(ora.Q4_K, x[i]), 1) for i in range(4)])
    parity = parity_of(got, want)
    wall, ev, steps, warm = timed_graph(gpu, step, 64, args.steps, args.warmup)
    chain(0)  # acts[0] holds a column for the gemv-only graph
    only = timed_graph(gpu, lambda i: gpu.enqueue_gemv(copies[i % 64], acts[i % 4], 1, y.ptr + 4 * (i % 64) * FF), 64, 1024, 64)[1]
    for i in range(4):
        chain(i)
    two = timed_graph(gpu, chain, 64, 1024, 64)[1]
    nbytes = FF * bm.row_bytes(bm.Q4_K, HIDDEN)
    ach = nbytes / (ev * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        col, n, t0 = ora.quantize_col(ora.Q4_K, x[0], avx2=True), 0, time.perf_counter()
        while time.perf_counter() - t0 < min(args.cpu_seconds, 3.0):
            ora.quantize_col(ora.Q4_K, x[n % 64], avx2=True)
            ora.gemv(ora.Q4_K, w, FF, HIDDEN, col, 1)
            n += 1
        cpu = {"value": (time.perf_counter() - t0) / n * 1e6, "unit": "us/gemv", "cores": 1, "kind": "port",
               "sample": f"{n} quantize + gemv calls of the same matrix, scalar restatement of qdot on 1 thread"}
    emit("q4k_gemv_us", wall * 1e3, "us/gemv", steps, warm, wall,
         "single Q4_K gemv 768 x 2048, one column, quantizer included: folded into the gemv launch (BASELINE.json configs[0])",
         {"event_ms_per_step": ev, "kernel_us": {"gemv_x": ev * 1e3, "gemv_alone": only * 1e3, "quantize_then_gemv": two * 1e3},
          "parity": parity, "algorithmic_bytes_per_launch": nbytes},
         {"bound": "hbm", "kernel": "k_gemv_x<Q4_K>", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
          "frac": ach / HBM_PEAK_GBS, "traffic": None}, cpu)
    gpu.close()


def bench_grouped(args, bm, ora, threads):
    """Config 3: the same layer, 16 tokens, expert-biased routing, grouped by expert."""
    m, sets = 16, 8
    wg, wu, wd = make_layer(ora, 0xB1000001, threads)
    x = np.random.default_rng(0xAC70001).standard_normal((m * sets, HIDDEN), dtype=np.float32)
    ids, wts = biased_routes(ora, m * sets, N_EXPERTS, TOP_K, 0x707E0001, bias_sigma=0.5)
    gpu = bm.Gpu(0)
    layers = [(gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, wg), gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, wu),
               gpu.weights(bm.Q6_K, N_EXPERTS * HIDDEN, FF, wd)) for _ in range(args.layers)]
    n_slots = m * TOP_K
    xd, sel, wt = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    y = gpu.buffer(np.float32, m * sets * HIDDEN)
    down = gpu.buffer(np.float32, n_slots * HIDDEN)
    act, act_h = gpu.act(bm.Q4_K, HIDDEN, m), gpu.act(bm.Q6_K, FF, n_slots)
    order, start = gpu.buffer(np.uint32, n_slots), gpu.buffer(np.uint32, N_EXPERTS + 1)
    tiles = gpu.buffer(np.uint32, gpu.tile_cap(n_slots, N_EXPERTS) + 1)

    def step(i, which=("tables", "quant", "gate_up", "down", "combine")):
        st = i % sets
        dg, du, dd = layers[i % len(layers)]
        s_ptr = sel.ptr + 4 * st * n_slots
        if "tables" in which and "quant" in which:  # the whole step: the two as one launch
            gpu.enqueue_tables_quantize(s_ptr, n_slots, N_EXPERTS, order, start, tiles, xd.ptr + 4 * st * m * HIDDEN, m, act)
        elif "tables" in which:
            gpu.enqueue_tables(s_ptr, n_slots, N_EXPERTS, order, start, tiles)
        elif "quant" in which:
            gpu.enqueue_quantize(xd.ptr + 4 * st * m * HIDDEN, m, act)
        if "gate_up" in which:
            gpu.enqueue_gate_up_tiles(dg, du, act, order, start, tiles, n_slots, FF, TOP_K, None, act_h)
        if "down" in which:
            gpu.enqueue_gemv_tiles(dd, act_h, order, start, tiles, n_slots, HIDDEN, down)
        if "combine" in which:
            gpu.enqueue_combine_tokens(down, wt.ptr + 4 * st * n_slots, None, HIDDEN, TOP_K, m, y.ptr + 4 * st * m * HIDDEN)

    step(0)
    want = ora.moe_forward(HIDDEN, FF, N_EXPERTS, (ora.Q4_K, ora.Q4_K, ora.Q6_K), wg, wu, wd, x[:m], ids[:m], wts[:m], TOP_K,
                           n_threads=threads).reshape(m, HIDDEN)
    parity = parity_of(y.download()[:m * HIDDEN].reshape(m, HIDDEN), want)
    wall, ev, steps, warm = timed_graph(gpu, step, 64, args.steps, args.warmup)
    step(0)  # leave set 0's tables for the single-kernel graphs
    kernel_us = {k: timed_graph(gpu, lambda i, k=k: step(i - i % sets, (k,)) if k in ("gate_up", "down") else step(i, (k,)),
                                64, 512, 64)[1] * 1e3 for k in ("tables", "quant", "gate_up", "down", "combine")}
    # the same 16 tokens through the per-slot fused step (bm_moe_decode, two launches): every slot reads its expert's rows
    # for itself, repeats come from the caches
    y2 = gpu.buffer(np.float32, m * sets * HIDDEN)

    def per_slot(i):
        st = i % sets
        dg, du, dd = layers[i % len(layers)]
        gpu.enqueue_moe_decode(dg, du, dd, xd.ptr + 4 * st * m * HIDDEN, sel.ptr + 4 * st * n_slots, wt.ptr + 4 * st * n_slots, None,
                               TOP_K, m, act_h, y2.ptr + 4 * st * m * HIDDEN)

    per_slot(0)
    per_slot_parity = parity_of(y2.download()[:m * HIDDEN].reshape(m, HIDDEN), want)
    per_slot_us = timed_graph(gpu, per_slot, 64, 512, 64)[1] * 1e3
    hit = np.mean([len(np.unique(ids[s * m:(s + 1) * m])) for s in range(sets)])
    per_expert = 2 * FF * bm.row_bytes(bm.Q4_K, HIDDEN) + HIDDEN * bm.row_bytes(bm.Q6_K, FF)
    nbytes = hit * per_expert
    ach = hit * 2 * FF * bm.row_bytes(bm.Q4_K, HIDDEN) / (kernel_us["gate_up"] * 1e-6) / 1e9
    cpu = cpu_layer_baseline(ora, args, threads, (ora.Q4_K, ora.Q4_K, ora.Q6_K), (HIDDEN, FF, N_EXPERTS), (wg, wu, wd), x, ids, wts,
                             TOP_K, m, nbytes)
    emit("moe_layer_decode_us_per_token", wall * 1e3 / m, "us/token", steps, warm, wall,
         "Qwen3-30B-A3B-shaped MoE layer, batched decode of 16 tokens grouped by expert, router logits N(0,1) + expert bias "
         "N(0,0.5) (BASELINE.json configs[2])",
         {"event_ms_per_step": ev, "kernel_us": kernel_us, "parity": parity, "distinct_experts_per_step": float(hit),
          "algorithmic_bytes_per_step": nbytes, "hbm_tbps": nbytes / (wall * 1e-3) / 1e12, "launches_per_step": 5,
          "per_slot_two_launches": {"us_per_step": per_slot_us, "us_per_token": per_slot_us / m, "parity": per_slot_parity,
                                    "note": "bm_moe_decode over the same tokens: not grouped, each slot streams its expert"}},
         {"bound": "hbm", "kernel": "k_gate_up_tiles<Q4_K>", "achieved": ach,
          "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": None}, cpu)
    gpu.close()


def prefill_leg(args, bm, ora, threads, gpu, stacks, layer, m, reps=16):
    """Config 4's step on a layer already on the device: quantize, route, gate and up GEMMs, SwiGLU quantizer, down GEMM,
    combine; 2048 tokens, top-8 of 128 experts, Zipf(1.1) popularity over a random expert permutation. Timed in both f32
    summing modes of bm_gemm (the integer block sums are the same exact ones in both): `fast` keeps the contract's 1e-4,
    `exact` the CPU path's eight-accumulator order bit for bit. Returns the figures as a dict."""
    wg, wu, wd = stacks
    dg, du, dd = layer
    x = np.random.default_rng(0xAC70001).standard_normal((m, HIDDEN), dtype=np.float32)
    ids, wts = biased_routes(ora, m, N_EXPERTS, TOP_K, 0x707E0001, zipf=1.1)
    n_slots = m * TOP_K
    xd, sel, wt = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    act, act_h = gpu.act(bm.Q4_K, HIDDEN, m), gpu.act(bm.Q6_K, FF, n_slots)
    g, u = gpu.buffer(np.float32, n_slots * FF), gpu.buffer(np.float32, n_slots * FF)
    down, y = gpu.buffer(np.float32, n_slots * HIDDEN), gpu.buffer(np.float32, m * HIDDEN)
    table = gpu.route(n_slots, N_EXPERTS)
    names = ("quant", "route", "gate", "up", "swiglu_quant", "down", "combine")

    def step(i, which=names):
        if "quant" in which and "route" in which:  # the whole step: the two as one launch
            table.fill_quantize(sel, n_slots, xd, m, act)
        elif "quant" in which:
            gpu.enqueue_quantize(xd, m, act)
        elif "route" in which:
            table.fill(sel, n_slots)
        if "gate" in which:
            gpu.enqueue_gemm(dg, FF, act, table, TOP_K, g)
        if "up" in which:
            gpu.enqueue_gemm(du, FF, act, table, TOP_K, u)
        if "swiglu_quant" in which:
            gpu.enqueue_swiglu_quant(g, u, n_slots, act_h)
        if "down" in which:
            gpu.enqueue_gemm(dd, HIDDEN, act_h, table, 0, down)
        if "combine" in which:
            gpu.enqueue_combine_tokens(down, wt, None, HIDDEN, TOP_K, m, y)

    n_chk = 4
    want = ora.moe_forward(HIDDEN, FF, N_EXPERTS, (ora.Q4_K, ora.Q4_K, ora.Q6_K), wg, wu, wd, x[:n_chk], ids[:n_chk], wts[:n_chk],
                           TOP_K, n_threads=threads).reshape(n_chk, HIDDEN)
    ops = 2.0 * n_slots * (2 * FF * HIDDEN + HIDDEN * FF)
    gate_ops = 2.0 * n_slots * FF * HIDDEN
    out = {}
    modes = (("fast", bm.GEMM_FAST), ("exact", bm.GEMM_EXACT)) + ((("fast_f16", bm.GEMM_FAST_F16),) if args.gemm_f16 else ())
    for mode, code in modes:
        gpu.set_gemm_mode(code)
        step(0)
        parity = parity_of(y.download()[:n_chk * HIDDEN].reshape(n_chk, HIDDEN), want)
        wall, ev, steps, warm = timed_graph(gpu, step, 2, 2 * reps, 4)
        kernel_us = {k: timed_graph(gpu, lambda i, k=k: step(i, (k,)), 2, 12, 2)[1] * 1e3 for k in names}
        out[mode] = {"ms_per_step": wall, "event_ms_per_step": ev, "steps": steps, "warmup": warm,
                     "tops": ops / (wall * 1e-3) / 1e12, "frac_of_5.0_POPs": ops / (wall * 1e-3) / 5.0e15,
                     "gate_gemm_tops": gate_ops / (kernel_us["gate"] * 1e-6) / 1e12,
                     "gate_gemm_frac_of_5.0_POPs": gate_ops / (kernel_us["gate"] * 1e-6) / 5.0e15,
                     "kernel_us": kernel_us, "parity": parity}
    gpu.set_gemm_mode(bm.GEMM_EXACT)
    hit = len(np.unique(ids))
    res = {"workload": f"Qwen3-30B-A3B-shaped MoE layer, prefill of {m} tokens, top-8 of 128 experts, Zipf(1.1) popularity "
                       "(BASELINE.json configs[3])",
           "mode": "fast: integer block sums exact on the int8 matrix cores, f32 sums within the contract's 1e-4 (bm_set_gemm_mode "
                   "BM_GEMM_FAST); `exact` beside it keeps the CPU path's f32 order bit for bit",
           "int8_ops_per_step": ops, "distinct_experts": hit,
           "weight_bytes_hit": hit * (2 * FF * bm.row_bytes(bm.Q4_K, HIDDEN) + HIDDEN * bm.row_bytes(bm.Q6_K, FF)),
           "us_per_token": out["fast"]["ms_per_step"] * 1e3 / m}
    res.update({k: out["fast"][k] for k in ("tops", "frac_of_5.0_POPs", "ms_per_step", "steps", "warmup", "parity", "gate_gemm_tops",
                                            "gate_gemm_frac_of_5.0_POPs", "kernel_us")})
    res["exact"] = out["exact"]
    if "fast_f16" in out:
        res["fast_f16"] = out["fast_f16"]
    for b in (xd, sel, wt, act, act_h, g, u, down, y, table):
        b.free()
    return res, (x, ids, wts)


def bench_prefill(args, bm, ora, threads):
    """Config 4: the same layer, prefill of 2048 tokens, Zipf(1.1) expert popularity."""
    m = args.prefill_tokens
    stacks = make_layer(ora, 0xB1000001, threads)
    gpu = bm.Gpu(0)
    layer = (gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, stacks[0]), gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, stacks[1]),
             gpu.weights(bm.Q6_K, N_EXPERTS * HIDDEN, FF, stacks[2]))
    res, (x, ids, wts) = prefill_leg(args, bm, ora, threads, gpu, stacks, layer, m)
    cpu = cpu_layer_baseline(ora, args, threads, (ora.Q4_K, ora.Q4_K, ora.Q6_K), (HIDDEN, FF, N_EXPERTS), stacks, x, ids, wts,
                             TOP_K, min(m, 64), 0)
    emit("prefill_int8_tops", res["tops"], "TOP/s", res["steps"], res["warmup"], res["ms_per_step"], res["workload"],
         {k: res[k] for k in ("mode", "int8_ops_per_step", "distinct_experts", "weight_bytes_hit", "us_per_token", "kernel_us",
                              "parity", "exact", "fast_f16") if k in res},
         {"bound": "mfma", "kernel": "k_gemm (gate GEMM, fast mode)", "achieved": res["gate_gemm_tops"], "peak": 5000.0,
          "unit": "TOP/s", "frac": res["gate_gemm_frac_of_5.0_POPs"], "traffic": None}, cpu, higher=True)
    gpu.close()


def random_blocks(rng, wtype, rows, k, block_bytes, d_off):
    """Random legal blocks with small f16 scales (IQ2_XXS stacks: the quantizer's search is too slow for 2.9 GB)."""
    nb = rows * (k // 256)
    w = rng.integers(0, 256, nb * block_bytes, dtype=np.uint8).reshape(nb, block_bytes)
    d = rng.uniform(0.001, 0.02, nb).astype(np.float16).view(np.uint16)
    w[:, d_off] = d & 0xFF
    w[:, d_off + 1] = d >> 8
    return w.reshape(-1)


def bench_dsv3(args, bm, ora, threads):
    """Config 5: DeepSeek-V3-shaped layer, 4 tokens, IQ2_XXS routed experts (grouped) + one Q6_K shared expert."""
    hidden, ff, n_experts, m, sets = 7168, 2048, 256, 4, 8
    rng = np.random.default_rng(0xB1000005)
    t0 = time.time()
    wg = random_blocks(rng, ora.IQ2_XXS, n_experts * ff, hidden, 66, 0)
    wu = random_blocks(rng, ora.IQ2_XXS, n_experts * ff, hidden, 66, 0)
    wd = random_blocks(rng, ora.IQ2_XXS, n_experts * hidden, ff, 66, 0)
    sg = random_blocks(rng, ora.Q6_K, ff, hidden, 210, 208)
    su = random_blocks(rng, ora.Q6_K, ff, hidden, 210, 208)
    sd = random_blocks(rng, ora.Q6_K, hidden, ff, 210, 208)
    log(f"[bench] stacks drawn ({(wg.nbytes * 2 + wd.nbytes) / 1e9:.2f} GB routed) in {time.time() - t0:.1f}s")
    x = np.random.default_rng(0xAC70005).standard_normal((m * sets, hidden), dtype=np.float32)
    ids, wts = biased_routes(ora, m * sets, n_experts, TOP_K, 0x707E0005)
    gpu = bm.Gpu(0)
    dg, du, dd = (gpu.weights(bm.IQ2_XXS, n_experts * ff, hidden, wg), gpu.weights(bm.IQ2_XXS, n_experts * ff, hidden, wu),
                  gpu.weights(bm.IQ2_XXS, n_experts * hidden, ff, wd))
    dsg, dsu, dsd = gpu.weights(bm.Q6_K, ff, hidden, sg), gpu.weights(bm.Q6_K, ff, hidden, su), gpu.weights(bm.Q6_K, hidden, ff, sd)
    n_slots = m * TOP_K
    xd, sel, wt = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    zeros, ones = gpu.upload(np.zeros(m, np.uint32)), gpu.upload(np.ones(m, np.float32))
    act, act6 = gpu.act(bm.IQ2_XXS, hidden, m), gpu.act(bm.Q6_K, hidden, m)
    act_h, act_sh = gpu.act(bm.IQ2_XXS, ff, n_slots), gpu.act(bm.Q6_K, ff, m)
    h, down = gpu.buffer(np.float32, n_slots * ff), gpu.buffer(np.float32, n_slots * hidden)
    sdown = gpu.buffer(np.float32, m * hidden)
    y = gpu.buffer(np.float32, m * sets * hidden)
    order, start = gpu.buffer(np.uint32, n_slots), gpu.buffer(np.uint32, n_experts + 1)
    tiles = gpu.buffer(np.uint32, gpu.tile_cap(n_slots, n_experts) + 1)

    sc = gpu.scratch(bm.IQ2_XXS, bm.IQ2_XXS, hidden, ff, n_experts, TOP_K, m)

    def step(i, which=("shared", "routed")):
        """The shared expert, then bm_moe_forward over the routed ones with the shared expert's rows as the added term
        ((routed sum + shared), the reference's grouping): at this shape its grouped path, which for so few slots an expert is
        the table, the per-slot gate . up launch from the token rows, the quantizer of h, the down tiles and the slot sum."""
        st = i % sets
        s_ptr, x_ptr = sel.ptr + 4 * st * n_slots, xd.ptr + 4 * st * m * hidden
        if "shared" in which:
            gpu.enqueue_quantize(x_ptr, m, act6)
            gpu.enqueue_gate_up(dsg, dsu, act6, zeros, m, ff, 1, None, act_sh)
            gpu.enqueue_gemv_sel(dsd, act_sh, zeros, m, hidden, sdown)
        if "routed" in which:
            gpu.enqueue_moe_forward(sc, dg, du, dd, x_ptr, s_ptr, wt.ptr + 4 * st * n_slots, sdown if "shared" in which else None, m,
                                    y.ptr + 4 * st * m * hidden)

    def tiles_step(i):
        """The same step on the tile launchers alone (what the grouped path was before: ten launches)."""
        st = i % sets
        s_ptr, x_ptr = sel.ptr + 4 * st * n_slots, xd.ptr + 4 * st * m * hidden
        gpu.enqueue_tables(s_ptr, n_slots, n_experts, order, start, tiles)
        gpu.enqueue_quantize(x_ptr, m, act)
        gpu.enqueue_gate_up_tiles(dg, du, act, order, start, tiles, n_slots, ff, TOP_K, h)
        gpu.enqueue_quantize_ord(h, start, n_experts, n_slots, act_h)
        gpu.enqueue_gemv_tiles(dd, act_h, order, start, tiles, n_slots, hidden, down)
        gpu.enqueue_quantize(x_ptr, m, act6)
        gpu.enqueue_gate_up(dsg, dsu, act6, zeros, m, ff, 1, None, act_sh)
        gpu.enqueue_gemv_sel(dsd, act_sh, zeros, m, hidden, sdown)
        gpu.enqueue_moe_combine(down, wt.ptr + 4 * st * n_slots, sdown, None, hidden, TOP_K, m, y.ptr + 4 * st * m * hidden)

    assert sc.path_for(m) == bm.PATH_GROUPED
    step(0)
    types = (ora.IQ2_XXS, ora.IQ2_XXS, ora.IQ2_XXS)
    routed = ora.moe_forward(hidden, ff, n_experts, types, wg, wu, wd, x[:m], ids[:m], wts[:m], TOP_K, n_threads=threads)
    shared = ora.moe_forward(hidden, ff, 1, (ora.Q6_K, ora.Q6_K, ora.Q6_K), sg, su, sd, x[:m], np.zeros((m, 1), np.uint32),
                             np.ones((m, 1), np.float32), 1, n_threads=threads)
    # (routed sum + shared expert), the reference's grouping (crates/gpu/src/moe_fused.rs:129-170)
    want = (np.asarray(routed, np.float32).reshape(m, hidden) + np.asarray(shared, np.float32).reshape(m, hidden)).astype(np.float32)
    parity = parity_of(y.download()[:m * hidden].reshape(m, hidden), want)
    wall, ev, steps, warm = timed_graph(gpu, step, 16, min(args.steps, 256), min(args.warmup, 32))
    kernel_us = {k: timed_graph(gpu, lambda i, k=k: step(i, (k,)), 16, 64, 16)[1] * 1e3 for k in ("routed", "shared")}
    tiles_step(0)
    tiles_parity = parity_of(y.download()[:m * hidden].reshape(m, hidden), want)
    tiles_us = timed_graph(gpu, tiles_step, 16, 128, 16)[1] * 1e3
    # the same tokens through the per-slot fused step: the shared expert first, its rows the term bm_moe_decode adds to
    # the slots' sum ((sum + shared), the same grouping); five launches, no tables
    y2 = gpu.buffer(np.float32, m * sets * hidden)

    def per_slot(i):
        st = i % sets
        s_ptr, x_ptr = sel.ptr + 4 * st * n_slots, xd.ptr + 4 * st * m * hidden
        gpu.enqueue_quantize(x_ptr, m, act6)
        gpu.enqueue_gate_up(dsg, dsu, act6, zeros, m, ff, 1, None, act_sh)
        gpu.enqueue_gemv_sel(dsd, act_sh, zeros, m, hidden, sdown)
        gpu.enqueue_moe_decode(dg, du, dd, x_ptr, s_ptr, wt.ptr + 4 * st * n_slots, sdown, TOP_K, m, act_h, y2.ptr + 4 * st * m * hidden, h=h)

    per_slot(0)
    per_slot_parity = parity_of(y2.download()[:m * hidden].reshape(m, hidden), want)
    per_slot_us = timed_graph(gpu, per_slot, 16, 128, 16)[1] * 1e3
    # the shared expert on a stream of its own beside the routed experts (a second context; fork and join by events, one graph):
    # the routed step without an added term, then (routed sum + shared) as a closing launch over one "slot" of weight 1
    side = bm.Gpu(0)
    forked, joined = gpu.event(), gpu.event()
    y3, routed_rows = gpu.buffer(np.float32, m * sets * hidden), gpu.buffer(np.float32, m * hidden)

    def two_streams(i):
        st = i % sets
        s_ptr, x_ptr = sel.ptr + 4 * st * n_slots, xd.ptr + 4 * st * m * hidden
        gpu.event_record(forked)
        side.event_wait(forked)
        side.enqueue_quantize(x_ptr, m, act6)
        side.enqueue_gate_up(dsg, dsu, act6, zeros, m, ff, 1, None, act_sh)
        side.enqueue_gemv_sel(dsd, act_sh, zeros, m, hidden, sdown)
        side.event_record(joined)
        gpu.enqueue_moe_forward(sc, dg, du, dd, x_ptr, s_ptr, wt.ptr + 4 * st * n_slots, None, m, routed_rows)
        gpu.event_wait(joined)
        gpu.enqueue_combine_tokens(routed_rows, ones, sdown, hidden, 1, m, y3.ptr + 4 * st * m * hidden)

    gpu.capture_begin()
    two_streams(0)
    g0 = gpu.capture_end()
    gpu.graph_launch(g0)
    gpu.sync()
    gpu.graph_destroy(g0)
    two_streams_parity = parity_of(y3.download()[:m * hidden].reshape(m, hidden), want)
    two_streams_us = timed_graph(gpu, two_streams, 16, 128, 16)[1] * 1e3
    assert side.fault() == (bm.FAULT_NONE, 0)
    side.close()
    hit = np.mean([len(np.unique(ids[s * m:(s + 1) * m])) for s in range(sets)])
    per_expert = (2 * ff * bm.row_bytes(bm.IQ2_XXS, hidden) + hidden * bm.row_bytes(bm.IQ2_XXS, ff))
    shared_bytes = 2 * ff * bm.row_bytes(bm.Q6_K, hidden) + hidden * bm.row_bytes(bm.Q6_K, ff)
    nbytes = hit * per_expert + shared_bytes
    ach = nbytes / (wall * 1e-3) / 1e9
    cpu = None
    emit("moe_layer_decode_us_per_token", wall * 1e3 / m, "us/token", steps, warm, wall,
         "DeepSeek-V3-shaped MoE layer decode, 4 tokens: hidden 7168, 256 IQ2_XXS experts of ff 2048 top-8 (bm_moe_forward) + one "
         "Q6_K shared expert; random legal blocks (BASELINE.json configs[4])",
         {"event_ms_per_step": ev, "kernel_us": kernel_us, "parity": parity, "distinct_experts_per_step": float(hit),
          "algorithmic_bytes_per_step": nbytes, "hbm_tbps": ach / 1e3,
          "tile_launchers_only_ten_launches": {"us_per_step": tiles_us, "us_per_token": tiles_us / m, "parity": tiles_parity},
          "per_slot_five_launches": {"us_per_step": per_slot_us, "us_per_token": per_slot_us / m, "parity": per_slot_parity,
                                     "note": "shared expert, then bm_moe_decode over the slots with its rows as the added term"},
          "shared_expert_on_a_stream_of_its_own": {"us_per_step": two_streams_us, "us_per_token": two_streams_us / m,
                                                   "parity": two_streams_parity,
                                                   "note": "two contexts forked and joined by events inside one graph; nine launches"}},
         {"bound": "hbm", "kernel": "whole step (8 launches)", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
          "frac": ach / HBM_PEAK_GBS, "traffic": None}, cpu)
    gpu.close()


def bench_dsv3_prefill(args, bm, ora, threads):
    """Config 7: the DeepSeek-V3-shaped routed experts at prefill, 2048 tokens: IQ2_XXS stacks on Q8_K columns through
    bm_gemm, in both f32 summing modes. A side measurement: BASELINE.json holds no prefill figure for this shape."""
    hidden, ff, n_experts, m = 7168, 2048, 256, 2048
    rng = np.random.default_rng(0xB1000007)
    t0 = time.time()
    wg = random_blocks(rng, ora.IQ2_XXS, n_experts * ff, hidden, 66, 0)
    wu = random_blocks(rng, ora.IQ2_XXS, n_experts * ff, hidden, 66, 0)
    wd = random_blocks(rng, ora.IQ2_XXS, n_experts * hidden, ff, 66, 0)
    log(f"[bench] stacks drawn ({(wg.nbytes * 2 + wd.nbytes) / 1e9:.2f} GB) in {time.time() - t0:.1f}s")
    x = np.random.default_rng(0xAC70007).standard_normal((m, hidden), dtype=np.float32)
    ids, wts = biased_routes(ora, m, n_experts, TOP_K, 0x707E0007, zipf=1.1)
    n_slots = m * TOP_K
    gpu = bm.Gpu(0)
    dg, du, dd = (gpu.weights(bm.IQ2_XXS, n_experts * ff, hidden, wg), gpu.weights(bm.IQ2_XXS, n_experts * ff, hidden, wu),
                  gpu.weights(bm.IQ2_XXS, n_experts * hidden, ff, wd))
    xd, sel, wt = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    act, act_h = gpu.act(bm.IQ2_XXS, hidden, m), gpu.act(bm.IQ2_XXS, ff, n_slots)
    g, u = gpu.buffer(np.float32, n_slots * ff), gpu.buffer(np.float32, n_slots * ff)
    down, y = gpu.buffer(np.float32, n_slots * hidden), gpu.buffer(np.float32, m * hidden)
    table = gpu.route(n_slots, n_experts)
    names = ("quant", "route", "gate", "up", "swiglu_quant", "down", "combine")

    def step(i, which=names):
        if "quant" in which and "route" in which:  # the whole step: the two as one launch
            table.fill_quantize(sel, n_slots, xd, m, act)
        elif "quant" in which:
            gpu.enqueue_quantize(xd, m, act)
        elif "route" in which:
            table.fill(sel, n_slots)
        if "gate" in which:
            gpu.enqueue_gemm(dg, ff, act, table, TOP_K, g)
        if "up" in which:
            gpu.enqueue_gemm(du, ff, act, table, TOP_K, u)
        if "swiglu_quant" in which:
            gpu.enqueue_swiglu_quant(g, u, n_slots, act_h)
        if "down" in which:
            gpu.enqueue_gemm(dd, hidden, act_h, table, 0, down)
        if "combine" in which:
            gpu.enqueue_combine_tokens(down, wt, None, hidden, TOP_K, m, y)

    n_chk = 2
    types = (ora.IQ2_XXS, ora.IQ2_XXS, ora.IQ2_XXS)
    want = ora.moe_forward(hidden, ff, n_experts, types, wg, wu, wd, x[:n_chk], ids[:n_chk], wts[:n_chk], TOP_K,
                           n_threads=threads).reshape(n_chk, hidden)
    ops = 2.0 * n_slots * 3 * ff * hidden
    gate_ops = 2.0 * n_slots * ff * hidden
    out = {}
    for mode, code in (("fast", bm.GEMM_FAST), ("exact", bm.GEMM_EXACT)):
        gpu.set_gemm_mode(code)
        step(0)
        parity = parity_of(y.download()[:n_chk * hidden].reshape(n_chk, hidden), want)
        wall, ev, steps, warm = timed_graph(gpu, step, 1, 6, 2)
        kernel_us = {k: timed_graph(gpu, lambda i, k=k: step(i, (k,)), 1, 4, 1)[1] * 1e3 for k in names}
        out[mode] = {"ms_per_step": wall, "event_ms_per_step": ev, "steps": steps, "warmup": warm,
                     "tops": ops / (wall * 1e-3) / 1e12, "frac_of_5.0_POPs": ops / (wall * 1e-3) / 5.0e15,
                     "gate_gemm_tops": gate_ops / (kernel_us["gate"] * 1e-6) / 1e12,
                     "gate_gemm_frac_of_5.0_POPs": gate_ops / (kernel_us["gate"] * 1e-6) / 5.0e15,
                     "kernel_us": kernel_us, "parity": parity}
        log(f"[bench] {mode}: {out[mode]}")
    gpu.set_gemm_mode(bm.GEMM_EXACT)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    f = out["fast"]
    emit("moe_layer_prefill_int8_tops", f["tops"], "TOP/s", f["steps"], f["warmup"], f["ms_per_step"],
         "DeepSeek-V3-shaped routed experts, prefill of 2048 tokens: hidden 7168, 256 IQ2_XXS experts of ff 2048 top-8, Zipf(1.1) "
         "popularity, Q8_K columns; random legal blocks (a side measurement; the shape is BASELINE.json configs[4]'s)",
         {"mode": "fast (BM_GEMM_FAST); `exact` beside it", "int8_ops_per_step": ops, "distinct_experts": int(len(np.unique(ids))),
          "fast": f, "exact": out["exact"]},
         {"bound": "mfma", "kernel": "k_gemm_iq<IQ2_XXS, fast> (gate)", "achieved": f["gate_gemm_tops"], "peak": 5000.0, "unit": "TOP/s",
          "frac": f["gate_gemm_frac_of_5.0_POPs"], "traffic": None}, None, higher=True)
    gpu.close()


def bench_paths(args, bm, ora, threads):
    """Config 8: bm_moe_forward's three paths over the number of tokens, on the headline layer with config 3's routing: the
    crossovers behind its automatic choice. A side measurement."""
    wg, wu, wd = make_layer(ora, 0xB1000001, threads)
    counts = (1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256, 512, 1024)
    if args.path_tokens:  # a few counts only (the run to put under a profiler)
        counts = tuple(sorted(int(t) for t in args.path_tokens.split(",")))
        assert all(1 <= t <= 1024 for t in counts), "--path-tokens: counts of 1 .. 1024"
    m_max, sets = counts[-1], 4
    x = np.random.default_rng(0xAC70001).standard_normal((m_max, HIDDEN), dtype=np.float32)
    ids, wts = biased_routes(ora, m_max * sets, N_EXPERTS, TOP_K, 0x707E0001, bias_sigma=0.5)
    gpu = bm.Gpu(0)
    layers = [(gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, wg), gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, wu),
               gpu.weights(bm.Q6_K, N_EXPERTS * HIDDEN, FF, wd)) for _ in range(args.layers)]
    xd, sel, wt = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    y = gpu.buffer(np.float32, m_max * HIDDEN)
    sc = gpu.scratch(bm.Q4_K, bm.Q6_K, HIDDEN, FF, N_EXPERTS, TOP_K, m_max)
    want = ora.moe_forward(HIDDEN, FF, N_EXPERTS, (ora.Q4_K, ora.Q4_K, ora.Q6_K), wg, wu, wd, x[:4], ids[:4], wts[:4], TOP_K,
                           n_threads=threads).reshape(4, HIDDEN)
    rows = []
    for m in counts:
        row = {"tokens": m}
        for name, path, mode in (("per_slot", bm.PATH_PER_SLOT, bm.GEMM_EXACT), ("grouped", bm.PATH_GROUPED, bm.GEMM_EXACT),
                                 ("gemm_exact", bm.PATH_GEMM, bm.GEMM_EXACT), ("gemm_fast", bm.PATH_GEMM, bm.GEMM_FAST)):
            sc.set_path(path)
            gpu.set_gemm_mode(mode)

            def step(i, m=m):
                dg, du, dd = layers[i % len(layers)]
                st = i % sets
                gpu.enqueue_moe_forward(sc, dg, du, dd, xd, sel.ptr + 4 * st * m * TOP_K, wt.ptr + 4 * st * m * TOP_K, None, m, y)

            step(0)
            if m >= 4:
                p = parity_of(y.download()[:4 * HIDDEN].reshape(4, HIDDEN), want)
                assert p["max_abs_normalised_err"] <= 1e-4, (name, m, p)
            unit = 16 if m <= 64 else 4
            row[name] = timed_graph(gpu, step, unit, max(2 * unit, min(256, 8192 // m)), unit)[1] * 1e3
        row["fastest_exact"] = min(("per_slot", "grouped", "gemm_exact"), key=lambda k: row[k])
        rows.append(row)
        log(f"[bench] {row}")
    gpu.set_gemm_mode(bm.GEMM_EXACT)
    sc.set_path(bm.PATH_AUTO)
    auto = {m: {bm.PATH_PER_SLOT: "per_slot", bm.PATH_GROUPED: "grouped", bm.PATH_GEMM: "gemm_exact"}[sc.path_for(m)] for m in counts}
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    worst = max(r[auto[r["tokens"]]] / r[r["fastest_exact"]] for r in rows)
    head = next((r for r in rows if r["tokens"] == 16), rows[0])
    emit("moe_layer_us_per_step_by_path", head["per_slot"], "us/step", 0, 0, head["per_slot"] * 1e-3,
         "Qwen3-30B-A3B-shaped MoE layer, 1 to 1024 tokens a step through each path of bm_moe_forward, config 3's routing "
         "(a side measurement: which path for how many tokens)",
         {"us_per_step": rows, "automatic_choice": auto, "automatic_over_fastest_worst_case": worst},
         {"bound": "hbm", "kernel": "n/a", "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None}, None)
    gpu.close()


def bench_card(args, bm, ora, threads):
    """Config 6 (a side measurement, not a BASELINE.json line): the card rule. The MoE down step of the reference's GPU
    tier at the headline layer's down shape (8 slots of 768 values against 2048 Q4_K rows of 8 of 128 resident experts:
    the q8_1 quantizer, then the 32-lane row walks), and one large Q4_K gemv by the same walk for its streaming rate."""
    rng = np.random.default_rng(0xB1000006)
    def q4k_blocks(rows, k):  # a finite dmin beside the finite d
        w = random_blocks(rng, bm.Q4_K, rows, k, 144, 0).reshape(-1, 144)
        w[:, 2:4] = rng.uniform(0.001, 0.02, w.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
        return w.reshape(-1)

    wd = q4k_blocks(N_EXPERTS * HIDDEN, FF)
    n_tok = args.tokens
    h = rng.uniform(-2, 2, (n_tok * TOP_K, FF)).astype(np.float32)
    ids = np.stack([rng.choice(N_EXPERTS, TOP_K, replace=False) for _ in range(n_tok)]).astype(np.uint32)
    gpu = bm.Gpu(0)
    copies = [gpu.weights(bm.Q4_K, N_EXPERTS * HIDDEN, FF, wd) for _ in range(args.layers)]
    hd, sel = gpu.upload(h, np.float32), gpu.upload(ids, np.uint32)
    codes, d8, s8 = gpu.buffer(np.int8, n_tok * TOP_K * FF), gpu.buffer(np.float32, n_tok * TOP_K * FF // 128), \
        gpu.buffer(np.int32, n_tok * TOP_K * FF // 32)
    y = gpu.buffer(np.float32, n_tok * TOP_K * HIDDEN)

    def planes(t):
        return codes.ptr + t * TOP_K * FF, d8.ptr + 4 * t * TOP_K * FF // 128, s8.ptr + 4 * t * TOP_K * FF // 32

    def quant(i):
        t = i % n_tok
        gpu.enqueue_card_quantize(hd.ptr + 4 * t * TOP_K * FF, TOP_K, FF, *planes(t))

    def down(i):
        t = i % n_tok
        gpu.enqueue_card_gemv_sel(copies[i % len(copies)], *planes(t), sel.ptr + 4 * t * TOP_K, TOP_K, HIDDEN,
                                  y.ptr + 4 * t * TOP_K * HIDDEN)

    def step(i):
        quant(i)
        down(i)

    for i in range(2):
        step(i)
    got = y.download()[:2 * TOP_K * HIDDEN]
    c, d, s, _ = ora.card_q8_1(h[:2 * TOP_K])
    want = ora.card_gemv_sel(ora.Q4_K, wd, N_EXPERTS, HIDDEN, FF, c, d, s, ids[:2].reshape(-1))
    parity = parity_of(got, want)
    wall, ev, steps, warm = timed_graph(gpu, step, n_tok, args.steps, args.warmup)
    kernel_us = {"card_quantize": timed_graph(gpu, quant, n_tok, 1024, 64)[1] * 1e3,
                 "card_gemv_sel": timed_graph(gpu, down, n_tok, 1024, 64)[1] * 1e3}
    nbytes = TOP_K * HIDDEN * bm.row_bytes(bm.Q4_K, FF)
    ach = nbytes / (kernel_us["card_gemv_sel"] * 1e-6) / 1e9
    # the walk's streaming rate: 32768 rows of 4096 values, four copies cycled
    rows_big, k_big = 32768, 4096
    wb = q4k_blocks(rows_big, k_big)
    big = [gpu.weights(bm.Q4_K, rows_big, k_big, wb) for _ in range(4)]
    xb = gpu.upload(rng.uniform(-2, 2, k_big).astype(np.float32), np.float32)
    cb, db, sb = gpu.buffer(np.int8, k_big), gpu.buffer(np.float32, k_big // 128), gpu.buffer(np.int32, k_big // 32)
    yb = gpu.buffer(np.float32, rows_big)
    gpu.enqueue_card_quantize(xb, 1, k_big, cb, db, sb)
    big_ms = timed_graph(gpu, lambda i: gpu.enqueue_card_gemv(big[i % 4], cb, db, sb, 1, yb), 8, 64, 8)[1]
    big_gbs = rows_big * bm.row_bytes(bm.Q4_K, k_big) / (big_ms * 1e-3) / 1e9
    cq, dq, sq, _ = ora.card_q8_1(xb.download())
    rb = bm.row_bytes(bm.Q4_K, k_big)
    big_parity = parity_of(yb.download()[-64:], ora.card_gemv(ora.Q4_K, wb[-64 * rb:], 64, k_big, cq, dq, sq))
    cpu = None
    if not args.no_cpu:
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < min(args.cpu_seconds, 10.0):
            t = n % n_tok
            c, d, s, _ = ora.card_q8_1(h[t * TOP_K:(t + 1) * TOP_K])
            ora.card_gemv_sel(ora.Q4_K, wd, N_EXPERTS, HIDDEN, FF, c, d, s, ids[t])
            n += 1
        cpu = {"value": (time.perf_counter() - t0) / n * 1e6, "unit": "us/token", "cores": 1, "kind": "port",
               "sample": f"{n} tokens' quantize + down step, scalar restatement of qdot's card mirrors on 1 thread"}
    emit("card_rule_down_step_us_per_token", wall * 1e3, "us/token", steps, warm, wall,
         "the card rule's MoE down step: 8 slots x 768 values, q8_1 quantizer + 32-lane Q4_K walks over 2048 rows of 8 of 128 "
         "experts; random legal blocks (not a BASELINE.json configuration)",
         {"event_ms_per_step": ev, "kernel_us": kernel_us, "parity": parity, "algorithmic_bytes_per_launch": nbytes,
          "large_gemv": {"rows": rows_big, "k": k_big, "ms": big_ms, "gb_per_s": big_gbs, "parity_last_64_rows": big_parity}},
         {"bound": "hbm", "kernel": "k_card_gemv_sel<Q4_K>", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
          "frac": ach / HBM_PEAK_GBS, "traffic": None}, cpu)
    gpu.close()


def timeline(args, bm, gpu, enqueue_step, type_names):
    """The decode step's two launches seen from inside: the measurement build's kernels leave the device's constant-rate
    counter (100 MHz) at marks in every workgroup; a graph of 193 steps is replayed three times and the last step's marks are
    read (cold rows: a different token and layer copy every step)."""
    import ctypes as C
    lib = gpu.lib
    lib.bm_timeline_read.restype = C.c_int
    lib.bm_timeline_read.argtypes = [C.c_void_p]
    gpu.capture_begin()
    for i in range(193):
        enqueue_step(i)
    graph = gpu.capture_end()
    for _ in range(3):
        gpu.graph_launch(graph)
    gpu.sync()
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    rows = 4096
    tr = np.zeros(rows * 8, np.uint64)
    rc = lib.bm_timeline_read(tr.ctypes.data)
    assert rc == 0, f"bm_timeline_read: {rc}"
    tr = tr.reshape(rows, 8).astype(np.int64)
    n_a, n_b = TOP_K * FF // 32, HIDDEN // (64 // TOP_K)
    a, b = tr[:n_a, :5], tr[rows // 2:rows // 2 + n_b, :7]
    t0 = a[:, 0].min()

    def stat(v):
        v = (v - t0) / 100.0
        return {"min": round(float(v.min()), 2), "median": round(float(np.median(v)), 2), "max": round(float(v.max()), 2)}
    out = {"unit": "us after the first workgroup of k_gate_up_x started", "gate": type_names[0], "down": type_names[1],
           "down_form": args.down_form,
           "k_gate_up_x": {"workgroups": n_a,
                           **{name: stat(a[:, i]) for i, name in enumerate(("start", "expert_id_known", "token_quantized", "rows_dotted", "h_block_stored"))}},
           "k_down_combine": {"workgroups": n_b,
                              **{name: stat(b[:, i]) for i, name in ((0, "start"), (4, "expert_id_known"), (5, "ring_asked_for"),
                                                                        (6, "columns_arrived"), (1, "columns_in_lds"),
                                                                        (2, "rows_dotted"), (3, "sum_stored"))}}}
    out["launch_boundary_us"] = round(out["k_down_combine"]["start"]["min"] - out["k_gate_up_x"]["h_block_stored"]["max"], 2)
    # the router launch of one token (norm, logits, routing: bm_norm_route), the same way: 65 launches in a graph, the last one's marks
    rng = np.random.default_rng(0x707E0001)
    router_d = gpu.upload(rng.standard_normal((N_EXPERTS, HIDDEN), dtype=np.float32) * np.float32(0.05), np.float32)
    xr = gpu.upload(rng.standard_normal((64, HIDDEN), dtype=np.float32), np.float32)
    gain_d = gpu.upload(np.ones(HIDDEN, np.float32), np.float32)
    normed_d, logits_d = gpu.buffer(np.float32, HIDDEN), gpu.buffer(np.float32, N_EXPERTS)
    ids_d, wts_d = gpu.buffer(np.uint32, TOP_K), gpu.buffer(np.float32, TOP_K)
    gpu.capture_begin()
    for i in range(65):
        gpu.enqueue_norm_route(router_d, xr.ptr + 4 * (i % 64) * HIDDEN, gain_d, 1e-6, 1, N_EXPERTS, HIDDEN, TOP_K, True, normed_d,
                               logits_d, None, ids_d, wts_d)
    graph = gpu.capture_end()
    for _ in range(3):
        gpu.graph_launch(graph)
    gpu.sync()
    lib.bm_router_timeline_read.restype = C.c_int
    lib.bm_router_timeline_read.argtypes = [C.c_void_p]
    rt = np.zeros(1024 * 8, np.uint64)
    rc = lib.bm_router_timeline_read(rt.ctypes.data)
    assert rc == 0, f"bm_router_timeline_read: {rc}"
    rt = rt.reshape(1024, 8).astype(np.int64)
    n_r = int(np.count_nonzero(rt[:, 0]))
    rt, wave = rt[:n_r - 1], rt[n_r - 1]  # the logits' workgroups, and behind them in the grid the token's routing workgroup
    r0 = min(rt[:, 0].min(), wave[0])
    out["k_norm_route"] = {"unit": "us after the launch's first workgroup started", "workgroups": n_r,
                           **{name: {"min": round(float((rt[:, i].min() - r0) / 100.0), 2), "median": round(float(np.median(rt[:, i] - r0) / 100.0), 2),
                                     "max": round(float((rt[:, i].max() - r0) / 100.0), 2)}
                              for i, name in enumerate(("start", "token_row_arrived", "normed", "rows_and_token_in_lds", "dots_done"))},
                           "routing_wave": {"start": round(float((wave[0] - r0) / 100.0), 2),
                                            "holds_every_logit": round(float((wave[4] - r0) / 100.0), 2),
                                            "maximum_known": round(float((wave[1] - r0) / 100.0), 2),
                                            "exponentials_summed": round(float((wave[2] - r0) / 100.0), 2),
                                            "probabilities_stored": round(float((wave[3] - r0) / 100.0), 2),
                                            "entries_ahead_counted_by_its_wave": round(float((wave[6] - r0) / 100.0), 2),
                                            "and_by_every_wave": round(float((wave[7] - r0) / 100.0), 2),
                                            "routed": round(float((wave[5] - r0) / 100.0), 2)}}
    print(json.dumps(out, indent=1), flush=True)
    gpu.close()


def handoff(bm, gpu, src, src_bytes):
    """What handing data from one workgroup to others costs inside a launch (a flag and 64 words through memory with device-scope
    stores and loads, the only scope another compute unit sees), to be read against the launch boundary of the decode step:
    pollers on the writer's XCD and on others, the rest of the chip idle, streaming reads, or the pollers' own compute units
    streaming too. Times from the writer's flag store to the poller holding the words, 20 launches a case."""
    import ctypes as C
    probe = load_probe()
    probe.bm_bench_probe_handoff.restype = C.c_int
    probe.bm_bench_probe_handoff.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_int, C.c_int]
    stream = gpu.lib.bm_ctx_stream(gpu.ctx)
    flag, out_d, sink = gpu.buffer(np.uint32, 128).fill_bytes(0), gpu.buffer(np.uint64, 2048), gpu.buffer(np.uint32, 256)
    same, other = (8, 16, 248), (1, 4, 255)
    res, gen = {"unit": "ns", "launches_a_case": 20, "writer": 0, "pollers_on_the_writers_xcd": list(same), "pollers_on_other_xcds": list(other)}, 0
    for load, name in ((0, "idle"), (1, "other_compute_units_stream"), (2, "every_compute_unit_streams")):
        lat = {w: [] for w in same + other}
        ack = []
        for _ in range(20):
            gen += 1
            out_d.fill_bytes(0)
            rc = probe.bm_bench_probe_handoff(stream, src, src_bytes, flag.ptr, out_d.ptr, sink.ptr, gen, load, 400)
            assert rc == 0, f"bm_bench_probe_handoff: {rc}"
            gpu.sync()
            o = out_d.download().reshape(256, 8).astype(np.int64)
            if gen == 1:
                res["workgroups_on_the_xcd_of_their_index_mod_8"] = int(sum(o[w, 0] == o[w % 8, 0] for w in range(256)))
            ack.append((o[0, 3] - o[0, 2]) * 10)
            for w in lat:
                assert o[w, 4] == 1, f"workgroup {w} did not see the words (polls {o[w, 5]})"
                lat[w].append((o[w, 3] - o[0, 2]) * 10)
        res[name] = {"flag_store_acknowledged": float(np.mean(ack)),
                     "same_xcd_mean": float(np.mean([lat[w] for w in same])), "same_xcd_max": float(np.max([lat[w] for w in same])),
                     "other_xcd_mean": float(np.mean([lat[w] for w in other])), "other_xcd_max": float(np.max([lat[w] for w in other]))}
    print(json.dumps(res, indent=1), flush=True)
    gpu.close()


def read_patterns(bm, gpu, layers, sel, n_tok):
    """What the two decode launches' requests cost with nothing computed, and what other ways of asking for the same bytes would
    (bloomery_amd/csrc/bench_probe.hip): graph replay over the cycling routings and layer copies as the timed step, us a launch."""
    import ctypes as C
    probe = load_probe()
    probe.bm_bench_probe_gate_up_rows.restype = C.c_int
    probe.bm_bench_probe_gate_up_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    probe.bm_bench_probe_down_rows.restype = C.c_int
    probe.bm_bench_probe_down_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
    stream = gpu.lib.bm_ctx_stream(gpu.ctx)
    sink = gpu.buffer(np.uint32, 4096)

    def timed(enqueue):
        return round(min(timed_graph(gpu, enqueue, 256, 1024, 256)[1] * 1e3 for _ in range(2)), 3)

    res = {"unit": "us a launch, graph replay, cold rows", "gate_up_bytes": TOP_K * 2 * FF * bm.row_bytes(bm.Q4_K, HIDDEN),
           "down_bytes": TOP_K * HIDDEN * bm.row_bytes(bm.Q6_K, FF), "gate_up": {}, "down": {}}
    for name, pattern, threads, ahead in (("quad_a_row_4_ahead_192x256_as_k_gate_up_x", 0, 256, 4), ("quad_a_row_8_ahead_192x256", 0, 256, 8),
                                          ("quad_a_row_4_ahead_256x192", 0, 192, 4), ("quad_a_row_8_ahead_256x192", 0, 192, 8),
                                          ("octet_a_row_pair_192x256", 1, 256, 8), ("octet_a_row_pair_256x192", 1, 192, 8),
                                          ("workgroup_contiguous_192x256", 2, 256, 8), ("workgroup_contiguous_256x192", 2, 192, 8),
                                          ("into_lds_nine_lanes_a_row_super_block_192x256", 3, 256, 8),
                                          ("into_lds_wave_rows_contiguous_192x256", 4, 256, 8)):
        def enqueue(i):
            dg, du, _ = layers[i % len(layers)]
            rc = probe.bm_bench_probe_gate_up_rows(stream, dg.dev_ptr, du.dev_ptr, sel.ptr + 4 * TOP_K * (i % n_tok), FF, pattern, threads,
                                                   ahead, sink.ptr)
            assert rc == 0, f"bm_bench_probe_gate_up_rows: {rc}"
        res["gate_up"][name] = timed(enqueue)
    planes = [gpu.buffer(np.uint8, N_EXPERTS * HIDDEN * 640).fill_bytes(0x11) for _ in range(4)]
    for name, layout in (("rows_of_630_bytes_as_they_are", 0), ("rows_as_planes_of_640_bytes", 1)):
        def enqueue(i):
            base = layers[i % len(layers)][2].dev_ptr if layout == 0 else planes[i % len(planes)].ptr
            rc = probe.bm_bench_probe_down_rows(stream, base, sel.ptr + 4 * TOP_K * (i % n_tok), HIDDEN, layout, sink.ptr)
            assert rc == 0, f"bm_bench_probe_down_rows: {rc}"
        res["down"][name] = timed(enqueue)
    print(json.dumps(res, indent=1), flush=True)
    gpu.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", type=int, default=2, choices=(1, 2, 3, 4, 5, 6, 7, 8),
                    help="1: one Q4_K gemv; 2 (default, the headline): Qwen3-shaped layer, 1 token; 3: the same layer, 16 tokens "
                         "grouped by expert; 4: prefill of 2048 tokens (int8 MFMA GEMM); 5: DeepSeek-V3-shaped layer, 4 tokens; "
                         "6: the card rule's down step (a side measurement); 7: DeepSeek-V3-shaped IQ2_XXS experts at prefill (a side "
                         "measurement); 8: the three paths of bm_moe_forward over the number of tokens (a side measurement)")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--path-tokens", default="", help="config 8 only: the token counts to run, comma separated (default: the whole sweep)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="config 2 only: no timing; 8 copies of 64 MiB by a plain kernel (the counters' calibration), then "
                         "256 eager steps - the run to put under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2048)
    ap.add_argument("--warmup", type=int, default=256)
    ap.add_argument("--layers", type=int, default=32,
                    help="distinct device copies of the layer cycled through: step i takes copy i %% layers, so with 64 tokens and 32 "
                         "copies two reads of the same expert of the same copy lie 32 steps = 780 MB apart, three times the memory-side "
                         "cache")
    ap.add_argument("--tokens", type=int, default=64, help="distinct tokens (and routings) cycled through")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--one-interval", action="store_true",
                    help="config 2 only: leave out the 32 replays with an event after each that give the median beside `value` (one replay "
                         "instead): for runs under a profiler, whose interception of a graph launch has crashed with events recorded between "
                         "the launches")
    ap.add_argument("--no-prefill", action="store_true", help="config 2 only: leave the prefill leg (config 4's step) out of the line")
    ap.add_argument("--types", default="q4_k,q6_k",
                    help="config 2 only: gate/up and down weight types (q3_k, q4_k, q5_k, q6_k, iq2_xxs, iq3_xxs, iq4_xs); other than the default is "
                         "a side measurement of that type, not the headline workload")
    ap.add_argument("--timeline", action="store_true",
                    help="config 2 only: no timing by events; the step's two launches through the measurement build of the library "
                         "(libbm_moe_hip_timeline.so), whose kernels leave the device's 100 MHz counter at marks inside every "
                         "workgroup; prints when each phase of each launch is reached")
    ap.add_argument("--down-form", choices=("ring", "split"), default="ring",
                    help="config 2 only: how the down launch walks a row (bm_set_down_form); `split` is the measured alternative, a side measurement")
    ap.add_argument("--gemm-f16", action="store_true",
                    help="prefill leg: also time the tolerance mode's f16-operand form (BM_GEMM_FAST_F16, Q4_K GEMMs), under `fast_f16`")
    ap.add_argument("--read-patterns", action="store_true",
                    help="config 2 only (Q4_K / Q6_K): no timing of the step; the decode launches' read patterns with nothing computed, "
                         "and other ways of asking for the same bytes")
    ap.add_argument("--handoff", action="store_true",
                    help="config 2 only: no timing of the step; what a hand-over between workgroups inside one launch costs (--layers 1 is enough)")
    ap.add_argument("--mode", choices=("two", "chain"), default="two",
                    help="two: bm_moe_decode, two launches with the quantizers folded in; chain: quantize, gate_up, down_combine")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus above 1 is not supported (nothing here shards)")

    import bloomery_amd as bm
    import ora

    if args.timeline:
        bm.load_library(os.path.join(ROOT, "bloomery_amd", "libbm_moe_hip_timeline.so"))
    threads = host_threads()
    if args.config != 2:
        return {1: bench_gemv, 3: bench_grouped, 4: bench_prefill, 5: bench_dsv3, 6: bench_card, 7: bench_dsv3_prefill, 8: bench_paths}[args.config](args, bm, ora, threads)
    names = {"q3_k": bm.Q3_K, "q4_k": bm.Q4_K, "q5_k": bm.Q5_K, "q6_k": bm.Q6_K, "iq2_xxs": bm.IQ2_XXS,
             "iq3_xxs": bm.IQ3_XXS, "iq4_xs": bm.IQ4_XS}
    try:
        gate_t, down_t = (names[v] for v in args.types.lower().split(","))
    except (KeyError, ValueError):
        sys.exit(f"bench.py: --types takes two of {sorted(names)} separated by a comma, got {args.types!r}")
    label = {v: k.upper() for k, v in names.items()}
    gate_n, down_n = label[gate_t], label[down_t]
    q8k = (bm.Q3_K, bm.IQ2_XXS, bm.IQ3_XXS, bm.IQ4_XS)
    types3 = (gate_t, gate_t, down_t)
    t0 = time.time()
    wg, wu, wd = make_layer(ora, 0xB1000001, threads, gate_t, down_t)
    x, ids, wts = make_tokens(ora, args.tokens, 0xAC70001)
    log(f"[bench] layer quantized ({(wg.nbytes + wu.nbytes + wd.nbytes) / 1e6:.1f} MB) in {time.time() - t0:.1f}s")

    gpu = bm.Gpu(0)
    layers = []
    for _ in range(args.layers):
        layers.append((gpu.weights(gate_t, N_EXPERTS * FF, HIDDEN, wg), gpu.weights(gate_t, N_EXPERTS * FF, HIDDEN, wu),
                       gpu.weights(down_t, N_EXPERTS * HIDDEN, FF, wd)))
    n_tok = args.tokens
    xd = gpu.upload(x, np.float32)
    sel = gpu.upload(ids, np.uint32)
    wt = gpu.upload(wts, np.float32)
    y = gpu.buffer(np.float32, n_tok * HIDDEN)
    act = gpu.act(gate_t, HIDDEN, 1)
    act_h = gpu.act(down_t, FF, TOP_K)
    fold_h = down_t not in q8k  # gate . up writes the down activation itself when that is a Q8_2_X4 column
    h = None if fold_h else gpu.buffer(np.float32, TOP_K * FF)  # else f32 rows, quantized by the down launch

    kernels = {"two": ("gate_up_x", "down"),
               "chain": ("quant", "gate_up", "down") if fold_h else ("quant", "gate_up", "quant_h", "down")}[args.mode]

    def enqueue_step(i, which=kernels):
        t = i % n_tok
        dg, du, dd = layers[i % len(layers)]
        if "gate_up_x" in which and "down" in which:
            gpu.enqueue_moe_decode(dg, du, dd, xd.ptr + 4 * t * HIDDEN, sel.ptr + 4 * t * TOP_K, wt.ptr + 4 * t * TOP_K,
                                   None, TOP_K, 1, act_h, y.ptr + 4 * t * HIDDEN, h=h)
            return
        if "gate_up_x" in which:
            gpu.enqueue_gate_up_x(dg, du, xd.ptr + 4 * t * HIDDEN, sel.ptr + 4 * t * TOP_K, TOP_K, 1, FF,
                                  act_h if fold_h else None, h=h)
        if "down" in which and not fold_h and args.mode == "two":
            gpu.enqueue_down_combine_h(dd, h, act_h, sel.ptr + 4 * t * TOP_K, wt.ptr + 4 * t * TOP_K, None, TOP_K, 1, HIDDEN,
                                       y.ptr + 4 * t * HIDDEN)
            return
        if "quant" in which:
            gpu.enqueue_quantize(xd.ptr + 4 * t * HIDDEN, 1, act)
        if "gate_up" in which:
            gpu.enqueue_gate_up(dg, du, act, sel.ptr + 4 * t * TOP_K, TOP_K, FF, TOP_K, h, act_h if fold_h else None)
        if "quant_h" in which:
            gpu.enqueue_quantize(h, TOP_K, act_h)
        if "down" in which:
            gpu.enqueue_down_combine(dd, act_h, sel.ptr + 4 * t * TOP_K, wt.ptr + 4 * t * TOP_K, None, TOP_K, 1, HIDDEN,
                                     y.ptr + 4 * t * HIDDEN)

    if args.down_form == "split":
        gpu.set_down_form(bm.DOWN_SPLIT)
    if args.read_patterns:
        assert (gate_t, down_t) == (bm.Q4_K, bm.Q6_K), "--read-patterns reads Q4_K gate/up and Q6_K down rows"
        return read_patterns(bm, gpu, layers, sel, n_tok)
    if args.handoff:
        return handoff(bm, gpu, layers[0][0].dev_ptr, N_EXPERTS * FF * bm.row_bytes(gate_t, HIDDEN))
    if args.timeline:
        return timeline(args, bm, gpu, enqueue_step, (gate_n, down_n))
    if args.traffic_probe:
        n = 1 << 24  # 64 MiB of f32 in, 64 MiB out: combine over one slot of weight 1 is a copy
        src, dst, one = gpu.buffer(np.float32, n).fill_bytes(0), gpu.buffer(np.float32, n), gpu.upload(np.ones(16, np.float32))
        for _ in range(8):
            gpu.enqueue_combine_tokens(src, one, None, n // 16, 1, 16, dst)
        for i in range(256):
            enqueue_step(i)
        gpu.sync()
        log("[bench] traffic probe done: 8 x k_combine copies of 67108864 B each way, 256 steps")
        gpu.close()
        return

    # parity first: the first tokens against the oracle, same seeded inputs
    parity = None
    if not args.no_parity:
        n_chk = min(4, n_tok)
        for i in range(n_chk):
            enqueue_step(i)
        got = y.download()[:n_chk * HIDDEN].reshape(n_chk, HIDDEN)
        want = ora.moe_forward(HIDDEN, FF, N_EXPERTS, types3, wg, wu, wd, x[:n_chk], ids[:n_chk],
                               wts[:n_chk], TOP_K, n_threads=threads).reshape(n_chk, HIDDEN)
        err = float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))
        parity = {"tokens": n_chk, "max_abs_normalised_err": err, "bit_identical": bool(np.array_equal(got, want))}
        log(f"[bench] parity {parity}")
        assert err <= 1e-4, parity

    # The timed region is exactly --steps steps behind exactly --warmup untimed ones: graphs of up to 256 steps (a token's
    # graph in a model of this size holds as many launches) replayed back to back, the remainder as a shorter graph. Everything
    # is enqueued before the first event can fire (two replays of the 256-step graph go first, untimed, so the device is busy
    # meanwhile), so the events bracket device time only; `value` is the event time of the region over its steps. Beside it, whatever --steps says: at least 32 replays of the 256-step graph with an event after
    # each, and their median, minimum and maximum (a replay is under three milliseconds of device time).
    unit = 256
    graphs = {}

    def graph_of(n):
        if n not in graphs:
            gpu.capture_begin()
            for i in range(n):
                enqueue_step(i)
            graphs[n] = gpu.capture_end()
        return graphs[n]

    def run_steps(n):
        for _ in range(n // unit):
            gpu.graph_launch(graph_of(unit))
        if n % unit:
            gpu.graph_launch(graph_of(n % unit))

    steps, warm = max(1, args.steps), max(0, args.warmup)
    for n in {unit, steps % unit, warm % unit} - {0}:
        graph_of(n)
    gpu.sync()
    e0, e1 = gpu.event(), gpu.event()
    t_start = time.perf_counter()
    run_steps(2 * unit)  # a lead-in that keeps the device busy while the host enqueues what follows: the events then see no idle gap
    run_steps(warm)
    gpu.event_record(e0)
    run_steps(steps)
    gpu.event_record(e1)
    gpu.sync()
    wall_ms = (time.perf_counter() - t_start) * 1e3
    ev_ms = gpu.event_elapsed_ms(e0, e1)
    ms_per_step = ev_ms / steps
    us_per_token = ms_per_step * 1e3
    graph = graph_of(unit)
    reps = 1 if args.one_interval else 32
    marks = [gpu.event() for _ in range(reps + 1)]
    gpu.event_record(marks[0])
    for r in range(reps):
        gpu.graph_launch(graph)
        gpu.event_record(marks[r + 1])
    gpu.sync()
    replay_us = sorted(gpu.event_elapsed_ms(marks[r], marks[r + 1]) * 1e3 / unit for r in range(reps))
    for ev in marks:
        gpu.event_destroy(ev)
    replay_stats = {"replays": reps, "steps_per_replay": unit, "median_us_per_token": replay_us[len(replay_us) // 2],
                    "min_us_per_token": replay_us[0], "max_us_per_token": replay_us[-1]}
    bytes_per_token = TOP_K * (2 * FF * bm.row_bytes(gate_t, HIDDEN) + HIDDEN * bm.row_bytes(down_t, FF))

    # per-kernel launch durations: a graph of one kernel only, over the same cycling inputs, between events on
    # the launch stream
    kernel_us = {}
    for name in kernels:
        gpu.capture_begin()
        for i in range(unit):
            enqueue_step(i, (name,))
        g1 = gpu.capture_end()
        gpu.graph_launch(g1)
        gpu.sync()
        gpu.event_record(e0)
        r = max(1, 1024 // unit)
        for _ in range(r):
            gpu.graph_launch(g1)
        gpu.event_record(e1)
        kernel_us[name] = gpu.event_elapsed_ms(e0, e1) * 1e3 / (r * unit)
        gpu.graph_destroy(g1)
    # the step before the layer, timed beside it (not part of `value`): norm + router logits, then softmax top-k
    rng_r = np.random.default_rng(0x707E0001)
    router_d = gpu.upload(rng_r.standard_normal((N_EXPERTS, HIDDEN), dtype=np.float32) * np.float32(0.05), np.float32)
    gain_d = gpu.upload(np.ones(HIDDEN, np.float32), np.float32)
    normed_d, logits_d = gpu.buffer(np.float32, HIDDEN), gpu.buffer(np.float32, N_EXPERTS)
    ids_d, wts_d = gpu.buffer(np.uint32, TOP_K), gpu.buffer(np.float32, TOP_K)
    router_us = {}
    for name in ("router_logits", "route_softmax", "norm_route_one_launch", "norm_route_with_column"):
        gpu.capture_begin()
        for i in range(unit):
            if name == "router_logits":
                gpu.enqueue_router_logits(router_d, xd.ptr + 4 * (i % n_tok) * HIDDEN, gain_d, 1e-6, 1, N_EXPERTS, HIDDEN,
                                          normed_d, logits_d)
            elif name == "route_softmax":
                gpu.enqueue_route_softmax(logits_d, 1, N_EXPERTS, TOP_K, True, None, ids_d, wts_d)
            elif name == "norm_route_one_launch":
                gpu.enqueue_norm_route(router_d, xd.ptr + 4 * (i % n_tok) * HIDDEN, gain_d, 1e-6, 1, N_EXPERTS, HIDDEN, TOP_K,
                                       True, normed_d, logits_d, None, ids_d, wts_d)
            else:  # the launch also leaves the token's quantized column; the normed f32 row is not stored
                gpu.enqueue_norm_route(router_d, xd.ptr + 4 * (i % n_tok) * HIDDEN, gain_d, 1e-6, 1, N_EXPERTS, HIDDEN, TOP_K,
                                       True, None, logits_d, None, ids_d, wts_d, act_x=act)
        g1 = gpu.capture_end()
        gpu.graph_launch(g1)
        gpu.sync()
        gpu.event_record(e0)
        r = max(1, 1024 // unit)
        for _ in range(r):
            gpu.graph_launch(g1)
        gpu.event_record(e1)
        router_us[name] = gpu.event_elapsed_ms(e0, e1) * 1e3 / (r * unit)
        gpu.graph_destroy(g1)
    # The layer from its residual row, router and experts together (three launches either way, the ids and weights the router's
    # own): the router launch leaves the normed f32 row and the fused expert step quantizes it in its first launch, or the
    # router launch leaves the quantized column and gate . up reads it. The residual added back is the input row.
    def from_residual(with_column):
        def enqueue(i):
            t = i % n_tok
            dg, du, dd = layers[i % len(layers)]
            xrow, yrow = xd.ptr + 4 * t * HIDDEN, y.ptr + 4 * t * HIDDEN
            if with_column:
                gpu.enqueue_norm_route(router_d, xrow, gain_d, 1e-6, 1, N_EXPERTS, HIDDEN, TOP_K, True, None, logits_d, None, ids_d,
                                       wts_d, act_x=act)
                gpu.enqueue_gate_up(dg, du, act, ids_d, TOP_K, FF, TOP_K, None, act_h)
                gpu.enqueue_down_combine(dd, act_h, ids_d, wts_d, xrow, TOP_K, 1, HIDDEN, yrow)
            else:
                gpu.enqueue_norm_route(router_d, xrow, gain_d, 1e-6, 1, N_EXPERTS, HIDDEN, TOP_K, True, normed_d, logits_d, None, ids_d,
                                       wts_d)
                gpu.enqueue_moe_decode(dg, du, dd, normed_d, ids_d, wts_d, xrow, TOP_K, 1, act_h, yrow, h=h)
        return enqueue

    residual_us = {"column_made_in_gate_up_x": timed_graph(gpu, from_residual(False), unit, 2048, 512)[1] * 1e3}
    if fold_h:
        residual_us["column_from_norm_route"] = timed_graph(gpu, from_residual(True), unit, 2048, 512)[1] * 1e3
        rows = []
        for way in (False, True):  # the two ways give the same bits
            from_residual(way)(0)
            rows.append(y.download()[:HIDDEN].copy())
        assert np.array_equal(rows[0].view(np.uint32), rows[1].view(np.uint32)), "the layer from its residual row, the two ways"
        residual_us["same_bits_both_ways"] = True
    gate_up_bytes = TOP_K * 2 * FF * bm.row_bytes(gate_t, HIDDEN)
    down_bytes = TOP_K * HIDDEN * bm.row_bytes(down_t, FF)
    # what the launches' times are to be read against, measured here: an empty launch, and launches that only fetch the
    # gate . up launch's bytes (cold: a different part of a different layer copy each time) with plain loads
    sink = gpu.buffer(np.uint32, 4096)
    probe = load_probe()
    stream = gpu.lib.bm_ctx_stream(gpu.ctx)
    stack_bytes = N_EXPERTS * FF * bm.row_bytes(gate_t, HIDDEN)
    spans = max(1, stack_bytes // gate_up_bytes)

    def plain_read(n_wg, nbytes):
        # 64 regions of the gate and up stacks of the four layer copies, one after the other: 900 MB between two reads of
        # the same bytes, so every read comes from HBM (the memory-side cache holds 256 MB)
        def enqueue(i):
            j = i % (len(layers) * 2 * spans)
            base = layers[j % len(layers)][(j // len(layers)) % 2].dev_ptr
            rc = probe.bm_bench_probe_read(stream, base + (j // (2 * len(layers))) * gate_up_bytes, nbytes, n_wg, sink.ptr)
            assert rc == 0, f"bm_bench_probe_read: {rc}"
        return min(timed_graph(gpu, enqueue, 64, 1024, 64)[1] * 1e3 for _ in range(2))

    calibration = {"empty_launch_us": plain_read(192, 0),
                   "plain_read_of_gate_up_bytes_us": {str(n): plain_read(n, gate_up_bytes) for n in (192, 1024, 2048)},
                   "plain_read_of_half_us": {str(n): plain_read(n, gate_up_bytes // 2) for n in (2048,)},
                   "note": "a plain read kernel (bloomery_amd/csrc/bench_probe.hip) under the same graph replay, cold: n workgroups fetch the gate . up launch's "
                           f"{gate_up_bytes} bytes (or half of them) with plain loads and do nothing else: no expert ids to read "
                           "first, no arithmetic, no output"}
    best = min(calibration["plain_read_of_gate_up_bytes_us"].values())
    calibration["plain_read_gbps"] = gate_up_bytes / (best * 1e-6) / 1e9
    half = calibration["plain_read_of_half_us"]["2048"]
    full = calibration["plain_read_of_gate_up_bytes_us"]["2048"]
    if full > half:
        calibration["streaming_gbps_between_half_and_whole"] = (gate_up_bytes - gate_up_bytes // 2) / ((full - half) * 1e-6) / 1e9
    gk = "gate_up_x" if args.mode == "two" else "gate_up"
    dominant, dom_bytes = (f"k_gate_up_x<{gate_n}>" if args.mode == "two" else f"k_gate_up<{gate_n}>"), gate_up_bytes
    achieved = dom_bytes / (kernel_us[gk] * 1e-6) / 1e9
    kernel_gbps = {gk: achieved, "down": down_bytes / (kernel_us["down"] * 1e-6) / 1e9}
    assert gpu.fault() == (bm.FAULT_NONE, 0)

    cpu = None
    if not args.no_cpu:
        pool = ora.lib.ora_pool_create(threads)
        try:
            for i in range(3):
                ora.moe_forward(HIDDEN, FF, N_EXPERTS, types3, wg, wu, wd, x[i % n_tok],
                                ids[i % n_tok], wts[i % n_tok], TOP_K, avx2_pool=pool)
            n, t_cpu = 0, time.perf_counter()
            while True:
                ora.moe_forward(HIDDEN, FF, N_EXPERTS, types3, wg, wu, wd, x[n % n_tok],
                                ids[n % n_tok], wts[n % n_tok], TOP_K, avx2_pool=pool)
                n += 1
                el = time.perf_counter() - t_cpu
                if el >= args.cpu_seconds and n >= 20:
                    break
        finally:
            ora.lib.ora_pool_destroy(pool)
        # the same on one thread, a shorter sample
        pool1 = ora.lib.ora_pool_create(1)
        try:
            ora.moe_forward(HIDDEN, FF, N_EXPERTS, types3, wg, wu, wd, x[0], ids[0], wts[0], TOP_K, avx2_pool=pool1)
            n1, t1 = 0, time.perf_counter()
            while True:
                ora.moe_forward(HIDDEN, FF, N_EXPERTS, types3, wg, wu, wd, x[n1 % n_tok], ids[n1 % n_tok], wts[n1 % n_tok], TOP_K,
                                avx2_pool=pool1)
                n1 += 1
                el1 = time.perf_counter() - t1
                if el1 >= args.cpu_seconds / 3 and n1 >= 10:
                    break
        finally:
            ora.lib.ora_pool_destroy(pool1)
        gbs = bytes_per_token * n / el / 1e9
        single = {"value": el1 / n1 * 1e6, "unit": "us/token", "cores": 1, "gb_per_s": bytes_per_token * n1 / el1 / 1e9,
                  "sample": f"{n1} tokens on one thread, {el1:.1f}s"}
        cpu = {"value": el / n * 1e6, "unit": "us/token", "cores": threads, "kind": "port", "single_thread": single,
               "sample": f"{n} tokens of the same layer and routings, AVX2 restatement of qdot on {threads} threads (the "
                         f"box's worker-pool size), {el:.1f}s; {gbs:.1f} GB/s of expert rows = {gbs / threads:.2f} GB/s a thread "
                         "(the reference documents about 12 GB/s a core and 130 GB/s on 32 cores for its own build, "
                         "docs/roofline.md:136-139, docs/performance.md:81-86)",
               "gb_per_s": gbs, "gb_per_s_per_thread": gbs / threads}

    out = {
        "metric": "moe_layer_decode_us_per_token",
        "value": us_per_token,
        "unit": "us/token",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warm,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "Qwen3-30B-A3B-shaped MoE layer decode, 1 token: hidden 2048, 128 experts x ff 768, "
                               f"{gate_n} gate/up + {down_n} down, softmax top-8 renormalised "
                               + ("(BASELINE.json configs[1])" if (gate_t, down_t) == (bm.Q4_K, bm.Q6_K)
                                  else "(BASELINE.json configs[1]'s shape with other weight types: a side measurement)"),
                   "layer_copies": len(layers), "distinct_tokens": n_tok, "launches_per_step": len(kernels), "mode": "hipGraph replay",
                   "down_form": args.down_form},
        "hbm_tbps": bytes_per_token / (us_per_token * 1e-6) / 1e12,
        "algorithmic_bytes_per_token": bytes_per_token,
        "wall_ms_lead_in_warmup_and_steps": wall_ms,
        "replay_us_per_token": replay_stats,
        "kernel_us": kernel_us,
        "kernel_gbps": kernel_gbps,
        "router_kernel_us": router_us,
        "layer_from_residual_row_us": residual_us,
        "calibration": calibration,
        "parity": parity,
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": GATE_UP_X_TRAFFIC_BYTES if args.mode == "two" and gate_t == bm.Q4_K else None,
                     "traffic_source": ("profiles/decode_qwen3_layer_hbm_traffic.md: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this "
                                        "kernel, collected offline, not in this run") if args.mode == "two" and gate_t == bm.Q4_K else None,
                     "algorithmic_bytes_per_launch": dom_bytes},
        "cpu_baseline": cpu,
    }
    if not args.no_prefill and (gate_t, down_t) == (bm.Q4_K, bm.Q6_K) and args.mode == "two":
        # the second leg of the metric, in the same line: config 4's step on the first layer copy
        out["prefill"], _ = prefill_leg(args, bm, ora, threads, gpu, (wg, wu, wd), layers[0], args.prefill_tokens)
        assert gpu.fault() == (bm.FAULT_NONE, 0)
    print(json.dumps(out), flush=True)
    gpu.close()


if __name__ == "__main__":
    main()
