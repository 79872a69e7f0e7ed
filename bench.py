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


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_layer(ora, seed, threads):
    """The layer's expert stacks: fp32 N(0, 0.02) quantized by the repo's K-quant rules (Q4_K, Q6_K `_ref`)."""
    rng = np.random.default_rng(seed)
    out = []
    for wtype, rows, k in ((ora.Q4_K, N_EXPERTS * FF, HIDDEN), (ora.Q4_K, N_EXPERTS * FF, HIDDEN),
                           (ora.Q6_K, N_EXPERTS * HIDDEN, FF)):
        rb = ora.row_bytes(wtype, k)
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2048)
    ap.add_argument("--warmup", type=int, default=256)
    ap.add_argument("--layers", type=int, default=4, help="distinct device copies of the layer cycled through")
    ap.add_argument("--tokens", type=int, default=64, help="distinct tokens (and routings) cycled through")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--mode", choices=("two", "single", "chain"), default="two",
                    help="two: bm_moe_decode in two launches (quantizers folded in); single: bm_moe_decode in one "
                         "launch; chain: quantize, gate_up, down_combine")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus above 1 is not supported (nothing here shards)")

    import bloomery_amd as bm
    import ora

    threads = min(os.cpu_count() or 1, 16)
    t0 = time.time()
    wg, wu, wd = make_layer(ora, 0xB1000001, threads)
    x, ids, wts = make_tokens(ora, args.tokens, 0xAC70001)
    log(f"[bench] layer quantized ({(wg.nbytes + wu.nbytes + wd.nbytes) / 1e6:.1f} MB) in {time.time() - t0:.1f}s")

    gpu = bm.Gpu(0)
    layers = []
    for _ in range(args.layers):
        layers.append((gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, wg), gpu.weights(bm.Q4_K, N_EXPERTS * FF, HIDDEN, wu),
                       gpu.weights(bm.Q6_K, N_EXPERTS * HIDDEN, FF, wd)))
    n_tok = args.tokens
    xd = gpu.upload(x, np.float32)
    sel = gpu.upload(ids, np.uint32)
    wt = gpu.upload(wts, np.float32)
    y = gpu.buffer(np.float32, n_tok * HIDDEN)
    act = gpu.act(bm.Q4_K, HIDDEN, 1)
    act_h = gpu.act(bm.Q6_K, FF, TOP_K)

    single = args.mode == "single"
    kernels = {"single": ("step",), "two": ("gate_up_x", "down"), "chain": ("quant", "gate_up", "down")}[args.mode]
    gpu.set_decode_plan(bm.PLAN_ONE_LAUNCH if single else bm.PLAN_TWO_LAUNCHES)

    def enqueue_step(i, which=kernels):
        t = i % n_tok
        dg, du, dd = layers[i % len(layers)]
        if "gate_up_x" in which and "down" in which:
            gpu.enqueue_moe_decode(dg, du, dd, xd.ptr + 4 * t * HIDDEN, sel.ptr + 4 * t * TOP_K, wt.ptr + 4 * t * TOP_K,
                                   None, TOP_K, 1, act_h, y.ptr + 4 * t * HIDDEN)
            return
        if "gate_up_x" in which:
            gpu.enqueue_gate_up_x(dg, du, xd.ptr + 4 * t * HIDDEN, sel.ptr + 4 * t * TOP_K, TOP_K, 1, FF, act_h)
        if "step" in which:
            gpu.enqueue_moe_decode(dg, du, dd, xd.ptr + 4 * t * HIDDEN, sel.ptr + 4 * t * TOP_K, wt.ptr + 4 * t * TOP_K,
                                   None, TOP_K, 1, act_h, y.ptr + 4 * t * HIDDEN)
        if "quant" in which:
            gpu.enqueue_quantize(xd.ptr + 4 * t * HIDDEN, 1, act)
        if "gate_up" in which:
            gpu.enqueue_gate_up(dg, du, act, sel.ptr + 4 * t * TOP_K, TOP_K, FF, TOP_K, None, act_h)
        if "down" in which:
            gpu.enqueue_down_combine(dd, act_h, sel.ptr + 4 * t * TOP_K, wt.ptr + 4 * t * TOP_K, None, TOP_K, 1, HIDDEN,
                                     y.ptr + 4 * t * HIDDEN)

    # parity first: the first tokens against the oracle, same seeded inputs
    parity = None
    if not args.no_parity:
        n_chk = min(4, n_tok)
        for i in range(n_chk):
            enqueue_step(i)
        got = y.download()[:n_chk * HIDDEN].reshape(n_chk, HIDDEN)
        want = ora.moe_forward(HIDDEN, FF, N_EXPERTS, (ora.Q4_K, ora.Q4_K, ora.Q6_K), wg, wu, wd, x[:n_chk], ids[:n_chk],
                               wts[:n_chk], TOP_K, n_threads=threads).reshape(n_chk, HIDDEN)
        err = float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))
        parity = {"tokens": n_chk, "max_abs_normalised_err": err, "bit_identical": bool(np.array_equal(got, want))}
        log(f"[bench] parity {parity}")
        assert err <= 1e-4, parity

    # one graph of `unit` steps; the timed region replays it
    unit = max(len(layers) * n_tok // np.gcd(len(layers), n_tok), 1)
    unit = min(max(int(unit), 64), 256)  # a graph of at least 64 steps: the replay call itself costs microseconds
    gpu.capture_begin()
    for i in range(unit):
        enqueue_step(i)
    graph = gpu.capture_end()
    reps_w = max(1, -(-args.warmup // unit))
    reps = max(1, -(-args.steps // unit))
    steps = reps * unit
    for _ in range(reps_w):
        gpu.graph_launch(graph)
    gpu.sync()
    e0, e1 = gpu.event(), gpu.event()
    t_start = time.perf_counter()
    gpu.event_record(e0)
    for _ in range(reps):
        gpu.graph_launch(graph)
    gpu.event_record(e1)
    gpu.sync()
    wall_ms = (time.perf_counter() - t_start) * 1e3
    ev_ms = gpu.event_elapsed_ms(e0, e1)
    ms_per_step = wall_ms / steps
    us_per_token = ms_per_step * 1e3
    bytes_per_token = TOP_K * (2 * FF * bm.row_bytes(bm.Q4_K, HIDDEN) + HIDDEN * bm.row_bytes(bm.Q6_K, FF))

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
    gate_up_bytes = TOP_K * 2 * FF * bm.row_bytes(bm.Q4_K, HIDDEN)
    down_bytes = TOP_K * HIDDEN * bm.row_bytes(bm.Q6_K, FF)
    if single:
        dominant, dom_bytes = "k_moe_decode<Q4_K, Q6_K>", bytes_per_token
        achieved = dom_bytes / (kernel_us["step"] * 1e-6) / 1e9
        kernel_gbps = {"step": achieved}
    else:
        gk = "gate_up_x" if args.mode == "two" else "gate_up"
        dominant, dom_bytes = ("k_gate_up_x<Q4_K>" if args.mode == "two" else "k_gate_up<Q4_K>"), gate_up_bytes
        achieved = dom_bytes / (kernel_us[gk] * 1e-6) / 1e9
        kernel_gbps = {gk: achieved, "down": down_bytes / (kernel_us["down"] * 1e-6) / 1e9}
    assert gpu.fault() == (bm.FAULT_NONE, 0)

    cpu = None
    if not args.no_cpu:
        pool = ora.lib.ora_pool_create(threads)
        try:
            for i in range(3):
                ora.moe_forward(HIDDEN, FF, N_EXPERTS, (ora.Q4_K, ora.Q4_K, ora.Q6_K), wg, wu, wd, x[i % n_tok],
                                ids[i % n_tok], wts[i % n_tok], TOP_K, avx2_pool=pool)
            n, t_cpu = 0, time.perf_counter()
            while True:
                ora.moe_forward(HIDDEN, FF, N_EXPERTS, (ora.Q4_K, ora.Q4_K, ora.Q6_K), wg, wu, wd, x[n % n_tok],
                                ids[n % n_tok], wts[n % n_tok], TOP_K, avx2_pool=pool)
                n += 1
                el = time.perf_counter() - t_cpu
                if el >= args.cpu_seconds and n >= 20:
                    break
        finally:
            ora.lib.ora_pool_destroy(pool)
        cpu = {"value": el / n * 1e6, "unit": "us/token", "cores": threads, "kind": "port",
               "sample": f"{n} tokens of the same layer and routings, AVX2 restatement of qdot on {threads} threads, "
                         f"{el:.1f}s; {bytes_per_token * n / el / 1e9:.1f} GB/s of expert rows"}

    out = {
        "metric": "moe_layer_decode_us_per_token",
        "value": us_per_token,
        "unit": "us/token",
        "n_gpus": 1,
        "steps": steps,
        "warmup": reps_w * unit,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "Qwen3-30B-A3B-shaped MoE layer decode, 1 token: hidden 2048, 128 experts x ff 768, "
                               "Q4_K gate/up + Q6_K down, softmax top-8 renormalised (BASELINE.json configs[1])",
                   "layer_copies": len(layers), "distinct_tokens": n_tok, "launches_per_step": len(kernels), "mode": "hipGraph replay"},
        "hbm_tbps": bytes_per_token / (us_per_token * 1e-6) / 1e12,
        "algorithmic_bytes_per_token": bytes_per_token,
        "event_ms_per_step": ev_ms / steps,
        "kernel_us": kernel_us,
        "kernel_gbps": kernel_gbps,
        "parity": parity,
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_launch": dom_bytes},
        "cpu_baseline": cpu,
    }
    print(json.dumps(out), flush=True)
    gpu.close()


if __name__ == "__main__":
    main()
