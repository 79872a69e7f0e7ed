"""GPU parity tests at the shapes the benchmark's configurations name, through the C ABI, against the CPU oracle on the
same seeded inputs: the DeepSeek-V3-shaped layer (IQ2_XXS routed experts over a resident subset, and over all 256, one Q6_K
shared expert, the shared-expert combine) on the grouped and on the per-slot path, and the prefill GEMMs at the Qwen3-shaped layer's
two matrix shapes under a skewed routing (an expert with three tiles, an expert with none). Also: a slot the host
serves through every gate . up entry, and stacks wrapped in place. Contracts: crates/gpu/src/iq_sel.rs:1357,1557,
crates/gpu/src/gemm/route.rs:351, crates/gpu/src/kquant/sel.rs:22-28, crates/gpu/src/moe_fused.rs:129-170."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora
from common import normal_f32
from test_gpu_decode import (Layer, assert_f32, gpu, grouped_tables_on_device, random_blocks, route,  # noqa: F401
                             run_fused_step)
from test_gpu_prefill import run_prefill

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------------- the DeepSeek-V3-shaped layer, 4 tokens

DS_HIDDEN, DS_FF, DS_TOPK, DS_TOKENS, DS_RESIDENT = 7168, 2048, 8, 4, 12


@pytest.fixture(scope="module")
def ds_layer(gpu):
    routed = Layer(gpu, (bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), DS_HIDDEN, DS_FF, DS_RESIDENT, 3100, cheap=True)
    shared = Layer(gpu, (bm.Q6_K, bm.Q6_K, bm.Q6_K), DS_HIDDEN, DS_FF, 1, 3200, cheap=True)
    rng = np.random.default_rng(3101)
    x = normal_f32(rng, (DS_TOKENS, DS_HIDDEN))
    ids, wts = route(rng, DS_TOKENS, DS_RESIDENT, DS_TOPK)
    zeros, ones = np.zeros((DS_TOKENS, 1), np.uint32), np.ones((DS_TOKENS, 1), np.float32)
    want_routed, want_h = routed.oracle(x, ids, wts, DS_TOPK)
    want_shared, _ = shared.oracle(x, zeros, ones, 1)
    # (routed sum + shared expert), the reference's grouping of the two adds
    want = (np.asarray(want_routed, np.float32) + np.asarray(want_shared, np.float32)).astype(np.float32)
    yield routed, shared, x, ids, wts, want, want_h, np.asarray(want_shared, np.float32)
    routed.free()
    shared.free()


def shared_expert_rows(gpu, shared, xd, m):
    """The shared expert as the one-expert case of the routed entries (crates/gpu/src/kquant/sel.rs:15-20): every id 0,
    a slot a token. Returns the buffer of its down rows."""
    zeros = gpu.upload(np.zeros(m, np.uint32))
    act6, act_sh = gpu.act(bm.Q6_K, DS_HIDDEN, m), gpu.act(bm.Q6_K, DS_FF, m)
    sdown = gpu.buffer(np.float32, m * DS_HIDDEN).fill_bytes(0xFF)
    gpu.enqueue_quantize(xd, m, act6)
    gpu.enqueue_gate_up(shared.dg, shared.du, act6, zeros, m, DS_FF, 1, None, act_sh)
    gpu.enqueue_gemv_sel(shared.dd, act_sh, zeros, m, DS_HIDDEN, sdown)
    return sdown, (zeros, act6, act_sh)


def test_deepseek_shaped_layer_grouped(gpu, ds_layer):
    routed, shared, x, ids, wts, want, want_h, want_shared = ds_layer
    m, n_slots = DS_TOKENS, DS_TOKENS * DS_TOPK
    gpu.fault_clear()
    sel, order, start, tiles = grouped_tables_on_device(gpu, ids.reshape(-1), DS_RESIDENT)
    xd, wd = gpu.upload(x, np.float32), gpu.upload(wts, np.float32)
    act, act_h = gpu.act(bm.IQ2_XXS, DS_HIDDEN, m), gpu.act(bm.IQ2_XXS, DS_FF, n_slots)
    h = gpu.buffer(np.float32, n_slots * DS_FF).fill_bytes(0xFF)
    down = gpu.buffer(np.float32, n_slots * DS_HIDDEN).fill_bytes(0xFF)
    y = gpu.buffer(np.float32, m * DS_HIDDEN).fill_bytes(0xFF)
    gpu.enqueue_quantize(xd, m, act)
    gpu.enqueue_gate_up_tiles(routed.dg, routed.du, act, order, start, tiles, n_slots, DS_FF, DS_TOPK, h)
    gpu.enqueue_quantize_ord(h, start, DS_RESIDENT, n_slots, act_h)
    gpu.enqueue_gemv_tiles(routed.dd, act_h, order, start, tiles, n_slots, DS_HIDDEN, down)
    sdown, keep = shared_expert_rows(gpu, shared, xd, m)
    gpu.enqueue_moe_combine(down, wd, sdown, None, DS_HIDDEN, DS_TOPK, m, y)
    got_h = h.download().reshape(n_slots, DS_FF)
    assert_f32(got_h, want_h.reshape(n_slots, DS_FF)[order.download()], "h by table entry")
    assert_f32(sdown.download(), want_shared, "shared expert rows")
    assert_f32(y.download(), want, "y = (routed + shared)")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (sel, order, start, tiles, xd, wd, act, act_h, h, down, y, sdown) + keep:
        b.free()


def test_deepseek_shaped_layer_with_all_256_experts_resident(gpu):
    """BASELINE configs[4] with its whole routed stack on the card: 256 IQ2_XXS experts of hidden 7168 / ff 2048 (2.9 GB of
    random legal blocks), 4 tokens, top-8 drawn over all 256. The grouped step and the per-slot step are separate kernels and
    must agree bit for bit on every slot's h and every token's y, and both are the oracle's (which only visits the 32 slots'
    experts, so the full comparison is affordable)."""
    n_experts, m, top_k = 256, DS_TOKENS, DS_TOPK
    n_slots = m * top_k
    routed = Layer(gpu, (bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), DS_HIDDEN, DS_FF, n_experts, 3300, cheap=True)
    try:
        rng = np.random.default_rng(3301)
        x = normal_f32(rng, (m, DS_HIDDEN))
        ids, wts = route(rng, m, n_experts, top_k)
        ids[1, 3] = 255  # the stack's last expert takes part
        ids[2, 0] = ids[0, 0]  # and one expert has two slots: a tile of two
        assert len(np.unique(ids[1])) == top_k and len(np.unique(ids[2])) == top_k
        want_y, want_h = routed.oracle(x, ids, wts, top_k)
        gpu.fault_clear()
        xd, sel_d, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
        # the per-slot step
        act_h = gpu.act(bm.IQ2_XXS, DS_FF, n_slots)
        h = gpu.buffer(np.float32, n_slots * DS_FF).fill_bytes(0xFF)
        y = gpu.buffer(np.float32, m * DS_HIDDEN).fill_bytes(0xFF)
        gpu.enqueue_moe_decode(routed.dg, routed.du, routed.dd, xd, sel_d, wd, None, top_k, m, act_h, y, h=h)
        h_slot, y_slot = h.download(), y.download()
        # the grouped step
        sel, order, start, tiles = grouped_tables_on_device(gpu, ids.reshape(-1), n_experts)
        act = gpu.act(bm.IQ2_XXS, DS_HIDDEN, m)
        act_g = gpu.act(bm.IQ2_XXS, DS_FF, n_slots)
        hg = gpu.buffer(np.float32, n_slots * DS_FF).fill_bytes(0xFF)
        down = gpu.buffer(np.float32, n_slots * DS_HIDDEN).fill_bytes(0xFF)
        yg = gpu.buffer(np.float32, m * DS_HIDDEN).fill_bytes(0xFF)
        gpu.enqueue_quantize(xd, m, act)
        gpu.enqueue_gate_up_tiles(routed.dg, routed.du, act, order, start, tiles, n_slots, DS_FF, top_k, hg)
        gpu.enqueue_quantize_ord(hg, start, n_experts, n_slots, act_g)
        gpu.enqueue_gemv_tiles(routed.dd, act_g, order, start, tiles, n_slots, DS_HIDDEN, down)
        gpu.enqueue_combine_tokens(down, wd, None, DS_HIDDEN, top_k, m, yg)
        h_grouped = hg.download().reshape(n_slots, DS_FF)
        assert np.array_equal(h_grouped.view(np.uint32), h_slot.reshape(n_slots, DS_FF)[order.download()].view(np.uint32)), "h: grouped against per slot"
        assert np.array_equal(yg.download().view(np.uint32), y_slot.view(np.uint32)), "y: grouped against per slot"
        assert_f32(h_slot, want_h, "h against the oracle")
        assert_f32(y_slot, want_y, "y against the oracle")
        assert gpu.fault() == (bm.FAULT_NONE, 0)
        for b in (xd, sel_d, wd, act_h, h, y, sel, order, start, tiles, act, act_g, hg, down, yg):
            b.free()
    finally:
        routed.free()


def test_long_rows_few_slots_an_expert_one_tile_launch(gpu, ds_layer):
    """With rows this long a tile launch has LDS for two columns, and with no more than two slots an expert of the stack
    on average the one launch takes every tile, a wider one in passes of two columns: three tokens that all name expert
    5 make a tile of three (two passes, the second of one column); every slot's h and down rows against the oracle."""
    routed = ds_layer[0]
    rng = np.random.default_rng(3150)
    m, top_k = 3, DS_TOPK
    n_slots = m * top_k  # 24 = 2 x the 12 experts of the stack
    x = normal_f32(rng, (m, DS_HIDDEN))
    ids = np.stack([np.concatenate([[5], rng.permutation([e for e in range(DS_RESIDENT) if e != 5])[:top_k - 1]]) for _ in range(m)])
    ids = np.stack([rng.permutation(row) for row in ids]).astype(np.uint32)
    wts = rng.uniform(0.05, 0.3, (m, top_k)).astype(np.float32)
    want_y, want_h = routed.oracle(x, ids, wts, top_k)
    gpu.fault_clear()
    sel, order, start, tiles = grouped_tables_on_device(gpu, ids.reshape(-1), DS_RESIDENT)
    counts = np.diff(start.download())
    assert counts[5] == 3 and n_slots <= 2 * DS_RESIDENT
    xd, wd = gpu.upload(x, np.float32), gpu.upload(wts, np.float32)
    act, act_h = gpu.act(bm.IQ2_XXS, DS_HIDDEN, m), gpu.act(bm.IQ2_XXS, DS_FF, n_slots)
    h = gpu.buffer(np.float32, n_slots * DS_FF).fill_bytes(0xFF)
    down = gpu.buffer(np.float32, n_slots * DS_HIDDEN).fill_bytes(0xFF)
    y = gpu.buffer(np.float32, m * DS_HIDDEN).fill_bytes(0xFF)
    gpu.enqueue_quantize(xd, m, act)
    gpu.enqueue_gate_up_tiles(routed.dg, routed.du, act, order, start, tiles, n_slots, DS_FF, top_k, h)
    gpu.enqueue_quantize_ord(h, start, DS_RESIDENT, n_slots, act_h)
    gpu.enqueue_gemv_tiles(routed.dd, act_h, order, start, tiles, n_slots, DS_HIDDEN, down)
    gpu.enqueue_combine_tokens(down, wd, None, DS_HIDDEN, top_k, m, y)
    assert_f32(h.download().reshape(n_slots, DS_FF), want_h.reshape(n_slots, DS_FF)[order.download()], "h by table entry")
    assert_f32(y.download(), want_y, "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (sel, order, start, tiles, xd, wd, act, act_h, h, down, y):
        b.free()


def test_deepseek_shaped_layer_slot_by_slot(gpu, ds_layer):
    """The same tokens through bm_moe_decode (its residual argument carrying the shared expert's rows, the same
    grouping of the adds) and through the plain chain bm_gate_up, bm_quantize, bm_gemv_sel, bm_moe_combine."""
    routed, shared, x, ids, wts, want, want_h, want_shared = ds_layer
    m, n_slots = DS_TOKENS, DS_TOKENS * DS_TOPK
    gpu.fault_clear()
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    sdown, keep = shared_expert_rows(gpu, shared, xd, m)
    act_h = gpu.act(bm.IQ2_XXS, DS_FF, n_slots)
    h = gpu.buffer(np.float32, n_slots * DS_FF).fill_bytes(0xFF)
    y = gpu.buffer(np.float32, m * DS_HIDDEN).fill_bytes(0xFF)
    gpu.enqueue_moe_decode(routed.dg, routed.du, routed.dd, xd, sel, wd, sdown, DS_TOPK, m, act_h, y, h=h)
    assert_f32(h.download(), want_h, "h")
    for s in (0, n_slots // 2, n_slots - 1):
        assert np.array_equal(act_h.download(s), ora.quantize_col(bm.IQ2_XXS, want_h[s * DS_FF:(s + 1) * DS_FF])), f"act_h {s}"
    assert_f32(y.download(), want, "y of the fused step")
    # the chain
    act = gpu.act(bm.IQ2_XXS, DS_HIDDEN, m)
    down = gpu.buffer(np.float32, n_slots * DS_HIDDEN).fill_bytes(0xFF)
    y2 = gpu.buffer(np.float32, m * DS_HIDDEN).fill_bytes(0xFF)
    h.fill_bytes(0xFF)
    gpu.enqueue_quantize(xd, m, act)
    gpu.enqueue_gate_up(routed.dg, routed.du, act, sel, n_slots, DS_FF, DS_TOPK, h)
    gpu.enqueue_quantize(h, n_slots, act_h)
    gpu.enqueue_gemv_sel(routed.dd, act_h, sel, n_slots, DS_HIDDEN, down)
    gpu.enqueue_moe_combine(down, wd, sdown, None, DS_HIDDEN, DS_TOPK, m, y2)
    assert_f32(y2.download(), want, "y of the chain")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (xd, sel, wd, sdown, act_h, h, y, act, down, y2) + keep:
        b.free()


# ------------------------------------------------------------ prefill at the layer's shapes under a skewed routing

def skewed_route(rng, m, n_experts, top_k):
    """Popularity falling with the expert's rank over a random permutation; the first expert of the permutation is in
    every token's choice (a run of m slots) and the last in none."""
    perm = rng.permutation(n_experts)
    bias = np.empty(n_experts, np.float32)
    bias[perm] = (-1.1 * np.log(np.arange(1, n_experts + 1))).astype(np.float32)
    bias[perm[0]], bias[perm[-1]] = 12.0, -60.0
    ids, wts = route(rng, m, n_experts, top_k, bias)
    return ids, wts, int(perm[0]), int(perm[-1])


def test_prefill_layer_shape_under_skewed_routing(gpu):
    """Config 4's layer (K 2048 with 768 rows, K 768 with 2048 rows): 160 tokens, top-4 of 16 resident experts. One
    expert owns 160 slots (tiles of 64, 64 and 32: both 32-slot parts of a tile and a ragged third), one owns none,
    the others' runs fall off with their rank."""
    hidden, ff, n_experts, m, top_k = 2048, 768, 16, 160, 4
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), hidden, ff, n_experts, 3300, cheap=True)
    rng = np.random.default_rng(3301)
    x = normal_f32(rng, (m, hidden))
    ids, wts, top, none = skewed_route(rng, m, n_experts, top_k)
    runs = np.bincount(ids.reshape(-1), minlength=n_experts)
    assert runs[top] == m > 128 and runs[none] == 0, runs
    gpu.fault_clear()
    y, g, u, act_h, down = run_prefill(gpu, L, x, ids, wts, top_k)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    n_slots = m * top_k
    flat = ids.reshape(-1)
    rb_g, rb_d = ora.row_bytes(bm.Q4_K, hidden), ora.row_bytes(bm.Q6_K, ff)
    # slots of the long run from each of its tiles, and of short runs: gate, up and down rows against the row dots
    long_run = np.flatnonzero(flat == top)
    picks = [int(long_run[i]) for i in (0, 63, 64, 100, 128, 159)] + [0, n_slots - 1]
    for s in picks:
        e, col = int(flat[s]), ora.quantize_col(bm.Q4_K, x[s // top_k])
        assert_f32(g[s * ff:(s + 1) * ff], ora.gemv(bm.Q4_K, L.wg[e * ff * rb_g:(e + 1) * ff * rb_g], ff, hidden, col, 1), f"gate slot {s}")
        assert_f32(u[s * ff:(s + 1) * ff], ora.gemv(bm.Q4_K, L.wu[e * ff * rb_g:(e + 1) * ff * rb_g], ff, hidden, col, 1), f"up slot {s}")
        hcol = ora.quantize_col(bm.Q6_K, want_h[s * ff:(s + 1) * ff])
        assert np.array_equal(act_h[s], hcol), f"act_h slot {s}"
        assert_f32(down[s * hidden:(s + 1) * hidden],
                   ora.gemv(bm.Q6_K, L.wd[e * hidden * rb_d:(e + 1) * hidden * rb_d], hidden, ff, hcol, 1), f"down slot {s}")
    assert_f32(y, want_y, "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    L.free()


def test_prefill_at_the_benchmarks_full_size_equals_the_slot_path(gpu):
    """The prefill configuration at its full size: 2048 tokens, top-8 of 128 resident experts under a Zipf routing, Q4_K
    gate / up (768 rows, K 2048), Q6_K down (2048 rows, K 768). The oracle would take minutes over 16384 slots, so the
    size-independent property stands in: the grouped GEMM step and the per-slot step are separate kernels over the same
    arithmetic and must agree bit for bit on every slot's down row and on every token's y; sampled slots' h columns are
    compared as bytes and their gate rows against the oracle's row dots. The tolerance mode's gate rows are held to the
    exact mode's, every slot."""
    hidden, ff, n_experts, m, top_k = 2048, 768, 128, 2048, 8
    n_slots = m * top_k
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), hidden, ff, n_experts, 3500, cheap=True)
    rng = np.random.default_rng(3501)
    x = normal_f32(rng, (m, hidden))
    bias = np.empty(n_experts, np.float32)
    bias[rng.permutation(n_experts)] = (-1.1 * np.log(np.arange(1, n_experts + 1))).astype(np.float32)
    ids, wts = route(rng, m, n_experts, top_k, bias)
    runs = np.bincount(ids.reshape(-1), minlength=n_experts)
    assert runs.max() > 1024 and runs.min() < 32, (runs.max(), runs.min())  # many tiles an expert, and less than a tile
    gpu.fault_clear()
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    act = gpu.act(bm.Q4_K, hidden, m)
    gpu.enqueue_quantize(xd, m, act)
    table = gpu.route(n_slots, n_experts)
    table.fill(sel, n_slots)
    g = gpu.buffer(np.float32, n_slots * ff).fill_bytes(0xFF)
    u = gpu.buffer(np.float32, n_slots * ff).fill_bytes(0xFF)
    sample = list(range(0, n_slots, 1021)) + [n_slots - 1]

    def gemm_step(fast):
        act_h = gpu.act(bm.Q6_K, ff, n_slots)
        down = gpu.buffer(np.float32, n_slots * hidden).fill_bytes(0xFF)
        y = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
        gpu.set_gemm_mode(bm.GEMM_FAST if fast else bm.GEMM_EXACT)
        try:
            gpu.enqueue_gemm(L.dg, ff, act, table, top_k, g)
            gpu.enqueue_gemm(L.du, ff, act, table, top_k, u)
            gpu.enqueue_swiglu_quant(g, u, n_slots, act_h)
            gpu.enqueue_gemm(L.dd, hidden, act_h, table, 0, down)
            gpu.enqueue_combine_tokens(down, wd, None, hidden, top_k, m, y)
            out = y.download(), down.download(), [act_h.download(s) for s in sample], g.download()
        finally:
            gpu.set_gemm_mode(bm.GEMM_EXACT)
        for b in (act_h, down, y):
            b.free()
        return out

    y_gemm, down_gemm, cols_gemm, g_gemm = gemm_step(False)
    # the per-slot step: gate . up with its folded quantizer, the slot gemv, the slot sum
    act_h = gpu.act(bm.Q6_K, ff, n_slots)
    down = gpu.buffer(np.float32, n_slots * hidden).fill_bytes(0xFF)
    y = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    gpu.enqueue_gate_up(L.dg, L.du, act, sel, n_slots, ff, top_k, None, act_h)
    gpu.enqueue_gemv_sel(L.dd, act_h, sel, n_slots, hidden, down)
    gpu.enqueue_combine_tokens(down, wd, None, hidden, top_k, m, y)
    y_slot, down_slot = y.download(), down.download()
    cols_slot = [act_h.download(s) for s in sample]
    assert np.array_equal(down_gemm.view(np.uint32), down_slot.view(np.uint32)), "down rows: GEMM against slot gemv"
    assert np.array_equal(y_gemm.view(np.uint32), y_slot.view(np.uint32)), "y: GEMM step against per-slot step"
    for s, a, b in zip(sample, cols_gemm, cols_slot):
        assert np.array_equal(a, b), f"h column of slot {s}"
    assert np.isfinite(y_gemm).all() and gpu.fault() == (bm.FAULT_NONE, 0)
    rb = ora.row_bytes(bm.Q4_K, hidden)
    flat = ids.reshape(-1)
    for s in sample[::4]:
        e, col = int(flat[s]), ora.quantize_col(bm.Q4_K, x[s // top_k])
        assert_f32(g_gemm[s * ff:(s + 1) * ff], ora.gemv(bm.Q4_K, L.wg[e * ff * rb:(e + 1) * ff * rb], ff, hidden, col, 1), f"gate slot {s}")
    # the tolerance mode, GEMM by GEMM on the same columns (through the layer a last-bit difference can flip a code of h)
    g_fast = gemm_step(True)[3].reshape(n_slots, ff)
    g_exact = g_gemm.reshape(n_slots, ff)
    worst = float((np.abs(g_fast - g_exact).max(axis=1) / np.abs(g_exact).max(axis=1)).max())
    assert worst <= 1e-5, f"tolerance mode, gate rows: {worst}"
    for b in (xd, sel, wd, act, table, g, u, act_h, down, y):
        b.free()
    L.free()


@pytest.mark.parametrize("m", (1, 16))
def test_decode_layer_with_all_128_experts_resident(gpu, m):
    """The headline configuration's layer with every one of its 128 experts resident (random legal blocks: the size is
    what is under test), one token and the sixteen of the grouped configuration: the fused per-slot step against the
    oracle, bit for bit, h columns included."""
    hidden, ff, n_experts, top_k = 2048, 768, 128, 8
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), hidden, ff, n_experts, 3600, cheap=True)
    rng = np.random.default_rng(3601 + m)
    x = normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, n_experts, top_k)
    resid = normal_f32(rng, (m, hidden))
    gpu.fault_clear()
    y, h, cols_h, cols_x = run_fused_step(gpu, L, x, ids, wts, top_k, resid=resid)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    assert_f32(h, want_h, "h")
    for s in range(m * top_k):
        assert np.array_equal(cols_h[s], ora.quantize_col(bm.Q6_K, want_h[s * ff:(s + 1) * ff])), f"act_h slot {s}"
    want = (np.asarray(want_y, np.float32).reshape(m, hidden) + resid).astype(np.float32)
    assert_f32(y, want.reshape(-1), "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    L.free()


# ------------------------------------------------------------------------ a host-served slot through gate . up

def test_gate_up_entries_skip_a_host_slot(gpu):
    """BM_HOST_SLOT through bm_gate_up, bm_gate_up_x and bm_moe_decode: no fault, the slot's rows of h and its
    activation column keep what they held, and y is the oracle's sum over the live slots."""
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 512, 256, 4, 3400)
    rng = np.random.default_rng(3401)
    m, top_k = 2, 3
    x = normal_f32(rng, (m, 512))
    ids = np.array([[1, bm.HOST_SLOT, 3], [2, 0, 1]], np.uint32)
    wts = np.array([[0.5, 0.3, 0.2], [0.2, 0.5, 0.3]], np.float32)
    live_ids, live_w = np.array([[1, 3]], np.uint32), np.array([[0.5, 0.2]], np.float32)
    want0, _ = L.oracle(x[:1], live_ids, live_w, 2)
    want1, want_h1 = L.oracle(x[1:], ids[1:], wts[1:], 3)
    gpu.fault_clear()
    # the fused step
    y, h, act_h, _ = run_fused_step(gpu, L, x, ids, wts, top_k)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    h = h.reshape(m * top_k, 256)
    assert np.all(h[1].view(np.uint32) == 0xFFFFFFFF), "the host's slot keeps its rows of h"
    assert_f32(h[3:].reshape(-1), want_h1, "h of the clean token")
    assert_f32(y[:512], want0, "token with a host slot")
    assert_f32(y[512:], want1, "clean token")
    # bm_gate_up and bm_gate_up_x on their own
    xd, sel = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32)
    act = gpu.act(bm.Q4_K, 512, m)
    for entry in ("gate_up", "gate_up_x"):
        ah = gpu.act(bm.Q6_K, 256, m * top_k)
        marker = np.full(bm.col_bytes(bm.Q6_K, 256), 0x5A, np.uint8)
        ah.upload(1, marker)
        hb = gpu.buffer(np.float32, m * top_k * 256).fill_bytes(0xFF)
        if entry == "gate_up":
            gpu.enqueue_quantize(xd, m, act)
            gpu.enqueue_gate_up(L.dg, L.du, act, sel, m * top_k, 256, top_k, hb, ah)
        else:
            gpu.enqueue_gate_up_x(L.dg, L.du, xd, sel, top_k, m, 256, ah, h=hb)
        got = hb.download().reshape(m * top_k, 256)
        assert gpu.fault() == (bm.FAULT_NONE, 0), entry
        assert np.all(got[1].view(np.uint32) == 0xFFFFFFFF), entry
        assert np.array_equal(ah.download(1), marker), f"{entry}: the host slot's activation column was written"
        assert_f32(got[3:].reshape(-1), want_h1, f"{entry}: h of the clean token")
        for s in (3, 4, 5):
            assert np.array_equal(ah.download(s), ora.quantize_col(bm.Q6_K, want_h1[(s - 3) * 256:(s - 2) * 256])), f"{entry} act_h {s}"
        ah.free()
        hb.free()
    for b in (xd, sel, act):
        b.free()
    L.free()


# ------------------------------------------------------------------------------------- stacks wrapped in place

@pytest.mark.parametrize("wtype,rows,k", ((bm.Q4_K, 96, 1024), (bm.Q6_K, 96, 768), (bm.IQ2_XXS, 96, 512)))
@pytest.mark.parametrize("shift", (0, 2))
def test_wrapped_weights_dot_like_uploaded_ones(gpu, wtype, rows, k, shift):
    """bm_weights_wrap over device memory the caller holds, also at a base that is only 2-byte aligned for the types
    whose rows are (Q6_K 210-byte and IQ2_XXS 66-byte blocks): bm_gemv_sel gives bm_weights_create's bits."""
    if wtype == bm.Q4_K and shift:
        pytest.skip("Q4_K rows are read with aligned 16-byte loads: a stack starts on a 16-byte boundary")
    rng = np.random.default_rng(3500 + k)
    n_experts, rpe = 3, rows // 3
    w = random_blocks(wtype, rows, k, rng)
    ids = np.array([2, 0, 1, 2], np.uint32)
    x = normal_f32(rng, (len(ids), k))
    act = gpu.act(wtype, k, len(ids))
    xd, sel = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32)
    gpu.enqueue_quantize(xd, len(ids), act)
    up = gpu.weights(wtype, rows, k, w)
    raw = gpu.buffer(np.uint8, w.size + 16)
    raw.upload(np.concatenate([np.zeros(shift, np.uint8), w]))
    wrapped = bm.DeviceTensor(gpu, wtype, rows, k, dev_ptr=raw.ptr + shift)
    ya = gpu.buffer(np.float32, len(ids) * rpe).fill_bytes(0xFF)
    yb = gpu.buffer(np.float32, len(ids) * rpe).fill_bytes(0xFF)
    gpu.enqueue_gemv_sel(up, act, sel, len(ids), rpe, ya)
    gpu.enqueue_gemv_sel(wrapped, act, sel, len(ids), rpe, yb)
    a, b = ya.download(), yb.download()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    rb = ora.row_bytes(wtype, k)
    for s, e in enumerate(ids):
        want = ora.gemv(wtype, w[int(e) * rpe * rb:(int(e) + 1) * rpe * rb], rpe, k, ora.quantize_col(wtype, x[s]), 1)
        assert_f32(b[s * rpe:(s + 1) * rpe], want, f"slot {s}")
    for t in (up, wrapped, raw, act, xd, sel, ya, yb):
        t.free()
