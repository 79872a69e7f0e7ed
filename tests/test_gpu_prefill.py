"""GPU parity tests of the prefill path (route table, grouped GEMM on the int8 matrix cores, SwiGLU quantizer),
through the C ABI, against the CPU oracle on the same seeded inputs. Every value of the grouped GEMM is the
one-column row dot's, so everything is compared bit for bit (and within the stated 1e-4 first).
Mirrors the reference's gate_gemm clauses (crates/gpu-gates/src/bin/gate_gemm.rs): table by definition, refused ids
-> NaN rows and ExpertId, Shared and PerSlot inputs, rows_per_expert a multiple of 16 that is not a whole slab."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora
from common import normal_f32
from test_gpu_decode import Layer, assert_f32, gpu, route, stack  # noqa: F401  (gpu is the module fixture)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_experts,n_slots,seed", ((128, 16384, 1), (3, 500, 2), (1, 64, 3), (1024, 4096, 4), (7, 1, 5)))
def test_route_table_is_the_definition(gpu, n_experts, n_slots, seed):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, n_experts, n_slots).astype(np.uint32)
    if n_experts == 128:  # skewed popularity, as a prefill batch has
        p = 1.0 / np.arange(1, n_experts + 1) ** 1.1
        ids = rng.choice(n_experts, n_slots, p=p / p.sum()).astype(np.uint32)
    gpu.fault_clear()
    table = gpu.route(n_slots, n_experts)
    ids_d = gpu.upload(ids, np.uint32)
    table.fill(ids_d, n_slots)
    cols, tiles, refused = table.read()
    want_cols, want_tiles, want_refused = ora.gemm_route(ids, n_experts)
    assert refused == want_refused == 0
    assert np.array_equal(cols, want_cols)
    assert np.array_equal(tiles, want_tiles)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    table.free()
    ids_d.free()


@pytest.mark.parametrize("n_experts,n_slots,seed", ((128, 40960, 11), (256, 16385, 12), (1024, 40960, 13), (511, 33000, 14),
                                                    (512, 2049, 15), (600, 8191, 16), (5, 129, 17)))
def test_route_table_made_by_several_workgroups(gpu, n_experts, n_slots, seed):
    """Lists long enough for several workgroups (each places a part of the slots), with host-served slots and refused ids
    among them, against the definition spelt with a stable sort: the live slots by expert, ascending inside an expert, then
    the refused ones ascending, then 0xffffffff for as many entries as slots are served elsewhere; tiles of at most 64."""
    rng = np.random.default_rng(seed)
    p = 1.0 / np.arange(1, n_experts + 1) ** 1.1
    ids = rng.permutation(n_experts)[rng.choice(n_experts, n_slots, p=p / p.sum())].astype(np.uint32)
    odd = rng.random(n_slots)
    ids[odd < 0.02] = bm.HOST_SLOT
    ids[(odd >= 0.02) & (odd < 0.03)] = n_experts + rng.integers(0, 1000, int(((odd >= 0.02) & (odd < 0.03)).sum()))
    live = np.flatnonzero(ids < n_experts)
    refused = np.flatnonzero((ids >= n_experts) & (ids != bm.HOST_SLOT))
    listed = live[np.argsort(ids[live], kind="stable")]
    want_cols = np.concatenate([listed, refused, np.full(n_slots - listed.size - refused.size, 0xFFFFFFFF)]).astype(np.uint32)
    counts = np.bincount(ids[live], minlength=n_experts)
    want_tiles, at = [], 0
    for e in range(n_experts):
        for j in range(0, int(counts[e]), 64):
            want_tiles.append((e, at + j, min(64, int(counts[e]) - j)))
        at += int(counts[e])
    gpu.fault_clear()
    table = gpu.route(n_slots, n_experts)
    ids_d = gpu.upload(ids, np.uint32)
    for rep in range(2):  # the second fill over the first one's table
        table.fill(ids_d, n_slots)
        cols, tiles, n_refused = table.read()
        assert n_refused == refused.size
        assert np.array_equal(cols, want_cols)
        assert np.array_equal(tiles, np.asarray(want_tiles, np.uint32).reshape(-1, 3))
    assert (gpu.fault()[1] & (1 << bm.SITE_EXPERT_ID)) != 0 if refused.size else gpu.fault() == (bm.FAULT_NONE, 0)
    gpu.fault_clear()
    table.free()
    ids_d.free()


@pytest.mark.parametrize("wtype,k,m,n_experts,top_k,seed", ((bm.Q4_K, 2048, 300, 128, 8, 1), (bm.IQ2_XXS, 1792, 5, 40, 3, 2),
                                                          (bm.Q6_K, 256, 1, 3, 2, 3), (bm.IQ4_XS, 512, 2100, 256, 8, 4)))
def test_route_table_and_quantizer_as_one_launch(gpu, wtype, k, m, n_experts, top_k, seed):
    """bm_route_fill_quantize leaves what bm_route_fill and bm_quantize leave: the table word for word and every column's
    bytes, in either column form, with a host-served slot and a refused id among the slots, twice in a row; rows that are not
    16-byte aligned go through the two launches and give the same."""
    rng = np.random.default_rng(7800 + seed)
    n_slots = m * top_k
    ids = rng.integers(0, n_experts, n_slots).astype(np.uint32)
    if n_slots > 4:
        ids[1], ids[3] = bm.HOST_SLOT, n_experts + 5
    x = normal_f32(rng, (m, k))
    sel, xd = gpu.upload(ids, np.uint32), gpu.upload(np.concatenate([np.zeros(1, np.float32), x.reshape(-1)]), np.float32)
    xa = gpu.upload(x, np.float32)
    want_t, want_act = gpu.route(n_slots, n_experts), gpu.act(wtype, k, m)
    gpu.fault_clear()
    want_t.fill(sel, n_slots)
    want_fault = gpu.fault()
    gpu.enqueue_quantize(xa, m, want_act)
    want = want_t.read()
    cols_to_check = sorted({0, m // 3, m // 2, m - 1})
    for x_ptr, what in ((xd.ptr + 4, "rows 4 bytes off a 16-byte boundary"), (xa, "aligned rows")):
        t, act = gpu.route(n_slots, n_experts), gpu.act(wtype, k, m)
        for rep in range(2):
            gpu.fault_clear()
            t.fill_quantize(sel, n_slots, x_ptr, m, act)
            got = t.read()
            assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]) and got[2] == want[2], what
            for c in cols_to_check:
                assert np.array_equal(act.download(c), want_act.download(c)), f"{what}: column {c}"
            assert np.array_equal(act.download(m - 1), ora.quantize_col(wtype, x[m - 1])), what
            assert gpu.fault() == want_fault, what
        t.free()
        act.free()
    gpu.fault_clear()
    for b in (want_t, want_act, sel, xd, xa):
        b.free()


def run_prefill(gpu, L, x, ids, wts, top_k):
    """quantize -> route -> gate GEMM, up GEMM (Shared) -> swiglu_quant -> down GEMM (PerSlot) -> combine
    (crates/gpu/src/arch/qwen3moe/wide.rs:1171-1225)."""
    m = x.shape[0]
    n_slots = m * top_k
    act = gpu.act(L.types[0], L.hidden, m)
    act_h = gpu.act(L.types[2], L.ff, n_slots)
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    table = gpu.route(n_slots, L.n_experts)
    g = gpu.buffer(np.float32, n_slots * L.ff).fill_bytes(0xFF)
    u = gpu.buffer(np.float32, n_slots * L.ff).fill_bytes(0xFF)
    down = gpu.buffer(np.float32, n_slots * L.hidden).fill_bytes(0xFF)
    y = gpu.buffer(np.float32, m * L.hidden).fill_bytes(0xFF)
    gpu.enqueue_quantize(xd, m, act)
    table.fill(sel, n_slots)
    gpu.enqueue_gemm(L.dg, L.ff, act, table, top_k, g)
    gpu.enqueue_gemm(L.du, L.ff, act, table, top_k, u)
    gpu.enqueue_swiglu_quant(g, u, n_slots, act_h)
    gpu.enqueue_gemm(L.dd, L.hidden, act_h, table, 0, down)
    gpu.enqueue_combine_tokens(down, wd, None, L.hidden, top_k, m, y)
    out = y.download(), g.download(), u.download(), [act_h.download(s) for s in range(n_slots)], down.download()
    for b in (act, act_h, xd, sel, wd, table, g, u, down, y):
        b.free()
    return out


def test_gemm_fast_mode_is_within_the_tolerance(gpu):
    """BM_GEMM_FAST keeps the exact integers and sums them in another f32 order: every value of one GEMM is within
    1e-4 (max-abs normalised over its row vector, the contract's tolerance) of the one-column dot, in practice far
    inside it. (Chained through the Q8 quantizer of h a last-bit difference can flip a code, which is why the exact
    mode is the default and the one the layer tests use.)"""
    from common import max_abs_normalised
    rng = np.random.default_rng(2200)
    worst = 0.0
    # the last cases: the f16 form of the tolerance mode (Q4_K), full slabs and a ragged one, tiles wider and narrower than 32 slots
    for wtype, k, rpe, mode in ((bm.Q4_K, 2048, 768, bm.GEMM_FAST), (bm.Q6_K, 768, 2048, bm.GEMM_FAST), (bm.Q5_K, 1024, 80, bm.GEMM_FAST),
                                (bm.IQ2_XXS, 1792, 208, bm.GEMM_FAST), (bm.Q4_K, 2048, 768, bm.GEMM_FAST_F16),
                                (bm.Q4_K, 512, 272, bm.GEMM_FAST_F16), (bm.Q6_K, 768, 96, bm.GEMM_FAST_F16)):
        n_experts, n_slots = 6, 150
        w = stack(wtype, n_experts * rpe, k, 2201)
        ids = rng.integers(0, n_experts, n_slots).astype(np.uint32)
        ids[ids == 5] = rng.integers(0, 2, int((ids == 5).sum())).astype(np.uint32)  # expert 5 idle, 0 and 1 past 32 slots
        ids[:3] = 5                                                                    # but for three slots: a narrow tile
        x = normal_f32(rng, (n_slots, k))
        dw, act = gpu.weights(wtype, n_experts * rpe, k, w), gpu.act(wtype, k, n_slots)
        xd, sel = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32)
        table = gpu.route(n_slots, n_experts)
        gpu.enqueue_quantize(xd, n_slots, act)
        table.fill(sel, n_slots)
        y = gpu.buffer(np.float32, n_slots * rpe).fill_bytes(0)
        gpu.set_gemm_mode(mode)
        try:
            gpu.enqueue_gemm(dw, rpe, act, table, 0, y)
            got = y.download().reshape(n_slots, rpe)
        finally:
            gpu.set_gemm_mode(bm.GEMM_EXACT)
        rb = ora.row_bytes(wtype, k)
        for s in range(0, n_slots, 7):
            e = int(ids[s])
            want = ora.gemv(wtype, w[e * rpe * rb:(e + 1) * rpe * rb], rpe, k, ora.quantize_col(wtype, x[s]), 1)
            err = max_abs_normalised(got[s], want)
            worst = max(worst, err)
            assert err <= 1e-4, f"type {wtype} slot {s}: max-abs normalised error {err}"
        for b in (dw, act, xd, sel, table, y):
            b.free()
    assert worst <= 1e-5, f"fast mode drifted further than f32 rounding explains: {worst}"


@pytest.mark.parametrize("types,hidden,ff,n_experts,m,top_k,cheap", (
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 512, 256, 6, 70, 3, False),      # 210 slots over 6 experts: runs of about 35, a tile each
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 16, 48, 8, True),     # config 4's layer shape, 384 slots
    ((bm.Q6_K, bm.Q6_K, bm.Q4_K), 768, 512, 3, 9, 2, False),       # the other type on each side; ragged tiles
    ((bm.Q5_K, bm.Q5_K, bm.Q5_K), 768, 512, 3, 40, 2, False),      # Q5_K on both sides: the Q4_K walk with a fifth bit
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), 1024, 512, 5, 60, 3, False),  # Q8_K columns on both sides; runs past one 32-slot half
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.Q6_K), 768, 256, 3, 11, 2, False),      # the two column forms in one layer
    ((bm.Q4_K, bm.Q4_K, bm.IQ2_XXS), 512, 768, 4, 30, 4, False),
    ((bm.IQ4_XS, bm.IQ4_XS, bm.IQ4_XS), 768, 512, 4, 50, 3, False),    # the other types on Q8_K columns: the IQ2_XXS kernel's
    ((bm.IQ3_XXS, bm.IQ3_XXS, bm.IQ3_XXS), 512, 768, 3, 44, 2, False),  # products over their own staging and f32 steps
    ((bm.Q3_K, bm.Q3_K, bm.Q3_K), 1024, 256, 5, 37, 4, False),
    ((bm.IQ3_XXS, bm.IQ3_XXS, bm.Q3_K), 768, 768, 3, 20, 3, False),
    ((bm.Q3_K, bm.Q3_K, bm.IQ4_XS), 512, 512, 6, 70, 2, False),
))
def test_prefill_layer_matches_the_oracle(gpu, types, hidden, ff, n_experts, m, top_k, cheap):
    L = Layer(gpu, types, hidden, ff, n_experts, 2000 + hidden, cheap=cheap)
    rng = np.random.default_rng(2001)
    x = normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, n_experts, top_k)
    gpu.fault_clear()
    y, g, u, act_h, down = run_prefill(gpu, L, x, ids, wts, top_k)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    # gate and up rows against the one-column dots
    rb = ora.row_bytes(types[0], hidden)
    for s in (0, m * top_k // 2, m * top_k - 1):
        e, col = int(ids.reshape(-1)[s]), ora.quantize_col(types[0], x[s // top_k])
        assert_f32(g[s * ff:(s + 1) * ff], ora.gemv(types[0], L.wg[e * ff * rb:(e + 1) * ff * rb], ff, hidden, col, 1), f"gate slot {s}")
        assert_f32(u[s * ff:(s + 1) * ff], ora.gemv(types[1], L.wu[e * ff * rb:(e + 1) * ff * rb], ff, hidden, col, 1), f"up slot {s}")
    for s in range(m * top_k):
        assert np.array_equal(act_h[s], ora.quantize_col(types[2], want_h[s * ff:(s + 1) * ff])), f"act_h slot {s}"
    assert_f32(y, want_y, "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    L.free()


@pytest.mark.parametrize("fast", (0, 1, 2))
def test_gemm_rows_not_a_whole_slab_and_refused_slots(gpu, fast):
    """rows_per_expert = 80 (a multiple of 16, not a whole slab of either mode's kernel); a refused id gets NaN rows and
    ExpertId. In the tolerance mode the live rows are held to the tolerance instead of to bits."""
    from common import max_abs_normalised
    rng = np.random.default_rng(2100)
    for wtype, k in ((bm.Q4_K, 1024), (bm.Q5_K, 512), (bm.Q6_K, 768), (bm.IQ2_XXS, 768), (bm.IQ3_XXS, 512), (bm.IQ4_XS, 768),
                     (bm.Q3_K, 1024)):
        rpe, n_experts, n_slots = 80, 4, 23
        w = stack(wtype, n_experts * rpe, k, 2101)
        ids = rng.integers(0, n_experts, n_slots).astype(np.uint32)
        ids[5] = 9   # past the stack
        x = normal_f32(rng, (n_slots, k))
        dw, act = gpu.weights(wtype, n_experts * rpe, k, w), gpu.act(wtype, k, n_slots)
        xd, sel = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32)
        table = gpu.route(n_slots, n_experts)
        gpu.fault_clear()
        gpu.set_layer(2)
        gpu.enqueue_quantize(xd, n_slots, act)
        table.fill(sel, n_slots)
        y = gpu.buffer(np.float32, n_slots * rpe).fill_bytes(0)
        gpu.set_gemm_mode(fast)  # 0: exact, 1: tolerance mode, 2: its f16 form
        try:
            gpu.enqueue_gemm(dw, rpe, act, table, 0, y)
            got = y.download().reshape(n_slots, rpe)
        finally:
            gpu.set_gemm_mode(bm.GEMM_EXACT)
        cols, tiles, refused = table.read()
        assert refused == 1 and cols[-1] == 5 and gpu.fault(2) == ((2 << 8) | bm.SITE_EXPERT_ID, 1 << bm.SITE_EXPERT_ID)
        assert np.isnan(got[5]).all()
        rb = ora.row_bytes(wtype, k)
        for s in range(n_slots):
            if s == 5:
                continue
            e = int(ids[s])
            want = ora.gemv(wtype, w[e * rpe * rb:(e + 1) * rpe * rb], rpe, k, ora.quantize_col(wtype, x[s]), 1)
            if fast:
                assert max_abs_normalised(got[s], want) <= 1e-4, f"type {wtype} slot {s}"
            else:
                assert_f32(got[s], want, f"type {wtype} slot {s}")
        gpu.set_layer(bm.LAYER_NONE)
        gpu.fault_clear()
        for b in (dw, act, xd, sel, table, y):
            b.free()


@pytest.mark.parametrize("fast", (0, 1, 2))
def test_gemm_column_that_is_not_finite(gpu, fast):
    """A token row with an infinity: the quantizer raises QuantColumn and leaves a NaN scale with zero codes
    (crates/gpu/src/lib.rs:925-933); the GEMM rows of that token's slots are NaN in either mode, and every other slot's
    rows are what they are without it."""
    from common import max_abs_normalised
    rng = np.random.default_rng(2150)
    wtype, k, rpe, n_experts, m, top_k = bm.Q4_K, 512, 96, 3, 20, 2
    n_slots = m * top_k
    w = stack(wtype, n_experts * rpe, k, 2151)
    ids = rng.integers(0, n_experts, (m, top_k)).astype(np.uint32)
    x = normal_f32(rng, (m, k))
    x[7, 100] = np.inf
    dw, act = gpu.weights(wtype, n_experts * rpe, k, w), gpu.act(wtype, k, m)
    xd, sel = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32)
    table = gpu.route(n_slots, n_experts)
    gpu.fault_clear()
    gpu.set_layer(4)
    gpu.enqueue_quantize(xd, m, act)
    table.fill(sel, n_slots)
    y = gpu.buffer(np.float32, n_slots * rpe).fill_bytes(0)
    gpu.set_gemm_mode(fast)  # 0: exact, 1: tolerance mode, 2: its f16 form
    try:
        gpu.enqueue_gemm(dw, rpe, act, table, top_k, y)
        got = y.download().reshape(n_slots, rpe)
    finally:
        gpu.set_gemm_mode(bm.GEMM_EXACT)
    assert gpu.fault(4)[1] & (1 << bm.SITE_QUANT_COLUMN)
    rb = ora.row_bytes(wtype, k)
    for s in range(n_slots):
        t, e = s // top_k, int(ids.reshape(-1)[s])
        if t == 7:
            assert np.isnan(got[s]).all(), f"slot {s} of the token that is not finite"
            continue
        want = ora.gemv(wtype, w[e * rpe * rb:(e + 1) * rpe * rb], rpe, k, ora.quantize_col(wtype, x[t]), 1)
        if fast:
            assert max_abs_normalised(got[s], want) <= 1e-4, f"slot {s}"
        else:
            assert_f32(got[s], want, f"slot {s}")
    gpu.set_layer(bm.LAYER_NONE)
    gpu.fault_clear()
    for b in (dw, act, xd, sel, table, y):
        b.free()


def test_prefill_refusals_are_named(gpu):
    w4 = gpu.weights(bm.Q4_K, 64, 512, np.zeros(64 * bm.row_bytes(bm.Q4_K, 512), np.uint8))
    wi = gpu.weights(bm.IQ4_XS, 64, 512, np.zeros(64 * bm.row_bytes(bm.IQ4_XS, 512), np.uint8))
    a512, aq8k = gpu.act(bm.Q4_K, 512, 8), gpu.act(bm.IQ4_XS, 512, 8)
    buf = gpu.buffer(np.float32, 4096)
    ids = gpu.upload(np.zeros(8, np.uint32))
    table = gpu.route(8, 2)
    cases = [(lambda: gpu.enqueue_gemm(w4, 32, a512, table, 0, buf), bm.ESHAPE, "filled")]
    for call, code, word in cases:
        with pytest.raises(bm.GpuError) as e:
            call()
        assert e.value.code == code and word in str(e.value), str(e.value)
    table.fill(ids, 8)
    cases = (
        (lambda: gpu.enqueue_gemm(w4, 24, a512, table, 0, buf), bm.ESHAPE, "multiple of 16"),
        (lambda: gpu.enqueue_gemm(w4, 16, a512, table, 0, buf), bm.ESHAPE, "experts"),
        (lambda: gpu.enqueue_gemm(w4, 32, a512, table, 3, buf), bm.ESHAPE, "whole tokens"),
        (lambda: gpu.enqueue_swiglu_quant(buf, buf, 9, a512), bm.ESHAPE, "n_cols"),
        (lambda: table.fill(ids, 9), bm.ESHAPE, "n_slots"),
        (lambda: gpu.route(50000, 2), bm.ESHAPE, "max_slots"),
        (lambda: gpu.route(8, 2000), bm.ESHAPE, "n_experts"),
    )
    for call, code, word in cases:
        with pytest.raises(bm.GpuError) as e:
            call()
        assert e.value.code == code and word in str(e.value), str(e.value)
    for b in (w4, wi, a512, aq8k, buf, ids, table):
        b.free()


def test_gemm_at_the_largest_route(gpu):
    """The route's limits (crates/gpu/src/gemm/mod.rs:97-101): 40960 slots over 1024 experts, one column a slot, with
    runs from empty to many tiles; every slot's 16 rows against the one-column dot, and the table by definition."""
    from test_gpu_decode import random_blocks
    n_experts, n_slots, rpe, k = 1024, 40960, 16, 256
    rng = np.random.default_rng(2600)
    w = random_blocks(bm.Q4_K, n_experts * rpe, k, rng)
    p = 1.0 / np.arange(1, n_experts + 1) ** 1.3     # skewed: the first experts own thousands of slots, the last none
    ids = rng.choice(n_experts, n_slots, p=p / p.sum()).astype(np.uint32)
    x = normal_f32(rng, (n_slots, k))
    dw, act = gpu.weights(bm.Q4_K, n_experts * rpe, k, w), gpu.act(bm.Q4_K, k, n_slots)
    xd, sel = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32)
    table = gpu.route(n_slots, n_experts)
    y = gpu.buffer(np.float32, n_slots * rpe).fill_bytes(0xFF)
    gpu.fault_clear()
    gpu.enqueue_quantize(xd, n_slots, act)
    table.fill(sel, n_slots)
    gpu.enqueue_gemm(dw, rpe, act, table, 0, y)
    got = y.download().reshape(n_slots, rpe)
    cols, tiles, refused = table.read()
    want_cols, want_tiles, want_refused = ora.gemm_route(ids, n_experts)
    assert refused == want_refused == 0 and np.array_equal(cols, want_cols) and np.array_equal(tiles, want_tiles)
    assert len(np.unique(ids)) < n_experts and np.bincount(ids).max() > 64 * 20
    rb = ora.row_bytes(bm.Q4_K, k)
    for s in np.concatenate([np.arange(0, n_slots, 97), [n_slots - 1]]):
        e = int(ids[s])
        want = ora.gemv(bm.Q4_K, w[e * rpe * rb:(e + 1) * rpe * rb], rpe, k, ora.quantize_col(bm.Q4_K, x[s]), 1)
        assert_f32(got[s], want, f"slot {s}")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    with pytest.raises(bm.GpuError) as e:
        gpu.route(n_slots + 1, n_experts)
    assert e.value.code == bm.ESHAPE and "max_slots" in str(e.value)
    for b in (dw, act, xd, sel, table, y):
        b.free()
