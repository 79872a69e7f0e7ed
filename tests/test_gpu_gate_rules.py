"""GPU parity tests of the gate . up rules through the C ABI against the oracle's restatement of the CPU path's rules
(crates/qdot/src/lib.rs:11492 swiglu_clamp, swiglu_oai, :11617 swiglu_gclamp) on the same seeded inputs: every entry
that applies a rule (bm_gate_up, bm_gate_up_x / bm_moe_decode, bm_gate_up_tiles, bm_swiglu_quant) gives the oracle's h
bit for bit, with limits chosen so that every clamp bites on part of the values; a sum that is not finite under a
clamped rule raises F32Product and comes out NaN (crates/gpu/src/kquant/act.rs:166-175). The rule travels with each
launch (GateUpArgs' act) or, where the launch passes none, comes from the context (bm_set_gate_rule): both ways are run.
SiTU-GLU calls a tanh that the reference does not pin to bits between its own card and host
(crates/model/src/ops.rs:2339-2343); its h is held to the reference's bound, 1e-5 relative, and its quantized columns
to one code."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora
from common import normal_f32
from test_gpu_decode import Layer, assert_f32, gpu, grouped_tables_on_device, route  # noqa: F401  (gpu: module fixture)

pytestmark = pytest.mark.gpu

RULES = ((bm.ACT_SWIGLU_CLAMP, 0.08), (bm.ACT_SWIGLU_OAI, 0.25), (bm.ACT_SWIGLU_GCLAMP, 0.2), (bm.ACT_SWIGLU_CLAMP, 0.0),
         (bm.ACT_SILU_MUL, 0.0))
SITU = (bm.ACT_SITU, 0.3)  # a beta small enough that the gate's tanh bends most values


def oracle_h(L, x, ids, rule, limit):
    """h[slot] = rule(gate row dots, up row dots) with the oracle's dots, and the share of values a clamp changed."""
    m, top_k = ids.shape
    rbg, rbu = ora.row_bytes(L.types[0], L.hidden), ora.row_bytes(L.types[1], L.hidden)
    out = np.empty((m * top_k, L.ff), np.float32)
    bitten = 0
    for t in range(m):
        col = ora.quantize_col(L.types[0], x[t])
        for k in range(top_k):
            e = int(ids[t, k])
            g = ora.gemv(L.types[0], L.wg[e * L.ff * rbg:(e + 1) * L.ff * rbg], L.ff, L.hidden, col)
            u = ora.gemv(L.types[1], L.wu[e * L.ff * rbu:(e + 1) * L.ff * rbu], L.ff, L.hidden, col)
            out[t * top_k + k], ok = ora.gate_rule(rule, limit, g, u)
            assert ok
            bitten += np.count_nonzero(out[t * top_k + k] != ora.swiglu(g, u))
    return out, bitten / out.size


@pytest.fixture(scope="module")
def layer(gpu):
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 6, 4100)  # the headline shape's rows, six experts
    yield L
    L.free()


@pytest.mark.parametrize("per_launch", (True, False), ids=("per-launch", "context"))
@pytest.mark.parametrize("rule,limit", RULES)
def test_every_gate_up_entry_applies_the_rule(gpu, layer, rule, limit, per_launch):
    L = layer
    arg = (rule, limit) if per_launch else None
    rng = np.random.default_rng(4200 + rule)
    m, top_k = 3, 2
    x = normal_f32(rng, (m, L.hidden))
    ids, wts = route(rng, m, L.n_experts, top_k)
    want, share = oracle_h(L, x, ids, rule, limit)
    if rule != bm.ACT_SILU_MUL and limit > 0:
        assert share > 0.05, f"the limit bites on {share:.1%} of the values only"
    n_slots = m * top_k
    xd, sel = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32)
    act, act_h = gpu.act(L.types[0], L.hidden, m), gpu.act(L.types[2], L.ff, n_slots)
    h = gpu.buffer(np.float32, n_slots * L.ff)
    gpu.fault_clear()
    if per_launch:
        gpu.set_gate_rule(bm.ACT_SWIGLU_OAI, 3.0)  # a context rule the launches must not take
    else:
        gpu.set_gate_rule(rule, limit)
    try:
        # the slot launcher, with its fused quantizer
        gpu.enqueue_quantize(xd, m, act)
        h.fill_bytes(0xFF)
        gpu.enqueue_gate_up(L.dg, L.du, act, sel, n_slots, L.ff, top_k, h, act_h, rule=arg)
        assert_f32(h.download(), want.reshape(-1), "bm_gate_up")
        for s in range(n_slots):
            assert np.array_equal(act_h.download(s), ora.quantize_col(L.types[2], want[s])), f"act_h slot {s}"
        # from the f32 row
        h.fill_bytes(0xFF)
        gpu.enqueue_gate_up_x(L.dg, L.du, xd, sel, top_k, m, L.ff, act_h, None, h, rule=arg)
        assert_f32(h.download(), want.reshape(-1), "bm_gate_up_x")
        # by tiles
        sel2, order, start, tiles = grouped_tables_on_device(gpu, ids.reshape(-1), L.n_experts)
        h.fill_bytes(0xFF)
        gpu.enqueue_gate_up_tiles(L.dg, L.du, act, order, start, tiles, n_slots, L.ff, top_k, h, rule=arg)
        got = h.download().reshape(n_slots, L.ff)
        assert_f32(got, want[order.download()], "bm_gate_up_tiles")  # entry-ordered rows
        # the prefill path's quantizer over given sums
        g = normal_f32(rng, (n_slots, L.ff)) * np.float32(0.5)
        u = normal_f32(rng, (n_slots, L.ff)) * np.float32(0.5)
        gd, ud = gpu.upload(g, np.float32), gpu.upload(u, np.float32)
        gpu.enqueue_swiglu_quant(gd, ud, n_slots, act_h, rule=arg)
        for s in range(n_slots):
            hv, ok = ora.gate_rule(rule, limit, g[s], u[s])
            assert ok and np.array_equal(act_h.download(s), ora.quantize_col(L.types[2], hv)), f"swiglu_quant column {s}"
        assert gpu.fault() == (bm.FAULT_NONE, 0)
        for b in (sel2, order, start, tiles, gd, ud):
            b.free()
    finally:
        gpu.set_gate_rule(bm.ACT_SILU_MUL)
        for b in (xd, sel, act, act_h, h):
            b.free()


@pytest.mark.parametrize("per_launch", (True, False), ids=("per-launch", "context"))
def test_the_whole_step_under_a_rule(gpu, layer, per_launch):
    """bm_moe_decode (and its variant that allocates nothing) under the OAI rule: the oracle's h through its down dots
    and combine."""
    L = layer
    rng = np.random.default_rng(4300)
    m, top_k, rule, limit = 2, 4, bm.ACT_SWIGLU_OAI, 0.25
    x = normal_f32(rng, (m, L.hidden))
    ids, wts = route(rng, m, L.n_experts, top_k)
    want_h, _ = oracle_h(L, x, ids, rule, limit)
    rbd = ora.row_bytes(L.types[2], L.ff)
    down = np.stack([ora.gemv(L.types[2], L.wd[int(e) * L.hidden * rbd:(int(e) + 1) * L.hidden * rbd], L.hidden, L.ff,
                              ora.quantize_col(L.types[2], want_h[s])) for s, e in enumerate(ids.reshape(-1))])
    want_y = ora.combine_tokens(down.reshape(-1), wts.reshape(-1), None, L.hidden, top_k, m)
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    act_h = gpu.act(L.types[2], L.ff, m * top_k)
    y = gpu.buffer(np.float32, m * L.hidden).fill_bytes(0xFF)
    arg = (rule, limit) if per_launch else None
    if not per_launch:
        gpu.set_gate_rule(rule, limit)
    try:
        gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wd, None, top_k, m, act_h, y, rule=arg)
        assert_f32(y.download(), want_y, "y")
        y.fill_bytes(0xFF)
        gpu.enqueue_moe_decode_noalloc(L.dg, L.du, L.dd, xd, sel, wd, None, top_k, m, y, rule=arg)
        assert_f32(y.download(), want_y, "y of bm_moe_decode_noalloc")
    finally:
        gpu.set_gate_rule(bm.ACT_SILU_MUL)
        for b in (xd, sel, wd, act_h, y):
            b.free()


def test_situ_rule_within_the_reference_bound(gpu, layer):
    """SiTU-GLU through every entry: h within 1e-5 relative of the oracle's (whose tanh is the host libm's, the device's
    may sit an ulp away); a quantized column's codes within one and its scale within an ulp; the whole step within the
    path's 1e-4."""
    L = layer
    rng = np.random.default_rng(4400)
    m, top_k = 2, 3
    x = normal_f32(rng, (m, L.hidden))
    ids, wts = route(rng, m, L.n_experts, top_k)
    want, share = oracle_h(L, x, ids, *SITU)
    assert share > 0.5
    n_slots = m * top_k
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    act, act_h = gpu.act(L.types[0], L.hidden, m), gpu.act(L.types[2], L.ff, n_slots)
    h = gpu.buffer(np.float32, n_slots * L.ff)
    y = gpu.buffer(np.float32, m * L.hidden)
    gpu.fault_clear()

    def close(got, what):
        got = got.reshape(want.shape)
        assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-30), what
        assert np.count_nonzero(got.view(np.uint32) == want.view(np.uint32)) > 0.5 * got.size, what  # the two tanh sit an ulp apart here and there

    try:
        gpu.enqueue_quantize(xd, m, act)
        gpu.enqueue_gate_up(L.dg, L.du, act, sel, n_slots, L.ff, top_k, h.fill_bytes(0xFF), act_h, rule=SITU)
        close(h.download(), "bm_gate_up")
        gpu.enqueue_gate_up_x(L.dg, L.du, xd, sel, top_k, m, L.ff, act_h, None, h.fill_bytes(0xFF), rule=SITU)
        close(h.download(), "bm_gate_up_x")
        sel2, order, start, tiles = grouped_tables_on_device(gpu, ids.reshape(-1), L.n_experts)
        gpu.enqueue_gate_up_tiles(L.dg, L.du, act, order, start, tiles, n_slots, L.ff, top_k, h.fill_bytes(0xFF), rule=SITU)
        got = h.download().reshape(n_slots, L.ff)
        back = np.empty_like(got)
        back[order.download()] = got
        close(back, "bm_gate_up_tiles")
        # the whole step against the oracle's h through its down dots: the path's tolerance
        rbd = ora.row_bytes(L.types[2], L.ff)
        down = np.stack([ora.gemv(L.types[2], L.wd[int(e) * L.hidden * rbd:(int(e) + 1) * L.hidden * rbd], L.hidden, L.ff,
                                  ora.quantize_col(L.types[2], want[s])) for s, e in enumerate(ids.reshape(-1))])
        want_y = ora.combine_tokens(down.reshape(-1), wts.reshape(-1), None, L.hidden, top_k, m)
        gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wd, None, top_k, m, act_h, y, rule=SITU)
        assert np.max(np.abs(y.download() - want_y)) <= 1e-4 * np.max(np.abs(want_y))
        # bm_swiglu_quant over given sums at the reference test's spread
        g = normal_f32(rng, (n_slots, L.ff)) * np.float32(6.0)
        u = normal_f32(rng, (n_slots, L.ff)) * np.float32(12.0)
        gd, ud = gpu.upload(g, np.float32), gpu.upload(u, np.float32)
        gpu.enqueue_swiglu_quant(gd, ud, n_slots, act_h, rule=(bm.ACT_SITU, 8.0))
        for s in range(n_slots):
            hv, ok = ora.gate_rule(bm.ACT_SITU, 8.0, g[s], u[s])
            got_v = ora.dequant_col(L.types[2], act_h.download(s), L.ff)
            want_v = ora.dequant_col(L.types[2], ora.quantize_col(L.types[2], hv), L.ff)
            step = np.max(np.abs(hv)) / 127.0
            assert ok and np.max(np.abs(got_v - want_v)) <= 1.01 * step, f"swiglu_quant column {s}"
        assert gpu.fault() == (bm.FAULT_NONE, 0)
        # beta must be finite and positive, refused by the entry before anything runs
        with pytest.raises(bm.GpuError) as e:
            gpu.enqueue_swiglu_quant(gd, ud, n_slots, act_h, rule=(bm.ACT_SITU, 0.0))
        assert e.value.code == bm.ESHAPE and "bm_swiglu_quant" in str(e.value) and "beta" in str(e.value)
        for b in (sel2, order, start, tiles, gd, ud):
            b.free()
    finally:
        for b in (xd, sel, wd, act, act_h, h, y):
            b.free()


@pytest.mark.parametrize("rule,limit", ((bm.ACT_SWIGLU_CLAMP, 7.0), (bm.ACT_SWIGLU_OAI, 7.0), (bm.ACT_SITU, 7.0),
                                        (bm.ACT_SWIGLU_GCLAMP, 7.0)))
def test_a_sum_that_is_not_finite_is_raised_not_clamped(gpu, rule, limit):
    k, n = 256, 3
    g = np.ones((n, k), np.float32)
    u = np.ones((n, k), np.float32)
    g[1, 40], u[2, 200] = np.inf, np.nan
    gd, ud = gpu.upload(g, np.float32), gpu.upload(u, np.float32)
    act = gpu.act(bm.Q6_K, k, n)
    gpu.fault_clear()
    gpu.set_layer(2)
    gpu.set_gate_rule(rule, limit)
    try:
        gpu.enqueue_swiglu_quant(gd, ud, n, act)
        w0, mask = gpu.fault(2)
        # the NaN the rule wrote is then met by the quantizer, which raises its own site (the lower code wins word 0)
        assert mask == (1 << bm.SITE_F32_PRODUCT) | (1 << bm.SITE_QUANT_COLUMN) and w0 == (2 << 8) + bm.SITE_QUANT_COLUMN
        hv, ok = ora.gate_rule(rule, limit, g[0], u[0])
        if rule != bm.ACT_SITU:
            assert ok and np.array_equal(act.download(0), ora.quantize_col(bm.Q6_K, hv))
    finally:
        gpu.set_gate_rule(bm.ACT_SILU_MUL)
        gpu.set_layer(0)
        gpu.fault_clear()
        for b in (gd, ud, act):
            b.free()


def test_rule_refusals_are_named(gpu):
    for rule, limit, word in ((bm.ACT_SWIGLU_CLAMP, np.inf, "finite"), (bm.ACT_SWIGLU_OAI, -1.0, "at least 0"),
                              (bm.ACT_SWIGLU_OAI, np.nan, "at least 0"), (bm.ACT_SWIGLU_GCLAMP, 0.0, "positive"),
                              (bm.ACT_SITU, -2.0, "beta"), (bm.ACT_SITU, np.inf, "beta"), (9, 1.0, "rule 9")):
        with pytest.raises(bm.GpuError) as e:
            gpu.set_gate_rule(rule, limit)
        assert word in str(e.value) and "bm_set_gate_rule" in str(e.value)
