"""Pins the rest of the oracle: expf / SwiGLU (crates/qdot/tests/qdot.rs:3927-4034, 8157-8230), router and combine
order (crates/model/src/moe.rs:246-279, crates/gpu/src/elem.rs:658-697), the weight quantizers' properties
(crates/gguf/src/kquant/tests.rs:5-60, crates/gguf/src/iq_quant/tests.rs:44-140) and the whole-layer step (scalar,
threaded and AVX2 forms must agree bit for bit)."""
import math

import numpy as np
import pytest

import ora
from common import iq4xs_rows, max_abs_normalised, normal_f32


# ----------------------------------------------------------------------------------------------- expf and SwiGLU

def test_expf_ik_tracks_libm():
    xs = np.concatenate([np.linspace(-87.0, 88.0, 4001), np.linspace(-1.0, 1.0, 2001), [0.0, -0.0]]).astype(np.float32)
    for x in xs:
        got = float(ora.expf_ik(x))
        want = math.exp(float(x))
        assert abs(got - want) <= 2.5e-7 * want, (x, got, want)


def test_expf_ik_special_paths():
    # |n| > 126 takes the two-step scale, |n| > 192 overflows or underflows outright (crates/qdot/src/lib.rs:3762-3771)
    assert ora.expf_ik(0.0) == np.float32(1.0)
    for x in (88.0, 88.5, 88.7):
        got, want = float(ora.expf_ik(x)), math.exp(float(np.float32(x)))
        assert abs(got - want) <= 3e-7 * want
    for x in (-88.0, -95.0, -100.0, -103.0):
        got, want = float(ora.expf_ik(x)), math.exp(float(np.float32(x)))
        assert abs(got - want) <= max(3e-7 * want, 1.5e-45)
    assert np.isinf(ora.expf_ik(89.0)) and np.isinf(ora.expf_ik(200.0)) and np.isinf(ora.expf_ik(1e30))
    assert ora.expf_ik(-104.5) == 0.0 and ora.expf_ik(-200.0) == 0.0 and ora.expf_ik(-1e30) == 0.0
    assert np.isnan(ora.expf_ik(np.nan))


def test_swiglu_is_divide_then_multiply_and_position_independent():
    rng = np.random.default_rng(1)
    g, u = normal_f32(rng, 777, 3.0), normal_f32(rng, 777, 2.0)
    out = ora.swiglu(g, u)
    for i in (0, 1, 7, 8, 9, 500, 776):
        e = ora.expf_ik(np.float32(0.0) - g[i])
        want = np.float32(np.float32(g[i] / np.float32(np.float32(1.0) + e)) * u[i])
        assert out[i].tobytes() == want.tobytes()
        assert ora.swiglu(g[i:i + 1], u[i:i + 1])[0].tobytes() == out[i].tobytes()
    ref = g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64))) * u.astype(np.float64)
    assert max_abs_normalised(out, ref) < 1e-6
    big = ora.swiglu(np.array([100.0, -100.0, 0.0], np.float32), np.array([2.0, 2.0, 5.0], np.float32))
    assert big[0] == 200.0 and abs(big[1]) < 1e-40 and big[2] == 0.0


def silu64(g):
    g = np.asarray(g, np.float64)
    return g / (1.0 + np.exp(-g))


def test_gate_rules_by_their_definitions():
    """The clamped rules against what their definitions fix (crates/qdot/tests/qdot.rs:4035-4046 ik_swiglu_clamp,
    :4158-4169 ref_swiglu_oai are transcriptions of the sources; here the cases a transcription could get wrong are
    worked by hand): which quantity each limit bites on, the +1 of the OAI rule, its alpha, the no-clamp threshold,
    NaN through every comparison, and the finite flag."""
    f = np.float32
    L = f(7.0)
    g = np.array([20.0, 20.0, 20.0, 1.0, 1.0, -30.0, 0.0, 7.0, 6.9999], f)
    u = np.array([3.0, 9.0, -9.0, 9.0, -0.5, 2.0, 5.0, 7.0, -7.0], f)
    s = ora.swiglu(g, np.ones_like(g))  # silu(g), pinned above
    # ik's clamp: the limit bites on silu(g), not on g
    out, ok = ora.gate_rule(1, L, g, u)
    want = np.minimum(s, L) * np.clip(u, -L, L)
    assert ok and out.tobytes() == want.astype(f).tobytes()
    assert out[0] == 21.0 and out[1] == 49.0 and out[2] == -49.0  # silu(20) = 20 > 7
    # the gate-first clamp: the limit bites on g before the activation: silu(7) < 7
    out4, ok = ora.gate_rule(4, L, g, u)
    s7 = ora.swiglu(np.array([7.0], f), np.ones(1, f))[0]
    assert ok and out4[0] == f(s7 * f(3.0)) and out4[1] == f(s7 * L) and out4[2] == f(s7 * -L)
    assert out4[3:].tobytes() == (ora.swiglu(np.minimum(g, L), np.ones_like(g)) * np.clip(u, -L, L))[3:].astype(f).tobytes()
    assert s7 < 7.0 and out4[0] != out[0]
    # the OAI rule: x / (1 + e^(-1.702 x)) * (y + 1), gate clamped from above only
    out2, ok = ora.gate_rule(2, L, g, u)
    x, y = np.minimum(g, L).astype(np.float64), np.clip(u, -L, L).astype(np.float64)
    ref = x / (1.0 + np.exp(-1.702 * x)) * (y + 1.0)
    assert ok and np.max(np.abs(out2 - ref)) <= 2e-6 * np.max(np.abs(ref))
    assert abs(out2[4] - 1.0 / (1.0 + np.exp(-1.702)) * 0.5) < 1e-6      # y + 1 with y = -0.5
    assert abs(out2[5] - (-30.0 / (1.0 + np.exp(1.702 * 30.0)) * 3.0)) < 1e-20  # no clamp from below on the gate
    e = ora.expf_ik(f(1.702) * (f(0.0) - f(1.0)))
    assert out2[3].tobytes() == f(f(f(1.0) / f(f(1.0) + e)) * f(8.0)).tobytes()  # op order: divide, then (y + 1)
    # a limit at or below 1e-6 (or NaN) clamps nothing under rules 1 and 4: the plain rule's bits
    plain = ora.swiglu(g, u)
    for lim in (0.0, 1e-6, -1.0, np.nan):
        for rule in (1, 4):
            o, ok = ora.gate_rule(rule, lim, g, u)
            assert ok and o.tobytes() == plain.tobytes()
    o, ok = ora.gate_rule(1, 2e-6, g, u)
    assert o.tobytes() != plain.tobytes()
    # rule 0 is swiglu; an unknown rule is refused
    assert ora.gate_rule(0, 5.0, g, u)[0].tobytes() == plain.tobytes()
    with pytest.raises(ValueError):
        ora.gate_rule(5, 1.0, g, u)
    # NaN through the comparisons: ik's clamp turns a NaN up into the limit and lets a NaN silu through; the other two
    # let a NaN up through (std::clamp); every clamping rule reports the block
    nan, inf = f(np.nan), f(np.inf)
    o, ok = ora.gate_rule(1, L, np.array([1.0, nan, inf], f), np.array([nan, 2.0, 2.0], f))
    assert not ok and o[0] == f(s[3] * L) and np.isnan(o[1]) and o[2] == 14.0
    for rule in (2, 4):
        o, ok = ora.gate_rule(rule, L, np.array([1.0, nan, inf, 1.0], f), np.array([nan, 2.0, 2.0, -inf], f))
        assert not ok and np.isnan(o[0]) and np.isnan(o[1]) and np.isfinite(o[2]) and np.isfinite(o[3])
    o, ok = ora.gate_rule(1, 0.0, np.array([inf], f), np.array([1.0], f))
    assert ok and not np.isfinite(o[0])  # below the threshold nothing is hidden, so nothing is reported
    # position independence
    rng = np.random.default_rng(5)
    gg, uu = normal_f32(rng, 333, 6.0), normal_f32(rng, 333, 6.0)
    for rule in (1, 2, 4):
        o, _ = ora.gate_rule(rule, 5.0, gg, uu)
        for i in (0, 7, 8, 332):
            assert ora.gate_rule(rule, 5.0, gg[i:i + 1], uu[i:i + 1])[0][0].tobytes() == o[i].tobytes()


def test_situ_rule_against_its_closed_form():
    """SiTU-GLU (rule 3) on the inputs and at the bound of the reference's own test (crates/model/src/ops.rs:7133-7153):
    beta tanh(g / beta) sigmoid(g) * 25 tanh(u / 25) in f64, 1e-5 relative. The bound notices the mistakes a restatement
    could make: the gate scaled by the up's beta, a missing sigmoid, the +1 of another rule, the betas swapped."""
    f = np.float32
    beta, lb, n = f(8.0), 25.0, 1024
    i = np.arange(n)
    g = ((i.astype(f) - f(512.0)) * f(0.07)).astype(f)
    u = (((i * 37 % n).astype(f) - f(512.0)) * f(0.1)).astype(f)
    out, ok = ora.gate_rule(3, beta, g, u)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = 8.0 * np.tanh(g64 / 8.0) / (1.0 + np.exp(-g64)) * (lb * np.tanh(u64 / lb))
    assert ok and np.all(np.abs(out - want) <= 1e-5 * np.abs(want) + 1e-30)
    for wrong in (25.0 * np.tanh(g64 / 25.0) / (1.0 + np.exp(-g64)) * (lb * np.tanh(u64 / lb)),
                  8.0 * np.tanh(g64 / 8.0) * (lb * np.tanh(u64 / lb)),
                  lb * np.tanh(g64 / lb) / (1.0 + np.exp(-g64)) * (8.0 * np.tanh(u64 / 8.0))):
        assert not np.all(np.abs(out - wrong) <= 1e-5 * np.abs(wrong) + 1e-30)
    # op order at one value: scale by the f32 reciprocal, tanh, scale back, then (a * s) * v
    e = ora.expf_ik(f(0.0) - f(1.5))
    a = f(np.tanh(np.float64(f(f(1.5) * f(f(1.0) / beta)))))  # a correctly rounded tanh; libm's may sit an ulp away
    sg = f(f(1.0) / f(f(1.0) + e))
    v = f(np.tanh(np.float64(f(f(-3.0) * f(f(1.0) / f(25.0))))))
    one, _ = ora.gate_rule(3, beta, np.array([1.5], f), np.array([-3.0], f))
    want1 = f(f(f(a * beta) * sg) * f(v * f(25.0)))
    assert abs(float(one[0]) - float(want1)) <= 4 * np.spacing(abs(want1))
    # a value that is not finite is reported, as situ_into refuses it
    for bad in (np.nan, np.inf, -np.inf):
        assert not ora.gate_rule(3, beta, np.array([1.0, bad], f), np.array([1.0, 1.0], f))[1]
        assert not ora.gate_rule(3, beta, np.array([1.0, 1.0], f), np.array([bad, 1.0], f))[1]


# ------------------------------------------------------------------------------------------- router and combine

def test_router_softmax_topk_renorm():
    rng = np.random.default_rng(2)
    for n_experts, top_k in ((128, 8), (256, 8), (8, 2), (4, 4)):
        logits = normal_f32(rng, n_experts)
        ids, w = ora.route_softmax_topk(logits, top_k)
        p = np.exp((logits - logits.max()).astype(np.float32)).astype(np.float32)
        p = (p / np.float32(p.astype(np.float64).sum())).astype(np.float32)
        order = sorted(range(n_experts), key=lambda e: (-p[e], e))[:top_k]
        assert list(ids) == order
        chosen = p[order]
        want = chosen / np.float32(chosen.astype(np.float64).sum())
        assert np.allclose(w, want, rtol=3e-7, atol=0)
        assert abs(float(w.astype(np.float64).sum()) - 1.0) < 1e-6
        ids2, w2 = ora.route_softmax_topk(logits, top_k, renorm=False)
        assert list(ids2) == order and np.allclose(w2, chosen, rtol=3e-7, atol=0)


def test_router_ties_go_to_the_smaller_id():
    logits = np.zeros(16, np.float32)
    logits[[3, 9, 12]] = 1.0
    ids, w = ora.route_softmax_topk(logits, 4)
    assert list(ids) == [3, 9, 12, 0]
    with pytest.raises(ora.OracleError):
        ora.route_softmax_topk(logits, 17)


def test_combine_is_slot_ascending_fma_then_residual():
    rng = np.random.default_rng(3)
    rows, n_slots, m = 40, 8, 3
    down, w, resid = normal_f32(rng, m * n_slots * rows), normal_f32(rng, m * n_slots), normal_f32(rng, m * rows)
    got = ora.combine_tokens(down, w, resid, rows, n_slots, m)
    d = down.reshape(m, n_slots, rows)
    for t in range(m):
        for r in (0, 17, rows - 1):
            acc = np.float32(0.0)
            for e in range(n_slots):
                # one rounding per term: the exact product added in f64 then rounded to f32 is the fma
                acc = np.float32(np.float64(w[t * n_slots + e]) * np.float64(d[t, e, r]) + np.float64(acc))
            want = np.float32(acc + resid[t * rows + r])
            assert got[t * rows + r].tobytes() == want.tobytes()
    assert np.array_equal(ora.combine_tokens(down, w, None, rows, n_slots, m),
                          ora.combine_tokens(down, w, np.zeros(m * rows, np.float32), rows, n_slots, m))
    # with a shared expert (crates/gpu/src/moe_fused.rs:129-170): (sum + shexp) + resid, not sum + (shexp + resid)
    one = np.ones(1, np.float32)
    got = ora.moe_combine(np.array([1e8], np.float32), one, np.array([-1e8], np.float32), one, 1, 1, 1)
    assert got[0] == 1.0  # the other grouping gives 1e8 + (-1e8 + 1) = 0
    got = ora.moe_combine(np.array([3.0], np.float32), np.array([0.5], np.float32), np.array([2.0], np.float32), None, 1, 1, 1)
    assert got[0] == 3.5
    sh = normal_f32(rng, m * rows)
    full = ora.moe_combine(down, w, sh, resid, rows, n_slots, m)
    base = ora.combine_tokens(down, w, None, rows, n_slots, m)
    assert np.array_equal(full, ((base + sh).astype(np.float32) + resid).astype(np.float32))


# ---------------------------------------------------------------------------------------------- weight quantizers

def wave_row(n, seed):
    """The reference's deterministic row (crates/gguf/src/kquant/tests.rs:5-15)."""
    out = np.empty(n, np.float32)
    for i in range(n):
        h = (i * 2654435761 + seed * 40503) & 0xFFFFFFFF
        ripple = np.float32(np.float32((h >> 8) & 0xFFFF) / np.float32(65536.0) - np.float32(0.5))
        out[i] = np.float32(np.sin(np.float32(np.float32(i) * np.float32(0.013) + np.float32(seed))) * np.float32(0.7)
                            + ripple * np.float32(0.3))
    return out


@pytest.mark.parametrize("wtype,bound", ((ora.Q4_K, 0.12), (ora.Q5_K, 0.06), (ora.Q6_K, 0.02)))
def test_kquant_round_trip_bounds(wtype, bound):
    x = wave_row(512, 3)
    q = ora.quantize_rows(wtype, x, 1, 512, n_threads=1)
    assert q.size == 512 // 256 * ora.BLOCK_BYTES[wtype]
    back = ora.dequant_row(wtype, q, 512)
    assert np.abs(x - back).max() < bound
    assert not ora.quantize_rows(wtype, np.zeros(256, np.float32), 1, 256).any(), "a zero row is zero bytes"


@pytest.mark.parametrize("wtype,rel", ((ora.Q4_K, 0.09), (ora.Q5_K, 0.045), (ora.Q6_K, 0.02), (ora.IQ2_XXS, 0.55)))
def test_quantizers_on_the_benchmark_distribution(wtype, rel):
    rng = np.random.default_rng(40 + wtype)
    x = normal_f32(rng, (16, 1024), 0.02)
    q = ora.quantize_rows(wtype, x, 16, 1024, n_threads=3)
    assert np.array_equal(q, ora.quantize_rows(wtype, x, 16, 1024, n_threads=1)), "rows are independent of the split"
    rb = ora.row_bytes(wtype, 1024)
    back = np.stack([ora.dequant_row(wtype, q[r * rb:(r + 1) * rb], 1024) for r in range(16)])
    err = np.sqrt(np.mean((back - x) ** 2)) / np.sqrt(np.mean(x ** 2))
    assert err < rel, err
    cos = float((back * x).sum() / np.sqrt((back ** 2).sum() * (x ** 2).sum()))
    assert cos > (0.8 if wtype == ora.IQ2_XXS else 0.99)


def test_kquant_refuses_non_finite_and_unaligned():
    x = np.ones(256, np.float32)
    x[3] = np.nan
    for wtype in (ora.Q4_K, ora.Q5_K, ora.Q6_K):
        with pytest.raises(ora.OracleError) as e:
            ora.quantize_rows(wtype, x, 1, 256)
        assert e.value.code == ora.ENONFINITE
    with pytest.raises(ora.OracleError) as e:
        ora.quantize_rows(ora.Q4_K, np.ones(300, np.float32), 1, 300)
    assert e.value.code == ora.EUNALIGNED


def test_iq2xxs_grid_tables_are_ggml_init():
    # crates/gguf/src/iq_quant/tests.rs:44-84: first point codes, map size, lists == naive (distance, index) sort
    codes, size, neg, words = ora.iq2xxs_grid_codes()
    assert size == 43692
    first8 = []
    for g in range(8):
        c = int(codes[g])
        first8.append(sum(((c >> (2 * k)) & 3) << (2 * k) for k in range(8)))
    assert first8 == [0, 2, 5, 8, 10, 17, 20, 32]
    assert neg == 43692 - 256
    assert len(set(int(c) for c in codes)) == 256


def test_iq2xxs_rows_quantize_and_read_back():
    # the reference's LCG row of few distinct levels with positive importance (crates/gguf/src/iq_quant/tests.rs:92-140)
    s = [7]

    def nxt():
        s[0] = (s[0] * 1103515245 + 12345) & 0xFFFFFFFF
        return s[0] >> 8

    levels = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    n = 4 * 256
    x = np.empty(n, np.float32)
    for i in range(n):
        r = nxt()
        v = np.float32(levels[r % 8]) * np.float32(0.01)
        x[i] = -v if r & 256 else v
    w = np.array([np.float32(0.1) + np.float32(nxt() % 1000) / np.float32(100.0) for _ in range(n)], np.float32)
    q = ora.quantize_row_iq2xxs(x, w)
    assert q.size == n // 256 * 66
    assert np.array_equal(q, ora.quantize_row_iq2xxs(x, w))
    y = ora.dequant_row(ora.IQ2_XXS, q, n).astype(np.float64)
    cos = float((x * y).sum() / np.sqrt((x.astype(np.float64) ** 2).sum() * (y ** 2).sum()))
    assert cos > 0.8, cos
    assert not ora.quantize_row_iq2xxs(np.zeros(256, np.float32), np.ones(256, np.float32)).any()


# ----------------------------------------------------------------------------------------------------- the layer

def small_layer(types, hidden, ff, n_experts, seed):
    rng = np.random.default_rng(seed)

    def rows(wtype, n, k):
        x = normal_f32(rng, (n, k), 0.02)
        return iq4xs_rows(x) if wtype == ora.IQ4_XS else ora.quantize_rows(wtype, x, n, k)

    return rows(types[0], n_experts * ff, hidden), rows(types[1], n_experts * ff, hidden), rows(types[2], n_experts * hidden, ff)


@pytest.mark.parametrize("types,hidden,ff", (((ora.Q4_K, ora.Q4_K, ora.Q6_K), 512, 256),
                                             ((ora.IQ2_XXS, ora.IQ2_XXS, ora.IQ2_XXS), 512, 256),
                                             ((ora.IQ4_XS, ora.IQ4_XS, ora.Q5_K), 512, 256)))
def test_layer_forms_agree_and_track_f64(types, hidden, ff):
    n_experts, top_k, m = 6, 3, 4
    wg, wu, wd = small_layer(types, hidden, ff, n_experts, 77)
    rng = np.random.default_rng(78)
    x = normal_f32(rng, (m, hidden))
    ids = np.empty((m, top_k), np.uint32)
    wts = np.empty((m, top_k), np.float32)
    for t in range(m):
        ids[t], wts[t] = ora.route_softmax_topk(normal_f32(rng, n_experts), top_k)
    y1, h1 = ora.moe_forward(hidden, ff, n_experts, types, wg, wu, wd, x, ids, wts, top_k, n_threads=1, want_h=True)
    y3 = ora.moe_forward(hidden, ff, n_experts, types, wg, wu, wd, x, ids, wts, top_k, n_threads=3)
    assert y1.tobytes() == y3.tobytes(), "the row split never changes a value"
    pool = ora.lib.ora_pool_create(3)
    try:
        y2, h2 = ora.moe_forward(hidden, ff, n_experts, types, wg, wu, wd, x, ids, wts, top_k, want_h=True,
                                 avx2_pool=pool)
    finally:
        ora.lib.ora_pool_destroy(pool)
    assert h1.tobytes() == h2.tobytes() and y1.tobytes() == y2.tobytes(), "AVX2 grouped form == scalar form"
    # against f64 on the dequantized weights and the raw activations: quantization error only
    rbg, rbd = ora.row_bytes(types[0], hidden), ora.row_bytes(types[2], ff)
    want = np.zeros((m, hidden))
    for t in range(m):
        for s in range(top_k):
            e = int(ids[t, s])
            G = np.stack([ora.dequant_row(types[0], wg[(e * ff + r) * rbg:(e * ff + r + 1) * rbg], hidden)
                          for r in range(ff)]).astype(np.float64)
            U = np.stack([ora.dequant_row(types[1], wu[(e * ff + r) * rbg:(e * ff + r + 1) * rbg], hidden)
                          for r in range(ff)]).astype(np.float64)
            D = np.stack([ora.dequant_row(types[2], wd[(e * hidden + r) * rbd:(e * hidden + r + 1) * rbd], ff)
                          for r in range(hidden)]).astype(np.float64)
            g, u = G @ x[t].astype(np.float64), U @ x[t].astype(np.float64)
            want[t] += float(wts[t, s]) * (D @ (g / (1.0 + np.exp(-g)) * u))
    assert max_abs_normalised(y1, want.reshape(-1)) < 0.05


def test_layer_refuses_bad_ids():
    types = (ora.Q4_K, ora.Q4_K, ora.Q6_K)
    wg, wu, wd = small_layer(types, 256, 256, 2, 5)
    x = np.ones(256, np.float32)
    with pytest.raises(ora.OracleError):
        ora.moe_forward(256, 256, 2, types, wg, wu, wd, x, np.array([2], np.uint32), np.array([1.0], np.float32), 1)


def test_grouped_table_by_hand():
    """The slot table and tile words of crates/gpu/src/q4k_sel.rs:20-41,562-680 on cases small enough to write out."""
    order, start, tiles, refused = ora.grouped_table([2, 0, 2, 1, 2], 3)
    assert list(order) == [1, 3, 0, 2, 4] and list(start) == [0, 1, 2, 5] and not refused
    assert list(tiles[:4]) == [3, (0 << 22) | 0, (1 << 22) | 1, (2 << 22) | 2]
    # a run of nine entries cuts into a tile of eight and a tile of one; the host's slot and a stale id join no run
    sel = [1] * 9 + [0xFFFFFFFF, 7]
    order, start, tiles, refused = ora.grouped_table(sel, 2)
    assert list(start) == [0, 0, 9] and list(order[:9]) == list(range(9)) and refused
    assert list(tiles[:3]) == [2, (1 << 22) | 0, (1 << 22) | 8]
    assert ora.tile_cap(11, 2) == 3 and ora.tile_cap(128, 128) == 128 and ora.tile_cap(16384, 128) == 2160


def test_gemm_route_by_hand():
    """crates/gpu/src/gemm/route.rs: grouped by expert, ascending inside, tiles of at most 64, refused slots last."""
    cols, tiles, refused = ora.gemm_route([1, 0, 5, 1, 1, 0], 3)
    assert list(cols) == [1, 5, 0, 3, 4, 2] and refused == 1
    assert tiles.tolist() == [[0, 0, 2], [1, 2, 3]]
    cols, tiles, refused = ora.gemm_route([2] * 130, 3)
    assert tiles.tolist() == [[2, 0, 64], [2, 64, 64], [2, 128, 2]] and refused == 0


# ------------------------------------------------------------------------- the norm and the router's logits

def fma32(a, b, c):
    """a * b + c rounded once to f32, exactly: the sum as a fraction, then the nearest of the f32 values around it
    (ties to the even mantissa)."""
    from fractions import Fraction
    r = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
    near = np.float32(float(r))
    best = None
    for cand in (np.nextafter(near, np.float32(-np.inf)), near, np.nextafter(near, np.float32(np.inf))):
        dist = abs(Fraction(float(cand)) - r)
        even = (int(np.float32(cand).view(np.uint32)) & 1) == 0
        if best is None or dist < best[0] or (dist == best[0] and even and not best[2]):
            best = (dist, cand, even)
    return np.float32(best[1])


def test_sum_of_squares_narrows_to_the_sequential_sum():
    # crates/qdot/tests/qdot.rs:4438-4455: the laned f64 sum against the left-to-right one, on its generator
    for n in (8, 512, 2048, 2048 + 5):
        x = ((np.arange(n) * 37 % 2001).astype(np.float32) - np.float32(1000.0)) * np.float32(0.0137)
        seq = 0.0
        for v in x:
            seq += float(np.float32(v * v))
        got = ora.sum_sq_f64(x)
        assert abs((got - seq) / seq) < 1e-14
        assert np.float32(got / n).tobytes() == np.float32(seq / n).tobytes()


def test_f32_row_dot_is_the_eight_lane_order():
    # crates/qdot/tests/qdot.rs:4460-4485, on its generators; the lanes re-derived with an exact fused multiply-add
    k = 2048
    w = ((np.arange(k) * 37 % 2001).astype(np.float32) - np.float32(1000.0)) * np.float32(0.0013)
    x = ((np.arange(k) * 91 % 1777).astype(np.float32) - np.float32(888.0)) * np.float32(0.0071)
    lane = [np.float32(x[l] * w[l]) for l in range(8)]
    for i in range(1, k // 8):
        for l in range(8):
            lane[l] = fma32(x[8 * i + l], w[8 * i + l], lane[l])
    s = [np.float32(lane[l] + lane[l + 4]) for l in range(4)]
    want = np.float32(np.float32(s[0] + s[2]) + np.float32(s[1] + s[3]))
    assert ora.dot_f32(w, x).tobytes() == want.tobytes()
    with pytest.raises(ora.OracleError) as e:
        ora.dot_f32(w[:12], x[:12])  # a width the lanes cannot take is the caller's
    assert e.value.code == ora.EUNALIGNED


def test_rms_norm_is_the_stated_formula():
    # crates/model/src/ops.rs:350-368: mean of squares narrowed to f32, eps inside the root, (scale * gain) * x
    rng = np.random.default_rng(91)
    for n, eps in ((256, 1e-6), (2048, 1e-5), (7168, 1e-6)):
        x, gain = normal_f32(rng, n, 3.0), normal_f32(rng, n, 1.0)
        mean = np.float32(np.sum(np.float32(x * x).astype(np.float64)) / n)
        scale = np.float32(1.0) / np.sqrt(np.float32(mean + np.float32(eps)), dtype=np.float32)
        want = (np.float32(scale) * gain).astype(np.float32) * x
        assert ora.rms_norm(x, gain, eps).tobytes() == want.astype(np.float32).tobytes()
    router = normal_f32(rng, (5, 64), 0.1)
    xs = normal_f32(rng, (3, 64))
    gain = normal_f32(rng, 64)
    normed, logits = ora.router_logits(router, xs, gain, 1e-6)
    for t in range(3):
        assert normed[t].tobytes() == ora.rms_norm(xs[t], gain, 1e-6).tobytes()
        assert [ora.dot_f32(router[e], normed[t]).tobytes() for e in range(5)] == [logits[t, e].tobytes() for e in range(5)]
    plain, logits0 = ora.router_logits(router, xs)
    assert plain.tobytes() == xs.tobytes() and logits0[1, 2] == ora.dot_f32(router[2], xs[1])
