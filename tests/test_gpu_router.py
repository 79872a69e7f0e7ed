"""GPU parity tests of the softmax router (bm_route_softmax) through the C ABI, against the CPU oracle's restatement
of the CPU path's router (crates/model/src/moe.rs:246-279) on the same seeded logits: ids exactly; weights and
probabilities within two units in the last place and bit for bit in all but a few per thousand (the CPU path's exp is
the host library's expf, the kernel's the f64 exp rounded to f32: each the correctly rounded value in all but rare
cases, and not the same rare cases; the stated tolerance of the path is 1e-4). Clauses follow the reference's router tests
(crates/gpu/src/route_softmax.rs:2035-2110): the rule's picks, ties toward the smaller id, a token with a logit that
is not finite."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora
from common import normal_f32
from test_gpu_decode import Layer, assert_f32, gpu  # noqa: F401  (gpu is the module fixture)

pytestmark = pytest.mark.gpu


def assert_ulp(got, want, what, ulps=2, odd_share=0.005):
    got, want = np.asarray(got, np.float32).ravel(), np.asarray(want, np.float32).ravel()
    assert np.isfinite(got).all(), what
    d = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))  # positive floats: ordered bits
    assert d.max() <= ulps, f"{what}: {int(d.max())} units in the last place apart"
    assert np.count_nonzero(d) <= max(1, int(odd_share * d.size)), f"{what}: {np.count_nonzero(d)} of {d.size} differ in bits"


def run_router(gpu, logits, top_k, renorm=True, want_probs=True):
    m, n_experts = logits.shape
    ld = gpu.upload(logits, np.float32)
    probs = gpu.buffer(np.float32, m * n_experts).fill_bytes(0xFF) if want_probs else None
    ids = gpu.buffer(np.uint32, m * top_k).fill_bytes(0xEE)
    wts = gpu.buffer(np.float32, m * top_k).fill_bytes(0xFF)
    gpu.enqueue_route_softmax(ld, m, n_experts, top_k, renorm, probs, ids, wts)
    out = (ids.download().reshape(m, top_k), wts.download().reshape(m, top_k),
           probs.download().reshape(m, n_experts) if want_probs else None)
    for b in (ld, probs, ids, wts):
        if b is not None:
            b.free()
    return out


def oracle_probs(logits):
    """The CPU path's softmax row: exp(l - max) in f32 (the host library's expf, as the oracle's C uses), the sum in
    f64 in expert order, one f32 divide."""
    one = ora.route_softmax_topk  # the top-1 weight without renormalising is the largest probability: pins the divide
    e = np.empty_like(logits)
    for t, row in enumerate(logits):
        # every probability through the oracle: route with top_k = n_experts, no renorm, then scatter by id
        ids, w = one(row, row.size, renorm=False)
        e[t, ids] = w
    return e


@pytest.mark.parametrize("n_experts,top_k,m,seed,renorm", ((128, 8, 512, 1, True), (256, 8, 64, 2, True), (100, 4, 33, 3, True),
                                                           (128, 8, 16, 4, False), (1024, 32, 8, 5, True), (5, 5, 7, 6, True),
                                                           (64, 1, 9, 7, True)))
def test_router_is_the_cpu_paths(gpu, n_experts, top_k, m, seed, renorm):
    rng = np.random.default_rng(seed)
    logits = np.stack([normal_f32(rng, n_experts) * np.float32(1 + (t % 5)) for t in range(m)])
    gpu.fault_clear()
    ids, wts, probs = run_router(gpu, logits, top_k, renorm)
    want_all = np.empty_like(wts)
    for t in range(m):
        want_ids, want_all[t] = ora.route_softmax_topk(logits[t], top_k, renorm=renorm)
        assert np.array_equal(ids[t], want_ids), t
    assert_ulp(wts, want_all, "weights")
    if n_experts <= 256:
        assert_ulp(probs, oracle_probs(logits), "probabilities")
    assert gpu.fault() == (bm.FAULT_NONE, 0)


def test_router_ties_go_to_the_smaller_id(gpu):
    logits = np.zeros((3, 128), np.float32)
    logits[1, [5, 77, 100]] = 2.0          # three equal winners, then equal losers
    logits[2] = np.float32(-3.5)
    logits[2, 127] = np.float32(-3.0)
    ids, wts, _ = run_router(gpu, logits, 4, want_probs=False)
    assert ids[0].tolist() == [0, 1, 2, 3]
    assert ids[1].tolist() == [5, 77, 100, 0]
    assert ids[2].tolist() == [127, 0, 1, 2]
    for t in range(3):
        want_ids, want_w = ora.route_softmax_topk(logits[t], 4)
        assert np.array_equal(ids[t], want_ids)
        assert_ulp(wts[t], want_w, f"weights of token {t}", odd_share=1.0)


@pytest.mark.parametrize("poison", (np.nan, np.inf, -np.inf))
def test_router_raises_on_a_logit_that_is_not_finite(gpu, poison):
    rng = np.random.default_rng(11)
    logits = np.stack([normal_f32(rng, 128) for _ in range(6)])
    logits[4, 93] = poison
    gpu.fault_clear()
    gpu.set_layer(3)
    ids, wts, probs = run_router(gpu, logits, 8)
    gpu.set_layer(0)
    w0, mask = gpu.fault(3)
    assert w0 == (3 << 8) + bm.SITE_ROUTER and mask == 1 << bm.SITE_ROUTER
    assert np.isnan(wts[4]).all() and np.isnan(probs[4]).all()
    assert (ids[4] == 0xEEEEEEEE).all()  # left as they stood
    for t in (0, 1, 2, 3, 5):
        want_ids, want_w = ora.route_softmax_topk(logits[t], 8)
        assert np.array_equal(ids[t], want_ids)
        assert_ulp(wts[t], want_w, f"weights of token {t}", odd_share=1.0)
    gpu.fault_clear()


def test_router_feeds_the_decode_step(gpu):
    """logits -> bm_route_softmax -> bm_moe_decode, ids and weights never leaving the device: the oracle's layer."""
    rng = np.random.default_rng(21)
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 512, 256, 16, 22)
    m, top_k = 3, 4
    x = np.stack([normal_f32(rng, L.hidden) for _ in range(m)])
    logits = np.stack([normal_f32(rng, L.n_experts) for _ in range(m)])
    ld, xd = gpu.upload(logits, np.float32), gpu.upload(x, np.float32)
    sel, wts = gpu.buffer(np.uint32, m * top_k), gpu.buffer(np.float32, m * top_k)
    act_h = gpu.act(L.types[2], L.ff, m * top_k)
    y = gpu.buffer(np.float32, m * L.hidden).fill_bytes(0xFF)
    gpu.enqueue_route_softmax(ld, m, L.n_experts, top_k, True, None, sel, wts)
    gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wts, None, top_k, m, act_h, y)
    got = y.download().reshape(m, L.hidden)
    routes = [ora.route_softmax_topk(logits[t], top_k) for t in range(m)]
    ids = np.stack([r[0] for r in routes])
    w = np.stack([r[1] for r in routes])
    want_y, _ = L.oracle(x, ids, w, top_k)
    assert (sel.download().reshape(m, top_k) == ids).all()
    err = np.max(np.abs(got.astype(np.float64) - np.asarray(want_y).reshape(m, L.hidden))) / np.max(np.abs(want_y))
    assert err <= 1e-6, err  # the weights may differ in their last place, nothing else does
    for b in (ld, xd, sel, wts, act_h, y):
        b.free()
    L.free()


def test_router_refusals_are_named(gpu):
    buf = gpu.buffer(np.float32, 4096)
    ids = gpu.buffer(np.uint32, 64)
    for args, word in (((1, 2048, 8), "n_experts"), ((1, 128, 33), "top_k"), ((1, 4, 5), "top_k"), ((0, 128, 8), "n_tokens")):
        with pytest.raises(bm.GpuError) as e:
            gpu.enqueue_route_softmax(buf, args[0], args[1], args[2], True, None, ids, buf)
        assert e.value.code == bm.ESHAPE and word in str(e.value) and "bm_route_softmax" in str(e.value)
    buf.free()
    ids.free()


# ------------------------------------------------------------------------- the norm and the router's logits

@pytest.mark.parametrize("n_experts,hidden,m,with_gain,seed", ((128, 2048, 5, True, 11), (256, 7168, 2, True, 12),
                                                               (128, 2048, 3, False, 13), (10, 64, 4, True, 14),
                                                               (7, 16384, 1, True, 15), (3, 64, 2000, True, 16)))
def test_router_logits_are_the_cpu_paths(gpu, n_experts, hidden, m, with_gain, seed):
    """bm_router_logits: the normed rows and the f32 logits bit for bit against the oracle's restatement of the CPU
    path's norm (crates/model/src/ops.rs:350-368) and eight-lane f32 row dot (crates/qdot/src/lib.rs:11349-11386).
    Shapes: the two benchmark layers', rows that are not a whole number of a workgroup's four, a row so long that a
    workgroup takes one router row at a time, and two thousand short rows for as many square roots (the hardware's is
    not the correctly rounded one)."""
    rng = np.random.default_rng(seed)
    router = normal_f32(rng, (n_experts, hidden), 0.05)
    x = np.stack([normal_f32(rng, hidden) * np.float32(10.0 ** rng.uniform(-2, 2)) for _ in range(m)])
    gain = (1.0 + normal_f32(rng, hidden, 0.2)).astype(np.float32) if with_gain else None
    eps = 1e-6
    rd, xd = gpu.upload(router, np.float32), gpu.upload(x, np.float32)
    gd = gpu.upload(gain, np.float32) if with_gain else None
    normed = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    logits = gpu.buffer(np.float32, m * n_experts).fill_bytes(0xFF)
    gpu.enqueue_router_logits(rd, xd, gd, eps, m, n_experts, hidden, normed, logits)
    want_n, want_l = ora.router_logits(router, x, gain, eps)
    assert_f32(normed.download(), want_n.reshape(-1), "normed rows")
    assert_f32(logits.download(), want_l.reshape(-1), "logits")
    # without the normed rows the logits are the same
    logits.fill_bytes(0xFF)
    gpu.enqueue_router_logits(rd, xd, gd, eps, m, n_experts, hidden, None, logits)
    assert np.array_equal(logits.download().view(np.uint32), want_l.reshape(-1).view(np.uint32))
    for b in (rd, xd, gd, normed, logits):
        if b is not None:
            b.free()


def test_layer_from_the_residual_row(gpu):
    """The layer from its input residual rows: norm and logits, routing, then the fused expert step on the normed rows,
    four launches, nothing through the host. The ids are the oracle's; with the kernel's own weights (within two units
    in the last place of the oracle's, see above) the layer's output is the oracle's bit for bit."""
    hidden, ff, n_experts, top_k, m = 2048, 768, 16, 4, 6
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), hidden, ff, n_experts, 4400)
    rng = np.random.default_rng(4401)
    router = normal_f32(rng, (n_experts, hidden), 0.05)
    gain = (1.0 + normal_f32(rng, hidden, 0.1)).astype(np.float32)
    x = normal_f32(rng, (m, hidden), 2.0)
    rd, xd, gd = gpu.upload(router, np.float32), gpu.upload(x, np.float32), gpu.upload(gain, np.float32)
    normed, logits = gpu.buffer(np.float32, m * hidden), gpu.buffer(np.float32, m * n_experts)
    ids, wts = gpu.buffer(np.uint32, m * top_k), gpu.buffer(np.float32, m * top_k)
    act_h, y = gpu.act(bm.Q6_K, ff, m * top_k), gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    gpu.fault_clear()
    gpu.enqueue_router_logits(rd, xd, gd, 1e-6, m, n_experts, hidden, normed, logits)
    gpu.enqueue_route_softmax(logits, m, n_experts, top_k, True, None, ids, wts)
    gpu.enqueue_moe_decode(L.dg, L.du, L.dd, normed, ids, wts, xd, top_k, m, act_h, y)   # the residual: the input rows
    want_n, want_l = ora.router_logits(router, x, gain, 1e-6)
    got_ids, got_w = ids.download().reshape(m, top_k), wts.download().reshape(m, top_k)
    for t in range(m):
        want_ids, want_w = ora.route_softmax_topk(want_l[t], top_k)
        assert list(got_ids[t]) == list(want_ids)
        assert_ulp(got_w[t], want_w, f"weights of token {t}", odd_share=1.0)
    want_y, _ = L.oracle(want_n, got_ids, got_w, top_k)
    assert_f32(y.download(), (want_y.reshape(m, hidden) + x).astype(np.float32).reshape(-1), "y + residual")
    # the same layer as three launches: the router launch leaves the quantized columns (with the tables the dots read), gate . up
    # takes them, down + combine closes
    act_x, y3 = gpu.act(bm.Q4_K, hidden, m), gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    ids3, wts3 = gpu.buffer(np.uint32, m * top_k), gpu.buffer(np.float32, m * top_k)
    gpu.enqueue_norm_route(rd, xd, gd, 1e-6, m, n_experts, hidden, top_k, True, None, logits, None, ids3, wts3, act_x=act_x)
    gpu.enqueue_gate_up(L.dg, L.du, act_x, ids3, m * top_k, ff, top_k, None, act_h)
    gpu.enqueue_down_combine(L.dd, act_h, ids3, wts3, xd, top_k, m, hidden, y3)
    assert np.array_equal(y3.download().view(np.uint32), y.download().view(np.uint32)), "three launches against four"
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (rd, xd, gd, normed, logits, ids, wts, act_h, y, act_x, y3, ids3, wts3):
        b.free()
    L.free()


@pytest.mark.parametrize("n_experts,hidden,m,top_k,with_gain,seed", ((128, 2048, 5, 8, True, 21), (256, 7168, 3, 8, True, 22),
                                                                      (10, 64, 70, 3, False, 23), (600, 256, 9, 6, True, 24),
                                                                      (7, 16384, 2, 2, True, 25), (3, 64, 4096, 1, True, 26)))
def test_norm_route_is_the_two_launches_in_one(gpu, n_experts, hidden, m, top_k, with_gain, seed):
    """bm_norm_route against bm_router_logits followed by bm_route_softmax on the same inputs: every output the same bits
    (normed rows, logits, probabilities, ids, weights), three launches in a row over the same hand-over words and then a
    smaller one, and under a graph replayed several times (the routing waves arm their words again without a memset)."""
    rng = np.random.default_rng(seed)
    router = normal_f32(rng, (n_experts, hidden), 0.05)
    x = np.stack([normal_f32(rng, hidden) * np.float32(10.0 ** rng.uniform(-1, 1)) for _ in range(m)])
    gain = (1.0 + normal_f32(rng, hidden, 0.2)).astype(np.float32) if with_gain else None
    eps = 1e-6
    rd, xd = gpu.upload(router, np.float32), gpu.upload(x, np.float32)
    gd = gpu.upload(gain, np.float32) if with_gain else None
    bufs = {}
    for tag in ("two", "one"):
        bufs[tag] = (gpu.buffer(np.float32, m * hidden), gpu.buffer(np.float32, m * n_experts), gpu.buffer(np.float32, m * n_experts),
                     gpu.buffer(np.uint32, m * top_k), gpu.buffer(np.float32, m * top_k))
    normed, logits, probs, ids, wts = bufs["two"]
    gpu.fault_clear()
    gpu.enqueue_router_logits(rd, xd, gd, eps, m, n_experts, hidden, normed, logits)
    gpu.enqueue_route_softmax(logits, m, n_experts, top_k, True, probs, ids, wts)
    want = [b.download() for b in bufs["two"]]
    normed, logits, probs, ids, wts = bufs["one"]

    # where the rows are whole super-blocks the launch also leaves the quantized columns, in either column form
    acts = [gpu.act(wt, hidden, m) for wt in (bm.Q4_K, bm.IQ2_XXS)] if hidden % 256 == 0 else [None]
    which = [0]

    def fused(tokens):
        gpu.enqueue_norm_route(rd, xd, gd, eps, tokens, n_experts, hidden, top_k, True, normed, logits, probs, ids, wts,
                               act_x=acts[which[0] % len(acts)])
        which[0] += 1

    def check(tokens, what):
        for b, w, per, name in zip(bufs["one"], want, (hidden, n_experts, n_experts, top_k, top_k),
                                   ("normed", "logits", "probs", "ids", "weights")):
            got = b.download()
            assert np.array_equal(got[:tokens * per].view(np.uint32), w[:tokens * per].view(np.uint32)), f"{what}: {name}"

    for rep in range(3):
        for b in bufs["one"]:
            b.fill_bytes(0xFF)
        fused(m)
        check(m, f"launch {rep}")
    if acts[0] is not None:  # the columns are the CPU path's bytes of the normed rows, and what bm_quantize makes of them
        normed_rows = want[0].reshape(m, hidden)
        for act, wt in zip(acts, (bm.Q4_K, bm.IQ2_XXS)):
            ref = gpu.act(wt, hidden, m)
            gpu.enqueue_quantize(bufs["two"][0], m, ref)
            for t in (0, m // 2, m - 1):
                col = act.download(t)
                assert np.array_equal(col, ora.quantize_col(wt, normed_rows[t])), f"act_x column {t}, type {wt}"
                assert np.array_equal(col, ref.download(t))
            ref.free()
    few = max(1, m // 2)
    for b in bufs["one"]:
        b.fill_bytes(0xFF)
    fused(few)
    check(few, "a smaller launch after a larger one")
    gpu.capture_begin()
    fused(m)
    g = gpu.capture_end()
    for rep in range(3):
        for b in bufs["one"]:
            b.fill_bytes(0xFF)
        gpu.graph_launch(g)
        gpu.sync()
        check(m, f"replay {rep}")
    gpu.graph_destroy(g)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (rd, xd, gd) + bufs["two"] + bufs["one"] + tuple(acts):
        if b is not None:
            b.free()


@pytest.mark.parametrize("n_experts,top_k", ((128, 8), (200, 6), (40, 4), (300, 8)))
def test_norm_route_picks_among_equal_probabilities(gpu, n_experts, top_k):
    """Router rows that repeat give logits that are equal bit for bit: the fused launch's picks (by counting, for up to 256
    experts, with the wave's rounds behind it when two entries tie) go to the smaller id as the two launches' and the
    oracle's do: a token whose winners tie, one whose ties lie past the picks, one whose row is zero (every expert ties),
    one without ties."""
    hidden, m = 256, 4
    rng = np.random.default_rng(4100 + n_experts)
    router = normal_f32(rng, (n_experts, hidden), 0.05)
    x = normal_f32(rng, (m, hidden))
    x[2] = 0.0
    l0 = ora.router_logits(router, x[:1], None, 0.0)[1][0]
    order = np.argsort(-l0, kind="stable")
    router[order[1]] = router[order[0]]            # token 0's two best tie (and every token's at those two ids)
    router[order[-1]] = router[order[-2]]          # and two of its worst
    rd, xd = gpu.upload(router, np.float32), gpu.upload(x, np.float32)
    out = {}
    for tag in ("two", "one"):
        out[tag] = (gpu.buffer(np.float32, m * n_experts), gpu.buffer(np.float32, m * n_experts), gpu.buffer(np.uint32, m * top_k).fill_bytes(0xFF),
                    gpu.buffer(np.float32, m * top_k))
    gpu.fault_clear()
    logits, probs, ids, wts = out["two"]
    gpu.enqueue_router_logits(rd, xd, None, 0.0, m, n_experts, hidden, None, logits)
    gpu.enqueue_route_softmax(logits, m, n_experts, top_k, True, probs, ids, wts)
    logits, probs, ids, wts = out["one"]
    for rep in range(2):
        gpu.enqueue_norm_route(rd, xd, None, 0.0, m, n_experts, hidden, top_k, True, None, logits, probs, ids, wts)
        for a, b, name in zip(out["one"], out["two"], ("logits", "probs", "ids", "weights")):
            assert np.array_equal(a.download().view(np.uint32), b.download().view(np.uint32)), f"call {rep}: {name}"
    got_l, got_ids = logits.download().reshape(m, n_experts), ids.download().reshape(m, top_k)
    assert got_l[0, order[0]] == got_l[0, order[1]] and sorted(got_ids[0, :2]) == sorted(order[:2]) and got_ids[0, 0] < got_ids[0, 1]
    assert got_ids[2].tolist() == list(range(top_k))
    for t in range(m):
        want_ids, _ = ora.route_softmax_topk(got_l[t], top_k)
        assert np.array_equal(got_ids[t], want_ids), f"token {t}"
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (rd, xd) + out["two"] + out["one"]:
        b.free()


def test_norm_route_gives_a_token_up_when_its_logits_do_not_come(gpu, monkeypatch):
    """The routing wave's wait is bounded: a context made with BM_NORM_ROUTE_POLLS=1 lets it look once, right after the
    launch started, when no logit of a single token's launch can be there yet; it then raises Router, leaves NaN weights,
    and every workgroup ends (the call returns, the context stays usable); bm_fault_clear arms the words again, and the
    module's own context, made without the variable, routes the same token."""
    n_experts, hidden, top_k = 128, 2048, 8
    rng = np.random.default_rng(77)
    router, x = normal_f32(rng, (n_experts, hidden), 0.05), normal_f32(rng, (1, hidden))
    monkeypatch.setenv("BM_NORM_ROUTE_POLLS", "1")
    hasty = bm.Gpu(0)
    monkeypatch.delenv("BM_NORM_ROUTE_POLLS")
    try:
        rd, xd = hasty.upload(router, np.float32), hasty.upload(x, np.float32)
        logits, ids, wts = hasty.buffer(np.float32, n_experts), hasty.buffer(np.uint32, top_k).fill_bytes(0), hasty.buffer(np.float32, top_k)
        for rep in range(2):
            hasty.fault_clear()
            wts.fill_bytes(0)
            hasty.enqueue_norm_route(rd, xd, None, 0.0, 1, n_experts, hidden, top_k, True, None, logits, None, ids, wts)
            assert hasty.fault()[1] == 1 << bm.SITE_ROUTER, f"call {rep}"
            assert np.isnan(wts.download()).all(), f"call {rep}"
            # the logits themselves are written whatever became of the routing
            assert np.array_equal(logits.download().view(np.uint32), ora.router_logits(router, x, None, 0.0)[1][0].view(np.uint32))
        hasty.fault_clear()
        for b in (rd, xd, logits, ids, wts):
            b.free()
    finally:
        hasty.close()
    rd, xd = gpu.upload(router, np.float32), gpu.upload(x, np.float32)
    logits, ids, wts = gpu.buffer(np.float32, n_experts), gpu.buffer(np.uint32, top_k), gpu.buffer(np.float32, top_k)
    gpu.fault_clear()
    gpu.enqueue_norm_route(rd, xd, None, 0.0, 1, n_experts, hidden, top_k, True, None, logits, None, ids, wts)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    want_ids, _ = ora.route_softmax_topk(logits.download(), top_k)
    assert np.array_equal(ids.download(), want_ids)
    for b in (rd, xd, logits, ids, wts):
        b.free()


def test_norm_route_raises_and_refuses_like_its_parts(gpu):
    """A logit that is not finite (a NaN in the token's row) raises Router from the fused launch too, and the other
    tokens are routed; the argument checks are the two entries' own, by name."""
    n_experts, hidden, m, top_k = 16, 256, 3, 4
    rng = np.random.default_rng(31)
    router, x = normal_f32(rng, (n_experts, hidden), 0.05), normal_f32(rng, (m, hidden))
    x[1, 7] = np.nan
    rd, xd = gpu.upload(router, np.float32), gpu.upload(x, np.float32)
    logits, ids, wts = gpu.buffer(np.float32, m * n_experts), gpu.buffer(np.uint32, m * top_k).fill_bytes(0), gpu.buffer(np.float32, m * top_k)
    gpu.fault_clear()
    gpu.set_layer(3)
    gpu.enqueue_norm_route(rd, xd, None, 0.0, m, n_experts, hidden, top_k, True, None, logits, None, ids, wts)
    assert gpu.fault(3) == ((3 << 8) | bm.SITE_ROUTER, 1 << bm.SITE_ROUTER)
    got_w = wts.download().reshape(m, top_k)
    assert np.isnan(got_w[1]).all() and np.isfinite(got_w[0]).all() and np.isfinite(got_w[2]).all()
    _, want_l = ora.router_logits(router, x, None, 0.0)
    for t in (0, 2):
        want_ids, _ = ora.route_softmax_topk(want_l[t], top_k)
        assert list(ids.download().reshape(m, top_k)[t]) == list(want_ids)
    gpu.set_layer(bm.LAYER_NONE)
    gpu.fault_clear()
    for call, word in ((lambda: gpu.enqueue_norm_route(rd, xd, None, 0.0, 4097, n_experts, hidden, top_k, True, None, logits, None, ids, wts), "4096"),
                       (lambda: gpu.enqueue_norm_route(rd, xd, None, 0.0, m, n_experts, hidden, 17, True, None, logits, None, ids, wts), "top_k"),
                       (lambda: gpu.enqueue_norm_route(rd, xd, None, 0.0, m, n_experts, 12, top_k, True, None, logits, None, ids, wts), "multiple of 8")):
        with pytest.raises(bm.GpuError) as e:
            call()
        assert e.value.code == bm.ESHAPE and word in str(e.value) and "bm_norm_route" in str(e.value)
    for b in (rd, xd, logits, ids, wts):
        b.free()
