"""GPU parity tests of the decode path, through the C ABI, against the CPU oracle on the same seeded inputs.

Bars: activation bytes bit-exact; per-block integer sums bit-exact; fp32 outputs within 1e-4 (max-abs normalised)
as the task states, and bit-exact where the kernels keep the reference's operation order (they do: every value
here is compared bit for bit as well, and a difference is reported with both numbers).
Mirrors the reference's gates: gate_q4k_sel (slot == one-expert gemv, duplicate ids, bad ids, HOST), gate_kquant,
gate_iq_sel, gate_moe_fused (crates/gpu-gates/src/bin/)."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora
from common import Lcg, iq4xs_rows, max_abs_normalised, normal_f32, q3k_rows

pytestmark = pytest.mark.gpu

TYPES = (bm.Q3_K, bm.Q4_K, bm.Q5_K, bm.Q6_K, bm.IQ2_XXS, bm.IQ3_XXS, bm.IQ4_XS)
Q8K_TYPES = (bm.Q3_K, bm.IQ2_XXS, bm.IQ3_XXS, bm.IQ4_XS)  # their activation columns are Q8_K, the others' Q8_2_X4
TIES = np.array([0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, -3.5, 0.25, 7.5, -7.5, 63.5, -63.5, 120.5, -120.5,
                 0.0, -0.0, 127.0, -127.0], np.float32)


@pytest.fixture(scope="module")
def gpu():
    g = bm.Gpu(0)
    yield g
    g.close()


def assert_f32(got, want, what):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    err = max_abs_normalised(got, want)
    assert err <= 1e-4, f"{what}: max-abs normalised error {err}"
    same = got.view(np.uint32) == want.view(np.uint32)
    assert same.all(), f"{what}: {np.count_nonzero(~same)} of {same.size} values differ in bits (err {err}); " \
                       f"first at {int(np.argmin(same))}: {got[np.argmin(same)]!r} vs {want[np.argmin(same)]!r}"


def random_blocks(wtype, rows, k, rng):
    """Raw random block bytes with sane f16 scales: every code pattern is a legal block."""
    bb = ora.BLOCK_BYTES[wtype]
    nb = k // 256
    w = rng.integers(0, 256, rows * nb * bb, dtype=np.uint8).reshape(rows * nb, bb)
    off = {ora.Q3_K: 108, ora.Q4_K: 0, ora.Q5_K: 0, ora.Q6_K: 208, ora.IQ2_XXS: 0, ora.IQ3_XXS: 0, ora.IQ4_XS: 0}[wtype]
    d = rng.uniform(-0.05, 0.05, rows * nb).astype(np.float16).view(np.uint16)
    w[:, off] = d & 0xFF
    w[:, off + 1] = d >> 8
    if wtype in (ora.Q4_K, ora.Q5_K):
        m = rng.uniform(0.0, 0.05, rows * nb).astype(np.float16).view(np.uint16)
        w[:, 2] = m & 0xFF
        w[:, 3] = m >> 8
    return w.reshape(-1)


def quantized(wtype, rows, k, seed):
    rng = np.random.default_rng(seed)
    x = normal_f32(rng, (rows, k), 0.02)
    if wtype == bm.IQ4_XS:  # the reference's gguf crate has no IQ4_XS quantizer: the test-side generator
        return iq4xs_rows(x)
    if wtype == bm.IQ3_XXS:  # nor an IQ3_XXS one: raw random blocks, every one of which is legal
        return random_blocks(wtype, rows, k, rng)
    if wtype == bm.Q3_K:  # a test-side generator: the oracle restates the quantizers of the benchmark's types only
        return q3k_rows(x)
    return ora.quantize_rows(wtype, x, rows, k, n_threads=8)


def stack(wtype, rows, k, seed):
    """Weights for a test: the repo's quantizer for the K-quants, and for IQ2_XXS (whose search is slow) a few
    quantized rows followed by raw random blocks."""
    if wtype != bm.IQ2_XXS or rows <= 64:
        return quantized(wtype, rows, k, seed)
    rng = np.random.default_rng(seed)
    head = quantized(wtype, 64, k, seed)
    return np.concatenate([head, random_blocks(wtype, rows - 64, k, rng)])


# ------------------------------------------------------------------------------------------------ quantizers

def kat_columns(k):
    """Edge columns of the reference's encoder tests (crates/qdot/tests/qdot.rs:4619-4944) at width k."""
    rng = Lcg(0xC0FFEE)
    cols = []
    x = np.array([rng.unit() for _ in range(k)], np.float32)
    cols.append(x)
    t = np.array([TIES[i % len(TIES)] for i in range(k)], np.float32)
    t[0::32] = 127.0
    t[32] = 254.0
    cols.append(t)
    sat = np.array([254.0 if j % 2 == 0 else -254.0 for j in range(k)], np.float32)
    sat[96:128] *= np.float32((127.0 - 127.0 / 512.0) / 254.0)
    cols.append(sat)
    cols.append(np.full(k, 1e-40, np.float32))
    cols.append(np.full(k, 1e-38, np.float32))
    z = np.array([rng.unit() * np.float32(3.0) for _ in range(k)], np.float32)
    z[0:64] = 0.0
    z[k // 2:k // 2 + 256] = 0.0
    cols.append(z)
    ties = np.array([rng.unit() * np.float32(0.4) for _ in range(k)], np.float32)
    ties[9], ties[200], ties[137] = 3.0, -3.0, 3.0
    ties[256 + 250], ties[256 + 3] = 3.0, -3.0
    cols.append(ties)
    sub = np.where(np.arange(k) % 2 == 0, 1.0, -1.0).astype(np.float32) * np.float32(127.0 * (64.49 / 64.0) * 2.0 ** -127)
    cols.append(sub)
    for mag in (1e-6, 1e-3, 1.0, 1e4):
        cols.append(np.array([rng.unit() * np.float32(mag) for _ in range(k)], np.float32))
    return np.stack(cols)


@pytest.mark.parametrize("wtype", (bm.Q4_K, bm.IQ2_XXS))
@pytest.mark.parametrize("k", (512, 2048))
def test_quantize_bytes_are_the_cpu_paths(gpu, wtype, k):
    x = kat_columns(k)
    m = x.shape[0]
    act = gpu.act(wtype, k, m)
    xd = gpu.upload(x, np.float32)
    gpu.enqueue_quantize(xd, m, act)
    for c in range(m):
        want = ora.quantize_col(wtype, x[c])
        got = act.download(c)
        assert np.array_equal(got, want), f"type {wtype} k {k} column {c}: {np.count_nonzero(got != want)} bytes differ"
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    act.free()
    xd.free()


def test_quantize_random_columns(gpu):
    rng = np.random.default_rng(7)
    for wtype, k in ((bm.Q4_K, 2048), (bm.Q5_K, 2304), (bm.Q6_K, 768), (bm.IQ2_XXS, 7168)):
        m = 40
        x = (normal_f32(rng, (m, k)) * (10.0 ** rng.uniform(-5, 4, (m, 1)))).astype(np.float32)
        act = gpu.act(wtype, k, m)
        xd = gpu.upload(x, np.float32)
        gpu.enqueue_quantize(xd, m, act)
        for c in range(m):
            assert np.array_equal(act.download(c), ora.quantize_col(wtype, x[c])), (wtype, c)
        act.free()
        xd.free()


def test_non_finite_activation_raises_quant_column(gpu):
    # crates/gpu/src/lib.rs:925-933: NaN scale, zero codes, fault site 1; the CPU path refuses the column instead
    for wtype, bb in ((bm.Q4_K, 144), (bm.IQ2_XXS, 296)):
        gpu.fault_clear()
        x = np.ones((1, 512), np.float32)
        x[0, 300] = np.inf
        act = gpu.act(wtype, 512, 1)
        xd = gpu.upload(x, np.float32)
        gpu.set_layer(3)
        gpu.enqueue_quantize(xd, 1, act)
        w0, mask = gpu.fault(3)
        assert w0 == (3 << 8) | bm.SITE_QUANT_COLUMN and mask == 1 << bm.SITE_QUANT_COLUMN
        col = act.download(0)
        good = ora.quantize_col(wtype, np.ones(256, np.float32))
        assert np.array_equal(col[:len(good)], good), "the clean block is untouched by its neighbour"
        if wtype == bm.Q4_K:
            grp = col[288:432]  # values 256..383; the bad block is the second of this group
            assert grp[2:4].view(np.uint16)[0] == 0x7FC0 and not grp[16 + 32:16 + 64].any() and grp[10:12].view(np.int16)[0] == 0
        else:
            blk = col[296:592]
            assert np.isnan(blk[0:4].view(np.float32)[0]) and not blk[4:].any()
        gpu.set_layer(bm.LAYER_NONE)
        gpu.fault_clear()
        assert gpu.fault(3) == (bm.FAULT_NONE, 0)
        act.free()
        xd.free()


# ------------------------------------------------------------------------------------------------ integer sums

@pytest.mark.parametrize("wtype", TYPES)
def test_block_sums_are_the_cpu_paths_integers(gpu, wtype):
    rng = np.random.default_rng(20 + wtype)
    for k in (256, 768, 2048):
        rows = 6
        w = np.concatenate([random_blocks(wtype, 3, k, rng), quantized(wtype, 3, k, 21)])
        x = normal_f32(rng, (2, k), 10.0 ** rng.uniform(-2, 2))
        wd, act = gpu.weights(wtype, rows, k, w), gpu.act(wtype, k, 2)
        xd = gpu.upload(x, np.float32)
        gpu.enqueue_quantize(xd, 2, act)
        out = gpu.buffer(np.int32, 16 * (k // 256))
        rb = ora.row_bytes(wtype, k)
        for row in range(rows):
            for col in range(2):
                gpu.enqueue_block_sums(wd, row, act, col, out)
                got = out.download().reshape(-1, 16)
                wrow, acol = w[row * rb:(row + 1) * rb], ora.quantize_col(wtype, x[col])
                if wtype in (bm.Q4_K, bm.Q5_K):
                    a, isum = ora.q4k_block_sums(wrow, acol, k, q5=wtype == bm.Q5_K)
                    assert np.array_equal(got[:, :8].reshape(-1), a) and np.array_equal(got[:, 8:].reshape(-1), isum)
                elif wtype == bm.Q3_K:
                    assert np.array_equal(got.reshape(-1), ora.q3k_block_sums(wrow, acol, k))
                elif wtype == bm.Q6_K:
                    assert np.array_equal(got.reshape(-1), ora.q6k_block_sums(wrow, acol, k))
                    assert np.array_equal(got.reshape(-1), ora.q6k_block_sums(wrow, acol, k, fold=True))
                elif wtype == bm.IQ4_XS:
                    i_b, lanes = ora.iq4xs_block_sums(wrow, acol, k)
                    assert np.array_equal(got[:, :8].reshape(-1), i_b) and np.array_equal(got[:, 8:].reshape(-1), lanes)
                    assert np.array_equal(lanes, ora.iq4xs_block_sums(wrow, acol, k, fold=True)[1])
                else:
                    i_b, sc, _, _ = ora.iq2xxs_block_sums(wrow, acol, k, iq3=wtype == bm.IQ3_XXS)
                    assert np.array_equal(got[:, :8].reshape(-1), i_b) and np.array_equal(got[:, 8:].reshape(-1), sc)
        for b in (wd, act, xd, out):
            b.free()


# -------------------------------------------------------------------------------------------------------- gemv

@pytest.mark.parametrize("wtype,rows,k", ((bm.Q4_K, 768, 2048), (bm.Q6_K, 2048, 768), (bm.IQ2_XXS, 300, 2048),
                                          (bm.Q4_K, 70, 256), (bm.Q6_K, 65, 1792), (bm.IQ2_XXS, 33, 7168),
                                          (bm.Q5_K, 96, 2304), (bm.Q5_K, 67, 1280), (bm.IQ4_XS, 200, 2560),
                                          (bm.IQ4_XS, 66, 768), (bm.IQ3_XXS, 130, 2048), (bm.IQ3_XXS, 40, 1280),
                                          (bm.Q3_K, 150, 2048), (bm.Q3_K, 70, 768)))
def test_gemv_matches_dot_row(gpu, wtype, rows, k):
    # config 1 is the first case: 768 x 2048 Q4_K against one 2048-vector
    rng = np.random.default_rng(30 + rows)
    w = stack(wtype, rows, k, 31 + rows)
    x = normal_f32(rng, (8, k))
    wd, act = gpu.weights(wtype, rows, k, w), gpu.act(wtype, k, 8)
    xd = gpu.upload(x, np.float32)
    gpu.enqueue_quantize(xd, 8, act)
    cols = np.concatenate([ora.quantize_col(wtype, x[c]) for c in range(8)])
    for m in (1, 3, 8):
        y = gpu.buffer(np.float32, rows * m).fill_bytes(0xFF)
        gpu.enqueue_gemv(wd, act, m, y)
        assert_f32(y.download(), ora.gemv(wtype, w, rows, k, cols, m), f"gemv type {wtype} {rows}x{k} m={m}")
        y.free()
    for b in (wd, act, xd):
        b.free()


@pytest.mark.parametrize("wtype,rows,k", ((bm.Q4_K, 768, 2048), (bm.Q6_K, 2048, 768), (bm.Q5_K, 67, 1280), (bm.Q4_K, 70, 4352),
                                          (bm.IQ2_XXS, 33, 7168), (bm.IQ4_XS, 66, 768), (bm.IQ3_XXS, 40, 1280),
                                          (bm.Q3_K, 150, 2048)))
def test_gemv_from_f32_folds_the_quantizer(gpu, wtype, rows, k):
    """bm_gemv_x: the quantizer and the gemv in one launch give the two launches' bits, for y and for the columns it
    leaves in act_out; a value that is not finite raises QuantColumn as bm_quantize does."""
    rng = np.random.default_rng(300 + rows)
    w = stack(wtype, rows, k, 301 + rows)
    x = normal_f32(rng, (3, k))
    x[1] *= np.float32(1e-3)
    wd, xd = gpu.weights(wtype, rows, k, w), gpu.upload(x, np.float32)
    cols = np.concatenate([ora.quantize_col(wtype, x[c]) for c in range(3)])
    gpu.fault_clear()
    for m, keep in ((1, False), (3, True)):
        y = gpu.buffer(np.float32, rows * m).fill_bytes(0xFF)
        act = gpu.act(wtype, k, 3) if keep else None
        gpu.enqueue_gemv_x(wd, xd, m, y, act)
        assert_f32(y.download(), ora.gemv(wtype, w, rows, k, cols, m), f"gemv_x type {wtype} {rows}x{k} m={m}")
        if keep:
            for c in range(m):
                assert np.array_equal(act.download(c), ora.quantize_col(wtype, x[c])), f"column {c} left in act_out"
            y2 = gpu.buffer(np.float32, rows * m).fill_bytes(0xFF)
            gpu.enqueue_gemv(wd, act, m, y2)  # the columns it left are whole: tables and all
            assert np.array_equal(y2.download().view(np.uint32), y.download().view(np.uint32))
            y2.free()
            act.free()
        y.free()
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    x[0, 5] = np.nan
    xd.upload(x)
    y = gpu.buffer(np.float32, rows)
    gpu.enqueue_gemv_x(wd, xd, 1, y)
    assert (gpu.fault()[0] & 0xFF) == bm.SITE_QUANT_COLUMN
    gpu.fault_clear()
    with pytest.raises(bm.GpuError) as e:
        gpu.enqueue_gemv_x(wd, xd, 0, y)
    assert e.value.code == bm.ESHAPE
    for b in (wd, xd, y):
        b.free()


def test_extreme_blocks(gpu):
    """Every code at its ends, zero, subnormal and negative block scales (crates/qdot/tests/qdot.rs:2615-2655)."""
    rng = np.random.default_rng(44)
    for wtype in TYPES:
        bb = ora.BLOCK_BYTES[wtype]
        rows_bytes = []
        for fill, dval in ((0xFF, 0.05), (0x00, 0.05), (0xFF, 0.0), (0xAA, 6e-8), (0x55, -0.03), (0x0F, 65504.0)):
            w = np.full(2 * bb, fill, np.uint8)
            for i in range(2):
                h = np.array([dval, abs(dval)], np.float16).view(np.uint8)
                off = {ora.Q3_K: 108, ora.Q4_K: 0, ora.Q5_K: 0, ora.Q6_K: 208, ora.IQ2_XXS: 0, ora.IQ3_XXS: 0, ora.IQ4_XS: 0}[wtype]
                w[i * bb + off:i * bb + off + 2] = h[0:2]
                if wtype in (ora.Q4_K, ora.Q5_K):
                    w[i * bb + 2:i * bb + 4] = h[2:4]
            rows_bytes.append(w)
        w = np.concatenate(rows_bytes)
        rows, k = len(rows_bytes), 512
        x = np.stack([np.full(k, 3.0, np.float32), normal_f32(rng, k), -np.abs(normal_f32(rng, k)),
                      normal_f32(rng, k, 1e-3)])
        wd, act = gpu.weights(wtype, rows, k, w), gpu.act(wtype, k, 4)
        xd = gpu.upload(x, np.float32)
        gpu.enqueue_quantize(xd, 4, act)
        y = gpu.buffer(np.float32, rows * 4)
        gpu.enqueue_gemv(wd, act, 4, y)
        cols = np.concatenate([ora.quantize_col(wtype, x[c]) for c in range(4)])
        want = ora.gemv(wtype, w, rows, k, cols, 4)
        got = y.download()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (wtype, got, want)
        for b in (wd, act, xd, y):
            b.free()


# ------------------------------------------------------------------------------------------- the expert chain

def route(rng, m, n_experts, top_k, bias=None):
    ids = np.empty((m, top_k), np.uint32)
    wts = np.empty((m, top_k), np.float32)
    for t in range(m):
        logits = normal_f32(rng, n_experts)
        if bias is not None:
            logits = (logits + bias).astype(np.float32)
        ids[t], wts[t] = ora.route_softmax_topk(logits, top_k)
    return ids, wts


class Layer:
    def __init__(self, gpu, types, hidden, ff, n_experts, seed, cheap=False):
        self.types, self.hidden, self.ff, self.n_experts = types, hidden, ff, n_experts
        if cheap:  # random legal blocks: a large stack without the quantizers' search
            rng = np.random.default_rng(seed)
            self.wg = random_blocks(types[0], n_experts * ff, hidden, rng)
            self.wu = random_blocks(types[1], n_experts * ff, hidden, rng)
            self.wd = random_blocks(types[2], n_experts * hidden, ff, rng)
        else:
            self.wg = stack(types[0], n_experts * ff, hidden, seed)
            self.wu = stack(types[1], n_experts * ff, hidden, seed + 1)
            self.wd = stack(types[2], n_experts * hidden, ff, seed + 2)
        self.dg = gpu.weights(types[0], n_experts * ff, hidden, self.wg)
        self.du = gpu.weights(types[1], n_experts * ff, hidden, self.wu)
        self.dd = gpu.weights(types[2], n_experts * hidden, ff, self.wd)

    def oracle(self, x, ids, wts, top_k):
        return ora.moe_forward(self.hidden, self.ff, self.n_experts, self.types, self.wg, self.wu, self.wd, x, ids,
                               wts, top_k, n_threads=8, want_h=True)

    def free(self):
        for b in (self.dg, self.du, self.dd):
            b.free()


def run_chain(gpu, L, x, ids, wts, top_k, fused):
    """quantize -> gate.up (-> quantize) -> down -> combine, as the reference's decode dispatch orders them
    (crates/gpu/src/arch/qwen3moe/dispatch.rs:1245-1436); `fused` takes the two fused launches instead."""
    m = x.shape[0]
    n_slots = m * top_k
    act = gpu.act(L.types[0], L.hidden, m)
    act_h = gpu.act(L.types[2], L.ff, n_slots)
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    h = gpu.buffer(np.float32, n_slots * L.ff).fill_bytes(0xFF)
    y = gpu.buffer(np.float32, m * L.hidden).fill_bytes(0xFF)
    gpu.enqueue_quantize(xd, m, act)
    if fused and L.types[2] not in Q8K_TYPES:  # the folded quantizer writes Q8_2_X4 columns
        gpu.enqueue_gate_up(L.dg, L.du, act, sel, n_slots, L.ff, top_k, h, act_h)
    else:
        gpu.enqueue_gate_up(L.dg, L.du, act, sel, n_slots, L.ff, top_k, h)
        gpu.enqueue_quantize(h, n_slots, act_h)
    if fused:
        gpu.enqueue_down_combine(L.dd, act_h, sel, wd, None, top_k, m, L.hidden, y)
    else:
        down = gpu.buffer(np.float32, n_slots * L.hidden).fill_bytes(0xFF)
        gpu.enqueue_gemv_sel(L.dd, act_h, sel, n_slots, L.hidden, down)
        gpu.enqueue_combine_tokens(down, wd, None, L.hidden, top_k, m, y)
    out = y.download(), h.download(), [act_h.download(s) for s in range(n_slots)]
    for b in (act, act_h, xd, sel, wd, h, y):
        b.free()
    return out


@pytest.mark.parametrize("fused", (False, True))
def test_qwen3_shaped_layer_one_token(gpu, fused):
    """Config 2 at its full shape with 16 of the 128 experts resident: hidden 2048, ff 768, Q4_K gate/up, Q6_K
    down, softmax top-8 renormalised, one token."""
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 16, 100)
    rng = np.random.default_rng(101)
    x = normal_f32(rng, (1, 2048))
    ids, wts = route(rng, 1, 16, 8)
    y, h, act_h = run_chain(gpu, L, x, ids, wts, 8, fused)
    want_y, want_h = L.oracle(x, ids, wts, 8)
    assert_f32(h, want_h, "h")
    for s in range(8):
        assert np.array_equal(act_h[s], ora.quantize_col(bm.Q6_K, want_h[s * 768:(s + 1) * 768])), f"act_h slot {s}"
    assert_f32(y, want_y, "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    L.free()


@pytest.mark.parametrize("fused", (False, True))
def test_gate_up_over_more_slots_than_one_grid_dimension_holds(gpu, fused):
    """bm_gate_up's grid counts the slots along its second dimension up to 32768 and the rest along the third: 4101 tokens of
    eight slots are 32808 slots, so the last 40 lie in the second plane. A small layer, every slot against the oracle."""
    types, hidden, ff, n_experts, m, top_k = (bm.Q4_K, bm.Q4_K, bm.Q6_K), 256, 256, 3, 4101, 8
    L = Layer(gpu, types, hidden, ff, n_experts, 977)
    rng = np.random.default_rng(978)
    x = normal_f32(rng, (m, hidden))
    ids = rng.integers(0, n_experts, size=(m, top_k)).astype(np.uint32)
    wts = (rng.random((m, top_k), dtype=np.float32) + np.float32(0.1)).astype(np.float32)
    y, h, act_h = run_chain(gpu, L, x, ids, wts, top_k, fused)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    assert_f32(h, want_h, "h")
    for s in (0, 1, 32767, 32768, 32769, 32807):
        assert np.array_equal(act_h[s], ora.quantize_col(types[2], want_h[s * ff:(s + 1) * ff])), f"act_h slot {s}"
    assert_f32(y, want_y, "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    L.free()


@pytest.mark.parametrize("types,hidden,ff,n_experts,m,top_k", (
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 12, 5, 4),
    ((bm.Q6_K, bm.Q6_K, bm.Q4_K), 512, 512, 5, 3, 2),
    ((bm.Q5_K, bm.Q5_K, bm.Q5_K), 768, 512, 4, 3, 2),
    ((bm.Q4_K, bm.Q4_K, bm.Q5_K), 512, 2304, 3, 2, 2),          # a Q5_K down stack over 2304-value rows
    ((bm.IQ4_XS, bm.IQ4_XS, bm.IQ4_XS), 768, 512, 4, 3, 2),
    ((bm.IQ4_XS, bm.IQ4_XS, bm.Q5_K), 512, 256, 3, 2, 3),       # Q8_K columns into gate / up, Q8_2_X4 into down
    ((bm.IQ3_XXS, bm.IQ3_XXS, bm.IQ3_XXS), 768, 512, 4, 3, 2),
    ((bm.Q3_K, bm.Q3_K, bm.Q3_K), 768, 512, 4, 3, 2),
    ((bm.Q3_K, bm.Q3_K, bm.Q5_K), 512, 256, 3, 2, 3),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ3_XXS), 512, 768, 3, 2, 3),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), 1024, 512, 6, 4, 3),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.Q6_K), 768, 256, 4, 2, 4),
))
@pytest.mark.parametrize("fused", (False, True))
def test_layers_of_every_type_and_several_tokens(gpu, types, hidden, ff, n_experts, m, top_k, fused):
    L = Layer(gpu, types, hidden, ff, n_experts, 200 + hidden)
    rng = np.random.default_rng(201)
    x = normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, n_experts, top_k)
    y, h, act_h = run_chain(gpu, L, x, ids, wts, top_k, fused)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    assert_f32(h, want_h, "h")
    for s in range(m * top_k):
        assert np.array_equal(act_h[s], ora.quantize_col(types[2], want_h[s * ff:(s + 1) * ff])), f"act_h slot {s}"
    assert_f32(y, want_y, "y")
    L.free()


def run_fused_step(gpu, L, x, ids, wts, top_k, resid=None, replays=1):
    """bm_moe_decode: the whole step with the quantizers folded in. Returns (y, h, act_h columns, act_x columns) of the
    last replay."""
    m = x.shape[0]
    n_slots = m * top_k
    act_x = gpu.act(L.types[0], L.hidden, m)
    act_h = gpu.act(L.types[2], L.ff, n_slots)
    xd, sel, wd = gpu.upload(x, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32)
    rd = gpu.upload(resid, np.float32) if resid is not None else None
    h = gpu.buffer(np.float32, n_slots * L.ff)
    y = gpu.buffer(np.float32, m * L.hidden)
    for _ in range(replays):
        h.fill_bytes(0xFF)
        y.fill_bytes(0xFF)
        gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wd, rd, top_k, m, act_h, y, act_x=act_x, h=h)
    out = (y.download(), h.download(), [act_h.download(s) for s in range(n_slots)],
           [act_x.download(t) for t in range(m)])
    for b in (act_x, act_h, xd, sel, wd, h, y) + ((rd,) if rd is not None else ()):
        b.free()
    return out


@pytest.mark.parametrize("types,hidden,ff,n_experts,m,top_k", (
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 16, 1, 8),   # config 2's shape: the whole-row variants
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 12, 5, 4),
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 1024, 512, 6, 3, 6),    # 64 / 6 rows a consumer workgroup: a ragged tail
    ((bm.Q4_K, bm.Q4_K, bm.Q4_K), 512, 512, 5, 4, 2),
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 4096, 256, 4, 2, 3),    # rows longer than one quantizer pass
    ((bm.Q5_K, bm.Q5_K, bm.Q6_K), 2048, 512, 4, 3, 4),    # Q5_K gate/up at the whole-row shape
    ((bm.Q5_K, bm.Q5_K, bm.Q5_K), 768, 256, 3, 2, 2),
    # the types on Q8_K columns: their quantizers folded into the two launches (the token's in every gate . up
    # workgroup, h's in every down workgroup), and the mixes of the two column forms
    ((bm.IQ4_XS, bm.IQ4_XS, bm.IQ4_XS), 2048, 768, 6, 3, 4),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ3_XXS), 1024, 512, 5, 2, 4),
    ((bm.Q3_K, bm.Q3_K, bm.Q6_K), 768, 512, 4, 5, 2),
    ((bm.Q4_K, bm.Q4_K, bm.IQ4_XS), 2048, 512, 4, 3, 4),
    ((bm.Q5_K, bm.Q5_K, bm.Q3_K), 512, 768, 3, 2, 3),
    ((bm.Q6_K, bm.Q6_K, bm.Q4_K), 768, 256, 3, 2, 2),
))
def test_fused_step_matches_the_chain_and_the_oracle(gpu, types, hidden, ff, n_experts, m, top_k):
    L = Layer(gpu, types, hidden, ff, n_experts, 600 + hidden + ff)
    rng = np.random.default_rng(601)
    x = normal_f32(rng, (m, hidden))
    resid = normal_f32(rng, (m, hidden))
    ids, wts = route(rng, m, n_experts, top_k)
    gpu.fault_clear()
    # three launches in a row over the same scratch
    y, h, act_h, act_x = run_fused_step(gpu, L, x, ids, wts, top_k, resid, replays=3)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    for t in range(m):
        assert np.array_equal(act_x[t], ora.quantize_col(types[0], x[t])), f"act_x token {t}"
    assert_f32(h, want_h, "h")
    for s in range(m * top_k):
        assert np.array_equal(act_h[s], ora.quantize_col(types[2], want_h[s * ff:(s + 1) * ff])), f"act_h slot {s}"
    assert_f32(y, (want_y.reshape(m, hidden) + resid).astype(np.float32).reshape(-1), "y + resid")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    L.free()


def test_fused_step_at_the_token_limit(gpu):
    """bm_moe_decode takes 1..=1024 tokens a launch: the limit itself against the oracle, one more refused by name."""
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 256, 256, 9, 650)
    rng = np.random.default_rng(651)
    m, top_k = 1024, 2
    x = normal_f32(rng, (m, L.hidden))
    ids, wts = route(rng, m, L.n_experts, top_k)
    gpu.fault_clear()
    y, h, _, _ = run_fused_step(gpu, L, x, ids, wts, top_k)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    assert_f32(h, want_h, "h")
    assert_f32(y, want_y, "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    xd, sel, wd = gpu.upload(np.zeros((m + 1, L.hidden), np.float32)), gpu.upload(np.zeros((m + 1, top_k), np.uint32)), \
        gpu.upload(np.zeros((m + 1, top_k), np.float32))
    act_h, yb = gpu.act(L.types[2], L.ff, (m + 1) * top_k), gpu.buffer(np.float32, (m + 1) * L.hidden)
    with pytest.raises(bm.GpuError) as e:
        gpu.enqueue_moe_decode(L.dg, L.du, L.dd, xd, sel, wd, None, top_k, m + 1, act_h, yb)
    assert e.value.code == bm.ESHAPE and "1025" in str(e.value)
    for b in (xd, sel, wd, act_h, yb):
        b.free()
    L.free()


def test_fused_step_refused_ids(gpu):
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 512, 256, 4, 700)
    rng = np.random.default_rng(701)
    x = normal_f32(rng, (2, 512))
    ids = np.array([[1, 9, 3], [2, 0, 1]], np.uint32)      # slot 1 names an expert past the stack
    wts = np.array([[0.5, 0.3, 0.2], [0.2, 0.5, 0.3]], np.float32)
    gpu.fault_clear()
    gpu.set_layer(4)
    y, h, _, _ = run_fused_step(gpu, L, x, ids, wts, 3)
    assert gpu.fault(4) == ((4 << 8) | bm.SITE_EXPERT_ID, 1 << bm.SITE_EXPERT_ID)
    assert np.isnan(h.reshape(6, 256)[1]).all()
    # the refused slot adds nothing: the same as the oracle over the live slots with the same weights
    live_ids, live_w = np.array([[1, 3], [2, 0]], np.uint32), np.array([[0.5, 0.2], [0.2, 0.5]], np.float32)
    want0, _ = L.oracle(x[:1], live_ids[:1], live_w[:1], 2)
    assert_f32(y[:512], want0, "token with a refused slot")
    want1, _ = L.oracle(x[1:], ids[1:], wts[1:], 3)
    assert_f32(y[512:], want1, "clean token")
    gpu.set_layer(bm.LAYER_NONE)
    gpu.fault_clear()
    L.free()


def test_uploaded_columns_dot_like_quantized_ones(gpu):
    """A column that arrives as bytes from a host tier (bm_act_upload) has its tables rebuilt on the device."""
    rng = np.random.default_rng(900)
    for wtype, rows, k in ((bm.Q4_K, 64, 1024), (bm.Q6_K, 64, 768), (bm.IQ2_XXS, 64, 512)):
        w = stack(wtype, rows, k, 901)
        x = normal_f32(rng, (2, k))
        cols = [ora.quantize_col(wtype, x[c]) for c in range(2)]
        dw, act = gpu.weights(wtype, rows, k, w), gpu.act(wtype, k, 2)
        for c in range(2):
            act.upload(c, cols[c])
            assert np.array_equal(act.download(c), cols[c])
        y = gpu.buffer(np.float32, rows * 2)
        gpu.enqueue_gemv(dw, act, 2, y)
        assert_f32(y.download(), ora.gemv(wtype, w, rows, k, np.concatenate(cols), 2), f"type {wtype}")
        for b in (dw, act, y):
            b.free()


# ------------------------------------------------------------------------------- several tokens, grouped by expert

def grouped_tables_on_device(gpu, ids_flat, n_experts):
    n_slots = ids_flat.size
    cap = gpu.tile_cap(n_slots, n_experts)
    assert cap == ora.tile_cap(n_slots, n_experts)
    sel = gpu.upload(ids_flat, np.uint32)
    order, start = gpu.buffer(np.uint32, n_slots).fill_bytes(0), gpu.buffer(np.uint32, n_experts + 1).fill_bytes(0xFF)
    tiles = gpu.buffer(np.uint32, cap + 1).fill_bytes(0)
    gpu.enqueue_buckets(sel, n_slots, n_experts, order, start)
    gpu.enqueue_tiles(start, n_experts, n_slots, tiles)
    return sel, order, start, tiles


@pytest.mark.parametrize("n_experts,n_slots,seed", ((128, 128, 1), (7, 40, 2), (1, 9, 3), (1024, 64, 4), (16, 1, 5)))
def test_grouped_tables_are_the_definition(gpu, n_experts, n_slots, seed):
    """order, start and the tile words against the table's definition (gate_q4k_sel's table clauses,
    crates/gpu-gates/src/bin/gate_q4k_sel.rs)."""
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, n_experts, n_slots).astype(np.uint32)
    if n_slots > 8:
        ids[3] = bm.HOST_SLOT      # served elsewhere: in no run, silently
    gpu.fault_clear()
    sel, order, start, tiles = grouped_tables_on_device(gpu, ids, n_experts)
    want_order, want_start, want_tiles, refused = ora.grouped_table(ids, n_experts)
    listed = int(want_start[-1])
    assert np.array_equal(start.download(), want_start)
    assert np.array_equal(order.download()[:listed], want_order[:listed])
    got_tiles = tiles.download()
    assert got_tiles[0] == want_tiles[0] and np.array_equal(got_tiles[1:1 + got_tiles[0]], want_tiles[1:1 + want_tiles[0]])
    assert not refused and gpu.fault() == (bm.FAULT_NONE, 0)
    # the two launches as one leave the same three tables
    o2, s2 = gpu.buffer(np.uint32, n_slots).fill_bytes(0), gpu.buffer(np.uint32, n_experts + 1).fill_bytes(0xFF)
    t2 = gpu.buffer(np.uint32, gpu.tile_cap(n_slots, n_experts) + 1).fill_bytes(0)
    gpu.enqueue_tables(sel, n_slots, n_experts, o2, s2, t2)
    assert np.array_equal(s2.download(), want_start) and np.array_equal(o2.download()[:listed], want_order[:listed])
    assert np.array_equal(t2.download()[:1 + got_tiles[0]], got_tiles[:1 + got_tiles[0]]) and gpu.fault() == (bm.FAULT_NONE, 0)
    for b in (sel, order, start, tiles, o2, s2, t2):
        b.free()


@pytest.mark.parametrize("wtype,k,m,n_experts,top_k,seed", ((bm.Q4_K, 2048, 16, 128, 8, 1), (bm.IQ2_XXS, 1792, 5, 40, 3, 2),
                                                          (bm.Q6_K, 256, 1, 3, 2, 3), (bm.IQ4_XS, 7168, 33, 256, 8, 4), (bm.Q5_K, 512, 70, 9, 4, 5)))
def test_tables_and_quantizer_as_one_launch(gpu, wtype, k, m, n_experts, top_k, seed):
    """bm_tables_quantize leaves what bm_tables and bm_quantize leave: the three tables word for word and every column's bytes,
    in either column form, with a host-served slot and an id past the stack among the slots (the one raises nothing, the other
    ExpertId, as in bm_tables), twice in a row; rows that are not 16-byte aligned go through the two launches and give the same."""
    rng = np.random.default_rng(7700 + seed)
    n_slots = m * top_k
    ids = rng.integers(0, n_experts, n_slots).astype(np.uint32)
    if n_slots > 4:
        ids[1], ids[3] = bm.HOST_SLOT, n_experts + 5
    x = normal_f32(rng, (m, k))
    x[0, 5] = 0.0
    sel, xd = gpu.upload(ids, np.uint32), gpu.upload(np.concatenate([np.zeros(1, np.float32), x.reshape(-1)]), np.float32)
    cap = gpu.tile_cap(n_slots, n_experts)
    want = (gpu.buffer(np.uint32, n_slots).fill_bytes(0), gpu.buffer(np.uint32, n_experts + 1).fill_bytes(0xFF), gpu.buffer(np.uint32, cap + 1).fill_bytes(0))
    want_act = gpu.act(wtype, k, m)
    gpu.fault_clear()
    gpu.enqueue_tables(sel, n_slots, n_experts, *want)
    want_fault = gpu.fault()
    gpu.enqueue_quantize(xd.ptr + 4, m, want_act)
    for x_ptr, what in ((xd.ptr + 4, "rows 4 bytes off a 16-byte boundary"), (None, "aligned rows")):
        xa = gpu.upload(x, np.float32) if x_ptr is None else None
        got = (gpu.buffer(np.uint32, n_slots).fill_bytes(0), gpu.buffer(np.uint32, n_experts + 1).fill_bytes(0xFF), gpu.buffer(np.uint32, cap + 1).fill_bytes(0))
        act = gpu.act(wtype, k, m)
        for rep in range(2):
            gpu.fault_clear()
            gpu.enqueue_tables_quantize(sel, n_slots, n_experts, *got, xa if xa is not None else x_ptr, m, act)
            listed = int(want[1].download()[-1])
            assert np.array_equal(got[1].download(), want[1].download()), what
            assert np.array_equal(got[0].download()[:listed], want[0].download()[:listed]), what
            n_t = int(want[2].download()[0])
            assert np.array_equal(got[2].download()[:1 + n_t], want[2].download()[:1 + n_t]), what
            for c in range(m):
                assert np.array_equal(act.download(c), want_act.download(c)), f"{what}: column {c}"
                if c in (0, m - 1):
                    assert np.array_equal(act.download(c), ora.quantize_col(wtype, x[c])), f"{what}: column {c} against the oracle"
            assert gpu.fault() == want_fault, what
        for b in got + (act,) + ((xa,) if xa is not None else ()):
            b.free()
    gpu.fault_clear()
    for b in want + (want_act, sel, xd):
        b.free()


def test_grouped_tables_refuse_bad_ids_and_bad_runs(gpu):
    ids = np.array([2, 9, 1, 2], np.uint32)   # 9 is past a stack of 4
    gpu.fault_clear()
    gpu.set_layer(3)
    sel, order, start, tiles = grouped_tables_on_device(gpu, ids, 4)
    assert gpu.fault(3) == ((3 << 8) | bm.SITE_EXPERT_ID, 1 << bm.SITE_EXPERT_ID)
    assert np.array_equal(start.download(), [0, 0, 1, 3, 3]) and np.array_equal(order.download()[:3], [2, 0, 3])
    # a run that ends past the table: no tiles, ExpertId (crates/gpu/src/q4k_sel.rs:606-651)
    gpu.fault_clear()
    start.upload(np.array([0, 2, 9, 3, 3], np.uint32))
    gpu.enqueue_tiles(start, 4, 4, tiles)
    assert tiles.download()[0] == 0 and gpu.fault(3)[0] == (3 << 8) | bm.SITE_EXPERT_ID
    gpu.set_layer(bm.LAYER_NONE)
    gpu.fault_clear()
    for b in (sel, order, start, tiles):
        b.free()


def run_grouped(gpu, L, x, ids, wts, top_k, fused_quant):
    """buckets -> tiles -> gate.up by tiles (-> quantize_ord) -> down by tiles -> combine: the reference's grouped
    decode (crates/gpu/src/arch/qwen3moe/dispatch.rs grouped branch; crates/gpu/src/kquant/tiles.rs)."""
    m = x.shape[0]
    n_slots = m * top_k
    sel, order, start, tiles = grouped_tables_on_device(gpu, ids.reshape(-1), L.n_experts)
    act = gpu.act(L.types[0], L.hidden, m)
    act_h = gpu.act(L.types[2], L.ff, n_slots)
    xd, wd = gpu.upload(x, np.float32), gpu.upload(wts, np.float32)
    h = gpu.buffer(np.float32, n_slots * L.ff).fill_bytes(0xFF)
    down = gpu.buffer(np.float32, n_slots * L.hidden).fill_bytes(0xFF)
    y = gpu.buffer(np.float32, m * L.hidden).fill_bytes(0xFF)
    gpu.enqueue_quantize(xd, m, act)
    if fused_quant and L.types[2] not in Q8K_TYPES:
        gpu.enqueue_gate_up_tiles(L.dg, L.du, act, order, start, tiles, n_slots, L.ff, top_k, h, act_h)
    else:
        gpu.enqueue_gate_up_tiles(L.dg, L.du, act, order, start, tiles, n_slots, L.ff, top_k, h)
        gpu.enqueue_quantize_ord(h, start, L.n_experts, n_slots, act_h)
    gpu.enqueue_gemv_tiles(L.dd, act_h, order, start, tiles, n_slots, L.hidden, down)
    gpu.enqueue_combine_tokens(down, wd, None, L.hidden, top_k, m, y)
    out = y.download(), h.download(), order.download(), down.download()
    for b in (sel, order, start, tiles, act, act_h, xd, wd, h, down, y):
        b.free()
    return out


@pytest.mark.parametrize("types,hidden,ff,n_experts,m,top_k", (
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 16, 16, 8),   # config 3's shape with 16 experts resident: long runs
    ((bm.Q4_K, bm.Q4_K, bm.Q6_K), 2048, 768, 128, 16, 8),  # config 3: 128 slots over 128 experts, skewed
    ((bm.Q6_K, bm.Q6_K, bm.Q4_K), 512, 512, 3, 7, 2),
    ((bm.Q5_K, bm.Q5_K, bm.Q5_K), 768, 512, 3, 9, 2),
    ((bm.IQ4_XS, bm.IQ4_XS, bm.IQ4_XS), 768, 512, 3, 9, 2),
    ((bm.IQ3_XXS, bm.IQ3_XXS, bm.IQ3_XXS), 768, 512, 3, 9, 2),
    ((bm.Q3_K, bm.Q3_K, bm.Q3_K), 768, 512, 3, 9, 2),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ2_XXS), 1024, 512, 5, 6, 3),
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.Q6_K), 768, 256, 4, 5, 4),
    # rows long enough that eight Q8_K columns pass the LDS mark where a tile launch goes as two, one for the tiles of
    # up to two slots and one for the wider ones: 18 slots over 6 experts give runs of both kinds
    ((bm.IQ2_XXS, bm.IQ2_XXS, bm.IQ4_XS), 5120, 4608, 6, 9, 2),
))
@pytest.mark.parametrize("fused_quant", (False, True))
def test_grouped_layer_matches_slot_by_slot(gpu, types, hidden, ff, n_experts, m, top_k, fused_quant):
    """Every slot of the grouped path holds its slot-by-slot value bit for bit (crates/gpu/src/kquant/tiles.rs:5-9);
    here against the oracle's slot-major layer on the same tokens."""
    if hidden >= 4096 and fused_quant:
        pytest.skip("Q8_K down columns: the folded quantizer does not apply, the other arm covers the case")
    if n_experts == 128 or hidden >= 4096:
        L = Layer(gpu, types, hidden, ff, n_experts, 1100, cheap=True)
    else:
        L = Layer(gpu, types, hidden, ff, n_experts, 1000 + hidden + n_experts)
    rng = np.random.default_rng(1001)
    x = normal_f32(rng, (m, hidden))
    bias = normal_f32(rng, n_experts, 0.5) if n_experts == 128 else None
    ids, wts = route(rng, m, n_experts, top_k, bias)
    if hidden >= 4096:
        runs = np.bincount(ids.reshape(-1), minlength=n_experts)
        assert (runs <= 2).any() and (runs > 2).any(), runs
    gpu.fault_clear()
    y, h, order, down = run_grouped(gpu, L, x, ids, wts, top_k, fused_quant)
    want_y, want_h = L.oracle(x, ids, wts, top_k)
    n_slots = m * top_k
    h, want_h = h.reshape(n_slots, ff), want_h.reshape(n_slots, ff)
    assert_f32(h, want_h[order], "h by table entry")   # entry j holds slot order[j]
    assert_f32(y, want_y, "y")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    L.free()


def test_grouped_skips_host_slots_and_refuses_stale_entries(gpu):
    L = Layer(gpu, (bm.Q4_K, bm.Q4_K, bm.Q6_K), 512, 256, 4, 1200)
    rng = np.random.default_rng(1201)
    m, top_k = 3, 2
    x = normal_f32(rng, (m, 512))
    ids = np.array([[1, bm.HOST_SLOT], [2, 1], [0, 3]], np.uint32)
    wts = normal_f32(rng, (m, top_k))
    gpu.fault_clear()
    y, h, order, down = run_grouped(gpu, L, x, ids, wts, top_k, True)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    down = down.reshape(m * top_k, 512)
    assert np.all(down[1].view(np.uint32) == 0xFFFFFFFF), "the host's slot keeps what it held"
    live = ids.copy()
    live[0, 1] = 1   # any live id: the slot's value is not compared
    _, want_h = L.oracle(x, live, wts, top_k)
    for s in (0, 2, 3, 4, 5):
        e = int(ids.reshape(-1)[s])
        rb = ora.row_bytes(bm.Q6_K, 256)
        want = ora.gemv(bm.Q6_K, L.wd[e * 512 * rb:(e + 1) * 512 * rb], 512, 256,
                        ora.quantize_col(bm.Q6_K, want_h[s * 256:(s + 1) * 256]), 1)
        assert_f32(down[s], want, f"slot {s}")
    L.free()


def test_slot_equals_one_expert_gemv_and_duplicate_ids(gpu):
    # gate_q4k_sel's first clauses (crates/gpu-gates/src/bin/gate_q4k_sel.rs:1-48)
    rng = np.random.default_rng(300)
    for wtype, k, rpe in ((bm.Q4_K, 768, 96), (bm.Q5_K, 1024, 72), (bm.Q6_K, 768, 2048 // 8), (bm.IQ2_XXS, 512, 80),
                          (bm.IQ4_XS, 1280, 40), (bm.IQ3_XXS, 768, 48), (bm.Q3_K, 512, 56)):
        n_experts, n_slots = 5, 7
        w = stack(wtype, n_experts * rpe, k, 301)
        sel = np.array([3, 0, 3, 4, 1, 3, 0], np.uint32)
        x = normal_f32(rng, (n_slots, k))
        wd, act = gpu.weights(wtype, n_experts * rpe, k, w), gpu.act(wtype, k, n_slots)
        xd, seld = gpu.upload(x, np.float32), gpu.upload(sel, np.uint32)
        gpu.enqueue_quantize(xd, n_slots, act)
        y = gpu.buffer(np.float32, n_slots * rpe).fill_bytes(0xFF)
        gpu.enqueue_gemv_sel(wd, act, seld, n_slots, rpe, y)
        got = y.download().reshape(n_slots, rpe)
        rb = ora.row_bytes(wtype, k)
        for s in range(n_slots):
            e = int(sel[s])
            want = ora.gemv(wtype, w[e * rpe * rb:(e + 1) * rpe * rb], rpe, k, ora.quantize_col(wtype, x[s]), 1)
            assert_f32(got[s], want, f"type {wtype} slot {s}")
        for b in (wd, act, xd, seld, y):
            b.free()


def test_bad_ids_raise_expert_id_and_host_is_silent(gpu):
    # crates/gpu/src/kquant/sel.rs:22-28, crates/gpu/src/q4k_sel.rs:968-972
    rng = np.random.default_rng(400)
    k, rpe, n_experts = 512, 64, 3
    w = quantized(bm.Q4_K, n_experts * rpe, k, 401)
    wd, act = gpu.weights(bm.Q4_K, n_experts * rpe, k, w), gpu.act(bm.Q4_K, k, 3)
    x = normal_f32(rng, (3, k))
    xd = gpu.upload(x, np.float32)
    gpu.enqueue_quantize(xd, 3, act)
    y = gpu.buffer(np.float32, 3 * rpe)
    # HOST: skipped silently, rows untouched
    gpu.fault_clear()
    y.upload(np.full(3 * rpe, 7.0, np.float32))
    seld = gpu.upload(np.array([1, bm.HOST_SLOT, 2], np.uint32))
    gpu.enqueue_gemv_sel(wd, act, seld, 3, rpe, y)
    got = y.download().reshape(3, rpe)
    assert (got[1] == 7.0).all() and not (got[0] == 7.0).any() and gpu.fault() == (bm.FAULT_NONE, 0)
    # an id past the stack: rows untouched and ExpertId raised under the launch's layer
    gpu.set_layer(9)
    y.upload(np.full(3 * rpe, 7.0, np.float32))
    seld.upload(np.array([1, 3, 2], np.uint32))
    gpu.enqueue_gemv_sel(wd, act, seld, 3, rpe, y)
    got = y.download().reshape(3, rpe)
    assert (got[1] == 7.0).all() and gpu.fault(9) == ((9 << 8) | bm.SITE_EXPERT_ID, 1 << bm.SITE_EXPERT_ID)
    # gate.up writes NaN into the refused slot's rows
    gpu.fault_clear()
    h = gpu.buffer(np.float32, 3 * rpe).fill_bytes(0)
    gpu.enqueue_gate_up(wd, wd, act, seld, 3, rpe, 1, h)
    hh = h.download().reshape(3, rpe)
    assert np.isnan(hh[1]).all() and np.isfinite(hh[0]).all() and np.isfinite(hh[2]).all()
    assert gpu.fault(9)[0] == (9 << 8) | bm.SITE_EXPERT_ID
    gpu.set_layer(bm.LAYER_NONE)
    gpu.fault_clear()
    for b in (wd, act, xd, y, seld, h):
        b.free()


def test_combine_adds_the_residual(gpu):
    rng = np.random.default_rng(500)
    rows, n_slots, m = 200, 8, 3
    down, w, resid = normal_f32(rng, m * n_slots * rows), normal_f32(rng, m * n_slots), normal_f32(rng, m * rows)
    dd, dw, dr = gpu.upload(down), gpu.upload(w), gpu.upload(resid)
    y = gpu.buffer(np.float32, m * rows)
    gpu.enqueue_combine_tokens(dd, dw, dr, rows, n_slots, m, y)
    assert_f32(y.download(), ora.combine_tokens(down, w, resid, rows, n_slots, m), "combine + resid")
    gpu.enqueue_combine_tokens(dd, dw, None, rows, n_slots, m, y)
    assert_f32(y.download(), ora.combine_tokens(down, w, None, rows, n_slots, m), "combine")
    # with a shared expert's rows (crates/gpu/src/moe_fused.rs:129-170): (sum + shexp) + resid, values chosen so that
    # the other grouping rounds differently
    shexp = (normal_f32(rng, m * rows) * np.float32(1e4)).astype(np.float32)
    big = (-shexp + normal_f32(rng, m * rows) * np.float32(1e-3)).astype(np.float32)
    ds, db = gpu.upload(shexp), gpu.upload(big)
    gpu.enqueue_moe_combine(dd, dw, ds, db, rows, n_slots, m, y)
    want = ora.moe_combine(down, w, shexp, big, rows, n_slots, m)
    assert_f32(y.download(), want, "moe_combine")
    other = ora.combine_tokens(down, w, (shexp + big).astype(np.float32), rows, n_slots, m)  # sum + (shexp + resid)
    assert np.count_nonzero(want != other) > rows  # the grouping matters on these values
    gpu.enqueue_moe_combine(dd, dw, ds, None, rows, n_slots, m, y)
    assert_f32(y.download(), ora.moe_combine(down, w, shexp, None, rows, n_slots, m), "moe_combine without resid")
    for b in (dd, dw, dr, y, ds, db):
        b.free()


def test_shape_refusals_are_named(gpu):
    # crates/gpu/src/q4k_sel.rs:990-1042: refused on the host, before any launch, with the entry point's name
    w4 = gpu.weights(bm.Q4_K, 64, 512, np.zeros(64 * bm.row_bytes(bm.Q4_K, 512), np.uint8))
    a512, a256, aq8k = gpu.act(bm.Q4_K, 512, 2), gpu.act(bm.Q4_K, 256, 2), gpu.act(bm.IQ2_XXS, 512, 2)
    buf = gpu.buffer(np.float32, 4096)
    sel = gpu.upload(np.zeros(8, np.uint32))
    cases = (
        (lambda: gpu.enqueue_gemv(w4, a256, 1, buf), bm.ESHAPE, "bm_gemv"),
        (lambda: gpu.enqueue_gemv(w4, aq8k, 1, buf), bm.ETYPE, "bm_gemv"),
        (lambda: gpu.enqueue_gemv(w4, a512, 3, buf), bm.ESHAPE, "bm_gemv"),
        (lambda: gpu.enqueue_gemv(w4, a512, 9, buf), bm.ESHAPE, "bm_gemv"),
        (lambda: gpu.enqueue_gemv_sel(w4, a512, sel, 2, 48, buf), bm.ESHAPE, "rows_per_expert"),
        (lambda: gpu.enqueue_gemv_sel(w4, a512, sel, 3, 32, buf), bm.ESHAPE, "n_slots"),
        (lambda: gpu.enqueue_gemv_sel(w4, a512, sel, 0, 32, buf), bm.ESHAPE, "n_slots"),
        (lambda: gpu.enqueue_gate_up(w4, w4, a512, sel, 5, 32, 2, buf), bm.ESHAPE, "bm_gate_up"),
        (lambda: gpu.enqueue_gate_up(w4, w4, a512, sel, 2, 32, 0, buf), bm.ESHAPE, "slots_per_col"),
        (lambda: gpu.enqueue_gate_up(w4, w4, a512, sel, 2, 32, 1, buf, a512), bm.ESHAPE, "act_h"),
        (lambda: gpu.enqueue_quantize(buf, 3, a512), bm.ESHAPE, "bm_quantize"),
        (lambda: gpu.enqueue_down_combine(w4, a512, sel, buf, None, 65, 1, 32, buf), bm.ESHAPE, "slots a token"),
        (lambda: gpu.weights(7, 4, 256, np.zeros(1024, np.uint8)), bm.ETYPE, "weight type"),
        (lambda: gpu.weights(bm.Q4_K, 4, 300, np.zeros(4096, np.uint8)), bm.ESHAPE, "256"),
        (lambda: gpu.act(bm.Q6_K, 100, 1), bm.ESHAPE, "256"),
    )
    for call, code, word in cases:
        with pytest.raises(bm.GpuError) as e:
            call()
        assert e.value.code == code and word in str(e.value), str(e.value)
    for b in (w4, a512, a256, aq8k, buf, sel):
        b.free()


def test_bench_probe_runs_and_refuses(gpu):
    """The benchmark's calibration launch (a library of its own, not the product's ABI): it fetches and leaves the
    source as it is; its geometry is checked on the host."""
    import ctypes as C
    import os
    path = os.path.join(os.path.dirname(bm.LIB_PATH), "libbm_bench_probe.so")
    assert os.path.exists(path), f"{path} is not built (make -C bloomery_amd/csrc)"
    lib = C.CDLL(path)
    lib.bm_bench_probe_read.restype = C.c_int
    lib.bm_bench_probe_read.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
    src = gpu.upload(np.arange(1 << 16, dtype=np.uint32), np.uint32)
    sink = gpu.buffer(np.uint32, 64).fill_bytes(0)
    stream = gpu.stream()
    assert lib.bm_bench_probe_read(stream, src.ptr, 0, 64, sink.ptr) == 0
    assert lib.bm_bench_probe_read(stream, src.ptr, 4 << 16, 64, sink.ptr) == 0
    assert lib.bm_bench_probe_read(stream, src.ptr, 4096 + 16, 7, sink.ptr) == 0
    gpu.sync()
    assert np.array_equal(src.download(), np.arange(1 << 16, dtype=np.uint32))
    assert lib.bm_bench_probe_read(stream, src.ptr, 24, 4, sink.ptr) == -1
    assert lib.bm_bench_probe_read(stream, src.ptr + 4, 64, 4, sink.ptr) == -1
    assert lib.bm_bench_probe_read(stream, src.ptr, 64, 0, sink.ptr) == -1
    src.free()
    sink.free()
    # the hand-over probe: every poller ends holding the writer's words, whatever the other workgroups do meanwhile
    lib.bm_bench_probe_handoff.restype = C.c_int
    lib.bm_bench_probe_handoff.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_int, C.c_int]
    big = gpu.buffer(np.uint32, 16 << 20).fill_bytes(1)
    flag, out, sink = gpu.buffer(np.uint32, 128).fill_bytes(0), gpu.buffer(np.uint64, 2048), gpu.buffer(np.uint32, 256)
    for gen, load in ((1, 0), (2, 1), (3, 2)):
        out.fill_bytes(0)
        assert lib.bm_bench_probe_handoff(stream, big.ptr, 64 << 20, flag.ptr, out.ptr, sink.ptr, gen, load, 100) == 0
        gpu.sync()
        o = out.download().reshape(256, 8)
        assert all(o[w, 4] == 1 for w in (8, 16, 248, 1, 4, 255)), o[[8, 16, 248, 1, 4, 255], 2:6]
        assert flag.download()[0] == gen
    assert lib.bm_bench_probe_handoff(stream, big.ptr, 1 << 20, flag.ptr, out.ptr, sink.ptr, 4, 0, 100) == -1
    assert lib.bm_bench_probe_handoff(stream, big.ptr, 64 << 20, flag.ptr, out.ptr, sink.ptr, 4, 3, 100) == -1
    assert lib.bm_bench_probe_handoff(stream, big.ptr, 64 << 20, None, out.ptr, sink.ptr, 4, 0, 100) == -1
    for b in (big, flag, out, sink):
        b.free()


@pytest.mark.parametrize("top_k,m,hidden", ((8, 3, 2048), (4, 2, 512), (2, 5, 72), (1, 1, 64), (3, 2, 256)))
def test_down_form_split_gives_the_rings_bits(gpu, top_k, m, hidden):
    """bm_set_down_form(BM_DOWN_SPLIT): the down + combine launch with a row's super-blocks dealt to the waves gives the bits of
    the default form (and so the oracle's), with a residual, a host-served slot and an id past the stack among the slots, at
    every number of slots a token it is built for; with three slots a token (64 is no multiple) the launch runs in the default
    form and the switch changes nothing. It refuses a form it does not know."""
    ff, n_experts = 768, 10
    rng = np.random.default_rng(9100 + top_k)
    wd = ora.quantize_rows(bm.Q6_K, normal_f32(rng, (n_experts * hidden, ff), 0.05), n_experts * hidden, ff)
    dd = gpu.weights(bm.Q6_K, n_experts * hidden, ff, wd)
    hrows = normal_f32(rng, (m * top_k, ff))
    act = gpu.act(bm.Q6_K, ff, m * top_k)
    hd = gpu.upload(hrows, np.float32)
    gpu.enqueue_quantize(hd, m * top_k, act)
    ids, wts = route(rng, m, n_experts, top_k)
    if top_k >= 2:
        ids[0, 1] = bm.HOST_SLOT
    if m >= 2:
        ids[1, 0] = n_experts + 3
    resid = normal_f32(rng, (m, hidden))
    sel, wt, rd = gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32), gpu.upload(resid, np.float32)
    ys = []
    try:
        for form in (bm.DOWN_RING, bm.DOWN_SPLIT, bm.DOWN_RING):
            gpu.set_down_form(form)
            gpu.fault_clear()
            y = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
            for _ in range(2):
                gpu.enqueue_down_combine(dd, act, sel, wt, rd, top_k, m, hidden, y)
            ys.append(y.download().copy())
            y.free()
            assert (gpu.fault()[0] != bm.FAULT_NONE) == (m >= 2)
        assert np.array_equal(ys[0].view(np.uint32), ys[1].view(np.uint32)), "split against ring"
        assert np.array_equal(ys[0].view(np.uint32), ys[2].view(np.uint32))
        with pytest.raises(bm.GpuError) as e:
            gpu.set_down_form(2)
        assert "bm_set_down_form" in str(e.value)
    finally:
        gpu.set_down_form(bm.DOWN_RING)
        gpu.fault_clear()
        for b in (dd, act, hd, sel, wt, rd):
            b.free()


@pytest.mark.parametrize("down_type,hidden,ff,n_experts,m,top_k", ((bm.Q6_K, 2048, 768, 10, 3, 8), (bm.Q4_K, 512, 512, 5, 4, 2),
                                                                    (bm.Q5_K, 768, 256, 4, 2, 3), (bm.IQ4_XS, 1024, 512, 6, 2, 4)))
def test_down_combine_from_f32_rows_for_either_column_form(gpu, down_type, hidden, ff, n_experts, m, top_k):
    """bm_down_combine_h quantizes the f32 rows of h itself, in the form the down stack dots against (Q8_2_X4 or Q8_K):
    y and the columns it leaves in act_h are the oracle's, for a stack of either form; a row that is not finite raises
    QuantColumn."""
    rng = np.random.default_rng(900 + ff)
    wd = stack(down_type, n_experts * hidden, ff, 901 + ff)
    dd = gpu.weights(down_type, n_experts * hidden, ff, wd)
    n_slots = m * top_k
    h = normal_f32(rng, (n_slots, ff))
    h[1] *= np.float32(1e-3)
    ids, wts = route(rng, m, n_experts, top_k)
    resid = normal_f32(rng, (m, hidden))
    hd, sel, wt, rd = gpu.upload(h, np.float32), gpu.upload(ids, np.uint32), gpu.upload(wts, np.float32), gpu.upload(resid, np.float32)
    act_h = gpu.act(down_type, ff, n_slots)
    y = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    gpu.fault_clear()
    gpu.enqueue_down_combine_h(dd, hd, act_h, sel, wt, rd, top_k, m, hidden, y)
    cols = [ora.quantize_col(down_type, h[s]) for s in range(n_slots)]
    for s in range(n_slots):
        assert np.array_equal(act_h.download(s), cols[s]), f"column {s}"
    rb = ora.row_bytes(down_type, ff)
    down = np.concatenate([ora.gemv(down_type, wd[int(ids.reshape(-1)[s]) * hidden * rb:], hidden, ff, cols[s]) for s in range(n_slots)])
    assert_f32(y.download(), ora.combine_tokens(down, wts, resid, hidden, top_k, m), "y")
    # against the launch that takes ready columns: the same bits
    y2 = gpu.buffer(np.float32, m * hidden).fill_bytes(0xFF)
    gpu.enqueue_down_combine(dd, act_h, sel, wt, rd, top_k, m, hidden, y2)
    assert np.array_equal(y.download().view(np.uint32), y2.download().view(np.uint32))
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    h[0, 3] = np.inf
    hd.upload(h)
    gpu.enqueue_down_combine_h(dd, hd, None, sel, wt, rd, top_k, m, hidden, y)
    assert (gpu.fault()[0] & 0xFF) == bm.SITE_QUANT_COLUMN
    gpu.fault_clear()
    for b in (dd, hd, sel, wt, rd, act_h, y, y2):
        b.free()
