"""The card rule on the GPU (bm_card_quantize, bm_card_gemv, bm_card_gemv_sel) against the oracle's restatement of the
reference's CPU mirrors (crates/qdot/src/lib.rs:2885 card_q8_1, :3558 card_q4k_dot_row, :3346 card_q3k_dot_row): the
three planes of a quantized column equal byte for byte, edge columns of the reference's own test included
(crates/qdot/tests/qdot.rs:7942-8040), and every row's walk equal bit for bit at every super-block count that exercises
the walks' guarded tails and the Q4_K walk's split prefix."""
import numpy as np
import pytest

import bloomery_amd as bm
import ora
from test_gpu_decode import gpu, random_blocks  # noqa: F401  (gpu is the module fixture)

pytestmark = pytest.mark.gpu
f32 = np.float32


def edge_columns():
    ties = np.zeros(512, f32)
    for i in range(512):
        j, sign = i % 128, 1.0 if (i // 128) % 2 == 0 else -1.0
        ties[i] = 127.0 if j == 0 else sign * (((j - 1) // 3) + (0.5, 0.0, 0.25)[(j - 1) % 3])
    near = np.zeros(1024, f32)
    near[0], i = 127.0, 1
    for m in range(127):
        for frac in (f32(0.5), f32(0.49999997), f32(0.50000006)):
            if i + 1 < near.size:
                near[i], near[i + 1] = f32(m) + frac, -(f32(m) + frac)
                i += 2
    near[128::128] = 127.0
    tiny = np.zeros(512, f32)
    tiny[128:256] = (np.arange(128, dtype=f32) - 64) * f32(1e-40)
    one = np.array([1], np.uint32).view(f32)[0]
    tiny[256], tiny[257] = one, -one
    tiny[384], tiny[385] = np.finfo(f32).tiny, -np.finfo(f32).tiny / f32(3)
    return {"ties": ties, "near ties": near, "tiny": tiny}


def planes(gpu, m, k):
    return gpu.buffer(np.int8, m * k).fill_bytes(0x55), gpu.buffer(np.float32, m * k // 128).fill_bytes(0x55), \
        gpu.buffer(np.int32, m * k // 32).fill_bytes(0x55)


def quantize(gpu, x):
    x = np.atleast_2d(np.asarray(x, f32))
    m, k = x.shape
    xd = gpu.upload(x, np.float32)
    codes, d8, s8 = planes(gpu, m, k)
    gpu.enqueue_card_quantize(xd, m, k, codes, d8, s8)
    out = codes.download().reshape(m, k), d8.download().reshape(m, -1), s8.download().reshape(m, -1)
    xd.free()
    return out, (codes, d8, s8)


def assert_planes(got, want, what):
    for name, g, w in zip(("codes", "d8", "s8"), got, want):
        g, w = np.ascontiguousarray(g), np.ascontiguousarray(w)
        same = g.view(np.uint8) == w.view(np.uint8)
        assert same.all(), f"{what}: {name} differs at {np.flatnonzero(~same.reshape(-1))[:8]}"


def test_quantizer_edge_columns(gpu):
    gpu.fault_clear()
    for what, col in edge_columns().items():
        got, bufs = quantize(gpu, col)
        assert_planes(got, ora.card_q8_1(col)[:3], what)
        for b in bufs:
            b.free()
    assert gpu.fault() == (bm.FAULT_NONE, 0)


@pytest.mark.parametrize("n_sb", (1, 2, 3, 9, 16, 64))
def test_quantizer_random_columns(gpu, n_sb):
    rng = np.random.default_rng(0xC0DE + n_sb)
    gpu.fault_clear()
    x = rng.uniform(-2, 2, (7, 256 * n_sb)).astype(f32)
    x[rng.integers(0, 7, 12), rng.integers(0, 256 * n_sb, 12)] *= 8
    x[1, :128] = 0
    x[3] *= f32(1e-30)
    x[4] *= f32(1e30)
    got, bufs = quantize(gpu, x)
    assert_planes(got, ora.card_q8_1(x)[:3], f"n_sb={n_sb}")
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    for b in bufs:
        b.free()


def test_a_refused_block_raises_quant_column(gpu):
    gpu.fault_clear()
    x = np.random.default_rng(3).uniform(-2, 2, (2, 512)).astype(f32)
    x[0, 129], x[1, 511] = np.nan, -np.inf
    gpu.set_layer(5)
    got, bufs = quantize(gpu, x)
    w0, mask = gpu.fault(5)
    assert w0 == (5 << 8) | bm.SITE_QUANT_COLUMN and mask == 1 << bm.SITE_QUANT_COLUMN
    want = ora.card_q8_1(x)
    assert list(want[3].reshape(-1)) == [False, True, False, False, False, False, False, True]
    assert_planes(got, want[:3], "refused")  # NaN scale (the same quiet NaN), zero codes and sums; the clean blocks as ever
    gpu.set_layer(bm.LAYER_NONE)
    gpu.fault_clear()
    for b in bufs:
        b.free()


def assert_bits(got, want, what):
    got, want = np.asarray(got, f32), np.asarray(want, f32)
    same = got.view(np.uint32) == want.view(np.uint32)
    assert same.all(), f"{what}: {np.count_nonzero(~same)} of {same.size} differ; first at {int(np.argmin(same))}: " \
                       f"{got[np.argmin(same)]!r} vs {want[np.argmin(same)]!r}"


@pytest.mark.parametrize("wtype", (bm.Q4_K, bm.Q3_K))
@pytest.mark.parametrize("n_sb", (1, 2, 3, 4, 5, 8, 9, 12, 16, 27))
def test_gemv_walks_are_the_mirrors(gpu, wtype, n_sb):
    rng = np.random.default_rng(0xC0DE41A2 + 100 * wtype + n_sb)
    rows, k, m = 21, 256 * n_sb, 3  # 21 rows: the last workgroup has five rows
    w = random_blocks(wtype, rows, k, rng)
    x = rng.uniform(-2, 2, (m, k)).astype(f32)
    x[0, rng.integers(0, k, 4)] *= 8
    (codes, d8, s8), bufs = quantize(gpu, x)
    dw = gpu.weights(wtype, rows, k, w)
    y = gpu.buffer(np.float32, rows * m).fill_bytes(0xFF)
    gpu.enqueue_card_gemv(dw, *bufs, m, y)
    assert_bits(y.download(), ora.card_gemv(wtype, w, rows, k, codes, d8, s8), f"type {wtype} n_sb {n_sb}")
    for b in bufs + (dw, y):
        b.free()


@pytest.mark.parametrize("wtype,k,rpe", ((bm.Q4_K, 768, 2048), (bm.Q3_K, 768, 2048), (bm.Q4_K, 2048, 77)))
def test_gemv_sel_takes_each_slots_expert(gpu, wtype, k, rpe):
    """The card tier's MoE down step at the benchmark layer's down shape (768 -> 2048, eight slots) and a ragged one."""
    rng = np.random.default_rng(77 + wtype + rpe)
    ne, n_slots = 5, 8
    w = random_blocks(wtype, ne * rpe, k, rng)
    x = rng.uniform(-2, 2, (n_slots, k)).astype(f32)
    sel = np.array([4, 0, 2, 2, 0xFFFFFFFF, 1, 3, 0], np.uint32)  # a duplicate and a host slot
    (codes, d8, s8), bufs = quantize(gpu, x)
    dw = gpu.weights(wtype, ne * rpe, k, w)
    seld = gpu.upload(sel, np.uint32)
    y = gpu.buffer(np.float32, n_slots * rpe).fill_bytes(0xFF)
    gpu.fault_clear()
    gpu.enqueue_card_gemv_sel(dw, *bufs, seld, n_slots, rpe, y)
    got = y.download().reshape(n_slots, rpe)
    assert gpu.fault() == (bm.FAULT_NONE, 0)
    assert (got[4].view(np.uint32) == 0xFFFFFFFF).all(), "a host slot's rows stay untouched"
    live = [s for s in range(n_slots) if s != 4]
    want = ora.card_gemv_sel(wtype, w, ne, rpe, k, codes[live], d8[live], s8[live], sel[live]).reshape(len(live), rpe)
    assert_bits(got[live], want, f"type {wtype}")
    # an id past the stack raises ExpertId and leaves its slot untouched
    sel[1] = ne
    seld.upload(sel)
    y.fill_bytes(0xFF)
    gpu.enqueue_card_gemv_sel(dw, *bufs, seld, n_slots, rpe, y)
    w0, mask = gpu.fault()
    assert (w0 & 0xFF) == bm.SITE_EXPERT_ID
    got = y.download().reshape(n_slots, rpe)
    assert (got[1].view(np.uint32) == 0xFFFFFFFF).all()
    assert_bits(got[0], want[0], "slot 0 beside the bad id")
    gpu.fault_clear()
    for b in bufs + (dw, seld, y):
        b.free()


def test_card_entries_refuse_by_name(gpu):
    rng = np.random.default_rng(9)
    dw6 = gpu.weights(bm.Q6_K, 8, 256, random_blocks(bm.Q6_K, 8, 256, rng))
    dw4 = gpu.weights(bm.Q4_K, 8, 256, random_blocks(bm.Q4_K, 8, 256, rng))
    codes, d8, s8 = planes(gpu, 1, 256)
    y, x = gpu.buffer(np.float32, 8), gpu.buffer(np.float32, 384)
    sel = gpu.upload(np.zeros(1, np.uint32), np.uint32)
    for call, code, word in (
        (lambda: gpu.enqueue_card_gemv(dw6, codes, d8, s8, 1, y), bm.ETYPE, "Q4_K (12) and Q3_K (11)"),
        (lambda: gpu.enqueue_card_quantize(x, 1, 384, codes, d8, s8), bm.ESHAPE, "whole 256-value super-blocks"),
        (lambda: gpu.enqueue_card_quantize(x, 0, 256, codes, d8, s8), bm.ESHAPE, "m >= 1"),
        (lambda: gpu.enqueue_card_gemv(dw4, codes, d8, s8, 0, y), bm.ESHAPE, "m = 0"),
        (lambda: gpu.enqueue_card_gemv_sel(dw4, codes, d8, s8, sel, 1, 3, y), bm.ESHAPE, "multiple of rows_per_expert"),
        (lambda: gpu.enqueue_card_gemv_sel(dw4, codes, d8, s8, sel, 0, 8, y), bm.ESHAPE, "n_slots >= 1"),
    ):
        with pytest.raises(bm.GpuError) as e:
            call()
        assert e.value.code == code and word in str(e.value), str(e.value)
    for b in (dw6, dw4, codes, d8, s8, y, x, sel):
        b.free()
