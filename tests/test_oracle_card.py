"""The card rule's oracle (oracle/card.c) pinned without the GPU: the q8_1 quantizer by the worked cases of the
reference's own test (crates/qdot/tests/qdot.rs:7942-8040) and an independent numpy restatement; the Q4_K and Q3_K row
walks by the reference test's f64 band around the dequantized dot (qdot.rs:8043-8098), by rows with one live lane whose
value is a short f32 chain worked here, and by a second spelling of each walk written from the device's loops
(crates/gpu/src/cores.rs:536-620: the pair loop over the guard-free prefix, then the guarded tail) over the codes the
independent block decoders give."""
import numpy as np
import pytest

import ora
from test_oracle_dots import q3k_decode, q4k_decode, random_blocks
from test_oracle_layer import fma32

f32 = np.float32


# ------------------------------------------------------------------------------------------------ the quantizer

def numpy_q8_1(x):
    """Written from the rule's text: d = amax / 127 (1 for a zero block), codes v / d rounded half away from zero and
    held to +-127, a sum per 32 codes; a block with a value that is not finite is a NaN scale over zero codes."""
    x = np.asarray(x, f32).reshape(-1, 128)
    bad = ~np.isfinite(x).all(axis=1)
    amax = np.abs(np.where(np.isfinite(x), x, 0)).max(axis=1)
    with np.errstate(all="ignore"):
        d = np.where(amax > 0, amax / f32(127), f32(1)).astype(f32)
        q = (x / d[:, None]).astype(f32)
        r = np.sign(q) * np.floor(np.abs(q).astype(np.float64) + 0.5)  # exact in f64: no second rounding at 0.49999997
        r = np.where(np.isnan(q), 0, np.clip(r, -127, 127))
    codes = np.where(bad[:, None], 0, r).astype(np.int8)
    d = np.where(bad, f32(np.nan), d).astype(f32)
    return codes.reshape(-1), d, codes.reshape(-1, 32).astype(np.int32).sum(axis=1), bad


def both(x, what):
    codes, d8, s8, refused = (a[0] for a in ora.card_q8_1(np.asarray(x, f32)[None, :]))
    c2, d2, s2, r2 = numpy_q8_1(x)
    assert np.array_equal(codes, c2), f"{what}: codes differ at {np.flatnonzero(codes != c2)[:8]}"
    assert np.array_equal(d8.view(np.uint32), d2.view(np.uint32)) and np.array_equal(s8, s2) and np.array_equal(refused, r2), what
    return codes, d8, s8, refused


def test_ties_round_half_away_from_zero():
    ties = np.zeros(512, f32)
    for i in range(512):
        j, sign = i % 128, 1.0 if (i // 128) % 2 == 0 else -1.0
        if j == 0:
            ties[i] = 127.0  # the scale is exactly 1
        else:
            m = float((j - 1) // 3)
            ties[i] = sign * (m + 0.5, m, m + 0.25)[(j - 1) % 3]
    codes, d8, _, _ = both(ties, "ties")
    assert (d8 == 1.0).all()
    want = np.minimum(np.floor(np.abs(ties).astype(np.float64) + 0.5), 127) * np.sign(ties)
    assert np.array_equal(codes.astype(np.float64), want)
    assert codes[1] == 1 and codes[7] == 3 and codes[128 + 1] == -1  # 0.5 -> 1, 2.5 -> 3 (half-even would give 0, 2)


def test_near_ties_and_the_clamp():
    near = np.zeros(1024, f32)
    near[0], i = 127.0, 1
    for m in range(127):
        for frac in (f32(0.5), f32(0.49999997), f32(0.50000006)):
            if i + 1 < near.size:
                near[i], near[i + 1] = f32(m) + frac, -(f32(m) + frac)
                i += 2
    near[128::128] = 127.0
    codes, _, _, _ = both(near, "near ties")
    assert codes[1] == 1 and codes[3] == 0 and codes[5] == 1  # 0.5, the float below it, the float above it
    assert np.abs(codes.astype(int)).max() == 127


def test_zero_subnormal_and_underflowed_scales():
    tiny = np.zeros(512, f32)
    tiny[128:256] = (np.arange(128, dtype=f32) - 64) * f32(1e-40)
    one = np.array([1], np.uint32).view(f32)[0]
    tiny[256], tiny[257] = one, -one
    tiny[384], tiny[385] = np.finfo(f32).tiny, -np.finfo(f32).tiny / f32(3)
    codes, d8, s8, refused = both(tiny, "tiny")
    assert d8[0] == 1.0 and not codes[:128].any()
    assert d8[2].view(np.uint32) == 0, "the smallest subnormal over 127 underflows to zero"
    assert tuple(codes[256:259]) == (127, -127, 0), "v / 0 is an infinity (the clamp's end), 0 / 0 a NaN (code 0)"
    assert codes[128] == -127 and codes[128 + 64] == 0 and codes[255] == 125 and not refused.any()


@pytest.mark.parametrize("n_sb", (1, 2, 3, 9, 16))
def test_random_columns_zero_blocks_and_refusals(n_sb):
    rng = np.random.default_rng(0xC0DE + n_sb)
    for case in range(8):
        col = rng.uniform(-2, 2, 256 * n_sb).astype(f32)
        col[rng.integers(0, col.size, 3)] *= 8
        if case % 4 == 1:
            col[:128] = 0
        if case % 4 == 2:
            col[129] = np.nan
        if case % 4 == 3:
            col[-1] = -np.inf
        codes, d8, s8, refused = both(col, f"random n_sb={n_sb} case={case}")
        assert np.array_equal(refused, ~np.isfinite(col.reshape(-1, 128)).all(axis=1))
        for b in np.flatnonzero(refused):
            assert np.isnan(d8[b]) and not codes[128 * b:128 * b + 128].any() and not s8[4 * b:4 * b + 4].any()
        assert np.array_equal(s8, codes.reshape(-1, 32).astype(np.int32).sum(axis=1))
    assert pytest.raises(ora.OracleError, ora.card_q8_1, np.zeros((1, 128), f32)).value.args[0].endswith("-1")


# ------------------------------------------------------------------------------------------------ the row walks

def butterfly(v):
    v = [f32(x) for x in v]
    for stride in (16, 8, 4, 2, 1):
        for lane in range(32):
            if lane & stride == 0:
                v[lane] = f32(v[lane] + v[lane | stride])
    return v[0]


def q4k_walk_by_the_device_loop(row, k, codes, d8, s8):
    """The device's loop shape (crates/gpu/src/cores.rs:568-617) over independently decoded blocks: iterations whose
    four super-blocks all exist go two at a time, the first term's product rounded before it is added, the second
    fused; what is left goes one at a time behind the guard, fused."""
    n_sb = k // 256
    blocks = [q4k_decode(row[144 * i:144 * i + 144]) for i in range(n_sb)]
    lanes = []
    for lane in range(32):
        s, grp = lane & 7, lane >> 3

        def term(it):
            sbp = 4 * it + grp
            q, _, (d, dmin, sc, mn) = blocks[sbp]
            c = codes[256 * sbp + 32 * s:256 * sbp + 32 * s + 32].astype(np.int64)
            a, b = int(((q[32 * s:32 * s + 32] - 8) * c).sum()), int(c.sum())
            assert b == s8[8 * sbp + s]
            cda = f32(f32(d) * f32(sc[s]))
            cdb = f32(f32(f32(8) * f32(d)) * f32(sc[s]) - f32(f32(dmin) * f32(mn[s])))  # crates/gpu/src/cores.rs:262
            return fma32(cda, f32(a), f32(cdb * f32(b))), d8[2 * sbp + (s >> 2)]

        f, it, full, iters = f32(0), 0, n_sb // 4, (n_sb + 3) // 4
        while it + 2 <= full:
            (x0, e0), (x1, e1) = term(it), term(it + 1)
            f = f32(f + f32(e0 * x0))
            f = fma32(e1, x1, f)
            it += 2
        while it < iters:
            if 4 * it + grp < n_sb:
                x, e = term(it)
                f = fma32(e, x, f)
            it += 1
        lanes.append(f)
    return butterfly(lanes)


def q3k_walk_by_the_device_loop(row, k, codes, d8):
    """Lane (half, w16) of iteration `it` takes super-block 2 it + half: the four values 4 (w16 & 7) .. + 3 of each
    32-value quarter of its 128-value half w16 >> 3, every quarter's integer dot times its 16-value group's scale,
    folded as fma(e * d, a, f)."""
    n_sb = k // 256
    blocks = [q3k_decode(row[110 * i:110 * i + 110]) for i in range(n_sb)]
    lanes = []
    for lane in range(32):
        w16, half = lane & 15, lane >> 4
        f = f32(0)
        for it in range((n_sb + 1) // 2):
            sbp = 2 * it + half
            if sbp >= n_sb:
                continue
            q, _, (d, sc) = blocks[sbp]
            a = 0
            for fld in range(4):
                at = 128 * (w16 >> 3) + 32 * fld + 4 * (w16 & 7)
                c = codes[256 * sbp + at:256 * sbp + at + 4].astype(np.int64)
                a += int((q[at:at + 4] * c).sum()) * sc[at // 16]
            f = fma32(f32(d8[2 * sbp + (w16 >> 3)] * f32(d)), f32(a), f)
        lanes.append(f)
    return butterfly(lanes)


def card_rows(wtype, rows, n_sb, rng):
    return random_blocks(wtype, rows * n_sb, rng).reshape(rows, -1)


@pytest.mark.parametrize("wtype", (ora.Q4_K, ora.Q3_K))
@pytest.mark.parametrize("n_sb", (1, 2, 3, 4, 5, 8, 9, 12, 16))
def test_walks_equal_the_device_loops_spelling_and_sit_in_the_f64_band(wtype, n_sb):
    rng = np.random.default_rng(0xC0DE41A2 + 100 * wtype + n_sb)
    k = 256 * n_sb
    w = card_rows(wtype, 3, n_sb, rng)
    x = rng.uniform(-2, 2, (2, k)).astype(f32)
    x[0, rng.integers(0, k, 4)] *= 8
    codes, d8, s8, _ = ora.card_q8_1(x)
    for r in range(3):
        deq = ora.dequant_row(wtype, w[r], k).astype(np.float64)
        for c in range(2):
            got = ora.card_dot_row(wtype, w[r], k, codes[c], d8[c], s8[c])
            want = q4k_walk_by_the_device_loop(w[r], k, codes[c], d8[c], s8[c]) if wtype == ora.Q4_K else \
                q3k_walk_by_the_device_loop(w[r], k, codes[c], d8[c])
            assert got.view(np.uint32) == want.view(np.uint32), f"row {r} col {c}: {got!r} vs {want!r}"
            terms = deq * (codes[c].astype(np.float64) * np.repeat(d8[c].astype(np.float64), 128))
            assert abs(float(got) - terms.sum()) <= 1e-5 * max(np.abs(terms).sum(), np.finfo(np.float64).tiny)
    # the gemv orders: y[r * m + c]; slots take their expert's rows
    y = ora.card_gemv(wtype, w.reshape(-1), 3, k, codes, d8, s8)
    assert y[1 * 2 + 1].view(np.uint32) == ora.card_dot_row(wtype, w[1], k, codes[1], d8[1], s8[1]).view(np.uint32)
    ys = ora.card_gemv_sel(wtype, w.reshape(-1), 3, 1, k, codes, d8, s8, [2, 0])
    assert ys[0].view(np.uint32) == y[2 * 2 + 0].view(np.uint32) and ys[1].view(np.uint32) == y[0 * 2 + 1].view(np.uint32)
    with pytest.raises(ora.OracleError):
        ora.card_gemv_sel(wtype, w.reshape(-1), 3, 1, k, codes, d8, s8, [3, 0])


def test_the_split_terms_round_their_product_first():
    """A row where the two roundings differ. Lane 0 is the only live lane (every other lane's codes are zero), with a
    term in iteration 0 and one in iteration 2. Over sixteen super-blocks the prefix is iterations 0 .. 3, so
    iteration 2's term is added as a rounded product; over twelve (prefix 0 .. 1, iteration 2 behind the guard) the same
    term is fused. Both are checked against the chain worked here, and some case must separate the two."""
    rng = np.random.default_rng(5)
    shown = False
    for _ in range(100):
        blk = random_blocks(ora.Q4_K, 1, rng)
        x = np.zeros(4096, f32)
        x[:32] = rng.uniform(-2, 2, 32)
        x[127] = 3.0  # a scale that is not a power of two
        x[2048:2080] = rng.uniform(-2, 2, 32)
        codes, d8, s8, _ = ora.card_q8_1(x)
        codes[0, 32:128], codes[0, 2080:2176] = 0, 0
        s8[0] = codes[0].reshape(-1, 32).astype(np.int32).sum(axis=1)
        zero = np.zeros(144, np.uint8)
        row16 = np.concatenate([blk] + [zero] * 7 + [blk] + [zero] * 7)
        q, _, (d, dmin, sc, mn) = q4k_decode(blk)

        def x_of(at):
            c = codes[0, at:at + 32].astype(np.int64)
            cda = f32(f32(d) * f32(sc[0]))
            cdb = f32(f32(f32(8) * f32(d)) * f32(sc[0]) - f32(f32(dmin) * f32(mn[0])))
            return fma32(cda, f32(int(((q[:32] - 8) * c).sum())), f32(cdb * f32(int(c.sum()))))

        x0, x2 = x_of(0), x_of(2048)
        f1 = f32(d8[0, 0] * x0)
        split, fused = f32(f1 + f32(d8[0, 16] * x2)), fma32(d8[0, 16], x2, f1)
        got16 = ora.card_dot_row(ora.Q4_K, row16, 4096, codes[0], d8[0], s8[0])
        got12 = ora.card_dot_row(ora.Q4_K, row16[:12 * 144], 3072, codes[0, :3072], d8[0, :24], s8[0, :96])
        assert got16.view(np.uint32) == split.view(np.uint32) and got12.view(np.uint32) == fused.view(np.uint32)
        shown = shown or split.view(np.uint32) != fused.view(np.uint32)
    assert shown, "no case separated the split order from the fused one"


def test_a_refused_block_gives_a_nan_dot():
    rng = np.random.default_rng(6)
    x = rng.uniform(-2, 2, 512).astype(f32)
    x[300] = np.inf
    codes, d8, s8, refused = ora.card_q8_1(x)
    assert list(refused[0]) == [False, False, True, False]
    for wtype in (ora.Q4_K, ora.Q3_K):
        assert np.isnan(ora.card_dot_row(wtype, card_rows(wtype, 1, 2, rng)[0], 512, codes[0], d8[0], s8[0]))
    for wtype in (ora.Q5_K, ora.Q6_K):
        with pytest.raises(ora.OracleError):
            ora.card_dot_row(wtype, np.zeros(1024, np.uint8), 512, codes[0], d8[0], s8[0])
