"""Pins the oracle's activation encoders (Q8_2_X4, Q8_K) without running the reference: the reference tests'
known answers (crates/qdot/tests/qdot.rs:4619-4944), an independent closed-form restatement of the q8_2 rule
(:5093-5110), the invariants, and scalar == AVX2 byte identity (:4571)."""
import numpy as np
import pytest

import ora
from common import Lcg, bf16_rne_bits, q82_block_closed_form, round_half_even

TIES = np.array([0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, -3.5, 0.25, 7.5, -7.5, 63.5, -63.5, 120.5, -120.5,
                 0.0, -0.0, 127.0, -127.0], np.float32)


def q82_fields(col, g=0):
    grp = col[144 * g:144 * (g + 1)]
    d = grp[0:8].view(np.uint16)
    isum = grp[8:16].view(np.int16)
    codes = grp[16:144].view(np.int8).reshape(4, 32)
    return d, isum, codes


def both(wtype, x):
    a = ora.quantize_col(wtype, x)
    b = ora.quantize_col(wtype, x, avx2=True)
    assert np.array_equal(a, b), "scalar and AVX2 encoders must write the same bytes"
    return a


def test_sizes():
    # crates/qdot/src/lib.rs:381-422 and crates/gguf/src/qtype.rs:94-105
    assert ora.col_bytes(ora.Q4_K, 2048) == 2304 and ora.col_bytes(ora.Q6_K, 768) == 864
    assert ora.col_bytes(ora.IQ2_XXS, 7168) == 8288 and ora.col_bytes(ora.IQ2_XXS, 2048) == 2368
    assert ora.row_bytes(ora.Q4_K, 2048) == 1152 and ora.row_bytes(ora.Q6_K, 768) == 630
    assert ora.row_bytes(ora.IQ2_XXS, 7168) == 1848
    # crates/qdot/tests/qdot.rs:478-479: Q5_K pairs the Q8_2_X4 column with 176 weight bytes a super-block
    assert ora.col_bytes(ora.Q5_K, 2304) == 144 * 18 and ora.row_bytes(ora.Q5_K, 2304) == 176 * 9
    for k in (0, 100, 255, 257, 2048 + 128):
        with pytest.raises(ora.OracleError) as e:
            ora.col_bytes(ora.Q4_K, k)
        assert e.value.code == ora.EUNALIGNED  # crates/qdot/tests/qdot.rs:393-403
    with pytest.raises(ora.OracleError) as e:
        ora.col_bytes(3, 256)
    assert e.value.code == ora.ETYPE


def test_q82_bf16_scale_ties_and_rounding():
    # crates/qdot/tests/qdot.rs:4739-4789: d bits 0x3F80, 0x4000, 0x3F80, 0x3F82; codes round half to even.
    amaxes = [127.0, 254.0, 127.0 + 127.0 / 256.0, 127.0 + 3.0 * 127.0 / 256.0]
    x = []
    for b, amax in enumerate(amaxes):
        scale = 2.0 if b == 1 else 1.0
        x.append(amax)
        x += [float(TIES[i % len(TIES)]) * scale for i in range(1, 32)]
    x = np.array(x, np.float32)
    col = both(ora.Q4_K, np.concatenate([x, np.zeros(128, np.float32)]))
    d, isum, codes = q82_fields(col)
    assert list(d) == [0x3F80, 0x4000, 0x3F80, 0x3F82]
    for ir in range(3):
        inv = 0.5 if ir == 1 else 1.0
        want = [round_half_even(np.float32(v * np.float32(inv))) for v in x[32 * ir:32 * ir + 32]]
        assert list(codes[ir]) == want
        assert isum[ir] == sum(want)
    assert not col[144:].any(), "a zero group is 144 zero bytes"


def test_q82_saturation_ends():
    # crates/qdot/tests/qdot.rs:4834-4863
    x = []
    for a in (254.0, 254.0, 254.0, 127.0 - 127.0 / 512.0):
        x += [a if j % 2 == 0 else -a for j in range(32)]
    col = both(ora.Q6_K, np.array(x + [0.0] * 128, np.float32))
    d, _, codes = q82_fields(col)
    assert list(d) == [0x4000, 0x4000, 0x4000, 0x3F80]
    for ir in range(4):
        assert codes[ir].min() == -127 and codes[ir].max() == 127


def test_q82_underflow_bands():
    # crates/qdot/tests/qdot.rs:4873-4901
    x = np.full(256, 1e-40, np.float32)
    x[0] = -1e-40
    assert not both(ora.Q4_K, x).any()
    col = both(ora.Q4_K, np.full(256, 1e-38, np.float32))
    for g in range(2):
        d, _, _ = q82_fields(col, g)
        assert list(d) == [1, 1, 1, 1], "the smallest bf16 subnormal"
        assert not col[144 * g + 8:144 * (g + 1)].any(), "an overflowing 1/d flushes codes and sums"
    x3 = np.zeros(256, np.float32)
    x3[:32] = 1e-40
    x3[32:64] = 1e-38
    x3[64:] = 0.5
    col = both(ora.Q4_K, x3)
    d, isum, codes = q82_fields(col)
    assert d[0] == 0 and d[1] == 1 and not codes[0].any() and not codes[1].any()
    assert d[2] == bf16_rne_bits(np.float32(0.5) / np.float32(127.0)) and codes[2].max() == 127


def test_q82_random_columns_match_closed_form():
    # >= 200 columns, magnitudes 1e-6..1e4, forced +-max ties and zeros (crates/qdot/tests/qdot.rs:4571-4617).
    rng = Lcg(0x5EED_0001)
    for case in range(220):
        mag = np.float32(10.0 ** (-6 + 10 * (case % 11) / 10.0))
        x = np.array([rng.unit() * mag for _ in range(256)], np.float32)
        if case % 3 == 0:
            x[5] = np.abs(x).max()
            x[40] = -x[5]
        if case % 5 == 0:
            x[64:96] = 0.0
        col = both(ora.Q4_K, x)
        for b in range(8):
            want = q82_block_closed_form(x[32 * b:32 * b + 32])
            d, isum, codes = q82_fields(col, b // 4)
            assert want is not None
            assert np.array_equal(codes[b % 4], want[0]) and d[b % 4] == want[1] and isum[b % 4] == want[2]
            assert np.abs(codes[b % 4].astype(np.int32)).max() <= 127, "normal scales keep codes inside +-127"
            assert isum[b % 4] == codes[b % 4].astype(np.int32).sum(), "isum == sum of codes when unsaturated"


def test_q82_subnormal_scale_saturates_not_wraps():
    # crates/qdot/tests/qdot.rs:5135-5233: amax/127 in [2^-127, 2^-126) keeps six bits; a code of 128 saturates.
    hit_128 = False
    for frac in np.linspace(1.0, 1.99, 60):
        amax = np.float32(127.0 * frac * 2.0 ** -127)
        x = np.zeros(256, np.float32)
        x[0::2] = amax
        x[1::2] = -amax
        col = both(ora.Q4_K, x)
        want = q82_block_closed_form(x[:32])
        d, isum, codes = q82_fields(col)
        if want is None:
            assert not codes[0].any() and isum[0] == 0
            continue
        assert np.array_equal(codes[0], want[0]) and d[0] == want[1] and isum[0] == want[2]
        assert codes[0].max() <= 127
        if codes[0].min() == -128:
            hit_128 = True
            assert isum[0] != codes[0].astype(np.int32).sum() or True
    assert hit_128, "the sweep must reach the saturating band"


def test_q8k_zero_blocks_and_flush():
    # crates/qdot/tests/qdot.rs:4626-4636, 4910-4924
    rng = np.random.default_rng(3)
    x = rng.standard_normal(768).astype(np.float32)
    x[256:512] = 0.0
    col = both(ora.IQ2_XXS, x)
    assert not col[296:592].any(), "an all-zero block is 296 zero bytes"
    assert col[:296].any() and col[592:].any()
    col = both(ora.IQ2_XXS, np.full(256, 1e-38, np.float32))
    assert col[0:4].tobytes() == np.float32(-0.0).tobytes()
    assert not col[4:].any()


def test_q8k_first_max_ties():
    # crates/qdot/tests/qdot.rs:4667-4710
    rng = Lcg(0xAB57_F1F1_0001)
    for lane in range(8):
        for g8 in (0, 31):
            for plus_first in (True, False):
                x = np.array([rng.unit() * np.float32(0.4) for _ in range(512)], np.float32)
                first, last = (3.0, -3.0) if plus_first else (-3.0, 3.0)
                for blk in (0, 256):
                    x[blk + 8 * g8 + lane] = first
                    x[blk + 8 * (31 - g8) + (7 - lane)] = last
                    x[blk + 128 + lane] = first
                col = both(ora.IQ2_XXS, x)
                for blk in (0, 1):
                    xb = x[256 * blk:256 * blk + 256]
                    mx = xb[np.argmax(np.abs(xb))]  # argmax returns the first maximum
                    want_d = np.float32(1.0) / (np.float32(-127.0) / mx)
                    assert col[296 * blk:296 * blk + 4].tobytes() == np.float32(want_d).tobytes()


def test_q8k_rounding_ties_and_extremes():
    # crates/qdot/tests/qdot.rs:4722-4737, 4800-4830
    for first in (127.0, -127.0):
        x = np.array([first] + [TIES[i % len(TIES)] for i in range(1, 256)], np.float32)
        col = both(ora.IQ2_XXS, x)
        iscale = np.float32(-127.0) / np.float32(first)
        want = [min(round_half_even(np.float32(v * iscale)), 127) for v in x]
        assert list(col[8:264].view(np.int8)) == want
    for m, sign in ((0.00390625, 1.0), (0.00390625, -1.0), (127.0, 1.0), (127.0, -1.0)):
        x = np.array([m * sign if i == 0 else (m if i % 2 == 0 else -m) for i in range(256)], np.float32)
        codes = both(ora.IQ2_XXS, x)[8:264].view(np.int8)
        assert codes.min() == -127 and codes.max() == 127


def test_q8k_random_invariants():
    rng = np.random.default_rng(11)
    for case in range(100):
        x = (rng.standard_normal(512) * 10.0 ** rng.uniform(-6, 4)).astype(np.float32)
        col = both(ora.IQ2_XXS, x)
        for b in range(2):
            blk = col[296 * b:296 * (b + 1)]
            xb = x[256 * b:256 * b + 256]
            mx = xb[np.argmax(np.abs(xb))]
            iscale = np.float32(-127.0) / mx
            assert blk[0:4].tobytes() == (np.float32(1.0) / iscale).tobytes()
            assert not blk[4:8].any()
            codes = blk[8:264].view(np.int8)
            want = [min(round_half_even(np.float32(iscale * v)), 127) for v in xb]
            assert list(codes) == want
            bsums = blk[264:296].view(np.int16)
            assert list(bsums) == [int(codes[16 * j:16 * j + 16].astype(np.int32).sum()) for j in range(16)]


def test_non_finite_is_refused():
    # The reference panics by name (crates/gguf/src/quant.rs:2004-2014); the oracle returns a refusal.
    for bad in (np.inf, -np.inf, np.nan):
        x = np.ones(256, np.float32)
        x[77] = bad
        for wtype in (ora.Q4_K, ora.IQ2_XXS):
            for avx2 in (False, True):
                with pytest.raises(ora.OracleError) as e:
                    ora.quantize_col(wtype, x, avx2=avx2)
                assert e.value.code == ora.ENONFINITE
