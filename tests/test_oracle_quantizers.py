"""Pins the oracle's weight quantizers (oracle/kquant.c, oracle/iq2xxs_quant.c), which restate the reference's
crates/gguf/src/kquant.rs and crates/gguf/src/iq_quant.rs. The reference holds no golden bytes for them (it checks them
against ggml on its own machine), so three things stand in:
  1. a second spelling written from the reference's text (tests/quant_restatement.py: vectors over all sub-blocks where
     the C walks one at a time) must give the same bytes on the reference tests' own row generators and on the
     benchmark's N(0, 0.02) rows;
  2. what the mathematics fixes: a row built from a legal block whose every product is exact must read back with zero
     error, and an IQ2_XXS group's stored signs must be the input's but for the one flip its parity bit forces, at the
     value the rule names;
  3. the comparison must notice a wrong constant: the same second spelling with one step fewer or more in the Q4_K
     search, or the other tie rule, gives different bytes on these very rows.
CPU only."""
import os

import numpy as np
import pytest

import ora
import quant_restatement as qr
from common import normal_f32
from test_oracle_layer import wave_row

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def tie_row(n, seed):
    """The reference's row of few distinct levels, ties everywhere, with positive importance
    (crates/gguf/src/iq_quant/tests.rs:92-111)."""
    s = [seed]

    def nxt():
        s[0] = (s[0] * 1103515245 + 12345) & 0xFFFFFFFF
        return s[0] >> 8

    levels = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    x = np.empty(n, np.float32)
    for i in range(n):
        r = nxt()
        v = np.float32(levels[r % 8]) * np.float32(0.01)
        x[i] = -v if r & 256 else v
    w = np.array([np.float32(0.1) + np.float32(nxt() % 1000) / np.float32(100.0) for _ in range(n)], np.float32)
    return x, w


def kquant_rows():
    rng = np.random.default_rng(5100)
    rows = [wave_row(2048, seed) for seed in (3, 9, 14)]
    rows += [normal_f32(rng, 2048, 0.02) for _ in range(24)]
    rows += [tie_row(2048, 7)[0], tie_row(2048, 8)[0]]
    sparse = normal_f32(rng, 2048, 0.02)
    sparse[::3] = 0.0
    sparse[256:512] = 0.0            # a zero block
    sparse[512:544] = 0.003          # a flat sub-block
    sparse[1024:1040] = 1e-20        # a group below the Q6_K floor
    rows.append(sparse)
    rows.append(np.abs(normal_f32(rng, 2048, 0.02)))   # all positive: the minimum is clamped to zero
    return np.stack(rows)


@pytest.mark.parametrize("wtype", (ora.Q4_K, ora.Q5_K, ora.Q6_K))
def test_kquant_bytes_equal_the_second_spelling(wtype):
    x = kquant_rows()
    got = ora.quantize_rows(wtype, x, x.shape[0], x.shape[1], n_threads=4)
    want = qr.quantize_q6k(x) if wtype == ora.Q6_K else qr.quantize_q45k(x, q5=wtype == ora.Q5_K)
    bb = ora.BLOCK_BYTES[wtype]
    diff = np.flatnonzero((got.reshape(-1, bb) != want.reshape(-1, bb)).any(axis=1))
    assert diff.size == 0, f"{diff.size} of {got.size // bb} blocks differ, first block {diff[:5]}"


def test_the_comparison_notices_a_wrong_step_count_or_tie_rule():
    x = kquant_rows()
    q4 = ora.quantize_rows(ora.Q4_K, x, x.shape[0], x.shape[1])
    assert not np.array_equal(q4, qr.quantize_q45k(x, nstep=19)), "one step fewer in the Q4_K search went unnoticed"
    assert not np.array_equal(q4, qr.quantize_q45k(x, nstep=21)), "one step more in the Q4_K search went unnoticed"
    assert not np.array_equal(q4, qr.quantize_q45k(x, q5=True)[:q4.size]), "the Q5_K constants went unnoticed"
    q6 = ora.quantize_rows(ora.Q6_K, x, x.shape[0], x.shape[1])
    # the last-maximum rule only matters where a group holds its largest magnitude twice with both signs: the tie rows
    assert not np.array_equal(q6, qr.quantize_q6k(x, first_max=False)), "the other maximum tie rule went unnoticed"


def exact_q4k_blocks(rng, n):
    """Legal Q4_K blocks whose dequantized values are exact f32 products: d = 2^-10, dmin = 2^-9, every sub-block uses
    level 0 and level 15, the largest scale and minimum codes are 63."""
    b = np.zeros((n, 144), np.uint8)
    for i in range(n):
        sc = rng.integers(1, 64, 8)
        m = rng.integers(0, 64, 8)
        sc[rng.integers(0, 8)] = 63
        m[rng.integers(0, 8)] = 63
        q = rng.integers(0, 16, (8, 32))
        q[:, 0], q[:, 1] = 0, 15
        b[i, 0:2] = np.array([2.0 ** -10], np.float16).view(np.uint8)
        b[i, 2:4] = np.array([2.0 ** -9], np.float16).view(np.uint8)
        b[i, 4:16] = qr.pack_scales(sc[None, :], m[None, :])[0]
        qq = q.reshape(4, 2, 32)
        b[i, 16:144] = (qq[:, 0] | (qq[:, 1] << 4)).reshape(-1)
    return b.reshape(-1)


def test_q4k_reads_an_exactly_representable_row_back_exactly():
    rng = np.random.default_rng(5200)
    blocks = exact_q4k_blocks(rng, 48)
    x = qr.dequant_q4k(blocks)
    assert np.array_equal(x, ora.dequant_row(ora.Q4_K, blocks, x.size)), "the two decoders agree on the construction"
    for quantize in (lambda v: ora.quantize_rows(ora.Q4_K, v, 1, v.size), qr.quantize_q45k):
        q = quantize(x)
        back = ora.dequant_row(ora.Q4_K, q, x.size)
        assert np.array_equal(back, x), f"max error {np.abs(back - x).max()}"
        assert np.array_equal(q.reshape(-1, 144)[:, :16], blocks.reshape(-1, 144)[:, :16]), "d, dmin and the scale codes come back"


def test_q6k_reads_an_exactly_representable_row_back_exactly():
    """d = 2^-12, the largest scale -128 (so the block's scale search lands on it), every group holds level -32."""
    rng = np.random.default_rng(5300)
    n = 48
    b = np.zeros((n, 210), np.uint8)
    for i in range(n):
        sc = rng.integers(-100, 101, 16)
        sc[sc == 0] = 7
        sc[rng.integers(0, 16)] = -128
        L = rng.integers(0, 64, (2, 4, 32))
        L[:, :, 0], L[:, :, 16] = 0, 0          # level -32 in each 16-value group
        ql = np.zeros((2, 64), np.int64)
        ql[:, 0:32] = (L[:, 0] & 15) | ((L[:, 2] & 15) << 4)
        ql[:, 32:64] = (L[:, 1] & 15) | ((L[:, 3] & 15) << 4)
        qh = (L[:, 0] >> 4) | ((L[:, 1] >> 4) << 2) | ((L[:, 2] >> 4) << 4) | ((L[:, 3] >> 4) << 6)
        b[i, 0:128], b[i, 128:192] = ql.reshape(-1), qh.reshape(-1)
        b[i, 192:208] = (sc & 0xFF).astype(np.uint8)
        b[i, 208:210] = np.array([2.0 ** -12], np.float16).view(np.uint8)
    blocks = b.reshape(-1)
    x = qr.dequant_q6k(blocks)
    assert np.array_equal(x, ora.dequant_row(ora.Q6_K, blocks, x.size))
    for quantize in (lambda v: ora.quantize_rows(ora.Q6_K, v, 1, v.size), qr.quantize_q6k):
        back = ora.dequant_row(ora.Q6_K, quantize(x), x.size)
        assert np.array_equal(back, x), f"max error {np.abs(back - x).max()}"


# ---------------------------------------------------------------------------------------------------- IQ2_XXS

@pytest.fixture(scope="module")
def grid():
    return qr.Grid(qr.read_iq2xxs_grid(os.path.join(ROOT, "oracle", "iq_tables.h")))


def test_the_second_spellings_grid_is_ggml_init(grid):
    # crates/gguf/src/iq_quant/tests.rs:44-84: the first point codes, and a list is the naive (distance, index) sort
    assert [int(u) for u in grid.word[:8]] == [0, 2, 5, 8, 10, 17, 20, 32]
    assert len(grid.on_grid) == 256
    codes, size, neg, _ = ora.iq2xxs_grid_codes()
    assert size == qr.KMAP_SIZE and np.array_equal(codes.astype(np.int64) & 0xFFFF, grid.word)
    for u in (1, 3, 4, 21845, 43691, 12345):
        kind, pts = grid.lookup(u)
        assert kind == "list"
        a = np.array([(u >> (2 * k)) & 3 for k in range(8)])
        d2 = [int(((2 * (grid.codes[g] - a)) ** 2).sum()) for g in range(256)]
        order = sorted(range(256), key=lambda g: (d2[g], g))
        kept = sorted(set(d2))[:2]
        assert pts == [g for g in order if d2[g] in kept]
    assert grid.lookup(qr.KMAP_SIZE) is None


def iq2_rows():
    rng = np.random.default_rng(5400)
    x_tie, w_tie = tie_row(1024, 7)
    rows = [(x_tie, w_tie), (x_tie, np.ones(1024, np.float32))]
    rows += [(normal_f32(rng, 1024, 0.02), np.ones(1024, np.float32)) for _ in range(3)]
    sparse = normal_f32(rng, 1024, 0.02)
    sparse[256:512] = 0.0
    sparse[512:544] = 0.0
    rows.append((sparse, np.ones(1024, np.float32)))
    return rows


def test_iq2xxs_bytes_equal_the_second_spelling(grid):
    for i, (x, w) in enumerate(iq2_rows()):
        got = ora.quantize_row_iq2xxs(x, w)
        want = qr.quantize_iq2xxs(x, w, grid)
        diff = np.flatnonzero((got.reshape(-1, 66) != want.reshape(-1, 66)).any(axis=1))
        assert diff.size == 0, f"row {i}: blocks {diff} differ"


def test_the_comparison_notices_a_shorter_scale_search(grid):
    rng = np.random.default_rng(5401)
    x, w = normal_f32(rng, 1024, 0.02), np.ones(1024, np.float32)
    assert not np.array_equal(ora.quantize_row_iq2xxs(x, w), qr.quantize_iq2xxs(x, w, grid, steps=5)), \
        "eleven trial scales for thirteen went unnoticed"


def test_iq2xxs_signs_are_the_inputs_but_for_the_parity_repair():
    """What the format fixes: a group of eight stores seven sign bits, the eighth being their parity, so a group with an
    odd number of negative values cannot keep them all. The quantizer flips the value of least weight x^2 (the first of
    equals) and fits the grid to it sign-reversed (crates/gguf/src/iq_quant.rs:489-514). So the stored signs are the
    input's in every group with an even count, and differ in exactly that one place in every other group."""
    odd_groups = 0
    for x, w in iq2_rows()[:4]:
        q = ora.quantize_row_iq2xxs(x, w).reshape(-1, 66)
        for b in range(q.shape[0]):
            xb = x[256 * b:256 * b + 256]
            if not q[b].any():
                continue
            sigma2 = np.float32(np.float32((xb.astype(np.float32) ** 2).sum(dtype=np.float32)) / np.float32(256.0))
            words = q[b, 2:66].copy().view(np.uint32).reshape(8, 2)
            for s in range(8):
                aux = int(words[s, 1])
                xs, ws = xb[32 * s:32 * s + 32], w[256 * b + 32 * s:256 * b + 32 * s + 32]
                if not xs.any():
                    continue
                weight = (ws * np.sqrt(sigma2 + xs * xs)).astype(np.float32)
                for k in range(4):
                    bits = (aux >> (7 * k)) & 127
                    bits |= (bin(bits).count("1") & 1) << 7      # crates/gguf/src/iq_tables.rs:13: bit 7 is the parity
                    stored = np.array([(bits >> i) & 1 for i in range(8)], bool)
                    neg = xs[8 * k:8 * k + 8] < 0
                    if neg.sum() % 2 == 0:
                        assert np.array_equal(stored, neg), (b, s, k)
                    else:
                        odd_groups += 1
                        sq = (weight[8 * k:8 * k + 8] * xs[8 * k:8 * k + 8]).astype(np.float32) * xs[8 * k:8 * k + 8]
                        flip = np.zeros(8, bool)
                        flip[int(np.argmin(sq))] = True
                        assert np.array_equal(stored, neg ^ flip), (b, s, k)
    assert odd_groups > 100
