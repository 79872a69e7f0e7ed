"""Pins the oracle's block decoders, integer sums and fp32 row dots without running the reference:
the ggml-made IQ2_XXS block the reference holds (crates/gguf/src/quant.rs:3678-3745), the codebook digests
(crates/gguf/src/iq_tables.rs:13,26), independent numpy decoders with brute-force integer sums, bit-equality of
the scalar and AVX2 restatements (the reference's first gate, crates/qdot/tests/qdot.rs:738,818,2664), tiles equal
to one column (:5697,6411,6176) and an f64 band around the dequantized dot (crates/qdot/tests/quant_rows.rs:44-66,
crates/qdot/tests/qdot.rs:2696-2757)."""
import hashlib
import json
import os
import struct

import numpy as np
import pytest

import ora
from common import KVALUES_IQ4NL, iq4xs_rows, normal_f32, q3k_rows

HERE = os.path.dirname(os.path.abspath(__file__))
TYPES = (ora.Q3_K, ora.Q4_K, ora.Q5_K, ora.Q6_K, ora.IQ2_XXS, ora.IQ3_XXS, ora.IQ4_XS)


# ---------------------------------------------------------------- independent numpy decoders (written from the
# layout tables, not from the oracle's C): integer codes per value and the f64 value of each weight.

def f16(b0, b1):
    return float(np.array([int(b0) | (int(b1) << 8)], np.uint16).view(np.float16)[0])


def parse_tables():
    """The codebook out of the shipped header, so the digest test covers what the kernels compile in."""
    import re
    out = {}
    for path in ("oracle/iq_tables.h", "bloomery_amd/csrc/iq2xxs_tables.h"):
        text = open(os.path.join(HERE, "..", path)).read()
        grid = [int(v, 16) for v in re.findall(r"0x([0-9a-f]{16})ULL", text)]
        ks = re.search(r"KSIGNS_IQ2XS\[128\] = \{(.*?)\};", text, re.S).group(1)
        out[path] = (grid, [int(v) for v in re.findall(r"\d+", ks)])
    return out


GRID, KSIGNS = parse_tables()["oracle/iq_tables.h"]


def parse_grid3():
    import re
    out = {}
    for path in ("oracle/iq_tables.h", "bloomery_amd/csrc/iq2xxs_tables.h"):
        text = open(os.path.join(HERE, "..", path)).read()
        body = re.search(r"IQ3XXS_GRID\[256\] = \{(.*?)\};", text, re.S).group(1)
        out[path] = [int(v, 16) for v in re.findall(r"0x([0-9a-f]{8})u", body)]
    return out


GRID3 = parse_grid3()["oracle/iq_tables.h"]


def q3k_decode(blk):
    """block_q3_K (crates/gguf/src/quant.rs:671-678): 32 high-bit bytes, 64 bytes of two-bit fields, twelve scale bytes
    (sixteen six-bit scales: four low bits in bytes 96..103, the two high bits in 104..107), d."""
    d = f16(blk[108], blk[109])
    sb = [int(v) for v in blk[96:108]]
    sc = []
    for j in range(16):
        low = (sb[j % 8] >> (4 * (j // 8))) & 15
        high = (sb[8 + j % 4] >> (2 * (j // 4))) & 3
        sc.append((low | (high << 4)) - 32)
    codes = np.zeros(256, np.int64)
    for n in range(256):
        half, field, cell = n // 128, (n // 32) % 4, n % 32
        low = (int(blk[32 + 32 * half + cell]) >> (2 * field)) & 3
        high = (int(blk[cell]) >> (4 * half + field)) & 1
        codes[n] = low - (0 if high else 4)
    vals = np.array([d * sc[n // 16] * codes[n] for n in range(256)], np.float64)
    return codes, vals, (d, sc)


def q4k_decode(blk):
    d, dmin = f16(blk[0], blk[1]), f16(blk[2], blk[3])
    q = [int(v) for v in blk[4:16]]
    sc, mn = [], []
    for j in range(8):
        if j < 4:
            sc.append(q[j] & 63)
            mn.append(q[j + 4] & 63)
        else:
            sc.append((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4))
            mn.append((q[j + 4] >> 4) | ((q[j] >> 6) << 4))
    qs = blk[16:144]
    codes = np.zeros(256, np.int64)
    for p in range(4):
        codes[64 * p:64 * p + 32] = qs[32 * p:32 * p + 32] & 0xF
        codes[64 * p + 32:64 * p + 64] = qs[32 * p:32 * p + 32] >> 4
    vals = np.array([d * sc[n // 32] * codes[n] - dmin * mn[n // 32] for n in range(256)], np.float64)
    return codes, vals, (d, dmin, sc, mn)


def q5k_decode(blk):
    """block_q5_K (crates/gguf/src/quant.rs:769-816): Q4_K's header, 32 high-bit bytes, then Q4_K's nibbles."""
    low, _, (d, dmin, sc, mn) = q4k_decode(np.concatenate([blk[0:16], blk[48:176]]))
    qh = blk[16:48]
    codes = low + np.array([((int(qh[n % 32]) >> (n // 32)) & 1) << 4 for n in range(256)], np.int64)
    vals = np.array([d * sc[n // 32] * codes[n] - dmin * mn[n // 32] for n in range(256)], np.float64)
    return codes, vals, (d, dmin, sc, mn)


def q6k_decode(blk):
    ql, qh, scb = blk[0:128], blk[128:192], blk[192:208].view(np.int8)
    d = f16(blk[208], blk[209])
    codes = np.zeros(256, np.int64)
    for c in range(2):
        for l in range(32):
            h = int(qh[32 * c + l])
            codes[128 * c + l] = (int(ql[64 * c + l]) & 0xF) | ((h & 3) << 4)
            codes[128 * c + 32 + l] = (int(ql[64 * c + 32 + l]) & 0xF) | (((h >> 2) & 3) << 4)
            codes[128 * c + 64 + l] = (int(ql[64 * c + l]) >> 4) | (((h >> 4) & 3) << 4)
            codes[128 * c + 96 + l] = (int(ql[64 * c + 32 + l]) >> 4) | (((h >> 6) & 3) << 4)
    codes -= 32
    vals = np.array([d * int(scb[n // 16]) * codes[n] for n in range(256)], np.float64)
    return codes, vals, (d, scb)


def iq2xxs_decode(blk):
    d = f16(blk[0], blk[1])
    codes = np.zeros(256, np.int64)
    scs = []
    for b in range(8):
        w = blk[2 + 8 * b:10 + 8 * b]
        aux = int(w[4]) | (int(w[5]) << 8) | (int(w[6]) << 16) | (int(w[7]) << 24)
        scs.append(aux >> 28)
        for l in range(4):
            g = GRID[int(w[l])]
            s = KSIGNS[(aux >> (7 * l)) & 127]
            for j in range(8):
                mag = (g >> (8 * j)) & 0xFF
                codes[32 * b + 8 * l + j] = -mag if (s >> j) & 1 else mag
    vals = np.array([d * (0.5 + scs[n // 32]) * 0.25 * codes[n] for n in range(256)], np.float64)
    return codes, vals, (d, scs)


def iq3xxs_decode(blk):
    """block_iq3_xxs (crates/gguf/src/quant.rs:1739-1747): d, 64 grid indices (eight a sub-block, four magnitudes a
    word), then a word a sub-block: four 7-bit sign indices and the scale in the top nibble."""
    d = f16(blk[0], blk[1])
    codes = np.zeros(256, np.int64)
    scs = []
    for b in range(8):
        aux = int(blk[66 + 4 * b]) | (int(blk[67 + 4 * b]) << 8) | (int(blk[68 + 4 * b]) << 16) | (int(blk[69 + 4 * b]) << 24)
        scs.append(aux >> 28)
        for l in range(4):
            s = KSIGNS[(aux >> (7 * l)) & 127]
            for j in range(8):
                g = GRID3[int(blk[2 + 8 * b + 2 * l + j // 4])]
                mag = (g >> (8 * (j % 4))) & 0xFF
                codes[32 * b + 8 * l + j] = -mag if (s >> j) & 1 else mag
    vals = np.array([d * (0.5 + scs[n // 32]) * 0.5 * codes[n] for n in range(256)], np.float64)
    return codes, vals, (d, scs)


def iq4xs_decode(blk):
    """block_iq4_xs (crates/gguf/src/quant.rs:1969-1976): d, scales_h, scales_l[4], then sixteen bytes a sub-block,
    low nibbles its first sixteen values, high nibbles the other sixteen."""
    d = f16(blk[0], blk[1])
    sh = int(blk[2]) | (int(blk[3]) << 8)
    ls = [(((int(blk[4 + b // 2]) >> (4 * (b % 2))) & 15) | (((sh >> (2 * b)) & 3) << 4)) - 32 for b in range(8)]
    codes = np.zeros(256, np.int64)
    for b in range(8):
        q = blk[8 + 16 * b:24 + 16 * b].astype(np.int64)
        codes[32 * b:32 * b + 16] = KVALUES_IQ4NL[q & 15]
        codes[32 * b + 16:32 * b + 32] = KVALUES_IQ4NL[q >> 4]
    vals = np.array([d * ls[n // 32] * codes[n] for n in range(256)], np.float64)
    return codes, vals, (d, ls)


DECODE = {ora.Q3_K: q3k_decode, ora.IQ3_XXS: iq3xxs_decode, ora.IQ4_XS: iq4xs_decode, ora.Q4_K: q4k_decode, ora.Q5_K: q5k_decode, ora.Q6_K: q6k_decode, ora.IQ2_XXS: iq2xxs_decode}


def act_codes(wtype, col, k):
    """Integer codes and f64 scales of an activation column, read from its bytes."""
    if wtype in ora.Q8K_TYPES:
        blocks = col.reshape(-1, 296)
        codes = np.concatenate([b[8:264].view(np.int8).astype(np.int64) for b in blocks])
        scale = np.concatenate([np.full(256, float(b[0:4].view(np.float32)[0])) for b in blocks])
    else:
        groups = col.reshape(-1, 144)
        codes = np.concatenate([g[16:144].view(np.int8).astype(np.int64) for g in groups])
        scale = np.concatenate([np.repeat((g[0:8].view(np.uint16).astype(np.uint32) << 16).view(np.float32)
                                          .astype(np.float64), 32) for g in groups])
    return codes[:k], scale[:k]


def random_blocks(wtype, nb, rng):
    """Raw random block bytes with sane f16 scales: every code pattern is a legal block."""
    bb = ora.BLOCK_BYTES[wtype]
    w = rng.integers(0, 256, nb * bb, dtype=np.uint8)
    for i in range(nb):
        h = np.array([rng.uniform(-0.1, 0.1), rng.uniform(0.0, 0.1)], np.float16).view(np.uint8)
        off = {ora.Q3_K: 108, ora.Q4_K: 0, ora.Q5_K: 0, ora.Q6_K: 208, ora.IQ2_XXS: 0, ora.IQ3_XXS: 0, ora.IQ4_XS: 0}[wtype]
        w[i * bb + off:i * bb + off + 2] = h[0:2]
        if wtype in (ora.Q4_K, ora.Q5_K):
            w[i * bb + 2:i * bb + 4] = h[2:4]
    return w


def quantized_rows(wtype, rows, k, seed):
    rng = np.random.default_rng(seed)
    x = normal_f32(rng, (rows, k), 0.02)
    if wtype == ora.IQ4_XS:
        return iq4xs_rows(x), x
    if wtype == ora.Q3_K:  # a test-side generator: the oracle restates the quantizers of the benchmark's types only
        return q3k_rows(x), x
    if wtype == ora.IQ3_XXS:  # no quantizer of this type in the reference's gguf crate: random legal blocks
        return random_blocks(wtype, rows * (k // 256), rng), x
    return ora.quantize_rows(wtype, x, rows, k, n_threads=4), x


# ------------------------------------------------------------------------------------------------ tables, decode

def test_codebook_digests_and_closed_form():
    for path, (grid, ks) in parse_tables().items():
        assert len(grid) == 256 and len(ks) == 128, path
        assert hashlib.md5(bytes(ks)).hexdigest() == "22df85f30ea9d4bde2651955dc97c39a", path
        assert hashlib.md5(struct.pack("<256Q", *grid)).hexdigest() == "fff55639176d84643cf2facd7a655c4d", path
        assert all(ks[i] == (i | ((bin(i).count("1") & 1) << 7)) for i in range(128)), path
        assert all(((g >> (8 * j)) & 0xFF) in (8, 25, 43) for g in grid for j in range(8)), path


def test_iq3xxs_grid_digest_and_structure():
    # crates/gguf/src/iq_tables.rs:293-295; every byte 4 + 8k or 62 (crates/gguf/src/quant.rs iq_tables_have_ggml_structure)
    for path, grid in parse_grid3().items():
        assert len(grid) == 256, path
        assert hashlib.md5(struct.pack("<256I", *grid)).hexdigest() == "0ee1848d3f04a5720691cb6e7daee92e", path
        assert all(((g >> (8 * j)) & 0xFF) in (4, 12, 20, 28, 36, 44, 52, 62) for g in grid for j in range(4)), path


def test_iq4_levels_digest():
    # crates/gguf/src/iq_tables.rs:432-436: md5 over the sixteen bytes; the shipped headers hold the same sixteen
    assert hashlib.md5(KVALUES_IQ4NL.astype(np.int8).tobytes()).hexdigest() == "5dc4c90c34afd4f896578cb08cb33249"
    import re
    for path in ("oracle/iq_tables.h", "bloomery_amd/csrc/iq2xxs_tables.h"):
        text = open(os.path.join(HERE, "..", path)).read()
        body = re.search(r"KVALUES_IQ4NL\[16\] = \{(.*?)\};", text, re.S).group(1)
        assert [int(v) for v in re.findall(r"-?\d+", body)] == list(KVALUES_IQ4NL), path
    # every level times every block scale is exact in f32 (crates/gguf/src/quant.rs:2693-2700), so the decoder's f64
    # product and the oracle's f32 one agree to the bit
    for bits in range(0, 0x7C00, 37):
        d = np.array([bits], np.uint16).view(np.float16).astype(np.float32)[0]
        for ls in (-32, -7, 1, 31):
            dl = np.float32(d * np.float32(ls))
            assert float(dl) == float(d) * ls
            assert all(float(np.float32(dl * np.float32(kv))) == float(dl) * int(kv) for kv in KVALUES_IQ4NL)


def test_iq2xxs_decodes_the_ggml_made_block():
    gold = json.load(open(os.path.join(HERE, "golden", "iq2xxs_ggml_block.json")))
    blk = np.array(gold["block"], np.uint8)
    got = ora.dequant_row(ora.IQ2_XXS, blk, 256)
    assert list(got.view(np.uint32)) == gold["want_f32_bits"]
    # the independent decoder agrees too, so it can stand as the brute-force side below
    _, vals, _ = iq2xxs_decode(blk)
    assert np.array_equal(vals.astype(np.float32), got)


@pytest.mark.parametrize("wtype", TYPES)
def test_dequant_matches_independent_decoder(wtype):
    rng = np.random.default_rng(100 + wtype)
    w = random_blocks(wtype, 6, rng)
    got = ora.dequant_row(wtype, w, 6 * 256)
    bb = ora.BLOCK_BYTES[wtype]
    want = np.concatenate([DECODE[wtype](w[i * bb:(i + 1) * bb])[1] for i in range(6)])
    # the oracle rounds each product in f32 as the reference does; the decoder is f64
    assert np.allclose(got, want, rtol=3e-7, atol=1e-12)


# -------------------------------------------------------------------------------------------------- integer sums

@pytest.mark.parametrize("wtype", TYPES)
def test_block_sums_equal_brute_force(wtype):
    rng = np.random.default_rng(200 + wtype)
    nb, k = 5, 5 * 256
    bb = ora.BLOCK_BYTES[wtype]
    for case in range(8):
        w = random_blocks(wtype, nb, rng)
        x = normal_f32(rng, k, 10.0 ** rng.uniform(-3, 3))
        col = ora.quantize_col(wtype, x)
        a, _ = act_codes(wtype, col, k)
        wc = np.concatenate([DECODE[wtype](w[i * bb:(i + 1) * bb])[0] for i in range(nb)])
        prod = wc * a
        if wtype in (ora.Q4_K, ora.Q5_K):
            got_a, got_isum = ora.q4k_block_sums(w, col, k, q5=wtype == ora.Q5_K)
            assert list(got_a) == [int(prod[32 * s:32 * s + 32].sum()) for s in range(nb * 8)]
            assert list(got_isum) == [int(a[32 * s:32 * s + 32].sum()) for s in range(nb * 8)]
        elif wtype == ora.Q3_K:
            assert list(ora.q3k_block_sums(w, col, k)) == [int(prod[16 * g:16 * g + 16].sum()) for g in range(nb * 16)]
        elif wtype == ora.Q6_K:
            want = [int(prod[16 * g:16 * g + 16].sum()) for g in range(nb * 16)]
            assert list(ora.q6k_block_sums(w, col, k)) == want
            assert list(ora.q6k_block_sums(w, col, k, fold=True)) == want, "no -128 code on these inputs"
        elif wtype == ora.IQ4_XS:
            i_b, lanes = ora.iq4xs_block_sums(w, col, k)
            assert list(i_b) == [int(prod[32 * b:32 * b + 32].sum()) for b in range(nb * 8)]
            for i in range(nb):
                ls = DECODE[wtype](w[i * bb:(i + 1) * bb])[2][1]
                want = [sum(ls[b] * int(prod[256 * i + 32 * b + 4 * l:256 * i + 32 * b + 4 * l + 4].sum()) for b in range(8))
                        for l in range(8)]
                assert list(lanes[8 * i:8 * i + 8]) == want
            assert ora.iq4xs_block_sums(w, col, k, fold=True)[1].tolist() == lanes.tolist(), "no -128 code on these inputs"
        else:
            off = 64 if wtype == ora.IQ3_XXS else 43
            i_b, sc, codes, fold = ora.iq2xxs_block_sums(w, col, k, iq3=wtype == ora.IQ3_XXS)
            assert list(i_b) == [int(prod[32 * b:32 * b + 32].sum()) for b in range(nb * 8)]
            for i in range(nb):
                s = [2 * DECODE[wtype](w[i * bb:(i + 1) * bb])[2][1][b] + 1 for b in range(8)]
                assert list(sc[8 * i:8 * i + 8]) == s
                bs = [int(a[256 * i + 32 * b:256 * i + 32 * b + 32].sum()) for b in range(8)]
                assert codes[i] == sum(s[b] * (int(i_b[8 * i + b]) + off * bs[b]) for b in range(8))
                assert fold[i] == sum(s[b] * bs[b] for b in range(8))


def test_q6k_sign_fold_differs_only_at_minus_128():
    # The reference's Q6_K kernel folds the weight's sign into the activation byte (crates/qdot/src/lib.rs:4539-4558);
    # -(-128) wraps, so a -128 code against a negative weight counts with the wrong sign there and nowhere else.
    rng = np.random.default_rng(5)
    w = random_blocks(ora.Q6_K, 1, rng)
    codes, _, _ = q6k_decode(w)
    amax = np.float32(127.0 * (64.49 / 64.0) * 2.0 ** -127)  # a subnormal bf16 scale rounding down: codes reach -128
    x = np.where(np.arange(256) % 2 == 0, amax, -amax).astype(np.float32)
    col = ora.quantize_col(ora.Q6_K, x)
    a, _ = act_codes(ora.Q6_K, col, 256)
    assert a.min() == -128
    plain = ora.q6k_block_sums(w, col, 256)
    fold = ora.q6k_block_sums(w, col, 256, fold=True)
    for g in range(16):
        want = sum(-256 * int(codes[16 * g + n]) for n in range(16) if a[16 * g + n] == -128 and codes[16 * g + n] < 0)
        assert int(plain[g]) - int(fold[g]) == want
    assert not np.array_equal(plain, fold)


def test_iq4xs_sign_fold_differs_only_at_minus_128():
    # The reference's IQ4_XS kernel folds a level's sign into the activation byte (crates/qdot/src/lib.rs:11127-11131);
    # -(-128) wraps, so a -128 code under a negative level counts with the wrong sign there and nowhere else. ik's
    # Q8_K encoder never writes -128, so the column is hand-made: random codes with -128 among them.
    rng = np.random.default_rng(6)
    w = random_blocks(ora.IQ4_XS, 2, rng)
    col = np.zeros(2 * 296, np.uint8)
    for i in range(2):
        col[296 * i:296 * i + 4] = np.array([0.01 * (i + 1)], np.float32).view(np.uint8)
        codes = rng.integers(-128, 128, 256).astype(np.int8)
        codes[rng.integers(0, 256, 24)] = -128
        col[296 * i + 8:296 * i + 264] = codes.view(np.uint8)
    a, _ = act_codes(ora.IQ4_XS, col, 512)
    plain = ora.iq4xs_block_sums(w, col, 512)[1]
    fold = ora.iq4xs_block_sums(w, col, 512, fold=True)[1]
    want = np.zeros(16, np.int64)
    for i in range(2):
        lv, _, (_, ls) = iq4xs_decode(w[136 * i:136 * (i + 1)])
        for n in range(256):
            if a[256 * i + n] == -128 and lv[n] < 0:
                want[8 * i + (n % 32) // 4] += -256 * ls[n // 32] * int(lv[n])
    assert (plain.astype(np.int64) - fold).tolist() == want.tolist() and want.any()
    # both restatements of the dot carry the fold: same bits, and the value the folded lanes give
    got = ora.dot_row(ora.IQ4_XS, w, col, 512)
    assert got.tobytes() == ora.dot_row(ora.IQ4_XS, w, col, 512, avx2=True).tobytes()
    acc = np.zeros(8, np.float32)
    for i in range(2):
        d = np.float32(f16(w[136 * i], w[136 * i + 1])) * col[296 * i:296 * i + 4].view(np.float32)[0]
        for l in range(8):
            acc[l] = np.float32(np.float64(d) * np.float64(np.float32(fold[8 * i + l])) + np.float64(acc[l]))
    t = [np.float32(acc[l] + acc[l + 4]) for l in range(4)]
    assert np.float32(np.float32(t[0] + t[2]) + np.float32(t[1] + t[3])) == got


# ------------------------------------------------------------------------------------------------------ fp32 dots

def extreme_cases(wtype, rng):
    """Hand-built blocks at the ends: all codes at their maximum, zero and subnormal scales, negative d."""
    bb = ora.BLOCK_BYTES[wtype]
    out = []
    for fill, dval in ((0xFF, 0.05), (0x00, 0.05), (0xFF, 0.0), (0xAA, 6e-8), (0x55, -0.03)):
        w = np.full(2 * bb, fill, np.uint8)
        for i in range(2):
            h = np.array([dval, abs(dval)], np.float16).view(np.uint8)
            off = {ora.Q3_K: 108, ora.Q4_K: 0, ora.Q5_K: 0, ora.Q6_K: 208, ora.IQ2_XXS: 0, ora.IQ3_XXS: 0, ora.IQ4_XS: 0}[wtype]
            w[i * bb + off:i * bb + off + 2] = h[0:2]
            if wtype in (ora.Q4_K, ora.Q5_K):
                w[i * bb + 2:i * bb + 4] = h[2:4]
        out.append(w)
    out.append(random_blocks(wtype, 2, rng))
    return out


@pytest.mark.parametrize("wtype", TYPES)
def test_scalar_and_avx2_dots_are_bit_identical(wtype):
    assert ora.lib.ora_avx2_supported()
    rng = np.random.default_rng(300 + wtype)
    for k in (256, 768, 2048):
        nb = k // 256
        for case in range(12):
            w = random_blocks(wtype, nb, rng)
            x = normal_f32(rng, k, 10.0 ** rng.uniform(-4, 3))
            if case % 4 == 0:
                x[rng.integers(0, k, 40)] = 0.0
            col = ora.quantize_col(wtype, x)
            a = ora.dot_row(wtype, w, col, k)
            b = ora.dot_row(wtype, w, col, k, avx2=True)
            assert a.tobytes() == b.tobytes(), (wtype, k, case, a, b)
    for w in extreme_cases(wtype, rng):
        for x in (np.full(512, 3.0, np.float32), normal_f32(rng, 512), -np.abs(normal_f32(rng, 512))):
            col = ora.quantize_col(wtype, x)
            assert ora.dot_row(wtype, w, col, 512).tobytes() == ora.dot_row(wtype, w, col, 512, avx2=True).tobytes()


@pytest.mark.parametrize("wtype", TYPES)
def test_quantized_weights_scalar_equals_avx2(wtype):
    k = 2048 if wtype != ora.Q6_K else 768
    rows = 24 if wtype != ora.IQ2_XXS else 6
    w, _ = quantized_rows(wtype, rows, k, 400 + wtype)
    rb = ora.row_bytes(wtype, k)
    rng = np.random.default_rng(401)
    col = ora.quantize_col(wtype, normal_f32(rng, k))
    for r in range(rows):
        a = ora.dot_row(wtype, w[r * rb:(r + 1) * rb], col, k)
        b = ora.dot_row(wtype, w[r * rb:(r + 1) * rb], col, k, avx2=True)
        assert a.tobytes() == b.tobytes()


@pytest.mark.parametrize("wtype", TYPES)
def test_tile_columns_equal_one_column(wtype):
    rng = np.random.default_rng(500 + wtype)
    k = 1024
    w = random_blocks(wtype, k // 256, rng)
    cols = [ora.quantize_col(wtype, normal_f32(rng, k, 10.0 ** rng.uniform(-2, 2))) for _ in range(8)]
    one = [ora.dot_row(wtype, w, c, k) for c in cols]
    for c in range(1, 9):
        got = ora.dot_row_cols(wtype, w, cols[:c], k)
        assert got.tobytes() == np.array(one[:c], np.float32).tobytes()
    with pytest.raises(ora.OracleError):
        ora.dot_row_cols(wtype, w, cols + cols[:1], k)  # crates/qdot/tests/qdot.rs:6502: TileShape


@pytest.mark.parametrize("wtype", TYPES)
def test_dot_within_f64_band_of_dequantized_dot(wtype):
    # |dot - exact| <= (nb_terms + 10) * 2^-24 * sum |w_i * a_i| (a Higham band with slack for the per-block scale
    # products), where exact is the f64 dot of the decoded weights and decoded activations.
    rng = np.random.default_rng(600 + wtype)
    bb = ora.BLOCK_BYTES[wtype]
    for k in (256, 2048):
        nb = k // 256
        for case in range(10):
            w = random_blocks(wtype, nb, rng) if case % 2 else quantized_rows(wtype, 1, k, 610 + case)[0]
            x = normal_f32(rng, k)
            col = ora.quantize_col(wtype, x)
            a_codes, a_scale = act_codes(wtype, col, k)
            act = a_codes * a_scale
            dq = ora.dequant_col(wtype, col, k).astype(np.float64)
            if wtype in ora.Q8K_TYPES:
                assert np.allclose(dq, act, rtol=1e-7, atol=0)  # an f32 scale times a code rounds once
            else:
                assert np.array_equal(dq, act), "a bf16 scale times an 8-bit code is exact in f32"
            if wtype in (ora.IQ2_XXS, ora.IQ3_XXS):
                # the kernel's own grouping: d/8 * (2s+1) * grid (IQ3_XXS: d/4), with the +43 (+64) offset folded out
                unit, both = (0.125, 86) if wtype == ora.IQ2_XXS else (0.25, 128)
                wv = np.concatenate([DECODE[wtype](w[i * bb:(i + 1) * bb])[1] for i in range(nb)])
                extra = np.concatenate([np.repeat([unit * abs(DECODE[wtype](w[i * bb:(i + 1) * bb])[2][0]) *
                                                   (2 * s + 1) * both for s in DECODE[wtype](w[i * bb:(i + 1) * bb])[2][1]],
                                                  32) for i in range(nb)])
                mag = np.sum((np.abs(wv) + extra) * np.abs(act))
                terms = 2 * nb + 10
            else:
                wv = np.concatenate([DECODE[wtype](w[i * bb:(i + 1) * bb])[1] for i in range(nb)])
                if wtype in (ora.Q4_K, ora.Q5_K):
                    # value = d*sc*q - dmin*m: bound with both parts' magnitudes
                    parts = []
                    for i in range(nb):
                        codes, _, (d, dmin, sc, mn) = DECODE[wtype](w[i * bb:(i + 1) * bb])
                        parts.append(np.array([abs(d) * sc[n // 32] * codes[n] + abs(dmin) * mn[n // 32]
                                               for n in range(256)]))
                    mag = np.sum(np.concatenate(parts) * np.abs(act))
                else:
                    mag = np.sum(np.abs(wv) * np.abs(act))
                terms = k // 32 + 10
            exact = float(np.sum(wv * act))
            got = float(ora.dot_row(wtype, w, col, k))
            assert abs(got - exact) <= terms * 2.0 ** -24 * 8 * mag + 1e-30, (wtype, k, case, got, exact)


def test_dot_row_refusals():
    # crates/qdot/src/lib.rs:1727-1779
    w = np.zeros(144 * 2, np.uint8)
    col = np.zeros(144 * 4, np.uint8)
    for k in (100, 255, 300):
        with pytest.raises(ora.OracleError) as e:
            ora.dot_row(ora.Q4_K, w, col, k)
        assert e.value.code == ora.EUNALIGNED
    with pytest.raises(ora.OracleError) as e:
        ora.dot_row(ora.Q4_K, w[:200], col, 512)
    assert e.value.code == ora.ESHORTROW
    with pytest.raises(ora.OracleError) as e:
        ora.dot_row(ora.Q4_K, w, col[:500], 512)
    assert e.value.code == ora.ESHORTCOL
    with pytest.raises(ora.OracleError) as e:
        ora.dot_row(7, w, col, 512)
    assert e.value.code == ora.ETYPE
    assert ora.dot_row(ora.Q4_K, w, col, 512) == 0.0
