"""Shared generators for the parity tests: seeded inputs and independent (numpy / pure Python) restatements the
oracle is checked against. Nothing here calls the HIP library."""
import numpy as np


class Lcg:
    """Knuth MMIX LCG, the generator the reference's encoder sweeps use (crates/qdot/tests/qdot.rs:4510-4525)."""

    def __init__(self, seed):
        self.s = seed & 0xFFFFFFFFFFFFFFFF

    def next_u32(self):
        self.s = (self.s * 6364136223846793005 + 1442695040888963407) & 0xFFFFFFFFFFFFFFFF
        return self.s >> 33

    def unit(self):
        return np.float32(np.float32(self.next_u32()) / np.float32(2147483648.0) - np.float32(1.0))


def bf16_rne_bits(x):
    u = int(np.float32(x).view(np.uint32))
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF


def bf16_to_f32(bits):
    return np.uint32(bits << 16).view(np.float32)


def round_half_even(v):
    """Independent of the magic-number form: numpy's rint rounds halves to even."""
    return int(np.rint(np.float64(v)))


def q82_block_closed_form(x):
    """ik's q8_2 rule for one 32-value block, restated independently (crates/qdot/tests/qdot.rs:5093-5110).
    Returns None where 1/d overflows (the encoders flush that block to zero)."""
    x = np.asarray(x, np.float32)
    amax = np.float32(np.max(np.abs(x)))
    t = bf16_rne_bits(amax / np.float32(127.0))
    d = bf16_to_f32(t)
    with np.errstate(divide="ignore", over="ignore"):
        inv = np.float32(1.0) / d if d > 0 else np.float32(0.0)
    if not np.isfinite(inv):
        return None
    codes, isum = [], 0
    for v in x:
        q = round_half_even(np.float32(v * inv))
        codes.append(max(-128, min(127, q)))
        isum += q
    isum = ((isum + 0x8000) & 0xFFFF) - 0x8000
    return np.array(codes, np.int8), t, isum


def normal_f32(rng, shape, sigma=1.0):
    return (rng.standard_normal(shape) * sigma).astype(np.float32)


def max_abs_normalised(got, want):
    """max |got - want| / max |want|: the metric the fp32 tolerance of 1e-4 is stated in."""
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    denom = np.max(np.abs(want))
    return float(np.max(np.abs(got - want)) / (denom if denom > 0 else 1.0))


KVALUES_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int64)


def iq4xs_rows(x):
    """IQ4_XS blocks (136 bytes a 256 values, crates/gguf/src/quant.rs:1969-1976) standing for the f32 rows x: a
    test-side generator, nearest level under one scale a 32 values. The reference's gguf crate has no IQ4_XS
    quantizer to follow; the tests only need blocks whose values look like weights, and every byte pattern is a legal
    block."""
    x = np.asarray(x, np.float32).reshape(-1, 256)
    out = np.zeros((x.shape[0], 136), np.uint8)
    for i, blk in enumerate(x):
        sub = blk.reshape(8, 32).astype(np.float64)
        amax = np.abs(sub).max(axis=1)
        d = np.float16(amax.max() / (127.0 * 31.0))
        df = float(d)
        ls = np.zeros(8, np.int64) if df == 0.0 else np.clip(np.rint(amax / (127.0 * df)), 1, 31).astype(np.int64)
        codes = np.zeros((8, 32), np.int64)
        for b in range(8):
            if df != 0.0:
                codes[b] = np.abs(sub[b][:, None] / (df * ls[b]) - KVALUES_IQ4NL[None, :]).argmin(axis=1)
        stored = ls + 32
        out[i, 0:2] = np.array([d], np.float16).view(np.uint8)
        sh = 0
        for b in range(8):
            sh |= int(stored[b] >> 4) << (2 * b)
            out[i, 4 + b // 2] |= int(stored[b] & 15) << (4 * (b % 2))
        out[i, 2], out[i, 3] = sh & 0xFF, sh >> 8
        out[i, 8:136] = (codes[:, :16] | (codes[:, 16:] << 4)).astype(np.uint8).reshape(-1)
    return out.reshape(-1)


def q3k_rows(x):
    """Q3_K blocks (110 bytes a 256 values, crates/gguf/src/quant.rs:671-678) standing for the f32 rows x: a test-side
    generator, nearest of the eight levels -4 .. 3 under one six-bit scale a 16 values. (The reference quantizes Q3_K
    with ggml's search; the tests only need blocks whose values look like weights, every byte pattern being legal.)"""
    x = np.asarray(x, np.float32).reshape(-1, 256)
    out = np.zeros((x.shape[0], 110), np.uint8)
    for i, blk in enumerate(x):
        grp = blk.reshape(16, 16).astype(np.float64)
        amax = np.abs(grp).max(axis=1)
        d = np.float16(amax.max() / (4.0 * 31.0))
        df = float(d)
        sc = np.zeros(16, np.int64) if df == 0.0 else np.clip(np.rint(amax / (4.0 * df)), 1, 31).astype(np.int64)
        u = np.full(256, 4, np.int64)
        if df != 0.0:
            u = (np.clip(np.rint(grp / (df * sc[:, None])), -4, 3).astype(np.int64) + 4).reshape(-1)
        for n in range(256):
            half, field, cell = n // 128, (n // 32) % 4, n % 32
            out[i, 32 + 32 * half + cell] |= int(u[n] & 3) << (2 * field)
            out[i, cell] |= int(u[n] >> 2) << (4 * half + field)
        s6 = sc + 32
        for k in range(4):  # crates/qdot/src/lib.rs:2187-2198
            out[i, 96 + k] = int(s6[k] & 15) | (int(s6[8 + k] & 15) << 4)
            out[i, 100 + k] = int(s6[4 + k] & 15) | (int(s6[12 + k] & 15) << 4)
            out[i, 104 + k] = int(s6[k] >> 4) | (int(s6[4 + k] >> 4) << 2) | (int(s6[8 + k] >> 4) << 4) | (int(s6[12 + k] >> 4) << 6)
        out[i, 108:110] = np.array([d], np.float16).view(np.uint8)
    return out.reshape(-1)
