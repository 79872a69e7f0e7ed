"""A second, independent spelling of the reference's weight quantizers, for pinning the oracle's C restatement
(oracle/kquant.c, oracle/iq2xxs_quant.c) byte for byte. Written from the reference's text, not from the C:
Q4_K / Q5_K `_ref` (crates/gguf/src/kquant.rs:239-318 make_qkx2_quants, :495-525 pack_scales / requant_levels, :528-660
kquant45_block), Q6_K `_ref` (:126-177 make_qx_quants, :787-842 q6k_block) and IQ2_XXS (crates/gguf/src/iq_quant.rs:
177-223 GridTables::new, :311-395 make_qp_quants, :401-437 iq2_best_neighbour, :440-637 iq2_xxs_sub, :867-881
iq2_xxs_finish). Every f32 operation is one numpy float32 operation (a product and a sum never fuse), sums run in the
reference's index order; where the C walks one sub-block at a time with scalar loops, the K-quant searches here run
over all sub-blocks of the input at once as vectors (the candidate loop and the 32-value accumulation stay sequential,
which is what fixes the rounding), so a slip in either spelling shows as differing bytes.

Parameters the reference fixes are arguments here (the step count of the Q4_K search, a tie rule) so that a test can
show that the comparison notices when one of them is wrong. Nothing here is used by the library or by the oracle."""
import re

import numpy as np

F = np.float32


def f32(v):
    return np.asarray(v, dtype=np.float32)


def nint(x):
    """crates/gguf/src/quant.rs:2222-2226: round to nearest even through one f32 add."""
    v = (f32(x) + F(12582912.0)).astype(np.float32)
    return (v.view(np.uint32) & np.uint32(0x007FFFFF)).astype(np.int64) - 0x00400000


def f16_bits(v):
    return np.asarray(v, np.float32).astype(np.float16).view(np.uint16)


def f16_value(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


# ------------------------------------------------------------------------------------------ Q4_K / Q5_K `_ref`

def make_qkx2(x, w, nmax, rmin, rdelta, nstep, strict=True):
    """x, w: [S, 32] f32. Returns (scale[S], the_min[S], levels[S, 32]). `strict`: an equal error does not replace the
    best so far (the reference's `<`)."""
    S = x.shape[0]
    mn, mx = x[:, 0].copy(), x[:, 0].copy()
    sum_w = w[:, 0].copy()
    sum_x = (sum_w * x[:, 0]).astype(np.float32)
    for i in range(1, 32):
        mn = np.where(x[:, i] < mn, x[:, i], mn)
        mx = np.where(x[:, i] > mx, x[:, i], mx)
        sum_w = (sum_w + w[:, i]).astype(np.float32)
        sum_x = (sum_x + (w[:, i] * x[:, i]).astype(np.float32)).astype(np.float32)
    mn = np.where(mn > 0, F(0), mn).astype(np.float32)
    flat = mx == mn
    nmaxf = F(nmax)
    with np.errstate(divide="ignore", invalid="ignore"):
        iscale = (nmaxf / (mx - mn).astype(np.float32)).astype(np.float32)
        scale = (F(1.0) / iscale).astype(np.float32)
        L = np.clip(nint((iscale[:, None] * (x - mn[:, None]).astype(np.float32)).astype(np.float32)), 0, nmax)
        best = np.zeros(S, np.float32)
        for i in range(32):
            diff = (((scale * L[:, i].astype(np.float32)).astype(np.float32) + mn).astype(np.float32) - x[:, i]).astype(np.float32)
            best = (best + (w[:, i] * (diff * diff).astype(np.float32)).astype(np.float32)).astype(np.float32)
        for step in range(nstep + 1):
            top = ((F(rmin) + (F(rdelta) * F(step)).astype(np.float32)).astype(np.float32) + nmaxf).astype(np.float32)
            iscale = (top / (mx - mn).astype(np.float32)).astype(np.float32)
            la = np.clip(nint((iscale[:, None] * (x - mn[:, None]).astype(np.float32)).astype(np.float32)), 0, nmax)
            sum_l, sum_l2, sum_xl = np.zeros(S, np.float32), np.zeros(S, np.float32), np.zeros(S, np.float32)
            for i in range(32):
                lf = la[:, i].astype(np.float32)
                wl = (w[:, i] * lf).astype(np.float32)
                sum_l = (sum_l + wl).astype(np.float32)
                sum_l2 = (sum_l2 + (wl * lf).astype(np.float32)).astype(np.float32)
                sum_xl = (sum_xl + (wl * x[:, i]).astype(np.float32)).astype(np.float32)
            d = ((sum_w * sum_l2).astype(np.float32) - (sum_l * sum_l).astype(np.float32)).astype(np.float32)
            ok = d > 0
            this_scale = (((sum_w * sum_xl).astype(np.float32) - (sum_x * sum_l).astype(np.float32)).astype(np.float32) / d).astype(np.float32)
            this_min = (((sum_l2 * sum_x).astype(np.float32) - (sum_l * sum_xl).astype(np.float32)).astype(np.float32) / d).astype(np.float32)
            pos = this_min > 0
            this_scale = np.where(pos, (sum_xl / sum_l2).astype(np.float32), this_scale).astype(np.float32)
            this_min = np.where(pos, F(0), this_min).astype(np.float32)
            cur = np.zeros(S, np.float32)
            for i in range(32):
                diff = (((this_scale * la[:, i].astype(np.float32)).astype(np.float32) + this_min).astype(np.float32) - x[:, i]).astype(np.float32)
                cur = (cur + (w[:, i] * (diff * diff).astype(np.float32)).astype(np.float32)).astype(np.float32)
            better = ok & ((cur < best) if strict else (cur <= best)) & ~flat
            L = np.where(better[:, None], la, L)
            best = np.where(better, cur, best).astype(np.float32)
            scale = np.where(better, this_scale, scale).astype(np.float32)
            mn = np.where(better, this_min, mn).astype(np.float32)
    scale = np.where(flat, F(0), scale).astype(np.float32)
    L = np.where(flat[:, None], 0, L)
    return scale, (-mn).astype(np.float32), L.astype(np.int64)


def pack_scales(ls, lm):
    """[B, 8] six-bit codes -> [B, 12] bytes (crates/gguf/src/kquant.rs:495-510)."""
    s = np.zeros((ls.shape[0], 12), np.int64)
    s[:, 0:4] = ls[:, 0:4] | ((ls[:, 4:8] >> 4) << 6)
    s[:, 4:8] = lm[:, 0:4] | ((lm[:, 4:8] >> 4) << 6)
    s[:, 8:12] = (ls[:, 4:8] & 15) | ((lm[:, 4:8] & 15) << 4)
    return s.astype(np.uint8)


def scale_min_k4(sc):
    """[B, 12] bytes -> (sc[B, 8], m[B, 8]) (crates/gguf/src/quant.rs:620-628)."""
    sc = sc.astype(np.int64)
    s, m = np.empty((sc.shape[0], 8), np.int64), np.empty((sc.shape[0], 8), np.int64)
    s[:, :4], m[:, :4] = sc[:, 0:4] & 63, sc[:, 4:8] & 63
    s[:, 4:] = (sc[:, 8:12] & 15) | ((sc[:, 0:4] >> 6) << 4)
    m[:, 4:] = (sc[:, 8:12] >> 4) | ((sc[:, 4:8] >> 6) << 4)
    return s, m


def quantize_q45k(x, q5=False, nstep=None, strict=True):
    """Rows of f32 (any shape, a multiple of 256 values) -> Q4_K (144 B) or Q5_K (176 B) blocks, the `_ref` rules."""
    x = f32(x).reshape(-1, 256)
    B = x.shape[0]
    nmax = 31 if q5 else 15
    rmin, rdelta, steps = (-0.5, 0.1, 15) if q5 else (-1.0, 0.1, 20)
    steps = steps if nstep is None else nstep
    xs = x.reshape(B * 8, 32)
    sum_x2 = np.zeros(B * 8, np.float32)
    for i in range(32):
        sum_x2 = (sum_x2 + (xs[:, i] * xs[:, i]).astype(np.float32)).astype(np.float32)
    av_x = np.sqrt((sum_x2 / F(32.0)).astype(np.float32)).astype(np.float32)
    w = (av_x[:, None] + np.abs(xs)).astype(np.float32)
    scale, the_min, L = make_qkx2(xs, w, nmax, rmin, rdelta, steps, strict)
    scales, mins, L = scale.reshape(B, 8), the_min.reshape(B, 8), L.reshape(B, 256)
    max_scale, max_min = np.zeros(B, np.float32), np.zeros(B, np.float32)
    for j in range(8):
        max_scale = np.where(scales[:, j] > max_scale, scales[:, j], max_scale).astype(np.float32)
        max_min = np.where(mins[:, j] > max_min, mins[:, j], max_min).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv_scale = np.where(max_scale > 0, (F(63.0) / max_scale).astype(np.float32), F(0)).astype(np.float32)
        inv_min = np.where(max_min > 0, (F(63.0) / max_min).astype(np.float32), F(0)).astype(np.float32)
    ls = np.minimum(nint((inv_scale[:, None] * scales).astype(np.float32)) & 0xFF, 63)   # `as u8`, then .min(63)
    lm = np.minimum(nint((inv_min[:, None] * mins).astype(np.float32)) & 0xFF, 63)
    sc = pack_scales(ls, lm)
    d_bits, dmin_bits = f16_bits((max_scale / F(63.0)).astype(np.float32)), f16_bits((max_min / F(63.0)).astype(np.float32))
    d, dmin = f16_value(d_bits), f16_value(dmin_bits)
    s6, m6 = scale_min_k4(sc)
    dd = (d[:, None] * s6.astype(np.float32)).astype(np.float32)
    dm = (dmin[:, None] * m6.astype(np.float32)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = nint((((x.reshape(B, 8, 32) + dm[:, :, None]).astype(np.float32)) / dd[:, :, None]).astype(np.float32))
    rel = np.clip(rel, 0, nmax)
    L = np.where((dd != 0)[:, :, None], rel, L.reshape(B, 8, 32)).reshape(B, 256)
    out = np.zeros((B, 176 if q5 else 144), np.uint8)
    out[:, 0:2] = d_bits.view(np.uint8).reshape(B, 2)
    out[:, 2:4] = dmin_bits.view(np.uint8).reshape(B, 2)
    out[:, 4:16] = sc
    Lq = L.reshape(B, 4, 2, 32)   # [64-value group][first / second 32][value]
    if q5:
        qh = np.zeros((B, 32), np.int64)
        for g in range(4):
            qh |= (Lq[:, g, 0] >> 4) << (2 * g)
            qh |= (Lq[:, g, 1] >> 4) << (2 * g + 1)
        out[:, 16:48] = qh.astype(np.uint8)
        out[:, 48:176] = ((Lq[:, :, 0] & 15) | ((Lq[:, :, 1] & 15) << 4)).reshape(B, 128).astype(np.uint8)
    else:
        out[:, 16:144] = (Lq[:, :, 0] | (Lq[:, :, 1] << 4)).reshape(B, 128).astype(np.uint8)
    return out.reshape(-1)


def dequant_q4k(blocks):
    """Q4_K blocks -> f32 values (crates/gguf/src/quant.rs:738-767), for the round-trip checks."""
    b = np.asarray(blocks, np.uint8).reshape(-1, 144)
    d, dmin = f16_value(b[:, 0:2].copy().view(np.uint16).reshape(-1)), f16_value(b[:, 2:4].copy().view(np.uint16).reshape(-1))
    s6, m6 = scale_min_k4(b[:, 4:16])
    qs = b[:, 16:144].reshape(-1, 4, 32).astype(np.int64)
    q = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 8, 32)
    dd = (d[:, None] * s6.astype(np.float32)).astype(np.float32)
    dm = (dmin[:, None] * m6.astype(np.float32)).astype(np.float32)
    return ((dd[:, :, None] * q.astype(np.float32)).astype(np.float32) - dm[:, :, None]).astype(np.float32).reshape(-1)


# ------------------------------------------------------------------------------------------------ Q6_K `_ref`

GROUP_MAX_EPS = F(1e-15)


def make_qx(x, nmax, first_max=True):
    """x: [G, n] f32, weights x^2. Returns (scale[G], levels[G, n] offset by nmax). `first_max`: of equal magnitudes the
    first one's signed value is the maximum (the reference's `ax > amax`)."""
    G, n = x.shape
    mx, amax = np.zeros(G, np.float32), np.zeros(G, np.float32)
    for i in range(n):
        ax = np.abs(x[:, i])
        take = (ax > amax) if first_max else (ax >= amax)
        mx = np.where(take, x[:, i], mx).astype(np.float32)
        amax = np.where(take, ax, amax).astype(np.float32)
    tiny = amax < GROUP_MAX_EPS
    nmaxf = F(nmax)

    def sums(iscale):
        li = np.clip(nint((iscale[:, None] * x).astype(np.float32)), -nmax, nmax - 1)
        sumlx, suml2 = np.zeros(G, np.float32), np.zeros(G, np.float32)
        for i in range(n):
            wgt = (x[:, i] * x[:, i]).astype(np.float32)
            lf = li[:, i].astype(np.float32)
            sumlx = (sumlx + ((wgt * x[:, i]).astype(np.float32) * lf).astype(np.float32)).astype(np.float32)
            suml2 = (suml2 + ((wgt * lf).astype(np.float32) * lf).astype(np.float32)).astype(np.float32)
        return li, sumlx, suml2

    with np.errstate(divide="ignore", invalid="ignore"):
        iscale = (-nmaxf / mx).astype(np.float32)
        L, sumlx, suml2 = sums(iscale)
        scale = np.where(suml2 != 0, (sumlx / suml2).astype(np.float32), F(0)).astype(np.float32)
        best = (scale * sumlx).astype(np.float32)
        for step in range(-9, 10):
            if step == 0:
                continue
            iscale = (-(nmaxf + (F(0.1) * F(step)).astype(np.float32)).astype(np.float32) / mx).astype(np.float32)
            li, sumlx, suml2 = sums(iscale)
            better = (suml2 > 0) & ((sumlx * sumlx).astype(np.float32) > (best * suml2).astype(np.float32)) & ~tiny
            L = np.where(better[:, None], li, L)
            scale = np.where(better, (sumlx / suml2).astype(np.float32), scale).astype(np.float32)
            best = np.where(better, (scale * sumlx).astype(np.float32), best).astype(np.float32)
    scale = np.where(tiny, F(0), scale).astype(np.float32)
    L = np.where(tiny[:, None], 0, L + nmax)
    return scale, L.astype(np.int64)


def quantize_q6k(x, first_max=True):
    x = f32(x).reshape(-1, 256)
    B = x.shape[0]
    scale, L = make_qx(x.reshape(B * 16, 16), 32, first_max)
    scales, L = scale.reshape(B, 16), L.reshape(B, 256)
    max_scale, max_abs = np.zeros(B, np.float32), np.zeros(B, np.float32)
    for ib in range(16):
        a = np.abs(scales[:, ib])
        take = a > max_abs
        max_scale = np.where(take, scales[:, ib], max_scale).astype(np.float32)
        max_abs = np.where(take, a, max_abs).astype(np.float32)
    zero = max_abs < GROUP_MAX_EPS
    with np.errstate(divide="ignore", invalid="ignore"):
        iscale = (F(-128.0) / max_scale).astype(np.float32)
        d_bits = f16_bits((F(1.0) / iscale).astype(np.float32))
        sc = np.minimum(127, nint((iscale[:, None] * scales).astype(np.float32)))
        sc = ((sc + 128) & 0xFF) - 128   # `as i8`
        d = f16_value(d_bits)
        dd = (d[:, None] * sc.astype(np.float32)).astype(np.float32)
        rel = np.clip(nint((x.reshape(B, 16, 16) / dd[:, :, None]).astype(np.float32)), -32, 31) + 32
    L = np.where((dd != 0)[:, :, None], rel, L.reshape(B, 16, 16)).reshape(B, 2, 4, 32)   # [half][quarter][value]
    out = np.zeros((B, 210), np.uint8)
    ql = np.zeros((B, 2, 64), np.int64)
    ql[:, :, 0:32] = (L[:, :, 0] & 15) | ((L[:, :, 2] & 15) << 4)
    ql[:, :, 32:64] = (L[:, :, 1] & 15) | ((L[:, :, 3] & 15) << 4)
    qh = (L[:, :, 0] >> 4) | ((L[:, :, 1] >> 4) << 2) | ((L[:, :, 2] >> 4) << 4) | ((L[:, :, 3] >> 4) << 6)
    out[:, 0:128] = ql.reshape(B, 128).astype(np.uint8)
    out[:, 128:192] = qh.reshape(B, 64).astype(np.uint8)
    out[:, 192:208] = (sc & 0xFF).astype(np.uint8)
    out[:, 208:210] = d_bits.view(np.uint8).reshape(B, 2)
    out[zero] = 0
    return out.reshape(-1)


def dequant_q6k(blocks):
    """Q6_K blocks -> f32 values (crates/gguf/src/quant.rs:826-859)."""
    b = np.asarray(blocks, np.uint8).reshape(-1, 210)
    ql, qh = b[:, 0:128].reshape(-1, 2, 64).astype(np.int64), b[:, 128:192].reshape(-1, 2, 32).astype(np.int64)
    sc = b[:, 192:208].astype(np.int8).astype(np.float32).reshape(-1, 2, 4, 2)
    d = f16_value(b[:, 208:210].copy().view(np.uint16).reshape(-1))
    q = np.empty((b.shape[0], 2, 4, 32), np.int64)
    q[:, :, 0] = (ql[:, :, 0:32] & 15) | ((qh & 3) << 4)
    q[:, :, 1] = (ql[:, :, 32:64] & 15) | (((qh >> 2) & 3) << 4)
    q[:, :, 2] = (ql[:, :, 0:32] >> 4) | (((qh >> 4) & 3) << 4)
    q[:, :, 3] = (ql[:, :, 32:64] >> 4) | (((qh >> 6) & 3) << 4)
    q = (q - 32).astype(np.float32).reshape(-1, 2, 4, 2, 16)
    v = (d[:, None, None, None, None] * sc[:, :, :, :, None]).astype(np.float32) * q
    return v.astype(np.float32).reshape(-1)


# ------------------------------------------------------------------------------------------------- IQ2_XXS

EPS_IQ2 = F(1e-15)
KMAP_SIZE = 43692


def read_iq2xxs_grid(header_path):
    """The 256 grid words out of a C table file (data: the md5 of these words is pinned by its own test)."""
    text = open(header_path).read()
    body = text[text.index("IQ2XXS_GRID"):]
    body = body[body.index("{") + 1:body.index("}")]
    words = [int(w, 16) for w in re.findall(r"0x[0-9a-fA-F]{16}", body)]
    assert len(words) == 256, len(words)
    return words


class Grid:
    """crates/gguf/src/iq_quant.rs:177-223: a grid point's eight 2-bit codes, the code word -> point map, and the
    neighbour list of a word that is no point: the points at the two smallest distinct squared distances, ordered by
    (distance, index). Lists are built when a word is first asked for."""

    def __init__(self, words):
        code_of = {0x08: 0, 0x19: 1, 0x2B: 2}
        self.codes = np.array([[code_of[(e >> (8 * k)) & 0xFF] for k in range(8)] for e in words], np.int64)   # [256, 8]
        self.word = (self.codes << (2 * np.arange(8))).sum(axis=1)
        self.on_grid = {int(u): g for g, u in enumerate(self.word)}
        self.lists = {}

    def lookup(self, u):
        """('point', g), ('list', [g ...]) or None past the map."""
        if u >= KMAP_SIZE:
            return None
        if u in self.on_grid:
            return "point", self.on_grid[u]
        if u not in self.lists:
            a = (u >> (2 * np.arange(8))) & 3
            d2 = ((2 * (self.codes - a[None, :])) ** 2).sum(axis=1)
            kept = np.unique(d2)[:2]
            self.lists[u] = [int(g) for v in kept for g in np.flatnonzero(d2 == v)]
        return "list", self.lists[u]


def _seq_sum(terms):
    s = F(0.0)
    for t in terms:
        s = F(s + t)
    return s


def make_qp(x, qw, nmax):
    """crates/gguf/src/iq_quant.rs:311-395: the scale only."""
    mx = F(0.0)
    for v in x:
        mx = v if v > mx else mx
    if mx < EPS_IQ2:
        return F(0.0)
    nmaxf = F(nmax)
    iscale = F(nmaxf / mx)
    scale = F(F(1.0) / iscale)
    l8 = nint((iscale * x).astype(np.float32)) & 0xFF   # ggml's uint8_t L
    diff = (x - (scale * l8.astype(np.float32)).astype(np.float32)).astype(np.float32)
    best = _seq_sum(((qw * diff).astype(np.float32) * diff).astype(np.float32))
    for step in range(-4, 5):
        if step == 0:
            continue
        isc = F(F(F(0.1) * F(step)) + nmaxf) / mx
        isc = F(isc)
        sc = F(F(1.0) / isc)
        li = np.minimum(nint((isc * x).astype(np.float32)), nmax)
        diff = (x - (sc * li.astype(np.float32)).astype(np.float32)).astype(np.float32)
        mse = _seq_sum(((qw * diff).astype(np.float32) * diff).astype(np.float32))
        if mse < best:
            best, iscale = mse, isc
    li = np.minimum(nint((iscale * x).astype(np.float32)), nmax)
    l8 = li & 0xFF
    lf = li.astype(np.float32)
    sumlx = _seq_sum(((qw * x).astype(np.float32) * lf).astype(np.float32))
    suml2 = _seq_sum(((qw * lf).astype(np.float32) * lf).astype(np.float32))
    for _ in range(5):
        changed = 0
        for i in range(32):
            w, cur = qw[i], F(float(l8[i]))
            slx = F(sumlx - F(F(w * x[i]) * cur))
            sl2 = F(suml2 - F(F(w * cur) * cur))
            if slx > 0 and sl2 > 0:
                new = min(int(nint(F(F(x[i] * sl2) / slx))), nmax)
                if new != int(l8[i]):
                    nl = F(new)
                    slx = F(slx + F(F(w * x[i]) * nl))
                    sl2 = F(sl2 + F(F(w * nl) * nl))
                    if F(F(slx * slx) * suml2) > F(F(sumlx * sumlx) * sl2):
                        l8[i] = new & 0xFF
                        sumlx, suml2 = slx, sl2
                        changed += 1
        if not changed:
            break
    return F(sumlx / suml2) if suml2 > 0 else F(0.0)


def iq2xxs_sub(xb, qw, sigma2, grid, first_least=True, steps=6):
    """One 32-value sub-block -> (w0, w1, scale) (crates/gguf/src/iq_quant.rs:471-637). `first_least`: of equal
    distances the list's first point wins (the reference's `<`); `steps`: the trial scales run from -steps to steps."""
    weight = (qw * np.sqrt((sigma2 + (xb * xb).astype(np.float32)).astype(np.float32)).astype(np.float32)).astype(np.float32)
    waux = np.sqrt(weight).astype(np.float32)
    xval = np.abs(xb).astype(np.float32)
    signs = [0, 0, 0, 0]
    for k in range(4):
        grp = slice(8 * k, 8 * k + 8)
        neg = xb[grp] < 0
        s = int((neg.astype(np.int64) << np.arange(8)).sum())
        if int(neg.sum()) % 2 == 1:
            sq = ((weight[grp] * xb[grp]).astype(np.float32) * xb[grp]).astype(np.float32)
            imin = int(np.argmin(sq))   # the first of the least
            xval[8 * k + imin] = -xval[8 * k + imin]
            s ^= 1 << imin
        signs[k] = s & 127
    mx = xval[0]
    for v in xval[1:]:
        mx = mx if mx > v else v
    if mx < EPS_IQ2:
        return 0, 0, F(0.0)
    scale = make_qp(xval, weight, 4)
    eff_max = F(scale * F(3.0))
    if eff_max <= 0:
        return 0, 0, F(0.0)

    def word_of(k, idv):
        c = np.clip(nint((F(0.5) * ((idv * xval[8 * k:8 * k + 8]).astype(np.float32) - F(1.0)).astype(np.float32)).astype(np.float32)), 0, 2)
        return int((c << (2 * np.arange(8))).sum()), c

    def nearest(points, k, sc):
        q = (2 * grid.codes[points] + 1).astype(np.float32)                      # [n, 8]
        diff = ((sc * q).astype(np.float32) - xval[None, 8 * k:8 * k + 8]).astype(np.float32)
        term = ((waux[None, 8 * k:8 * k + 8] * diff).astype(np.float32) * diff).astype(np.float32)
        d2 = np.zeros(len(points), np.float32)
        for i in range(8):
            d2 = (d2 + term[:, i]).astype(np.float32)
        at = int(np.argmin(d2)) if first_least else int(len(d2) - 1 - np.argmin(d2[::-1]))
        return points[at]

    def snap(idv, sc, want_point):
        lv = np.zeros(32, np.int64)
        pts = []
        for k in range(4):
            u, c = word_of(k, idv)
            hit = grid.lookup(u)
            assert hit is not None, "a code word past the map"
            if hit[0] == "point":
                g = hit[1]
                lv[8 * k:8 * k + 8] = grid.codes[g] if want_point else c
            else:
                g = nearest(hit[1], k, sc)
                lv[8 * k:8 * k + 8] = grid.codes[g]
            pts.append(g)
        return lv, pts

    def sums(lv):
        q = (2 * lv + 1).astype(np.float32)
        sumqx = _seq_sum(((weight * xval).astype(np.float32) * q).astype(np.float32))
        sumq2 = _seq_sum(((weight * q).astype(np.float32) * q).astype(np.float32))
        return sumqx, sumq2

    L = np.zeros(32, np.int64)
    best = F(0.0)
    for step in range(-steps, steps + 1):
        idv = F(F(F(5.0) + F(F(step) * F(0.1))) / eff_max)
        this_scale = F(F(1.0) / idv)
        la, _ = snap(idv, this_scale, False)
        sumqx, sumq2 = sums(la)
        if sumq2 > 0 and F(sumqx * sumqx) > F(best * sumq2):
            scale = F(sumqx / sumq2)
            best = F(scale * sumqx)
            L = la
    if scale > 0:
        idv = F(F(1.0) / scale)
        L, _ = snap(idv, scale, True)
        sumqx, sumq2 = sums(L)
        if sumq2 > 0:
            scale = F(sumqx / sumq2)
    if scale < 0:
        scale = F(-scale)
        signs = [~s & 127 for s in signs]
    w0 = w1 = 0
    for k in range(4):
        u = int((L[8 * k:8 * k + 8] << (2 * np.arange(8))).sum())
        hit = grid.lookup(u)
        assert hit is not None and hit[0] == "point", "the final levels are no grid point"
        w0 |= hit[1] << (8 * k)
        w1 |= signs[k] << (7 * k)
    return w0, w1, scale


def quantize_iq2xxs(x, qw, grid, first_least=True, steps=6):
    """A row of f32 (a multiple of 256 values) with importance qw -> IQ2_XXS blocks (66 B)."""
    x, qw = f32(x).reshape(-1, 256), f32(qw).reshape(-1, 256)
    out = np.zeros((x.shape[0], 66), np.uint8)
    for b in range(x.shape[0]):
        sigma2 = F(_seq_sum((x[b] * x[b]).astype(np.float32)) / F(256.0))
        subs = [iq2xxs_sub(x[b, 32 * s:32 * s + 32], qw[b, 32 * s:32 * s + 32], sigma2, grid, first_least, steps) for s in range(8)]
        m = F(0.0)
        for _, _, sc in subs:
            m = m if m > sc else sc
        if m == 0:
            continue
        d = F(m / F(31.0))
        idv = F(F(1.0) / d)
        words = []
        for w0, w1, sc in subs:
            lvl = int(np.clip(nint(F(F(0.5) * F(F(idv * sc) - F(1.0)))), 0, 15))
            words += [w0, w1 | (lvl << 28)]
        out[b, 0:2] = f16_bits(d).reshape(1).view(np.uint8)
        out[b, 2:66] = np.array(words, np.uint32).view(np.uint8)
    return out.reshape(-1)
