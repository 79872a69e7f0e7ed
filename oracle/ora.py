"""TEST INFRASTRUCTURE ONLY: ctypes view of the CPU oracle (oracle/libbm_oracle.so).

Imported by the test suite, the smoke check and the benchmark's CPU-baseline leg; never by the package.
The library is built by `make -C oracle` (or `__graft_entry__.build()`); loading it never compiles.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbm_oracle.so")

Q3_K, Q4_K, Q5_K, Q6_K, IQ2_XXS, IQ3_XXS, IQ4_XS = 11, 12, 13, 14, 16, 18, 23
BLOCK_BYTES = {Q3_K: 110, Q4_K: 144, Q5_K: 176, Q6_K: 210, IQ2_XXS: 66, IQ3_XXS: 98, IQ4_XS: 136}
Q8K_TYPES = (Q3_K, IQ2_XXS, IQ3_XXS, IQ4_XS)  # the types whose activation column is ik's Q8_K; the others take Q8_2_X4

EUNALIGNED, ETYPE, ESHORTROW, ESHORTCOL, ENONFINITE, ESHAPE, ESTATUS = -1, -2, -3, -4, -5, -6, -7

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int32)
_u32p = C.POINTER(C.c_uint32)


class MoeLayer(C.Structure):
    _fields_ = [
        ("hidden", C.c_int), ("ff", C.c_int), ("n_experts", C.c_int),
        ("gate_type", C.c_int), ("up_type", C.c_int), ("down_type", C.c_int),
        ("wg", C.c_void_p), ("wu", C.c_void_p), ("wd", C.c_void_p),
    ]


def _load():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is not built: run `make -C oracle`")
    lib = C.CDLL(LIB_PATH)
    sig = {
        "ora_col_bytes": (C.c_int, [C.c_int, C.c_int]),
        "ora_row_bytes": (C.c_int, [C.c_int, C.c_int]),
        "ora_quantize_col": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_avx2_quantize_col": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_dot_row": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]),
        "ora_gemv": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_avx2_dot_row": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_avx2_dot_row_cols": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
        "ora_avx2_supported": (C.c_int, []),
        "ora_q3k_block_sums": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_q4k_block_sums": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
        "ora_q5k_block_sums": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
        "ora_q6k_block_sums": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
        "ora_iq2xxs_block_sums": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_void_p]),
        "ora_iq3xxs_block_sums": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_void_p]),
        "ora_iq4xs_block_sums": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
        "ora_dequant_row": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_dequant_col": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_expf_ik": (C.c_float, [C.c_float]),
        "ora_swiglu": (None, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_gate_rule": (C.c_int, [C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_sum_sq_f64": (C.c_double, [C.c_void_p, C.c_int]),
        "ora_rms_norm": (None, [C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_void_p]),
        "ora_dot_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_card_q8_1": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
        "ora_card_dot_row": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
        "ora_card_gemv": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_card_gemv_sel": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_void_p, C.c_int, C.c_void_p]),
        "ora_router_logits": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_void_p,
                                        C.c_void_p]),
        "ora_route_softmax_topk": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
        "ora_combine_tokens": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
        "ora_moe_combine": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
        "ora_quantize_row_q4k": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
        "ora_quantize_row_q6k": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
        "ora_quantize_row_iq2xxs": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
        "ora_quantize_rows": (C.c_int, [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int]),
        "ora_iq2xxs_grid_codes": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
        "ora_moe_forward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
                                      C.c_void_p, C.c_int]),
        "ora_pool_create": (C.c_void_p, [C.c_int]),
        "ora_pool_destroy": (None, [C.c_void_p]),
        "ora_avx2_moe_forward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                           C.c_int, C.c_void_p, C.c_void_p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


class OracleError(Exception):
    def __init__(self, code):
        super().__init__(f"oracle refusal {code}")
        self.code = code


def _check(rc):
    if rc != 0:
        raise OracleError(rc)


def col_bytes(wtype, k):
    n = lib.ora_col_bytes(wtype, k)
    if n < 0:
        raise OracleError(n)
    return n


def row_bytes(wtype, k):
    n = lib.ora_row_bytes(wtype, k)
    if n < 0:
        raise OracleError(n)
    return n


def quantize_col(wtype, x, avx2=False):
    """One f32 column -> the activation bytes the weight type `wtype` dots against."""
    x = _f32(x)
    out = np.empty(col_bytes(wtype, x.size), np.uint8)
    fn = lib.ora_avx2_quantize_col if avx2 else lib.ora_quantize_col
    _check(fn(wtype, _p(x), x.size, _p(out)))
    return out


def dot_row(wtype, wrow, acol, k, avx2=False):
    wrow, acol = _u8(wrow), _u8(acol)
    out = C.c_float()
    if avx2:
        if wrow.size < row_bytes(wtype, k) or acol.size < col_bytes(wtype, k):
            raise OracleError(ESHAPE)
        _check(lib.ora_avx2_dot_row(wtype, _p(wrow), _p(acol), k, C.byref(out)))
    else:
        _check(lib.ora_dot_row(wtype, _p(wrow), wrow.size, _p(acol), acol.size, k, C.byref(out)))
    return np.float32(out.value)


def dot_row_cols(wtype, wrow, acols, k):
    """AVX2 tile: one row against 1..8 columns."""
    wrow = _u8(wrow)
    acols = [_u8(a) for a in acols]
    ptrs = (C.c_void_p * len(acols))(*[a.ctypes.data for a in acols])
    out = np.empty(len(acols), np.float32)
    _check(lib.ora_avx2_dot_row_cols(wtype, _p(wrow), ptrs, len(acols), k, _p(out)))
    return out


def gemv(wtype, w, rows, k, act, m=1):
    """y[r * m + c] = row r . column c; `act` holds m columns back to back."""
    w, act = _u8(w), _u8(act)
    assert w.size >= rows * row_bytes(wtype, k) and act.size >= m * col_bytes(wtype, k)
    y = np.empty(rows * m, np.float32)
    _check(lib.ora_gemv(wtype, _p(w), rows, k, _p(act), m, _p(y)))
    return y


def q4k_block_sums(wrow, acol, k, q5=False):
    """Per 32-value sub-block: sum of code * activation, and the column's stored isum (Q4_K; with q5 a Q5_K row)."""
    nb = k // 256
    a = np.empty(nb * 8, np.int32)
    s = np.empty(nb * 8, np.int32)
    (lib.ora_q5k_block_sums if q5 else lib.ora_q4k_block_sums)(_p(_u8(wrow)), _p(_u8(acol)), nb, _p(a), _p(s))
    return a, s


def q6k_block_sums(wrow, acol, k, fold=False):
    nb = k // 256
    s = np.empty(nb * 16, np.int32)
    lib.ora_q6k_block_sums(_p(_u8(wrow)), _p(_u8(acol)), nb, int(fold), _p(s))
    return s


def q3k_block_sums(wrow, acol, k):
    """Per 16-value group the sum of (code - 4) * activation."""
    nb = k // 256
    s = np.empty(nb * 16, np.int32)
    lib.ora_q3k_block_sums(_p(_u8(wrow)), _p(_u8(acol)), nb, _p(s))
    return s


def iq2xxs_block_sums(wrow, acol, k, iq3=False):
    """Per sub-block the signed sum and the scale 2s + 1, per super-block the CPU lanes' two aggregates (IQ2_XXS; with
    iq3 an IQ3_XXS row)."""
    nb = k // 256
    i = np.empty(nb * 8, np.int32)
    sc = np.empty(nb * 8, np.int32)
    codes = np.empty(nb, np.int32)
    fold = np.empty(nb, np.int32)
    (lib.ora_iq3xxs_block_sums if iq3 else lib.ora_iq2xxs_block_sums)(_p(_u8(wrow)), _p(_u8(acol)), nb, _p(i), _p(sc),
                                                                      _p(codes), _p(fold))
    return i, sc, codes, fold


def iq4xs_block_sums(wrow, acol, k, fold=False):
    """Per sub-block the sum of level * activation; per super-block the eight scaled lane sums the CPU path holds."""
    nb = k // 256
    i = np.empty(nb * 8, np.int32)
    lanes = np.empty(nb * 8, np.int32)
    lib.ora_iq4xs_block_sums(_p(_u8(wrow)), _p(_u8(acol)), nb, int(fold), _p(i), _p(lanes))
    return i, lanes


def dequant_row(wtype, src, k):
    src = _u8(src)
    out = np.empty(k, np.float32)
    _check(lib.ora_dequant_row(wtype, _p(src), k, _p(out)))
    return out


def dequant_col(wtype, acol, k):
    out = np.empty(k, np.float32)
    _check(lib.ora_dequant_col(wtype, _p(_u8(acol)), k, _p(out)))
    return out


def expf_ik(x):
    return np.float32(lib.ora_expf_ik(C.c_float(float(x))))


def swiglu(gate, up):
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    lib.ora_swiglu(_p(gate), _p(up), gate.size, _p(out))
    return out


def gate_rule(rule, limit, gate, up):
    """(out, finite): a gate . up rule of the CPU path over two vectors; `finite` is the reference functions' flag."""
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    rc = lib.ora_gate_rule(int(rule), float(limit), _p(gate), _p(up), gate.size, _p(out))
    if rc < 0:
        raise ValueError(f"no gate rule {rule}")
    return out, bool(rc)


def route_softmax_topk(logits, top_k, renorm=True):
    logits = _f32(logits)
    ids = np.empty(top_k, np.uint32)
    w = np.empty(top_k, np.float32)
    _check(lib.ora_route_softmax_topk(_p(logits), logits.size, top_k, int(renorm), _p(ids), _p(w)))
    return ids, w


def combine_tokens(down, w, resid, rows, n_slots, m):
    down, w = _f32(down), _f32(w)
    y = np.empty(rows * m, np.float32)
    rp = _p(_f32(resid)) if resid is not None else None
    lib.ora_combine_tokens(_p(down), _p(w), rp, rows, n_slots, m, _p(y))
    return y


def moe_combine(down, w, shexp, resid, rows, n_slots, m):
    down, w, shexp = _f32(down), _f32(w), _f32(shexp)
    y = np.empty(rows * m, np.float32)
    rp = _p(_f32(resid)) if resid is not None else None
    lib.ora_moe_combine(_p(down), _p(w), _p(shexp), rp, rows, n_slots, m, _p(y))
    return y


TILE_COLS, TILE_E_SHIFT, HOST_SLOT = 8, 22, 0xFFFFFFFF


def tile_cap(n_slots, n_experts):
    """crates/gpu/src/q4k_sel.rs:96-98."""
    return min(n_slots, (n_slots + (TILE_COLS - 1) * n_experts) // TILE_COLS)


def grouped_table(sel, n_experts):
    """The grouped slot table and its tile table by definition (crates/gpu/src/q4k_sel.rs:20-41, grouped_buckets
    :480-560, grouped_tiles :562-680): order = the slots by expert, ascending inside a run; start = the runs' bounds;
    tiles = [count, (e << 22) | j ...] with j stepping by 8 through each run, padded with zeros to tile_cap + 1
    words. Ids at or past n_experts (the host's included) join no run. Returns (order, start, tiles, refused) with
    refused = an id past the stack that is not the host's was met."""
    sel = np.asarray(sel, np.uint32).reshape(-1)
    n_slots = sel.size
    order = [s for e in range(n_experts) for s in range(n_slots) if int(sel[s]) == e]
    start = [0]
    for e in range(n_experts):
        start.append(start[-1] + int(np.count_nonzero(sel == e)))
    words = []
    for e in range(n_experts):
        for j in range(start[e], start[e + 1], TILE_COLS):
            words.append((e << TILE_E_SHIFT) | j)
    cap = tile_cap(n_slots, n_experts)
    assert len(words) <= cap
    tiles = np.zeros(cap + 1, np.uint32)
    tiles[0] = len(words)
    tiles[1:1 + len(words)] = words
    refused = bool(np.any((sel >= n_experts) & (sel != HOST_SLOT)))
    return (np.asarray(order + [0] * (n_slots - len(order)), np.uint32), np.asarray(start, np.uint32), tiles, refused)


GEMM_BN = 64


def gemm_route(ids, n_experts):
    """The prefill route table by definition (crates/gpu/src/gemm/route.rs:1-4,109-125,351-362): the slots grouped
    by expert, ascending slot order inside an expert, the refused slots (an id at or past the stack) at the end in
    ascending order; tiles of at most 64 slots as rows (expert, start, len). Returns (cols, tiles, refused count)."""
    ids = np.asarray(ids, np.uint32).reshape(-1)
    cols, tiles = [], []
    for e in range(n_experts):
        run = [s for s in range(ids.size) if int(ids[s]) == e]
        for j in range(0, len(run), GEMM_BN):
            tiles.append((e, len(cols) + j, min(GEMM_BN, len(run) - j)))
        cols += run
    refused = [s for s in range(ids.size) if int(ids[s]) >= n_experts]
    return (np.asarray(cols + refused, np.uint32), np.asarray(tiles, np.uint32).reshape(-1, 3), len(refused))


def quantize_rows(wtype, x, rows, k, n_threads=8):
    """rows x k f32 -> GGUF block bytes, rows back to back."""
    x = _f32(x).reshape(rows, k)
    out = np.empty(rows * row_bytes(wtype, k), np.uint8)
    _check(lib.ora_quantize_rows(wtype, _p(x), rows, k, _p(out), n_threads))
    return out


def quantize_row_iq2xxs(x, qw):
    x, qw = _f32(x), _f32(qw)
    out = np.empty(row_bytes(IQ2_XXS, x.size), np.uint8)
    _check(lib.ora_quantize_row_iq2xxs(_p(x), _p(qw), x.size, _p(out)))
    return out


def iq2xxs_grid_codes():
    codes = np.empty(256, np.uint32)
    neg, words = C.c_int(), C.c_int()
    size = lib.ora_iq2xxs_grid_codes(_p(codes), C.byref(neg), C.byref(words))
    return codes, size, neg.value, words.value


def _layer(hidden, ff, n_experts, types, wg, wu, wd):
    L = MoeLayer(hidden, ff, n_experts, types[0], types[1], types[2], wg.ctypes.data, wu.ctypes.data, wd.ctypes.data)
    return L


def moe_forward(hidden, ff, n_experts, types, wg, wu, wd, x, ids, wts, top_k, n_threads=1, want_h=False,
                avx2_pool=None):
    """One layer step; x[m][hidden], ids/wts[m][top_k] -> y[m][hidden] (and h[m*top_k][ff])."""
    wg, wu, wd = _u8(wg), _u8(wu), _u8(wd)
    x = _f32(x)
    m = x.size // hidden
    ids = np.ascontiguousarray(ids, np.uint32)
    wts = _f32(wts)
    L = _layer(hidden, ff, n_experts, types, wg, wu, wd)
    y = np.empty(m * hidden, np.float32)
    h = np.empty(m * top_k * ff, np.float32) if want_h else None
    hp = _p(h) if want_h else None
    if avx2_pool is not None:
        rc = lib.ora_avx2_moe_forward(avx2_pool, C.byref(L), _p(x), m, _p(ids), _p(wts), top_k, _p(y), hp)
    else:
        rc = lib.ora_moe_forward(C.byref(L), _p(x), m, _p(ids), _p(wts), top_k, _p(y), hp, n_threads)
    _check(rc)
    return (y, h) if want_h else y


def sum_sq_f64(x):
    x = np.ascontiguousarray(x, np.float32)
    return float(lib.ora_sum_sq_f64(_p(x), x.size))


def rms_norm(x, gain, eps):
    x, gain = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(gain, np.float32)
    out = np.empty(x.size, np.float32)
    lib.ora_rms_norm(_p(x), _p(gain), float(eps), x.size, _p(out))
    return out


def dot_f32(w, x):
    w, x = np.ascontiguousarray(w, np.float32), np.ascontiguousarray(x, np.float32)
    out = np.empty(1, np.float32)
    _check(lib.ora_dot_f32(_p(w), _p(x), x.size, _p(out)))
    return out[0]


def router_logits(router, x, gain=None, eps=0.0):
    """(normed rows, logits) of the tokens x[m, hidden] against the f32 router rows router[n_experts, hidden]."""
    router, x = np.ascontiguousarray(router, np.float32), np.ascontiguousarray(x, np.float32)
    n_experts, hidden = router.shape
    m = x.size // hidden
    g = None if gain is None else np.ascontiguousarray(gain, np.float32)
    normed = np.empty((m, hidden), np.float32)
    logits = np.empty((m, n_experts), np.float32)
    _check(lib.ora_router_logits(_p(router), n_experts, hidden, _p(x), _p(g) if g is not None else None, float(eps), m,
                                 _p(normed), _p(logits)))
    return normed, logits


# ------------------------------------------------------------------------------------------------ the card rule

def card_q8_1(x):
    """The GPU tier's q8_1 form of the columns x[m, k] (crates/qdot/src/lib.rs:2885 card_q8_1): (codes i8 [m, k],
    d8 f32 [m, k / 128], s8 i32 [m, k / 32], refused bool [m, k / 128])."""
    x = np.atleast_2d(_f32(x))
    m, k = x.shape
    codes, d8 = np.empty((m, k), np.int8), np.empty((m, k // 128), np.float32)
    s8, refused = np.empty((m, k // 32), np.int32), np.empty((m, k // 128), np.uint8)
    for c in range(m):
        rc = lib.ora_card_q8_1(_p(x[c]), k, _p(codes[c]), _p(d8[c]), _p(s8[c]), _p(refused[c]))
        if rc < 0:
            raise OracleError(rc)
    return codes, d8, s8, refused.astype(bool)


def card_dot_row(wtype, wrow, k, codes, d8, s8):
    out = np.empty(1, np.float32)
    _check(lib.ora_card_dot_row(wtype, _p(_u8(wrow)), k, _p(np.ascontiguousarray(codes, np.int8)), _p(_f32(d8)),
                                _p(np.ascontiguousarray(s8, np.int32)), _p(out)))
    return out[0]


def card_gemv(wtype, w, rows, k, codes, d8, s8):
    """y[r * m + c] over the m columns of (codes, d8, s8) as card_q8_1 returns them."""
    codes, d8, s8 = np.ascontiguousarray(codes, np.int8), _f32(d8), np.ascontiguousarray(s8, np.int32)
    m = codes.size // k
    y = np.empty(rows * m, np.float32)
    _check(lib.ora_card_gemv(wtype, _p(_u8(w)), rows, k, _p(codes), _p(d8), _p(s8), m, _p(y)))
    return y


def card_gemv_sel(wtype, w, n_experts, rows_per_expert, k, codes, d8, s8, sel):
    """y[s * rows_per_expert + r]: slot s's column against the rows of expert sel[s]."""
    codes, d8, s8 = np.ascontiguousarray(codes, np.int8), _f32(d8), np.ascontiguousarray(s8, np.int32)
    sel = np.ascontiguousarray(sel, np.uint32)
    y = np.empty(sel.size * rows_per_expert, np.float32)
    _check(lib.ora_card_gemv_sel(wtype, _p(_u8(w)), n_experts, rows_per_expert, k, _p(codes), _p(d8), _p(s8), _p(sel),
                                 sel.size, _p(y)))
    return y
