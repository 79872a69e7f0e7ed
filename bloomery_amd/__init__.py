"""bloomery_amd: MI355X-native quantized MoE expert matmul (Q3_K / Q4_K / Q5_K / Q6_K / IQ2_XXS / IQ3_XXS / IQ4_XS x Q8) behind the kernel-call
surface of the reference's crates/gpu.

This module is a thin ctypes view of the C ABI in include/bm_moe.h (bloomery_amd/libbm_moe_hip.so, hand-written
HIP for gfx950). The names mirror the reference's host objects: `Gpu` (crates/gpu/src/lib.rs:2529), `DeviceTensor`
(crates/gpu/src/tensor.rs:588), `Q8Act` (:811) and the `enqueue_*` launchers; a refusal raises `GpuError` with the
library's message, as the reference returns `GpuError::Shape` / `Driver`.

There is no CPU fallback: without the built library, or without a GPU, every entry raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbm_moe_hip.so")

Q3_K, Q4_K, Q5_K, Q6_K, IQ2_XXS, IQ3_XXS, IQ4_XS = 11, 12, 13, 14, 16, 18, 23
FAULT_NONE = 0xFFFFFFFF
LAYER_NONE = 0xFFFF
SITE_QUANT_COLUMN, SITE_ROUTER, SITE_EXPERT_ID = 1, 5, 7
GEMM_EXACT, GEMM_FAST, GEMM_FAST_F16 = 0, 1, 2
DOWN_RING, DOWN_SPLIT = 0, 1
PATH_AUTO, PATH_PER_SLOT, PATH_GROUPED, PATH_GEMM = 0, 1, 2, 3
ACT_SILU_MUL, ACT_SWIGLU_CLAMP, ACT_SWIGLU_OAI, ACT_SITU, ACT_SWIGLU_GCLAMP = 0, 1, 2, 3, 4
SITE_F32_PRODUCT = 21
HOST_SLOT = 0xFFFFFFFF

OK, ESHAPE, EDRIVER, ETYPE, EARG, EFAULT = 0, -1, -2, -3, -4, -5

# Every symbol include/bm_moe.h declares: (restype, argtypes).
_vp, _i, _i64, _u32 = C.c_void_p, C.c_int, C.c_int64, C.c_uint32
SYMBOLS = {
    "bm_version": (_i, []),
    "bm_ctx_create": (_i, [_i, C.POINTER(_vp)]),
    "bm_ctx_create_on_stream": (_i, [_i, _vp, C.POINTER(_vp)]),
    "bm_ctx_destroy": (None, [_vp]),
    "bm_ctx_stream": (_vp, [_vp]),
    "bm_ctx_sync": (_i, [_vp]),
    "bm_last_error": (C.c_char_p, [_vp]),
    "bm_set_layer": (_i, [_vp, _u32]),
    "bm_fault_read": (_i, [_vp, _u32, C.POINTER(_u32), C.POINTER(_u32)]),
    "bm_fault_clear": (_i, [_vp]),
    "bm_fault_word_dev": (_vp, [_vp]),
    "bm_row_bytes": (_i64, [_i, _i]),
    "bm_col_bytes": (_i64, [_i, _i]),
    "bm_dev_alloc": (_i, [_vp, C.c_size_t, C.POINTER(_vp)]),
    "bm_dev_free": (_i, [_vp, _vp]),
    "bm_dev_upload": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "bm_dev_download": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "bm_dev_memset": (_i, [_vp, _vp, _i, C.c_size_t]),
    "bm_weights_create": (_i, [_vp, _i, _i64, _i, _vp, C.POINTER(_vp)]),
    "bm_weights_wrap": (_i, [_vp, _i, _i64, _i, _vp, C.POINTER(_vp)]),
    "bm_weights_destroy": (None, [_vp]),
    "bm_weights_dev": (_vp, [_vp]),
    "bm_act_create": (_i, [_vp, _i, _i, _i, C.POINTER(_vp)]),
    "bm_act_destroy": (None, [_vp]),
    "bm_act_download": (_i, [_vp, _vp, _i, _vp]),
    "bm_act_upload": (_i, [_vp, _vp, _i, _vp]),
    "bm_quantize": (_i, [_vp, _vp, _i, _vp]),
    "bm_gemv": (_i, [_vp, _vp, _vp, _i, _vp]),
    "bm_gate_up": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _vp]),
    "bm_tables": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp]),
    "bm_tables_quantize": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "bm_gemv_x": (_i, [_vp, _vp, _vp, _i, _vp, _vp]),
    "bm_gemv_sel": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "bm_combine_tokens": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "bm_down_combine": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "bm_down_combine_h": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "bm_moe_decode": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "bm_moe_decode_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "bm_gate_up_x": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "bm_tile_cap": (_i, [_i, _i]),
    "bm_buckets": (_i, [_vp, _vp, _i, _i, _vp, _vp]),
    "bm_tiles": (_i, [_vp, _vp, _i, _i, _vp]),
    "bm_quantize_ord": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "bm_gate_up_tiles": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _vp]),
    "bm_gemv_tiles": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "bm_route_create": (_i, [_vp, _i, _i, C.POINTER(_vp)]),
    "bm_route_destroy": (None, [_vp]),
    "bm_route_fill": (_i, [_vp, _vp, _i, _vp]),
    "bm_route_fill_quantize": (_i, [_vp, _vp, _i, _vp, _vp, _i, _vp]),
    "bm_route_read": (_i, [_vp, _vp, _vp, _vp, C.POINTER(_i), C.POINTER(_i)]),
    "bm_gemm": (_i, [_vp, _vp, _i, _vp, _vp, _i, _vp]),
    "bm_swiglu_quant": (_i, [_vp, _vp, _vp, _i, _vp, _vp]),
    "bm_swiglu_quant_sel": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "bm_moe_combine": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "bm_set_gate_rule": (_i, [_vp, _i, C.c_float]),
    "bm_route_softmax": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "bm_router_logits": (_i, [_vp, _vp, _vp, _vp, C.c_float, _i, _i, _i, _vp, _vp]),
    "bm_scratch_create": (_i, [_vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "bm_scratch_destroy": (None, [_vp]),
    "bm_scratch_set_path": (_i, [_vp, _i, _i, _i]),
    "bm_scratch_path_for": (_i, [_vp, _i]),
    "bm_moe_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp]),
    "bm_norm_route": (_i, [_vp, _vp, _vp, _vp, C.c_float, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "bm_card_quantize": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp]),
    "bm_card_gemv": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "bm_card_gemv_sel": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "bm_gguf_open": (_i, [C.c_char_p, C.POINTER(_vp)]),
    "bm_gguf_open_split": (_i, [C.c_char_p, C.POINTER(_vp)]),
    "bm_gguf_close": (None, [_vp]),
    "bm_gguf_last_error": (C.c_char_p, []),
    "bm_gguf_version": (_i, [_vp]),
    "bm_gguf_tensor_count": (_i64, [_vp]),
    "bm_gguf_tensor_at": (_i, [_vp, _i64, _vp]),
    "bm_gguf_find": (_i, [_vp, C.c_char_p, _vp]),
    "bm_gguf_get_u64": (_i, [_vp, C.c_char_p, C.POINTER(C.c_uint64)]),
    "bm_gguf_get_f32": (_i, [_vp, C.c_char_p, C.POINTER(C.c_float)]),
    "bm_gguf_get_str": (C.c_char_p, [_vp, C.c_char_p]),
    "bm_weights_from_gguf": (_i, [_vp, _vp, C.c_char_p, C.POINTER(_vp), C.POINTER(_i), C.POINTER(_i)]),
    "bm_set_gemm_mode": (_i, [_vp, _i]),
    "bm_set_down_form": (_i, [_vp, _i]),
    "bm_block_sums": (_i, [_vp, _vp, _i64, _vp, _i, _vp]),
    "bm_capture_begin": (_i, [_vp]),
    "bm_capture_end": (_i, [_vp, C.POINTER(_vp)]),
    "bm_graph_launch": (_i, [_vp, _vp]),
    "bm_graph_destroy": (None, [_vp]),
    "bm_event_create": (_i, [_vp, C.POINTER(_vp)]),
    "bm_event_record": (_i, [_vp, _vp]),
    "bm_event_wait": (_i, [_vp, _vp]),
    "bm_event_elapsed_ms": (_i, [_vp, _vp, _vp, C.POINTER(C.c_float)]),
    "bm_event_destroy": (None, [_vp]),
}


class GpuError(RuntimeError):
    """A refusal of the library: `code` is the C ABI's return value, the text its bm_last_error message."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


_lib = None


def load_library(path=LIB_PATH):
    """Load the built library and bind every declared symbol. Never compiles; raises when the file is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise GpuError(EDRIVER, f"{path} is not built: run __graft_entry__.build() (hipcc, gfx950); there is no CPU path")
    lib = C.CDLL(path)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def row_bytes(wtype, k):
    return int(load_library().bm_row_bytes(wtype, k))


def col_bytes(wtype, k):
    return int(load_library().bm_col_bytes(wtype, k))


class DeviceBuffer:
    """A typed device allocation (the reference's DeviceBuffer<T>)."""

    def __init__(self, gpu, dtype, count):
        self.gpu, self.dtype, self.count = gpu, np.dtype(dtype), int(count)
        p = _vp()
        gpu._check(gpu.lib.bm_dev_alloc(gpu.ctx, self.count * self.dtype.itemsize, C.byref(p)))
        self.ptr = p.value

    @property
    def nbytes(self):
        return self.count * self.dtype.itemsize

    def upload(self, host):
        host = np.ascontiguousarray(host, self.dtype).reshape(-1)
        assert host.size <= self.count
        self.gpu._check(self.gpu.lib.bm_dev_upload(self.gpu.ctx, self.ptr, host.ctypes.data, host.nbytes))
        return self

    def download(self, count=None):
        out = np.empty(self.count if count is None else count, self.dtype)
        self.gpu._check(self.gpu.lib.bm_dev_download(self.gpu.ctx, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def fill_bytes(self, byte):
        self.gpu._check(self.gpu.lib.bm_dev_memset(self.gpu.ctx, self.ptr, byte, self.nbytes))
        return self

    def free(self):
        if self.ptr:
            self.gpu.lib.bm_dev_free(self.gpu.ctx, self.ptr)
            self.ptr = None


class DeviceTensor:
    """An expert stack or one matrix: rows of GGUF block bytes on the device."""

    def __init__(self, gpu, wtype, rows, k, host_bytes=None, dev_ptr=None):
        self.gpu, self.wtype, self.rows, self.k = gpu, wtype, int(rows), int(k)
        h = _vp()
        if host_bytes is not None:
            host_bytes = np.ascontiguousarray(host_bytes, np.uint8)
            need = self.rows * row_bytes(wtype, k) if row_bytes(wtype, k) > 0 else 0
            if host_bytes.size < need:
                raise GpuError(ESHAPE, f"DeviceTensor: {host_bytes.size} bytes for {rows} rows of {need // max(rows, 1)}")
            gpu._check(gpu.lib.bm_weights_create(gpu.ctx, wtype, self.rows, self.k, host_bytes.ctypes.data, C.byref(h)))
        else:
            gpu._check(gpu.lib.bm_weights_wrap(gpu.ctx, wtype, self.rows, self.k, dev_ptr, C.byref(h)))
        self.handle = h.value

    @property
    def dev_ptr(self):
        return self.gpu.lib.bm_weights_dev(self.handle)

    def free(self):
        if self.handle:
            self.gpu.lib.bm_weights_destroy(self.handle)
            self.handle = None


class _GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("type", _i), ("n_dims", _i), ("dims", C.c_uint64 * 4), ("offset", C.c_uint64),
                ("nbytes", C.c_uint64), ("data", _vp)]


class Gguf:
    """A model file's header and mapping (crates/gguf/src/lib.rs Gguf): tensors by name, key-values, and a tensor as a
    weight stack on a Gpu. Host code: opening and reading need no GPU. With split=True the path is a model's first
    shard and the object answers for the whole split set (crates/gguf/src/lib.rs Split)."""

    def __init__(self, path, split=False):
        self.lib = load_library()
        h = _vp()
        rc = (self.lib.bm_gguf_open_split if split else self.lib.bm_gguf_open)(os.fsencode(path), C.byref(h))
        if rc:
            raise GpuError(rc, self.lib.bm_gguf_last_error().decode(errors="replace"))
        self.handle = h.value

    def _tensor(self, t):
        return {"name": t.name.decode(errors="replace"), "type": t.type, "dims": [int(t.dims[d]) for d in range(t.n_dims)],
                "offset": int(t.offset), "nbytes": int(t.nbytes), "data": t.data}

    @property
    def version(self):
        return self.lib.bm_gguf_version(self.handle)

    def tensors(self):
        out = []
        for i in range(self.lib.bm_gguf_tensor_count(self.handle)):
            t = _GgufTensor()
            rc = self.lib.bm_gguf_tensor_at(self.handle, i, C.byref(t))
            if rc:
                raise GpuError(rc, self.lib.bm_gguf_last_error().decode(errors="replace"))
            out.append(self._tensor(t))
        return out

    def find(self, name):
        t = _GgufTensor()
        rc = self.lib.bm_gguf_find(self.handle, name.encode(), C.byref(t))
        if rc:
            raise GpuError(rc, self.lib.bm_gguf_last_error().decode(errors="replace"))
        return self._tensor(t)

    def data(self, name):
        """The tensor's bytes, copied out of the mapping."""
        t = self.find(name)
        return np.ctypeslib.as_array(C.cast(t["data"], C.POINTER(C.c_uint8)), (t["nbytes"],)).copy() if t["nbytes"] else \
            np.empty(0, np.uint8)

    def get_u64(self, key):
        v = C.c_uint64()
        rc = self.lib.bm_gguf_get_u64(self.handle, key.encode(), C.byref(v))
        if rc:
            raise GpuError(rc, self.lib.bm_gguf_last_error().decode(errors="replace"))
        return v.value

    def get_f32(self, key):
        v = C.c_float()
        rc = self.lib.bm_gguf_get_f32(self.handle, key.encode(), C.byref(v))
        if rc:
            raise GpuError(rc, self.lib.bm_gguf_last_error().decode(errors="replace"))
        return v.value

    def get_str(self, key):
        v = self.lib.bm_gguf_get_str(self.handle, key.encode())
        return v.decode(errors="replace") if v is not None else None

    def weights(self, gpu, name):
        """The tensor as a DeviceTensor on `gpu`, with (rows_per_expert, n_experts) of an expert stack."""
        h, rpe, ne = _vp(), _i(), _i()
        gpu._check(self.lib.bm_weights_from_gguf(gpu.ctx, self.handle, name.encode(), C.byref(h), C.byref(rpe), C.byref(ne)))
        t = self.find(name)
        w = DeviceTensor.__new__(DeviceTensor)
        w.gpu, w.wtype, w.rows, w.k, w.handle = gpu, t["type"], rpe.value * ne.value, t["dims"][0], h.value
        return w, rpe.value, ne.value

    def close(self):
        if self.handle:
            self.lib.bm_gguf_close(self.handle)
            self.handle = None


class Q8Act:
    """Quantized activation scratch: m_cap columns of k values in the form weight type `wtype` dots against."""

    def __init__(self, gpu, wtype, k, m_cap):
        self.gpu, self.wtype, self.k, self.m_cap = gpu, wtype, int(k), int(m_cap)
        h = _vp()
        gpu._check(gpu.lib.bm_act_create(gpu.ctx, wtype, self.k, self.m_cap, C.byref(h)))
        self.handle = h.value

    def download(self, col):
        out = np.empty(col_bytes(self.wtype, self.k), np.uint8)
        self.gpu._check(self.gpu.lib.bm_act_download(self.gpu.ctx, self.handle, col, out.ctypes.data))
        return out

    def upload(self, col, host_bytes):
        host_bytes = np.ascontiguousarray(host_bytes, np.uint8)
        assert host_bytes.size == col_bytes(self.wtype, self.k)
        self.gpu._check(self.gpu.lib.bm_act_upload(self.gpu.ctx, self.handle, col, host_bytes.ctypes.data))

    def free(self):
        if self.handle:
            self.gpu.lib.bm_act_destroy(self.handle)
            self.handle = None


class Route:
    """A prefill route table (GemmRoute, crates/gpu/src/gemm/route.rs:109)."""

    def __init__(self, gpu, max_slots, n_experts):
        self.gpu, self.max_slots, self.n_experts = gpu, max_slots, n_experts
        h = _vp()
        gpu._check(gpu.lib.bm_route_create(gpu.ctx, max_slots, n_experts, C.byref(h)))
        self.handle = h

    def fill(self, ids, n_slots):
        self.gpu._check(self.gpu.lib.bm_route_fill(self.gpu.ctx, _ptr(ids), n_slots, self.handle))
        self.n_slots = n_slots

    def fill_quantize(self, ids, n_slots, x, m, act):
        """fill and Gpu.enqueue_quantize(x, m, act) as one launch (same table, same column bytes)."""
        self.gpu._check(self.gpu.lib.bm_route_fill_quantize(self.gpu.ctx, _ptr(ids), n_slots, self.handle, _ptr(x), m, act.handle))
        self.n_slots = n_slots

    def read(self):
        """(cols, tiles as rows of (expert, start, len), refused count) of the last fill."""
        cap = self.n_slots // 64 + min(self.n_experts, self.n_slots)
        cols = np.empty(self.n_slots, np.uint32)
        tiles = np.zeros(2 * cap, np.uint32)
        n, r = _i(), _i()
        self.gpu._check(self.gpu.lib.bm_route_read(self.gpu.ctx, self.handle, cols.ctypes.data_as(_vp),
                                                   tiles.ctypes.data_as(_vp), C.byref(n), C.byref(r)))
        t = tiles[:2 * n.value].reshape(-1, 2)
        return cols, np.stack([t[:, 0], t[:, 1] & 0xFFFF, t[:, 1] >> 16], axis=1), r.value

    def free(self):
        if self.handle:
            self.gpu.lib.bm_route_destroy(self.handle)
            self.handle = None


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, DeviceBuffer):
        return x.ptr
    return x  # a raw device address (e.g. torch.Tensor.data_ptr())


class GateAct(C.Structure):
    """bm_gate_act: a gate . up launch's own rule and its limit (SiTU: the gate's beta)."""
    _fields_ = [("rule", C.c_int), ("limit", C.c_float)]


def _rule(rule):
    """None (the context's rule) or (ACT_*, limit) as the bm_gate_act a launch takes."""
    if rule is None:
        return None
    code, limit = rule
    return C.cast(C.pointer(GateAct(int(code), float(limit))), C.c_void_p)


class Scratch:
    """bm_scratch: what bm_moe_forward's three paths keep between their launches, for up to max_tokens tokens."""

    def __init__(self, gpu, gate_type, down_type, hidden, ff, n_experts, n_slots_per_token, max_tokens):
        self.gpu = gpu
        h = _vp()
        gpu._check(gpu.lib.bm_scratch_create(gpu.ctx, gate_type, down_type, hidden, ff, n_experts, n_slots_per_token, max_tokens,
                                             C.byref(h)))
        self.handle = h.value

    def set_path(self, path, grouped_from=0, gemm_from=0):
        self.gpu._check(self.gpu.lib.bm_scratch_set_path(self.handle, path, grouped_from, gemm_from))

    def path_for(self, m):
        return self.gpu.lib.bm_scratch_path_for(self.handle, m)

    def free(self):
        if self.handle:
            self.gpu.lib.bm_scratch_destroy(self.handle)
            self.handle = None


class Gpu:
    """A device context: stream, fault word and the launchers (the reference's `Gpu` and its kernel structs)."""

    def __init__(self, device=0, stream=None):
        self.lib = load_library()
        ctx = _vp()
        if stream is None:
            rc = self.lib.bm_ctx_create(device, C.byref(ctx))
        else:
            rc = self.lib.bm_ctx_create_on_stream(device, stream, C.byref(ctx))
        if rc != OK:
            raise GpuError(rc, self.lib.bm_last_error(None).decode(errors="replace"))
        self.ctx = ctx.value

    def _check(self, rc):
        if rc != OK:
            raise GpuError(rc, self.lib.bm_last_error(self.ctx).decode(errors="replace"))

    def close(self):
        if self.ctx:
            self.lib.bm_ctx_destroy(self.ctx)
            self.ctx = None

    # -- context
    def stream(self):
        return self.lib.bm_ctx_stream(self.ctx)

    def sync(self):
        self._check(self.lib.bm_ctx_sync(self.ctx))

    def set_layer(self, layer):
        self._check(self.lib.bm_set_layer(self.ctx, layer))

    def fault(self, layer=LAYER_NONE):
        w0, mask = _u32(), _u32()
        self._check(self.lib.bm_fault_read(self.ctx, layer, C.byref(w0), C.byref(mask)))
        return w0.value, mask.value

    def fault_clear(self):
        self._check(self.lib.bm_fault_clear(self.ctx))

    # -- buffers
    def buffer(self, dtype, count, host=None):
        b = DeviceBuffer(self, dtype, count)
        if host is not None:
            b.upload(host)
        return b

    def upload(self, host, dtype=None):
        host = np.ascontiguousarray(host, dtype)
        return DeviceBuffer(self, host.dtype, host.size).upload(host)

    def weights(self, wtype, rows, k, host_bytes):
        return DeviceTensor(self, wtype, rows, k, host_bytes=host_bytes)

    def act(self, wtype, k, m_cap):
        return Q8Act(self, wtype, k, m_cap)

    # -- graphs and events
    def capture_begin(self):
        self._check(self.lib.bm_capture_begin(self.ctx))

    def capture_end(self):
        g = _vp()
        self._check(self.lib.bm_capture_end(self.ctx, C.byref(g)))
        return g.value

    def graph_launch(self, graph):
        self._check(self.lib.bm_graph_launch(self.ctx, graph))

    def graph_destroy(self, graph):
        self.lib.bm_graph_destroy(graph)

    def event(self):
        e = _vp()
        self._check(self.lib.bm_event_create(self.ctx, C.byref(e)))
        return e.value

    def event_record(self, event):
        self._check(self.lib.bm_event_record(self.ctx, event))

    def event_wait(self, event):
        """What is enqueued on this context's stream from here on waits for `event` (another context's record): Stream::wait."""
        self._check(self.lib.bm_event_wait(self.ctx, event))

    def event_elapsed_ms(self, start, stop):
        ms = C.c_float()
        self._check(self.lib.bm_event_elapsed_ms(self.ctx, start, stop, C.byref(ms)))
        return ms.value

    def event_destroy(self, event):
        self.lib.bm_event_destroy(event)

    # -- launchers (asynchronous on the context's stream)
    def enqueue_quantize(self, x, m, act):
        self._check(self.lib.bm_quantize(self.ctx, _ptr(x), m, act.handle))

    def enqueue_gemv(self, w, act, m, y):
        self._check(self.lib.bm_gemv(self.ctx, w.handle, act.handle, m, _ptr(y)))

    def enqueue_gate_up(self, wg, wu, act, sel, n_slots, rows_per_expert, slots_per_col, h, act_h=None, rule=None):
        """rule: (ACT_*, limit) for this launch (GateUpArgs' act), None for the context's."""
        self._check(self.lib.bm_gate_up(self.ctx, wg.handle, wu.handle, act.handle, _ptr(sel), n_slots, rows_per_expert,
                                        slots_per_col, _rule(rule), _ptr(h), act_h.handle if act_h is not None else None))

    def enqueue_gemv_sel(self, w, act, sel, n_slots, rows_per_expert, y):
        self._check(self.lib.bm_gemv_sel(self.ctx, w.handle, act.handle, _ptr(sel), n_slots, rows_per_expert, _ptr(y)))

    def enqueue_combine_tokens(self, down, w, resid, rows, n_slots, m, y):
        self._check(self.lib.bm_combine_tokens(self.ctx, _ptr(down), _ptr(w), _ptr(resid), rows, n_slots, m, _ptr(y)))

    def enqueue_moe_combine(self, down, w, shexp, resid, rows, n_slots, m, y):
        """moe_combine (crates/gpu/src/moe_fused.rs:129-170): (slot sum + shared expert) + residual."""
        self._check(self.lib.bm_moe_combine(self.ctx, _ptr(down), _ptr(w), _ptr(shexp), _ptr(resid) if resid is not None else None,
                                            rows, n_slots, m, _ptr(y)))

    def enqueue_down_combine(self, w, act, sel, wts, resid, n_slots_per_token, m, rows_per_expert, y):
        self._check(self.lib.bm_down_combine(self.ctx, w.handle, act.handle, _ptr(sel), _ptr(wts), _ptr(resid),
                                             n_slots_per_token, m, rows_per_expert, _ptr(y)))

    def enqueue_down_combine_h(self, w, h, act_h, sel, wts, resid, n_slots_per_token, m, rows_per_expert, y):
        """bm_down_combine from the f32 rows of h, quantized in the launch in the form the stack dots against (act_h may be None)."""
        self._check(self.lib.bm_down_combine_h(self.ctx, w.handle, _ptr(h), act_h.handle if act_h is not None else None,
                                               _ptr(sel), _ptr(wts), _ptr(resid), n_slots_per_token, m, rows_per_expert,
                                               _ptr(y)))

    def enqueue_moe_decode(self, wg, wu, wd, x, sel, wts, resid, n_slots_per_token, m, act_h, y, act_x=None, h=None, rule=None):
        """The whole layer step with the quantizers folded in (bm_moe_decode), two launches. A down stack on Q8_K
        columns needs h (f32 scratch of m * n_slots_per_token * ff values)."""
        self._check(self.lib.bm_moe_decode(self.ctx, wg.handle, wu.handle, wd.handle, _ptr(x), _ptr(sel), _ptr(wts),
                                           _ptr(resid), n_slots_per_token, m, _rule(rule), act_h.handle,
                                           act_x.handle if act_x is not None else None, _ptr(h), _ptr(y)))

    def enqueue_moe_decode_noalloc(self, wg, wu, wd, x, sel, wts, resid, n_slots_per_token, m, y, rule=None):
        """bm_moe_decode in two launches with the scratch between them held by the library: nothing is allocated."""
        self._check(self.lib.bm_moe_decode_noalloc(self.ctx, wg.handle, wu.handle, wd.handle, _ptr(x), _ptr(sel), _ptr(wts),
                                                   _ptr(resid), n_slots_per_token, m, _rule(rule), _ptr(y)))

    def enqueue_gate_up_x(self, wg, wu, x, sel, n_slots_per_token, m, rows_per_expert, act_h, act_x=None, h=None, rule=None):
        self._check(self.lib.bm_gate_up_x(self.ctx, wg.handle, wu.handle, _ptr(x), _ptr(sel), n_slots_per_token, m,
                                          rows_per_expert, _rule(rule), act_h.handle if act_h is not None else None,
                                          act_x.handle if act_x is not None else None, _ptr(h)))

    def enqueue_gemv_x(self, w, x, m, y, act_out=None):
        """Quantizer and gemv in one launch: y[r * m + c] from the f32 columns x[m, k]."""
        self._check(self.lib.bm_gemv_x(self.ctx, w.handle, _ptr(x), m, act_out.handle if act_out is not None else None, _ptr(y)))

    # -- the card rule: the reference GPU tier's q8_1 columns and 32-lane row walks
    def enqueue_card_quantize(self, x, m, k, codes, d8, s8):
        self._check(self.lib.bm_card_quantize(self.ctx, _ptr(x), m, k, _ptr(codes), _ptr(d8), _ptr(s8)))

    def enqueue_card_gemv(self, w, codes, d8, s8, m, y):
        self._check(self.lib.bm_card_gemv(self.ctx, w.handle, _ptr(codes), _ptr(d8), _ptr(s8), m, _ptr(y)))

    def enqueue_card_gemv_sel(self, w, codes, d8, s8, sel, n_slots, rows_per_expert, y):
        self._check(self.lib.bm_card_gemv_sel(self.ctx, w.handle, _ptr(codes), _ptr(d8), _ptr(s8), _ptr(sel), n_slots,
                                              rows_per_expert, _ptr(y)))

    # -- grouped decode: the slot table by expert and the tile launchers
    def tile_cap(self, n_slots, n_experts):
        return self.lib.bm_tile_cap(n_slots, n_experts)

    def enqueue_buckets(self, sel, n_slots, n_experts, order, start):
        self._check(self.lib.bm_buckets(self.ctx, _ptr(sel), n_slots, n_experts, _ptr(order), _ptr(start)))

    def enqueue_tables(self, sel, n_slots, n_experts, order, start, tiles):
        """enqueue_buckets and enqueue_tiles as one launch."""
        self._check(self.lib.bm_tables(self.ctx, _ptr(sel), n_slots, n_experts, _ptr(order), _ptr(start), _ptr(tiles)))

    def enqueue_tables_quantize(self, sel, n_slots, n_experts, order, start, tiles, x, m, act):
        """enqueue_tables and enqueue_quantize as one launch (same tables, same column bytes)."""
        self._check(self.lib.bm_tables_quantize(self.ctx, _ptr(sel), n_slots, n_experts, _ptr(order), _ptr(start), _ptr(tiles), _ptr(x), m,
                                                act.handle))

    def enqueue_tiles(self, start, n_experts, n_slots, tiles):
        self._check(self.lib.bm_tiles(self.ctx, _ptr(start), n_experts, n_slots, _ptr(tiles)))

    def enqueue_quantize_ord(self, x, start, n_experts, m_cols, act):
        self._check(self.lib.bm_quantize_ord(self.ctx, _ptr(x), _ptr(start), n_experts, m_cols, act.handle))

    def enqueue_gate_up_tiles(self, wg, wu, act, order, start, tiles, n_slots, rows_per_expert, slots_per_col, h,
                              act_h=None, rule=None):
        self._check(self.lib.bm_gate_up_tiles(self.ctx, wg.handle, wu.handle, act.handle, _ptr(order), _ptr(start),
                                              _ptr(tiles), n_slots, rows_per_expert, slots_per_col, _rule(rule), _ptr(h),
                                              act_h.handle if act_h is not None else None))

    def enqueue_gemv_tiles(self, w, act, order, start, tiles, n_slots, rows_per_expert, y):
        self._check(self.lib.bm_gemv_tiles(self.ctx, w.handle, act.handle, _ptr(order), _ptr(start), _ptr(tiles),
                                           n_slots, rows_per_expert, _ptr(y)))

    # -- prefill
    def route(self, max_slots, n_experts):
        return Route(self, max_slots, n_experts)

    def enqueue_gemm(self, w, rows_per_expert, act, route, top_k, y):
        """top_k > 0: every slot of a token reads the token's column; 0: a column a slot."""
        self._check(self.lib.bm_gemm(self.ctx, w.handle, rows_per_expert, act.handle, route.handle, top_k, _ptr(y)))

    def set_gate_rule(self, rule, limit=0.0):
        """The Act of the gate . up launches that follow and pass no rule of their own (crates/gpu/src/kquant/act.rs:21-57)."""
        self._check(self.lib.bm_set_gate_rule(self.ctx, rule, float(limit)))

    def set_gemm_mode(self, mode):
        self._check(self.lib.bm_set_gemm_mode(self.ctx, mode))

    def set_down_form(self, form):
        """DOWN_RING (default) or DOWN_SPLIT: how the down + combine launch walks a row; the same bits (bm_set_down_form)."""
        self._check(self.lib.bm_set_down_form(self.ctx, form))

    def enqueue_swiglu_quant(self, g, u, n_cols, act, rule=None, sel=None, n_experts=0):
        """With sel: only the columns of slots whose expert is on the stack (a host-served slot's column is left as it is)."""
        if sel is not None:
            self._check(self.lib.bm_swiglu_quant_sel(self.ctx, _ptr(g), _ptr(u), _ptr(sel), n_experts, n_cols, _rule(rule), act.handle))
            return
        self._check(self.lib.bm_swiglu_quant(self.ctx, _ptr(g), _ptr(u), n_cols, _rule(rule), act.handle))

    def enqueue_route_softmax(self, logits, n_tokens, n_experts, top_k, renorm, probs, ids, weights):
        """RouterKernels::enqueue_route (crates/gpu/src/route_softmax.rs:1643): softmax, top-k, renormalised weights."""
        self._check(self.lib.bm_route_softmax(self.ctx, _ptr(logits), n_tokens, n_experts, top_k, int(bool(renorm)),
                                              _ptr(probs) if probs is not None else None, _ptr(ids), _ptr(weights)))

    def scratch(self, gate_type, down_type, hidden, ff, n_experts, n_slots_per_token, max_tokens):
        return Scratch(self, gate_type, down_type, hidden, ff, n_experts, n_slots_per_token, max_tokens)

    def enqueue_moe_forward(self, scratch, wg, wu, wd, x, sel, wts, resid, m, y, rule=None):
        """The expert step for any number of tokens (bm_moe_forward): per slot, grouped by expert or the grouped GEMM,
        by the number of tokens."""
        self._check(self.lib.bm_moe_forward(self.ctx, scratch.handle, wg.handle, wu.handle, wd.handle, _ptr(x), _ptr(sel), _ptr(wts),
                                            _ptr(resid), m, _rule(rule), _ptr(y)))

    def enqueue_norm_route(self, router, x, gain, eps, n_tokens, n_experts, hidden, top_k, renorm, normed, logits, probs, ids, weights,
                           act_x=None):
        """enqueue_router_logits and enqueue_route_softmax as one launch (bm_norm_route): the same bits in every output. With act_x
        the launch also leaves the normed rows as quantized columns (the bytes enqueue_quantize makes of `normed`)."""
        self._check(self.lib.bm_norm_route(self.ctx, _ptr(router), _ptr(x), _ptr(gain) if gain is not None else None, float(eps),
                                           n_tokens, n_experts, hidden, top_k, int(bool(renorm)),
                                           _ptr(normed) if normed is not None else None, _ptr(logits),
                                           _ptr(probs) if probs is not None else None, _ptr(ids), _ptr(weights),
                                           act_x.handle if act_x is not None else None))

    def enqueue_router_logits(self, router, x, gain, eps, n_tokens, n_experts, hidden, normed, logits):
        """The FFN norm (gain None: none) and the router's f32 logits, the step before enqueue_route_softmax
        (bm_router_logits); normed (optional) receives the normed rows."""
        self._check(self.lib.bm_router_logits(self.ctx, _ptr(router), _ptr(x), _ptr(gain) if gain is not None else None,
                                              float(eps), n_tokens, n_experts, hidden,
                                              _ptr(normed) if normed is not None else None, _ptr(logits)))

    def enqueue_block_sums(self, w, row, act, col, out):
        self._check(self.lib.bm_block_sums(self.ctx, w.handle, row, act.handle, col, _ptr(out)))
