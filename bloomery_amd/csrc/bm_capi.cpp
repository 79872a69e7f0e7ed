// The C ABI of libbm_moe_hip.so (include/bm_moe.h): handles, the host-side geometry checks the reference's
// launchers make before a launch (crates/gpu/src/q4k_sel.rs:990-1042 and its siblings), and the calls into the
// kernels. Refusals carry a message naming the entry point and the lengths, as GpuError::Shape does.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>

#include <hip/hip_runtime.h>

#include "../../include/bm_moe.h"
#include "bm_kernels.h"

// bm_norm_route's hand-over words: one a (token, expert) of the largest launch it takes
static constexpr size_t kRouteHandWords = (size_t)bmk::kNormRouteMaxTokens * bmk::kRouteMaxExperts;

struct bm_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool own_stream = false;
    uint32_t *fault = nullptr;
    uint32_t layer = BM_LAYER_NONE;
    uint32_t *route_hand = nullptr; // bm_norm_route's hand-over words, one a (token, expert), bmk::kRouteArmed between launches
    // polls a routing wave of bm_norm_route waits for its logits (BM_NORM_ROUTE_POLLS in the environment when the context is
    // made, for the tests of the give-up path: the kernels end normally either way)
    uint32_t route_polls = bmk::kRoutePolls;
    int gemm_mode = BM_GEMM_EXACT;
    int down_form = BM_DOWN_RING;
    bmk::GateRule rule = {0u, 0.0f}; // silu(g) * u
    std::string err;
};

struct bm_weights {
    bm_ctx *ctx;
    int wtype;
    int64_t rows;
    int k;
    uint8_t *dev;
    bool owned;
};

struct bm_act {
    bm_ctx *ctx;
    int wtype; // the weight type whose activation form this is
    int k, m_cap;
    uint8_t *dev;
};

static thread_local std::string g_err;

static int fail(bm_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    if (ctx) ctx->err = buf;
    return code;
}

static int driver(bm_ctx *ctx, const char *what, hipError_t e) {
    if (e == hipSuccess) return BM_OK;
    return fail(ctx, BM_EDRIVER, "%s: %s", what, hipGetErrorString(e));
}

static bool known_type(int t) {
    return t == BM_TYPE_Q3_K || t == BM_TYPE_Q4_K || t == BM_TYPE_Q5_K || t == BM_TYPE_Q6_K || t == BM_TYPE_IQ2_XXS || t == BM_TYPE_IQ3_XXS || t == BM_TYPE_IQ4_XS;
}
// Q8_2_X4 for Q4_K, Q5_K and Q6_K, Q8_K for Q3_K, IQ2_XXS, IQ3_XXS and IQ4_XS (crates/gguf/src/qtype.rs host_act).
static int act_form(int t) { return t == BM_TYPE_Q3_K || t == BM_TYPE_IQ2_XXS || t == BM_TYPE_IQ3_XXS || t == BM_TYPE_IQ4_XS ? 1 : 0; }
// Bytes between two columns of a bm_act on the device (the CPU path's bytes plus the dot kernels' tables).
static size_t dev_col_bytes(int wtype, int k) { return (size_t)bmk::act_col_bytes(wtype, k); }

extern "C" {

int bm_version(void) { return 101; }

int64_t bm_row_bytes(int wtype, int k) {
    if (!known_type(wtype)) return BM_ETYPE;
    if (k <= 0 || k % 256 != 0) return BM_ESHAPE;
    const int bb = wtype == BM_TYPE_Q3_K ? 110 : wtype == BM_TYPE_Q4_K ? 144 : wtype == BM_TYPE_Q5_K ? 176 : wtype == BM_TYPE_Q6_K ? 210 : wtype == BM_TYPE_IQ4_XS ? 136 : wtype == BM_TYPE_IQ3_XXS ? 98 : 66;
    return (int64_t)(k / 256) * bb;
}

int64_t bm_col_bytes(int wtype, int k) {
    if (!known_type(wtype)) return BM_ETYPE;
    if (k <= 0 || k % 256 != 0) return BM_ESHAPE;
    return (int64_t)(k / 256) * (act_form(wtype) ? 296 : 288);
}

const char *bm_last_error(const bm_ctx *ctx) { return ctx ? ctx->err.c_str() : g_err.c_str(); }

static int ctx_make(int device, hipStream_t stream, bool own, bm_ctx **out) {
    if (!out) return fail(nullptr, BM_EARG, "bm_ctx_create: out is NULL");
    *out = nullptr;
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return fail(nullptr, BM_EDRIVER, "bm_ctx_create: hipSetDevice(%d): %s", device, hipGetErrorString(e));
    // the device address of the library's static scratch (bm_moe_decode_noalloc), looked up once a device
    e = bmk::static_scratch_init(device);
    if (e != hipSuccess) return fail(nullptr, BM_EDRIVER, "bm_ctx_create: hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
    bm_ctx *c = new (std::nothrow) bm_ctx();
    if (!c) return fail(nullptr, BM_EDRIVER, "bm_ctx_create: out of host memory");
    c->device = device;
    if (const char *polls = getenv("BM_NORM_ROUTE_POLLS")) {
        const long v = atol(polls);
        if (v >= 1 && v <= (long)bmk::kRoutePolls) c->route_polls = (uint32_t)v;
    }
    if (own) {
        e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking); // default priority
        if (e != hipSuccess) {
            delete c;
            return fail(nullptr, BM_EDRIVER, "bm_ctx_create: hipStreamCreate: %s", hipGetErrorString(e));
        }
        c->own_stream = true;
    } else {
        c->stream = stream;
    }
    e = hipMalloc((void **)&c->fault, sizeof(uint32_t) * BM_FAULT_WORDS);
    if (e == hipSuccess) {
        // word 0 all ones, the masks zero: synchronous here, load time
        e = hipMemset(c->fault, 0, sizeof(uint32_t) * BM_FAULT_WORDS);
        if (e == hipSuccess) e = hipMemset(c->fault, 0xff, sizeof(uint32_t));
    }
    if (e == hipSuccess) {
        e = hipMalloc((void **)&c->route_hand, sizeof(uint32_t) * kRouteHandWords);
        if (e == hipSuccess) e = hipMemsetD32(reinterpret_cast<hipDeviceptr_t>(c->route_hand), (int)bmk::kRouteArmed, kRouteHandWords);
    }
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        if (c->fault) (void)hipFree(c->fault);
        if (c->route_hand) (void)hipFree(c->route_hand);
        if (c->own_stream) (void)hipStreamDestroy(c->stream);
        delete c;
        return fail(nullptr, BM_EDRIVER, "bm_ctx_create: fault word: %s", hipGetErrorString(e));
    }
    *out = c;
    return BM_OK;
}

int bm_ctx_create(int device, bm_ctx **out) { return ctx_make(device, nullptr, true, out); }

int bm_ctx_create_on_stream(int device, void *hip_stream, bm_ctx **out) {
    return ctx_make(device, (hipStream_t)hip_stream, false, out);
}

void bm_ctx_destroy(bm_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(ctx->fault);
    (void)hipFree(ctx->route_hand);
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

void *bm_ctx_stream(bm_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int bm_ctx_sync(bm_ctx *ctx) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_ctx_sync: ctx is NULL");
    return driver(ctx, "bm_ctx_sync", hipStreamSynchronize(ctx->stream));
}

int bm_set_layer(bm_ctx *ctx, uint32_t layer) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_set_layer: ctx is NULL");
    if (layer > BM_LAYER_NONE) return fail(ctx, BM_ESHAPE, "bm_set_layer: layer %u is past %u", layer, BM_LAYER_NONE);
    ctx->layer = layer;
    return BM_OK;
}

uint32_t *bm_fault_word_dev(bm_ctx *ctx) { return ctx ? ctx->fault : nullptr; }

int bm_fault_read(bm_ctx *ctx, uint32_t layer, uint32_t *word0, uint32_t *mask) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_fault_read: ctx is NULL");
    if (layer > BM_LAYER_NONE) return fail(ctx, BM_ESHAPE, "bm_fault_read: layer %u is past %u", layer, BM_LAYER_NONE);
    int rc = driver(ctx, "bm_fault_read: sync", hipStreamSynchronize(ctx->stream));
    if (rc) return rc;
    if (word0) rc = driver(ctx, "bm_fault_read", hipMemcpy(word0, ctx->fault, 4, hipMemcpyDeviceToHost));
    if (!rc && mask) rc = driver(ctx, "bm_fault_read", hipMemcpy(mask, ctx->fault + 1 + layer, 4, hipMemcpyDeviceToHost));
    return rc;
}

static bmk::Launch launch_of(bm_ctx *ctx) { return bmk::Launch{ctx->stream, ctx->fault, ctx->layer, ctx->rule, ctx->down_form}; }
static int rule_checked(bm_ctx *ctx, const char *what, int rule, float limit, bmk::GateRule *out);
// The launch state of a gate . up entry: the entry's own rule when the caller passes one, else the context's.
static int launch_under(bm_ctx *ctx, const char *what, const bm_gate_act *act, bmk::Launch *L) {
    *L = launch_of(ctx);
    return act ? rule_checked(ctx, what, act->rule, act->limit, &L->rule) : BM_OK;
}

int bm_fault_clear(bm_ctx *ctx) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_fault_clear: ctx is NULL");
    bmk::Launch L = launch_of(ctx);
    hipError_t e = bmk::fill_u32(L, ctx->fault + 1, 0u, BM_FAULT_WORDS - 1);
    if (e == hipSuccess) e = bmk::fill_u32(L, ctx->fault, BM_FAULT_NONE, 1);
    // a launch that did not run to its end may have left words of its hand-over behind
    if (e == hipSuccess) e = bmk::fill_u32(L, ctx->route_hand, bmk::kRouteArmed, kRouteHandWords);
    return driver(ctx, "bm_fault_clear", e);
}

// ------------------------------------------------------------------------------------------------ buffers

int bm_dev_alloc(bm_ctx *ctx, size_t bytes, void **out_dev) {
    if (!ctx || !out_dev) return fail(ctx, BM_EARG, "bm_dev_alloc: NULL argument");
    return driver(ctx, "bm_dev_alloc", hipMalloc(out_dev, bytes ? bytes : 1));
}

int bm_dev_free(bm_ctx *ctx, void *dev) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_dev_free: ctx is NULL");
    return driver(ctx, "bm_dev_free", hipFree(dev));
}

int bm_dev_upload(bm_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    if (!ctx || !dst_dev || !src_host) return fail(ctx, BM_EARG, "bm_dev_upload: NULL argument");
    int rc = driver(ctx, "bm_dev_upload: sync", hipStreamSynchronize(ctx->stream));
    if (rc) return rc;
    return driver(ctx, "bm_dev_upload", hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
}

int bm_dev_download(bm_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    if (!ctx || !dst_host || !src_dev) return fail(ctx, BM_EARG, "bm_dev_download: NULL argument");
    int rc = driver(ctx, "bm_dev_download: sync", hipStreamSynchronize(ctx->stream));
    if (rc) return rc;
    return driver(ctx, "bm_dev_download", hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
}

int bm_dev_memset(bm_ctx *ctx, void *dst_dev, int byte, size_t bytes) {
    if (!ctx || !dst_dev) return fail(ctx, BM_EARG, "bm_dev_memset: NULL argument");
    int rc = driver(ctx, "bm_dev_memset: sync", hipStreamSynchronize(ctx->stream));
    if (rc) return rc;
    rc = driver(ctx, "bm_dev_memset", hipMemset(dst_dev, byte, bytes));
    if (rc) return rc;
    return driver(ctx, "bm_dev_memset: sync", hipDeviceSynchronize());
}

static int weights_make(bm_ctx *ctx, const char *what, int wtype, int64_t rows, int k, const void *host,
                        const void *dev, bm_weights **out) {
    if (!ctx || !out) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    *out = nullptr;
    if (!known_type(wtype)) return fail(ctx, BM_ETYPE, "%s: weight type %d has no kernel (11 Q3_K, 12 Q4_K, 13 Q5_K, 14 Q6_K, 16 IQ2_XXS, 18 IQ3_XXS, 23 IQ4_XS)", what, wtype);
    if (k <= 0 || k % 256 != 0) return fail(ctx, BM_ESHAPE, "%s: k = %d is not a whole number of 256-value super-blocks", what, k);
    if (rows <= 0) return fail(ctx, BM_ESHAPE, "%s: rows = %lld must be positive", what, (long long)rows);
    const size_t bytes = (size_t)rows * (size_t)bm_row_bytes(wtype, k);
    bm_weights *w = new (std::nothrow) bm_weights{ctx, wtype, rows, k, nullptr, false};
    if (!w) return fail(ctx, BM_EDRIVER, "%s: out of host memory", what);
    if (host) {
        // 16 spare bytes: the last row's vector loads never leave the allocation
        hipError_t e = hipMalloc((void **)&w->dev, bytes + 16);
        if (e == hipSuccess) e = hipMemcpy(w->dev, host, bytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            if (w->dev) (void)hipFree(w->dev);
            delete w;
            return driver(ctx, what, e);
        }
        w->owned = true;
    } else {
        if (!dev) {
            delete w;
            return fail(ctx, BM_EARG, "%s: dev_bytes is NULL", what);
        }
        if ((wtype == BM_TYPE_Q4_K || wtype == BM_TYPE_Q5_K) && ((uintptr_t)dev & 15) != 0) {
            delete w;
            return fail(ctx, BM_ESHAPE, "%s: Q4_K and Q5_K rows are read with 16-byte loads, dev_bytes %p is not 16-byte aligned", what, dev);
        }
        if (wtype == BM_TYPE_IQ4_XS && ((uintptr_t)dev & 7) != 0) {
            delete w;
            return fail(ctx, BM_ESHAPE, "%s: IQ4_XS block headers are read with 8-byte loads, dev_bytes %p is not 8-byte aligned", what, dev);
        }
        if (((uintptr_t)dev & 1) != 0) {
            delete w;
            return fail(ctx, BM_ESHAPE, "%s: dev_bytes %p is not 2-byte aligned", what, dev);
        }
        w->dev = (uint8_t *)dev;
    }
    *out = w;
    return BM_OK;
}

int bm_weights_create(bm_ctx *ctx, int wtype, int64_t rows, int k, const void *host_bytes, bm_weights **out) {
    if (!host_bytes) return fail(ctx, BM_EARG, "bm_weights_create: host_bytes is NULL");
    return weights_make(ctx, "bm_weights_create", wtype, rows, k, host_bytes, nullptr, out);
}

int bm_weights_wrap(bm_ctx *ctx, int wtype, int64_t rows, int k, const void *dev_bytes, bm_weights **out) {
    return weights_make(ctx, "bm_weights_wrap", wtype, rows, k, nullptr, dev_bytes, out);
}

void bm_weights_destroy(bm_weights *w) {
    if (!w) return;
    if (w->owned) (void)hipFree(w->dev);
    delete w;
}

const void *bm_weights_dev(const bm_weights *w) { return w ? w->dev : nullptr; }

int bm_act_create(bm_ctx *ctx, int wtype, int k, int m_cap, bm_act **out) {
    if (!ctx || !out) return fail(ctx, BM_EARG, "bm_act_create: NULL argument");
    *out = nullptr;
    if (!known_type(wtype)) return fail(ctx, BM_ETYPE, "bm_act_create: weight type %d has no activation form here", wtype);
    if (k <= 0 || k % 256 != 0) return fail(ctx, BM_ESHAPE, "bm_act_create: activation columns are whole 256-value super-blocks, k = %d", k);
    if (m_cap <= 0) return fail(ctx, BM_ESHAPE, "bm_act_create: m_cap = %d must be positive", m_cap);
    bm_act *a = new (std::nothrow) bm_act{ctx, wtype, k, m_cap, nullptr};
    if (!a) return fail(ctx, BM_EDRIVER, "bm_act_create: out of host memory");
    const size_t bytes = (size_t)m_cap * dev_col_bytes(wtype, k);
    hipError_t e = hipMalloc((void **)&a->dev, bytes);
    if (e == hipSuccess) e = hipMemset(a->dev, 0, bytes);
    if (e == hipSuccess) e = hipDeviceSynchronize(); // the fill runs on the null stream; the context's does not wait for it
    if (e != hipSuccess) {
        if (a->dev) (void)hipFree(a->dev);
        delete a;
        return driver(ctx, "bm_act_create", e);
    }
    *out = a;
    return BM_OK;
}

void bm_act_destroy(bm_act *act) {
    if (!act) return;
    (void)hipFree(act->dev);
    delete act;
}

int bm_act_download(bm_ctx *ctx, const bm_act *act, int col, void *host_bytes) {
    if (!ctx || !act || !host_bytes) return fail(ctx, BM_EARG, "bm_act_download: NULL argument");
    if (col < 0 || col >= act->m_cap) return fail(ctx, BM_ESHAPE, "bm_act_download: column %d of %d", col, act->m_cap);
    // a column starts with the CPU path's bytes
    return bm_dev_download(ctx, host_bytes, act->dev + (size_t)col * dev_col_bytes(act->wtype, act->k),
                           (size_t)bm_col_bytes(act->wtype, act->k));
}

int bm_act_upload(bm_ctx *ctx, bm_act *act, int col, const void *host_bytes) {
    if (!ctx || !act || !host_bytes) return fail(ctx, BM_EARG, "bm_act_upload: NULL argument");
    if (col < 0 || col >= act->m_cap) return fail(ctx, BM_ESHAPE, "bm_act_upload: column %d of %d", col, act->m_cap);
    uint8_t *dst = act->dev + (size_t)col * dev_col_bytes(act->wtype, act->k);
    int rc = bm_dev_upload(ctx, dst, host_bytes, (size_t)bm_col_bytes(act->wtype, act->k));
    if (rc || act_form(act->wtype) != 0) return rc;
    return driver(ctx, "bm_act_upload: tables", bmk::q82_tables(launch_of(ctx), dst, 1, act->k));
}

// ------------------------------------------------------------------------------------------------ launchers

int bm_quantize(bm_ctx *ctx, const float *x_dev, int m, bm_act *act) {
    const char *what = "bm_quantize";
    if (!ctx || !x_dev || !act) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (m < 1 || m > act->m_cap) return fail(ctx, BM_ESHAPE, "%s: m = %d columns, act holds %d", what, m, act->m_cap);
    return driver(ctx, what, bmk::quantize(launch_of(ctx), act->wtype, x_dev, m, act->k, act->dev));
}

// A weight stack and an activation of one form and one k.
static int check_pair(bm_ctx *ctx, const char *what, const bm_weights *w, const bm_act *act) {
    if (act_form(w->wtype) != act_form(act->wtype))
        return fail(ctx, BM_ETYPE, "%s: weight type %d dots %s columns, act was made for type %d", what, w->wtype,
                    act_form(w->wtype) ? "Q8_K" : "Q8_2_X4", act->wtype);
    if (w->k != act->k) return fail(ctx, BM_ESHAPE, "%s: weight rows hold k = %d values, act columns %d", what, w->k, act->k);
    return BM_OK;
}

int bm_gemv(bm_ctx *ctx, const bm_weights *w, const bm_act *act, int m, float *y_dev) {
    const char *what = "bm_gemv";
    if (!ctx || !w || !act || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int rc = check_pair(ctx, what, w, act);
    if (rc) return rc;
    if (m < 1 || m > 8 || m > act->m_cap)
        return fail(ctx, BM_ESHAPE, "%s: m = %d columns outside 1..=8 or past act's %d", what, m, act->m_cap);
    const int per = bmk::gemv_max_cols(w->wtype, w->k);
    if (per < 1) return fail(ctx, BM_ESHAPE, "%s: one column of k = %d does not fit the workgroup's LDS", what, w->k);
    bmk::Launch L = launch_of(ctx);
    for (int c0 = 0; c0 < m; c0 += per) {
        const int mc = m - c0 < per ? m - c0 : per;
        rc = driver(ctx, what, bmk::gemv(L, w->wtype, w->dev, w->rows, w->k, act->dev, m, c0, mc, y_dev));
        if (rc) return rc;
    }
    return BM_OK;
}

int bm_gemv_x(bm_ctx *ctx, const bm_weights *w, const float *x_dev, int m, bm_act *act_out, float *y_dev) {
    const char *what = "bm_gemv_x";
    if (!ctx || !w || !x_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (m < 1 || m > 65535) return fail(ctx, BM_ESHAPE, "%s: m = %d columns (1 .. 65535)", what, m);
    if (((uintptr_t)x_dev & 15) != 0) return fail(ctx, BM_ESHAPE, "%s: x_dev %p must be 16-byte aligned", what, (const void *)x_dev);
    if (act_out) {
        int rc = check_pair(ctx, what, w, act_out);
        if (rc) return rc;
        if (act_out->m_cap < m) return fail(ctx, BM_ESHAPE, "%s: act_out holds %d columns, m = %d", what, act_out->m_cap, m);
    }
    if (bmk::gemv_x_lds(w->wtype, w->k) > (size_t)bmk::kMaxLds)
        return fail(ctx, BM_ESHAPE, "%s: one column of k = %d does not fit the workgroup's LDS", what, w->k);
    return driver(ctx, what, bmk::gemv_x(launch_of(ctx), w->wtype, w->dev, w->rows, w->k, x_dev, m, act_out ? act_out->dev : nullptr, y_dev));
}

// rows a positive multiple of rows_per_expert (crates/gpu/src/q4k_sel.rs:1013-1023).
static int check_stack(bm_ctx *ctx, const char *what, const bm_weights *w, int rows_per_expert, int *n_experts) {
    if (rows_per_expert <= 0 || w->rows % rows_per_expert != 0)
        return fail(ctx, BM_ESHAPE, "%s: w.rows() %lld must be a positive multiple of rows_per_expert %d", what,
                    (long long)w->rows, rows_per_expert);
    const int64_t n = w->rows / rows_per_expert;
    if (n > 0x7fffffff) return fail(ctx, BM_ESHAPE, "%s: %lld experts", what, (long long)n);
    *n_experts = (int)n;
    return BM_OK;
}

int bm_gate_up(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_act *act, const uint32_t *sel_dev,
               int n_slots, int rows_per_expert, int slots_per_col, const bm_gate_act *rule, float *h_dev, bm_act *act_h) {
    const char *what = "bm_gate_up";
    if (!ctx || !wg || !wu || !act || !sel_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (!h_dev && !act_h) return fail(ctx, BM_EARG, "%s: neither h_dev nor act_h to write", what);
    if (wg->wtype != wu->wtype)
        return fail(ctx, BM_ETYPE, "%s: gate is type %d and up type %d; one launch reads one type", what, wg->wtype, wu->wtype);
    int rc = check_pair(ctx, what, wg, act);
    if (rc) return rc;
    if (wu->k != wg->k || wu->rows != wg->rows)
        return fail(ctx, BM_ESHAPE, "%s: gate is %lld x %d, up %lld x %d", what, (long long)wg->rows, wg->k, (long long)wu->rows, wu->k);
    int n_experts = 0;
    rc = check_stack(ctx, what, wg, rows_per_expert, &n_experts);
    if (rc) return rc;
    if (n_slots < 1) return fail(ctx, BM_ESHAPE, "%s: need n_slots >= 1, got %d", what, n_slots);
    if (slots_per_col < 1) return fail(ctx, BM_ESHAPE, "%s: slots_per_col = %d must be at least 1", what, slots_per_col);
    if ((int64_t)n_slots > (int64_t)act->m_cap * slots_per_col)
        return fail(ctx, BM_ESHAPE, "%s: n_slots %d needs %d columns at %d slots a column, act holds %d", what, n_slots,
                    (n_slots + slots_per_col - 1) / slots_per_col, slots_per_col, act->m_cap);
    uint8_t *ah = nullptr;
    if (act_h) {
        if (act_form(act_h->wtype) != 0)
            return fail(ctx, BM_ETYPE, "%s: the fused quantizer writes Q8_2_X4 columns; act_h was made for type %d (Q8_K)", what, act_h->wtype);
        if (act_h->k != rows_per_expert)
            return fail(ctx, BM_ESHAPE, "%s: act_h columns hold k = %d values, a slot writes rows_per_expert = %d", what, act_h->k, rows_per_expert);
        if (act_h->m_cap < n_slots)
            return fail(ctx, BM_ESHAPE, "%s: a column of act_h per slot: %d slots, act_h holds %d", what, n_slots, act_h->m_cap);
        ah = act_h->dev;
    }
    bmk::Launch L;
    if ((rc = launch_under(ctx, what, rule, &L)) != 0) return rc;
    return driver(ctx, what, bmk::gate_up(L, wg->wtype, wg->dev, wu->dev, n_experts, wg->k, act->dev, sel_dev,
                                          n_slots, rows_per_expert, slots_per_col, h_dev, ah));
}

int bm_gemv_sel(bm_ctx *ctx, const bm_weights *w, const bm_act *act, const uint32_t *sel_dev, int n_slots,
                int rows_per_expert, float *y_dev) {
    const char *what = "bm_gemv_sel";
    if (!ctx || !w || !act || !sel_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int rc = check_pair(ctx, what, w, act);
    if (rc) return rc;
    int n_experts = 0;
    rc = check_stack(ctx, what, w, rows_per_expert, &n_experts);
    if (rc) return rc;
    if (n_slots < 1) return fail(ctx, BM_ESHAPE, "%s: need n_slots >= 1, got %d", what, n_slots);
    if (act->m_cap < n_slots)
        return fail(ctx, BM_ESHAPE, "%s: an activation column per slot: act.m() = %d must be at least n_slots = %d", what, act->m_cap, n_slots);
    return driver(ctx, what, bmk::gemv_sel(launch_of(ctx), w->wtype, w->dev, n_experts, w->k, act->dev, sel_dev, n_slots,
                                           rows_per_expert, y_dev));
}

int bm_combine_tokens(bm_ctx *ctx, const float *down_dev, const float *w_dev, const float *resid_dev, int rows,
                      int n_slots, int m, float *y_dev) {
    const char *what = "bm_combine_tokens";
    if (!ctx || !down_dev || !w_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (rows < 1 || n_slots < 1 || m < 1)
        return fail(ctx, BM_ESHAPE, "%s: rows %d, n_slots %d and m %d must all be positive", what, rows, n_slots, m);
    return driver(ctx, what, bmk::combine_tokens(launch_of(ctx), down_dev, w_dev, nullptr, resid_dev, rows, n_slots, m, y_dev));
}

int bm_moe_combine(bm_ctx *ctx, const float *down_dev, const float *w_dev, const float *shexp_dev, const float *resid_dev,
                   int rows, int n_slots, int m, float *y_dev) {
    const char *what = "bm_moe_combine";
    if (!ctx || !down_dev || !w_dev || !shexp_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (rows < 1 || n_slots < 1 || m < 1)
        return fail(ctx, BM_ESHAPE, "%s: rows %d, n_slots %d and m %d must all be positive", what, rows, n_slots, m);
    return driver(ctx, what, bmk::combine_tokens(launch_of(ctx), down_dev, w_dev, shexp_dev, resid_dev, rows, n_slots, m, y_dev));
}

int bm_down_combine(bm_ctx *ctx, const bm_weights *w, const bm_act *act, const uint32_t *sel_dev,
                    const float *w_dev, const float *resid_dev, int n_slots_per_token, int m, int rows_per_expert,
                    float *y_dev) {
    const char *what = "bm_down_combine";
    if (!ctx || !w || !act || !sel_dev || !w_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int rc = check_pair(ctx, what, w, act);
    if (rc) return rc;
    int n_experts = 0;
    rc = check_stack(ctx, what, w, rows_per_expert, &n_experts);
    if (rc) return rc;
    if (n_slots_per_token < 1 || n_slots_per_token > bmk::kMaxCombineSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d slots a token outside 1..=%d", what, n_slots_per_token, bmk::kMaxCombineSlots);
    if (m < 1) return fail(ctx, BM_ESHAPE, "%s: need m >= 1 tokens, got %d", what, m);
    if ((int64_t)m * n_slots_per_token > act->m_cap)
        return fail(ctx, BM_ESHAPE, "%s: an activation column per slot: %d tokens x %d slots, act holds %d", what, m,
                    n_slots_per_token, act->m_cap);
    const size_t lds = (size_t)n_slots_per_token * dev_col_bytes(act->wtype, act->k) + 4096;
    if (lds > (size_t)bmk::kMaxLds)
        return fail(ctx, BM_ESHAPE, "%s: %d columns of k = %d do not fit the workgroup's LDS; use bm_gemv_sel and bm_combine_tokens", what,
                    n_slots_per_token, act->k);
    return driver(ctx, what, bmk::down_combine(launch_of(ctx), w->wtype, w->dev, n_experts, w->k, act->dev, sel_dev, w_dev,
                                               resid_dev, n_slots_per_token, m, rows_per_expert, y_dev));
}

int bm_down_combine_h(bm_ctx *ctx, const bm_weights *w, const float *h_dev, bm_act *act_h, const uint32_t *sel_dev,
                      const float *w_dev, const float *resid_dev, int n_slots_per_token, int m, int rows_per_expert,
                      float *y_dev) {
    const char *what = "bm_down_combine_h";
    if (!ctx || !w || !h_dev || !sel_dev || !w_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int n_experts = 0;
    int rc = check_stack(ctx, what, w, rows_per_expert, &n_experts);
    if (rc) return rc;
    if (n_slots_per_token < 1 || n_slots_per_token > bmk::kMaxCombineSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d slots a token outside 1..=%d", what, n_slots_per_token, bmk::kMaxCombineSlots);
    if (m < 1) return fail(ctx, BM_ESHAPE, "%s: need m >= 1 tokens, got %d", what, m);
    if (act_h && (act_form(act_h->wtype) != act_form(w->wtype) || act_h->k != w->k || (int64_t)act_h->m_cap < (int64_t)m * n_slots_per_token))
        return fail(ctx, BM_ESHAPE, "%s: act_h must hold %d columns of k = %d in the form type %d dots against; it holds %d of k = %d (type %d)",
                    what, m * n_slots_per_token, w->k, w->wtype, act_h->m_cap, act_h->k, act_h->wtype);
    if (((uintptr_t)h_dev & 15) != 0) return fail(ctx, BM_ESHAPE, "%s: h_dev %p is not 16-byte aligned", what, (const void *)h_dev);
    const size_t lds = (size_t)n_slots_per_token * dev_col_bytes(w->wtype, w->k) + 12288;
    if (lds > (size_t)bmk::kMaxLds)
        return fail(ctx, BM_ESHAPE, "%s: %d columns of k = %d do not fit the workgroup's LDS; use bm_quantize, bm_gemv_sel and "
                    "bm_combine_tokens", what, n_slots_per_token, w->k);
    return driver(ctx, what, bmk::down_combine_hq(launch_of(ctx), w->wtype, w->dev, n_experts, w->k, h_dev, act_h ? act_h->dev : nullptr,
                                                  sel_dev, w_dev, resid_dev, n_slots_per_token, m, rows_per_expert, y_dev));
}

int bm_gate_up_x(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const float *x_dev, const uint32_t *sel_dev,
                 int n_slots_per_token, int m, int rows_per_expert, const bm_gate_act *rule, bm_act *act_h, bm_act *act_x,
                 float *h_dev) {
    const char *what = "bm_gate_up_x";
    if (!ctx || !wg || !wu || !x_dev || !sel_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (!act_h && !h_dev) return fail(ctx, BM_EARG, "%s: neither act_h nor h_dev: the launch would have no output", what);
    if (wg->wtype != wu->wtype)
        return fail(ctx, BM_ETYPE, "%s: gate is type %d and up type %d; one launch reads one type", what, wg->wtype, wu->wtype);
    if (wu->k != wg->k || wu->rows != wg->rows)
        return fail(ctx, BM_ESHAPE, "%s: gate is %lld x %d, up %lld x %d", what, (long long)wg->rows, wg->k, (long long)wu->rows, wu->k);
    const int hidden = wg->k, ff = rows_per_expert;
    int n_experts = 0;
    int rc = check_stack(ctx, what, wg, ff, &n_experts);
    if (rc) return rc;
    if (ff % 256 != 0) return fail(ctx, BM_ESHAPE, "%s: rows_per_expert = %d is not a whole number of 256-value super-blocks", what, ff);
    if (n_slots_per_token < 1 || m < 1 || m > bmk::kMaxDecodeTokens)
        return fail(ctx, BM_ESHAPE, "%s: %d slots a token, m = %d tokens (1..=%d)", what, n_slots_per_token, m, bmk::kMaxDecodeTokens);
    if (act_h && (act_form(act_h->wtype) != 0 || act_h->k != ff || (int64_t)act_h->m_cap < (int64_t)m * n_slots_per_token))
        return fail(ctx, BM_ESHAPE,
                    "%s: act_h must hold %d Q8_2_X4 columns of k = %d (the launch folds that quantizer only; pass NULL and h_dev for a "
                    "down stack on Q8_K columns); it holds %d of k = %d (type %d)",
                    what, m * n_slots_per_token, ff, act_h->m_cap, act_h->k, act_h->wtype);
    if (act_x && (act_form(act_x->wtype) != act_form(wg->wtype) || act_x->k != hidden || act_x->m_cap < m))
        return fail(ctx, BM_ESHAPE, "%s: act_x must hold %d %s columns of k = %d; it holds %d of k = %d (type %d)", what, m,
                    act_form(wg->wtype) ? "Q8_K" : "Q8_2_X4", hidden, act_x->m_cap, act_x->k, act_x->wtype);
    if (((uintptr_t)x_dev & 15) != 0) return fail(ctx, BM_ESHAPE, "%s: x_dev %p is not 16-byte aligned", what, (const void *)x_dev);
    if (dev_col_bytes(wg->wtype, hidden) + 8192 > (size_t)bmk::kMaxLds)
        return fail(ctx, BM_ESHAPE, "%s: a column of hidden = %d does not fit the workgroup's LDS", what, hidden);
    bmk::Launch L;
    if ((rc = launch_under(ctx, what, rule, &L)) != 0) return rc;
    return driver(ctx, what,
                  bmk::gate_up_x(L, wg->wtype, x_dev, wg->dev, wu->dev, n_experts, hidden, ff, sel_dev, n_slots_per_token, m,
                                 act_x ? act_x->dev : nullptr, act_h ? act_h->dev : nullptr, h_dev));
}

int bm_moe_decode(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_weights *wd, const float *x_dev,
                  const uint32_t *sel_dev, const float *w_dev, const float *resid_dev, int n_slots_per_token, int m,
                  const bm_gate_act *rule, bm_act *act_h, bm_act *act_x, float *h_dev, float *y_dev) {
    const char *what = "bm_moe_decode";
    if (!ctx || !wg || !wu || !wd || !x_dev || !sel_dev || !w_dev || !act_h || !y_dev)
        return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (wg->wtype != wu->wtype)
        return fail(ctx, BM_ETYPE, "%s: gate is type %d and up type %d; one launch reads one type", what, wg->wtype, wu->wtype);
    if (!bmk::moe_decode_supported(wg->wtype, wd->wtype))
        return fail(ctx, BM_ETYPE, "%s: no kernel for gate/up type %d with down type %d", what, wg->wtype, wd->wtype);
    if (wu->k != wg->k || wu->rows != wg->rows)
        return fail(ctx, BM_ESHAPE, "%s: gate is %lld x %d, up %lld x %d", what, (long long)wg->rows, wg->k, (long long)wu->rows, wu->k);
    const int hidden = wg->k, ff = wd->k;
    int n_experts = 0, n_down = 0;
    int rc = check_stack(ctx, what, wg, ff, &n_experts);
    if (!rc) rc = check_stack(ctx, what, wd, hidden, &n_down);
    if (rc) return rc;
    if (n_down != n_experts)
        return fail(ctx, BM_ESHAPE, "%s: gate/up hold %d experts of %d rows, down %d experts of %d rows", what, n_experts, ff, n_down, hidden);
    if (n_slots_per_token < 1 || n_slots_per_token > bmk::kMaxCombineSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d slots a token outside 1..=%d", what, n_slots_per_token, bmk::kMaxCombineSlots);
    if (m < 1 || m > bmk::kMaxDecodeTokens)
        return fail(ctx, BM_ESHAPE, "%s: m = %d tokens outside 1..=%d", what, m, bmk::kMaxDecodeTokens);
    if (act_form(act_h->wtype) != act_form(wd->wtype) || act_h->k != ff || (int64_t)act_h->m_cap < (int64_t)m * n_slots_per_token)
        return fail(ctx, BM_ESHAPE, "%s: act_h must hold %d %s columns of k = %d; it holds %d of k = %d (type %d)", what,
                    m * n_slots_per_token, act_form(wd->wtype) ? "Q8_K" : "Q8_2_X4", ff, act_h->m_cap, act_h->k, act_h->wtype);
    if (act_x && (act_form(act_x->wtype) != act_form(wg->wtype) || act_x->k != hidden || act_x->m_cap < m))
        return fail(ctx, BM_ESHAPE, "%s: act_x must hold %d %s columns of k = %d; it holds %d of k = %d (type %d)", what, m,
                    act_form(wg->wtype) ? "Q8_K" : "Q8_2_X4", hidden, act_x->m_cap, act_x->k, act_x->wtype);
    if (act_form(wd->wtype) != 0 && !h_dev)
        return fail(ctx, BM_EARG, "%s: a down stack on Q8_K columns needs h_dev: the gate . up launch leaves h there as f32 rows and "
                    "the down launch quantizes them", what);
    if (((uintptr_t)x_dev & 15) != 0) return fail(ctx, BM_ESHAPE, "%s: x_dev %p is not 16-byte aligned", what, (const void *)x_dev);
    if (h_dev && ((uintptr_t)h_dev & 15) != 0) return fail(ctx, BM_ESHAPE, "%s: h_dev %p is not 16-byte aligned", what, (const void *)h_dev);
    const size_t lds_a = dev_col_bytes(wg->wtype, hidden) + 8192;
    const size_t lds_b = (size_t)n_slots_per_token * dev_col_bytes(wd->wtype, ff) + 12288;
    if (lds_a > (size_t)bmk::kMaxLds || lds_b > (size_t)bmk::kMaxLds)
        return fail(ctx, BM_ESHAPE, "%s: hidden = %d or %d columns of ff = %d do not fit the workgroup's LDS; use the separate launches", what,
                    hidden, n_slots_per_token, ff);
    bmk::Launch L;
    if ((rc = launch_under(ctx, what, rule, &L)) != 0) return rc;
    return driver(ctx, what,
                  bmk::moe_decode(L, wg->wtype, wd->wtype, x_dev, wg->dev, wu->dev, wd->dev, n_experts, hidden, ff, sel_dev,
                                  w_dev, resid_dev, n_slots_per_token, m, act_x ? act_x->dev : nullptr, act_h->dev, h_dev, y_dev));
}

int bm_moe_decode_noalloc(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_weights *wd, const float *x_dev,
                          const uint32_t *sel_dev, const float *w_dev, const float *resid_dev, int n_slots_per_token, int m,
                          const bm_gate_act *rule, float *y_dev) {
    const char *what = "bm_moe_decode_noalloc";
    if (!ctx || !wg || !wu || !wd || !x_dev || !sel_dev || !w_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (wg->wtype != wu->wtype)
        return fail(ctx, BM_ETYPE, "%s: gate is type %d and up type %d; one launch reads one type", what, wg->wtype, wu->wtype);
    if (!bmk::moe_decode_supported(wg->wtype, wd->wtype))
        return fail(ctx, BM_ETYPE, "%s: no kernel for gate/up type %d with down type %d", what, wg->wtype, wd->wtype);
    if (wu->k != wg->k || wu->rows != wg->rows)
        return fail(ctx, BM_ESHAPE, "%s: gate is %lld x %d, up %lld x %d", what, (long long)wg->rows, wg->k, (long long)wu->rows, wu->k);
    const int hidden = wg->k, ff = wd->k;
    int n_experts = 0, n_down = 0;
    int rc = check_stack(ctx, what, wg, ff, &n_experts);
    if (!rc) rc = check_stack(ctx, what, wd, hidden, &n_down);
    if (rc) return rc;
    if (n_down != n_experts)
        return fail(ctx, BM_ESHAPE, "%s: gate/up hold %d experts of %d rows, down %d experts of %d rows", what, n_experts, ff, n_down, hidden);
    if (n_slots_per_token < 1 || n_slots_per_token > bmk::kMaxCombineSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d slots a token outside 1..=%d", what, n_slots_per_token, bmk::kMaxCombineSlots);
    if (m < 1 || m > bmk::kMaxDecodeTokens)
        return fail(ctx, BM_ESHAPE, "%s: m = %d tokens outside 1..=%d", what, m, bmk::kMaxDecodeTokens);
    if ((size_t)m * (size_t)n_slots_per_token * (size_t)ff > bmk::kStaticValues)
        return fail(ctx, BM_ESHAPE, "%s: %d tokens x %d slots x ff = %d is %zu values of h; the library's static scratch holds %zu "
                    "(use bm_moe_decode with caller-held act_h past that)", what, m, n_slots_per_token, ff,
                    (size_t)m * (size_t)n_slots_per_token * (size_t)ff, (size_t)bmk::kStaticValues);
    if (((uintptr_t)x_dev & 15) != 0) return fail(ctx, BM_ESHAPE, "%s: x_dev %p is not 16-byte aligned", what, (const void *)x_dev);
    const size_t lds_a = dev_col_bytes(wg->wtype, hidden) + 8192;
    const size_t lds_b = (size_t)n_slots_per_token * dev_col_bytes(wd->wtype, ff) + 12288;
    if (lds_a > (size_t)bmk::kMaxLds || lds_b > (size_t)bmk::kMaxLds)
        return fail(ctx, BM_ESHAPE, "%s: hidden = %d or %d columns of ff = %d do not fit the workgroup's LDS; use the separate launches", what,
                    hidden, n_slots_per_token, ff);
    bmk::Launch L;
    if ((rc = launch_under(ctx, what, rule, &L)) != 0) return rc;
    return driver(ctx, what,
                  bmk::moe_decode_static(L, ctx->device, wg->wtype, wd->wtype, x_dev, wg->dev, wu->dev, wd->dev, n_experts,
                                         hidden, ff, sel_dev, w_dev, resid_dev, n_slots_per_token, m, y_dev));
}

// ------------------------------------------------------------------------------------------ grouped decode

int bm_tile_cap(int n_slots, int n_experts) {
    if (n_slots < 0 || n_experts < 1) return BM_ESHAPE;
    return bmk::tile_cap(n_slots, n_experts);
}

int bm_buckets(bm_ctx *ctx, const uint32_t *sel_dev, int n_slots, int n_experts, uint32_t *order_dev, uint32_t *start_dev) {
    const char *what = "bm_buckets";
    if (!ctx || !sel_dev || !order_dev || !start_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_experts < 1 || n_experts > bmk::kBucketExperts || n_slots < 1 || n_slots > bmk::kTileMaxSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d places over %d experts (1..=%d experts, 1..=%d places)", what, n_slots, n_experts,
                    bmk::kBucketExperts, bmk::kTileMaxSlots);
    return driver(ctx, what, bmk::buckets(launch_of(ctx), sel_dev, n_slots, n_experts, order_dev, start_dev));
}

int bm_tiles(bm_ctx *ctx, const uint32_t *start_dev, int n_experts, int n_slots, uint32_t *tiles_dev) {
    const char *what = "bm_tiles";
    if (!ctx || !start_dev || !tiles_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_experts < 1 || n_experts > bmk::kBucketExperts || n_slots < 1 || n_slots > bmk::kTileMaxSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d slots over %d experts (1..=%d experts, at most %d slots)", what, n_slots, n_experts,
                    bmk::kBucketExperts, bmk::kTileMaxSlots);
    return driver(ctx, what, bmk::tiles(launch_of(ctx), start_dev, n_experts, n_slots, tiles_dev));
}

int bm_tables(bm_ctx *ctx, const uint32_t *sel_dev, int n_slots, int n_experts, uint32_t *order_dev, uint32_t *start_dev,
              uint32_t *tiles_dev) {
    const char *what = "bm_tables";
    if (!ctx || !sel_dev || !order_dev || !start_dev || !tiles_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_experts < 1 || n_experts > bmk::kBucketExperts || n_slots < 1 || n_slots > bmk::kTileMaxSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d places over %d experts (1..=%d experts, 1..=%d places)", what, n_slots, n_experts,
                    bmk::kBucketExperts, bmk::kTileMaxSlots);
    return driver(ctx, what, bmk::tables(launch_of(ctx), sel_dev, n_slots, n_experts, order_dev, start_dev, tiles_dev));
}

int bm_tables_quantize(bm_ctx *ctx, const uint32_t *sel_dev, int n_slots, int n_experts, uint32_t *order_dev, uint32_t *start_dev,
                       uint32_t *tiles_dev, const float *x_dev, int m, bm_act *act) {
    const char *what = "bm_tables_quantize";
    if (!ctx || !sel_dev || !order_dev || !start_dev || !tiles_dev || !x_dev || !act) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_experts < 1 || n_experts > bmk::kBucketExperts || n_slots < 1 || n_slots > bmk::kTileMaxSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d places over %d experts (1..=%d experts, 1..=%d places)", what, n_slots, n_experts,
                    bmk::kBucketExperts, bmk::kTileMaxSlots);
    if (m < 1 || m > act->m_cap) return fail(ctx, BM_ESHAPE, "%s: m = %d columns, act holds %d", what, m, act->m_cap);
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15) != 0 || act->k % 256 != 0) { // rows the one launch does not read: the two launches
        int rc = bm_tables(ctx, sel_dev, n_slots, n_experts, order_dev, start_dev, tiles_dev);
        return rc ? rc : bm_quantize(ctx, x_dev, m, act);
    }
    return driver(ctx, what, bmk::tables_quant(launch_of(ctx), sel_dev, n_slots, n_experts, order_dev, start_dev, tiles_dev, act->wtype,
                                               x_dev, m, act->k, act->dev));
}

int bm_quantize_ord(bm_ctx *ctx, const float *x_dev, const uint32_t *start_dev, int n_experts, int m_cols, bm_act *act) {
    const char *what = "bm_quantize_ord";
    if (!ctx || !x_dev || !start_dev || !act) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_experts < 1) return fail(ctx, BM_ESHAPE, "%s: n_experts = %d", what, n_experts);
    if (m_cols < 1 || m_cols > act->m_cap)
        return fail(ctx, BM_ESHAPE, "%s: %d columns of %d values into %d columns", what, m_cols, act->k, act->m_cap);
    return driver(ctx, what, bmk::quantize(launch_of(ctx), act->wtype, x_dev, m_cols, act->k, act->dev, start_dev + n_experts));
}

// The table arguments every tile launcher takes.
static int check_table(bm_ctx *ctx, const char *what, const uint32_t *order, const uint32_t *start, const uint32_t *tiles,
                       int n_slots, int n_experts) {
    if (!order || !start || !tiles) return fail(ctx, BM_EARG, "%s: NULL table", what);
    if (n_experts > bmk::kBucketExperts)
        return fail(ctx, BM_ESHAPE, "%s: the stack holds %d experts, a tile word names at most %d", what, n_experts, bmk::kBucketExperts);
    if (n_slots < 1 || n_slots > bmk::kTileMaxSlots)
        return fail(ctx, BM_ESHAPE, "%s: n_slots = %d outside 1..=%d", what, n_slots, bmk::kTileMaxSlots);
    return BM_OK;
}

int bm_gate_up_tiles(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_act *act, const uint32_t *order_dev,
                     const uint32_t *start_dev, const uint32_t *tiles_dev, int n_slots, int rows_per_expert,
                     int slots_per_col, const bm_gate_act *rule, float *h_dev, bm_act *act_h) {
    const char *what = "bm_gate_up_tiles";
    if (!ctx || !wg || !wu || !act) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (!h_dev && !act_h) return fail(ctx, BM_EARG, "%s: neither h_dev nor act_h to write", what);
    if (wg->wtype != wu->wtype)
        return fail(ctx, BM_ETYPE, "%s: gate is type %d and up type %d; one launch reads one type", what, wg->wtype, wu->wtype);
    int rc = check_pair(ctx, what, wg, act);
    if (rc) return rc;
    if (wu->k != wg->k || wu->rows != wg->rows)
        return fail(ctx, BM_ESHAPE, "%s: gate is %lld x %d, up %lld x %d", what, (long long)wg->rows, wg->k, (long long)wu->rows, wu->k);
    int n_experts = 0;
    rc = check_stack(ctx, what, wg, rows_per_expert, &n_experts);
    if (!rc) rc = check_table(ctx, what, order_dev, start_dev, tiles_dev, n_slots, n_experts);
    if (rc) return rc;
    if (slots_per_col < 1) return fail(ctx, BM_ESHAPE, "%s: slots_per_col = %d must be at least 1", what, slots_per_col);
    if ((int64_t)n_slots > (int64_t)act->m_cap * slots_per_col)
        return fail(ctx, BM_ESHAPE, "%s: n_slots %d needs %d columns at %d slots a column, act holds %d", what, n_slots,
                    (n_slots + slots_per_col - 1) / slots_per_col, slots_per_col, act->m_cap);
    uint8_t *ah = nullptr;
    if (act_h) {
        if (act_form(act_h->wtype) != 0)
            return fail(ctx, BM_ETYPE, "%s: the fused quantizer writes Q8_2_X4 columns; act_h was made for type %d (Q8_K)", what, act_h->wtype);
        if (act_h->k != rows_per_expert)
            return fail(ctx, BM_ESHAPE, "%s: act_h columns hold k = %d values, an entry writes rows_per_expert = %d", what, act_h->k, rows_per_expert);
        if (act_h->m_cap < n_slots)
            return fail(ctx, BM_ESHAPE, "%s: a column of act_h per table entry: %d slots, act_h holds %d", what, n_slots, act_h->m_cap);
        ah = act_h->dev;
    }
    if (bmk::tiles_lds(wg->wtype, wg->k) == 0)
        return fail(ctx, BM_ESHAPE, "%s: eight columns of k = %d do not fit the workgroup's LDS; use bm_gate_up", what, wg->k);
    bmk::Launch L;
    if ((rc = launch_under(ctx, what, rule, &L)) != 0) return rc;
    return driver(ctx, what, bmk::gate_up_tiles(L, wg->wtype, wg->dev, wu->dev, n_experts, wg->k, act->dev, act->m_cap,
                                                order_dev, start_dev, tiles_dev, n_slots, rows_per_expert, slots_per_col, h_dev, ah));
}

int bm_gemv_tiles(bm_ctx *ctx, const bm_weights *w, const bm_act *act, const uint32_t *order_dev, const uint32_t *start_dev,
                  const uint32_t *tiles_dev, int n_slots, int rows_per_expert, float *y_dev) {
    const char *what = "bm_gemv_tiles";
    if (!ctx || !w || !act || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int rc = check_pair(ctx, what, w, act);
    if (rc) return rc;
    int n_experts = 0;
    rc = check_stack(ctx, what, w, rows_per_expert, &n_experts);
    if (!rc) rc = check_table(ctx, what, order_dev, start_dev, tiles_dev, n_slots, n_experts);
    if (rc) return rc;
    if (act->m_cap < n_slots)
        return fail(ctx, BM_ESHAPE, "%s: an activation column per table entry: act.m() = %d must be at least n_slots = %d", what,
                    act->m_cap, n_slots);
    if (bmk::tiles_lds(w->wtype, w->k) == 0)
        return fail(ctx, BM_ESHAPE, "%s: eight columns of k = %d do not fit the workgroup's LDS; use bm_gemv_sel", what, w->k);
    return driver(ctx, what, bmk::gemv_tiles(launch_of(ctx), w->wtype, w->dev, n_experts, w->k, act->dev, order_dev, start_dev,
                                             tiles_dev, n_slots, rows_per_expert, y_dev));
}

// ------------------------------------------------------------------------------------------------ prefill

struct bm_route {
    bm_ctx *ctx;
    int max_slots, n_experts;
    int filled; // the slot count of the last fill, 0: never filled
    uint32_t *cols, *tiles, *n_tiles;
};

int bm_route_create(bm_ctx *ctx, int max_slots, int n_experts, bm_route **out) {
    const char *what = "bm_route_create";
    if (!ctx || !out) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    *out = nullptr;
    if (max_slots < 1 || max_slots > bmk::kGemmMaxSlots)
        return fail(ctx, BM_ESHAPE, "%s: 1 <= max_slots <= %d, got %d", what, bmk::kGemmMaxSlots, max_slots);
    if (n_experts < 1 || n_experts > bmk::kGemmMaxExperts)
        return fail(ctx, BM_ESHAPE, "%s: 1 <= n_experts <= %d, got %d", what, bmk::kGemmMaxExperts, n_experts);
    bm_route *r = new (std::nothrow) bm_route{ctx, max_slots, n_experts, 0, nullptr, nullptr, nullptr};
    if (!r) return fail(ctx, BM_EDRIVER, "%s: out of host memory", what);
    const size_t words = (size_t)max_slots + 2 * (size_t)bmk::gemm_max_tiles(max_slots, n_experts) + 3;
    hipError_t e = hipMalloc((void **)&r->cols, words * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMemset(r->cols, 0, words * sizeof(uint32_t));
    if (e == hipSuccess) e = hipDeviceSynchronize(); // as in bm_act_create
    if (e != hipSuccess) {
        if (r->cols) (void)hipFree(r->cols);
        delete r;
        return driver(ctx, what, e);
    }
    r->tiles = r->cols + max_slots;
    r->n_tiles = r->tiles + 2 * (size_t)bmk::gemm_max_tiles(max_slots, n_experts);
    *out = r;
    return BM_OK;
}

void bm_route_destroy(bm_route *route) {
    if (!route) return;
    (void)hipFree(route->cols);
    delete route;
}

int bm_route_fill(bm_ctx *ctx, const uint32_t *ids_dev, int n_slots, bm_route *route) {
    const char *what = "bm_route_fill";
    if (!ctx || !ids_dev || !route) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_slots < 1 || n_slots > route->max_slots)
        return fail(ctx, BM_ESHAPE, "%s: 1 <= n_slots <= the table's %d slots, got %d", what, route->max_slots, n_slots);
    int rc = driver(ctx, what, bmk::route(launch_of(ctx), ids_dev, n_slots, route->n_experts, route->cols, route->tiles, route->n_tiles));
    if (!rc) route->filled = n_slots;
    return rc;
}

int bm_route_fill_quantize(bm_ctx *ctx, const uint32_t *ids_dev, int n_slots, bm_route *route, const float *x_dev, int m, bm_act *act) {
    const char *what = "bm_route_fill_quantize";
    if (!ctx || !ids_dev || !route || !x_dev || !act) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_slots < 1 || n_slots > route->max_slots)
        return fail(ctx, BM_ESHAPE, "%s: 1 <= n_slots <= the table's %d slots, got %d", what, route->max_slots, n_slots);
    if (m < 1 || m > act->m_cap) return fail(ctx, BM_ESHAPE, "%s: m = %d columns, act holds %d", what, m, act->m_cap);
    if ((reinterpret_cast<uintptr_t>(x_dev) & 15) != 0 || act->k % 256 != 0) { // rows the one launch does not read: the two launches
        int rc = bm_quantize(ctx, x_dev, m, act);
        return rc ? rc : bm_route_fill(ctx, ids_dev, n_slots, route);
    }
    int rc = driver(ctx, what, bmk::route(launch_of(ctx), ids_dev, n_slots, route->n_experts, route->cols, route->tiles, route->n_tiles,
                                          act->wtype, x_dev, m, act->k, act->dev));
    if (!rc) route->filled = n_slots;
    return rc;
}

int bm_route_read(bm_ctx *ctx, const bm_route *route, uint32_t *cols_host, uint32_t *tiles_host, int *n_tiles, int *n_refused) {
    const char *what = "bm_route_read";
    if (!ctx || !route || !n_tiles || !n_refused) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (!route->filled) return fail(ctx, BM_ESHAPE, "%s: the table was never filled", what);
    uint32_t counts[2];
    int rc = bm_dev_download(ctx, counts, route->n_tiles, sizeof counts);
    if (rc) return rc;
    const int cap = bmk::gemm_max_tiles(route->filled, route->n_experts);
    if ((int)counts[0] > cap || (int)counts[1] > route->filled)
        return fail(ctx, BM_ESHAPE, "%s: tile count %u (of %d) or refused count %u (of %d slots) is past the table", what, counts[0], cap,
                    counts[1], route->filled);
    *n_tiles = (int)counts[0];
    *n_refused = (int)counts[1];
    if (cols_host) rc = bm_dev_download(ctx, cols_host, route->cols, sizeof(uint32_t) * (size_t)route->filled);
    if (!rc && tiles_host && counts[0]) rc = bm_dev_download(ctx, tiles_host, route->tiles, sizeof(uint32_t) * 2 * counts[0]);
    return rc;
}

int bm_gemm(bm_ctx *ctx, const bm_weights *w, int rows_per_expert, const bm_act *act, const bm_route *route, int top_k, float *y_dev) {
    const char *what = "bm_gemm";
    if (!ctx || !w || !act || !route || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (!route->filled) return fail(ctx, BM_ESHAPE, "%s: a filled route table (bm_route_fill first)", what);
    if (!bmk::gemm_supported(w->wtype))
        return fail(ctx, BM_ETYPE, "%s: weight type %d has no grouped GEMM here (Q4_K, Q5_K, Q6_K and IQ2_XXS do); use the tile launchers", what, w->wtype);
    int rc = check_pair(ctx, what, w, act);
    if (rc) return rc;
    if (rows_per_expert <= 0 || rows_per_expert % 16 != 0)
        return fail(ctx, BM_ESHAPE, "%s: rows_per_expert must be a positive multiple of 16, got %d", what, rows_per_expert);
    if (w->rows != (int64_t)route->n_experts * rows_per_expert)
        return fail(ctx, BM_ESHAPE, "%s: the stack has %lld rows, the route %d experts of %d rows", what, (long long)w->rows,
                    route->n_experts, rows_per_expert);
    const int n_slots = route->filled;
    int slot_div = 1;
    if (top_k > 0) {
        if (n_slots % top_k != 0) return fail(ctx, BM_ESHAPE, "%s: %d slots are not whole tokens of top_k %d", what, n_slots, top_k);
        slot_div = top_k;
    } else if (top_k < 0) {
        return fail(ctx, BM_ESHAPE, "%s: top_k = %d (0: a column a slot)", what, top_k);
    }
    if (act->m_cap < n_slots / slot_div)
        return fail(ctx, BM_ESHAPE, "%s: %d slots read %d activation columns, act holds %d", what, n_slots, n_slots / slot_div, act->m_cap);
    // the kernels address the columns and an expert's rows by 32-bit offsets
    if ((uint64_t)(n_slots / slot_div) * dev_col_bytes(act->wtype, act->k) >= (1ull << 32) ||
        (uint64_t)rows_per_expert * (uint64_t)bm_row_bytes(w->wtype, w->k) >= (1ull << 32))
        return fail(ctx, BM_ESHAPE, "%s: %d columns of k = %d or %d rows an expert pass 4 GiB, the kernels' offset range", what,
                    n_slots / slot_div, act->k, rows_per_expert);
    return driver(ctx, what, bmk::gemm(launch_of(ctx), w->wtype, w->dev, route->n_experts, rows_per_expert, w->k, act->dev, route->cols,
                                       route->tiles, route->n_tiles, n_slots, slot_div, y_dev, ctx->gemm_mode));
}

// ------------------------------------------------------------------------- one entry for every batch size

struct bm_scratch {
    bm_ctx *ctx;
    int gate_type, down_type, hidden, ff, n_experts, spt, max_tokens;
    bm_act *act_x, *act_h;
    float *g, *u, *down;           // f32 rows: g (also the per-slot and grouped paths' h) and u of slots x ff, down of slots x hidden
    uint32_t *order, *start, *tiles; // the grouped table
    bm_route *route;               // the GEMM path's table
    int path, grouped_from, gemm_from, gemm_from_fast;
};

void bm_scratch_destroy(bm_scratch *s) {
    if (!s) return;
    bm_act_destroy(s->act_x);
    bm_act_destroy(s->act_h);
    (void)hipFree(s->g);
    (void)hipFree(s->u);
    (void)hipFree(s->down);
    (void)hipFree(s->order);
    bm_route_destroy(s->route);
    delete s;
}

int bm_scratch_create(bm_ctx *ctx, int gate_type, int down_type, int hidden, int ff, int n_experts, int n_slots_per_token,
                      int max_tokens, bm_scratch **out) {
    const char *what = "bm_scratch_create";
    if (!ctx || !out) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    *out = nullptr;
    if (!bmk::moe_decode_supported(gate_type, down_type))
        return fail(ctx, BM_ETYPE, "%s: no kernels for gate/up type %d with down type %d", what, gate_type, down_type);
    if (hidden < 256 || hidden % 256 != 0 || ff < 256 || ff % 256 != 0)
        return fail(ctx, BM_ESHAPE, "%s: hidden = %d and ff = %d must be positive multiples of 256", what, hidden, ff);
    if (n_experts < 1 || n_experts > bmk::kBucketExperts)
        return fail(ctx, BM_ESHAPE, "%s: n_experts = %d outside 1..=%d", what, n_experts, bmk::kBucketExperts);
    if (n_slots_per_token < 1 || n_slots_per_token > bmk::kMaxCombineSlots)
        return fail(ctx, BM_ESHAPE, "%s: %d slots a token outside 1..=%d", what, n_slots_per_token, bmk::kMaxCombineSlots);
    if (max_tokens < 1 || (int64_t)max_tokens * n_slots_per_token > bmk::kGemmMaxSlots)
        return fail(ctx, BM_ESHAPE, "%s: max_tokens = %d at %d slots a token is outside 1..=%d slots", what, max_tokens,
                    n_slots_per_token, bmk::kGemmMaxSlots);
    bm_scratch *s = new (std::nothrow) bm_scratch{};
    if (!s) return fail(ctx, BM_EDRIVER, "%s: out of host memory", what);
    s->ctx = ctx;
    s->gate_type = gate_type, s->down_type = down_type, s->hidden = hidden, s->ff = ff, s->n_experts = n_experts;
    s->spt = n_slots_per_token, s->max_tokens = max_tokens;
    // the crossovers measured on MI355X at the Qwen3-30B-A3B layer shape (Q4_K gate/up, Q6_K down, top-8 of 128):
    // tokens   per slot   grouped   GEMM exact   GEMM tolerance mode   (us a step)
    //     16       67        86        190          118
    //     24       92        88        217          130
    //    128      400       188        336          201
    //    192      580       246        370          214
    //    256      767       296        392          230
    //    512     1491       534        481          289
    s->path = BM_PATH_AUTO, s->grouped_from = 22, s->gemm_from = 448, s->gemm_from_fast = 96;
    // a gate/up stack on Q8_K columns (Q3_K, IQ2_XXS, IQ3_XXS, IQ4_XS): its tile launchers are bound by the type's decode, which
    // the GEMM does once a row and super-block for all of a tile's slots, so the exact GEMM is ahead much earlier (same layer
    // shape, us a step, grouped / GEMM: IQ4_XS 48 tokens 180 / 170, 96 tokens 265 / 185, 2048 tokens 3202 / 907; IQ2_XXS 64
    // tokens 168 / 196, 96 tokens 230 / 212, 2048 tokens 2682 / 995; IQ3_XXS 96 tokens 241 / 215; Q3_K 24 tokens 112 / 103)
    if (act_form(gate_type) != 0) s->gemm_from = 96;
    // ... and where the down stack is on Q8_K columns too and the experts are large, the grouped step - for few slots an
    // expert the per-slot gate . up launch and the down tiles, see bm_moe_forward - is ahead of the per-slot step from the first
    // token: every workgroup of the per-slot down launch encodes all of a token's h rows itself, work that grows with hidden x ff
    // (DeepSeek-V3 shape, hidden 7168, ff 2048, IQ2_XXS, us a step per slot / grouped: 1 token 61.5 / 57.9, 4 tokens 171 / 147,
    // 16 tokens 589 / 481; at hidden 2048, ff 768 the per-slot step leads up to 12 tokens: 1 token 16.0 / 23.7)
    if (act_form(gate_type) != 0 && act_form(down_type) != 0 && (int64_t)hidden * ff >= ((int64_t)1 << 23)) s->grouped_from = 1;
    const size_t slots = (size_t)max_tokens * n_slots_per_token;
    int rc = bm_act_create(ctx, gate_type, hidden, max_tokens, &s->act_x);
    if (!rc) rc = bm_act_create(ctx, down_type, ff, (int)slots, &s->act_h);
    if (!rc) rc = bm_route_create(ctx, (int)slots, n_experts, &s->route);
    if (!rc) {
        (void)hipSetDevice(ctx->device);
        const size_t table = slots + (size_t)n_experts + 1 + (size_t)bmk::tile_cap((int)slots, n_experts) + 1;
        hipError_t e = hipMalloc((void **)&s->g, slots * ff * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void **)&s->u, slots * ff * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void **)&s->down, slots * hidden * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void **)&s->order, table * sizeof(uint32_t));
        if (e == hipSuccess) e = hipMemset(s->order, 0, table * sizeof(uint32_t));
        if (e == hipSuccess) e = hipDeviceSynchronize();
        if (e != hipSuccess) rc = fail(ctx, BM_EDRIVER, "%s: %zu slots of scratch: %s", what, slots, hipGetErrorString(e));
        s->start = s->order + slots;
        s->tiles = s->start + n_experts + 1;
    }
    if (rc) {
        const std::string keep = ctx->err;
        bm_scratch_destroy(s);
        ctx->err = keep;
        return rc;
    }
    *out = s;
    return BM_OK;
}

int bm_scratch_set_path(bm_scratch *s, int path, int grouped_from, int gemm_from) {
    const char *what = "bm_scratch_set_path";
    if (!s) return fail(nullptr, BM_EARG, "%s: scratch is NULL", what);
    if (path != BM_PATH_AUTO && path != BM_PATH_PER_SLOT && path != BM_PATH_GROUPED && path != BM_PATH_GEMM)
        return fail(s->ctx, BM_EARG, "%s: path %d is not one of BM_PATH_AUTO, BM_PATH_PER_SLOT, BM_PATH_GROUPED, BM_PATH_GEMM", what, path);
    if (path == BM_PATH_GEMM && !(bmk::gemm_supported(s->gate_type) && bmk::gemm_supported(s->down_type)))
        return fail(s->ctx, BM_ETYPE, "%s: no grouped GEMM for types %d / %d", what, s->gate_type, s->down_type);
    if (grouped_from < 0 || gemm_from < 0)
        return fail(s->ctx, BM_ESHAPE, "%s: the crossovers are token counts (0: keep), got %d and %d", what, grouped_from, gemm_from);
    s->path = path;
    if (grouped_from) s->grouped_from = grouped_from;
    if (gemm_from) s->gemm_from = s->gemm_from_fast = gemm_from;
    return BM_OK;
}

// Whether the per-slot step's two launches fit a workgroup's LDS at this shape (bm_moe_decode refuses a shape past it: the
// token's column beside the quantizer's staging, and a token's slot columns beside the closing sum's operands).
static bool per_slot_fits(const bm_scratch *s) {
    const size_t lds_a = dev_col_bytes(s->gate_type, s->hidden) + 8192;
    const size_t lds_b = (size_t)s->spt * dev_col_bytes(s->down_type, s->ff) + 12288;
    return lds_a <= (size_t)bmk::kMaxLds && lds_b <= (size_t)bmk::kMaxLds;
}

int bm_scratch_path_for(const bm_scratch *s, int m) {
    if (!s || m < 1 || m > s->max_tokens) return BM_ESHAPE;
    const bool gemm_ok = bmk::gemm_supported(s->gate_type) && bmk::gemm_supported(s->down_type);
    const bool per_slot_ok = m <= bmk::kMaxDecodeTokens && per_slot_fits(s);
    if (s->path != BM_PATH_AUTO) {
        if (s->path == BM_PATH_PER_SLOT && !per_slot_ok) return BM_PATH_GROUPED;
        return s->path;
    }
    if (m < s->grouped_from && per_slot_ok) return BM_PATH_PER_SLOT;
    if (m < (s->ctx->gemm_mode != BM_GEMM_EXACT ? s->gemm_from_fast : s->gemm_from) || !gemm_ok) return BM_PATH_GROUPED;
    return BM_PATH_GEMM;
}

int bm_moe_forward(bm_ctx *ctx, bm_scratch *s, const bm_weights *wg, const bm_weights *wu, const bm_weights *wd,
                   const float *x_dev, const uint32_t *sel_dev, const float *w_dev, const float *resid_dev, int m,
                   const bm_gate_act *rule, float *y_dev) {
    const char *what = "bm_moe_forward";
    if (!ctx || !s || !wg || !wu || !wd || !x_dev || !sel_dev || !w_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (s->ctx != ctx) return fail(ctx, BM_EARG, "%s: the scratch was made on another context", what);
    if (wg->wtype != s->gate_type || wu->wtype != s->gate_type || wd->wtype != s->down_type || wg->k != s->hidden || wd->k != s->ff)
        return fail(ctx, BM_ESHAPE, "%s: the scratch was made for types %d / %d at hidden %d, ff %d; the stacks are %d / %d / %d at %d, %d",
                    what, s->gate_type, s->down_type, s->hidden, s->ff, wg->wtype, wu->wtype, wd->wtype, wg->k, wd->k);
    if (wg->rows != (int64_t)s->n_experts * s->ff || wu->rows != wg->rows || wd->rows != (int64_t)s->n_experts * s->hidden)
        return fail(ctx, BM_ESHAPE, "%s: the scratch was made for %d experts; the stacks hold %lld, %lld and %lld rows", what,
                    s->n_experts, (long long)wg->rows, (long long)wu->rows, (long long)wd->rows);
    if (m < 1 || m > s->max_tokens) return fail(ctx, BM_ESHAPE, "%s: m = %d tokens, the scratch holds 1..=%d", what, m, s->max_tokens);
    const int spt = s->spt, n_slots = m * spt, hidden = s->hidden, ff = s->ff, n_experts = s->n_experts;
    const bool down_q8k = act_form(s->down_type) != 0;
    switch (bm_scratch_path_for(s, m)) {
    case BM_PATH_PER_SLOT:
        return bm_moe_decode(ctx, wg, wu, wd, x_dev, sel_dev, w_dev, resid_dev, spt, m, rule, s->act_h, nullptr,
                             down_q8k ? s->g : nullptr, y_dev);
    case BM_PATH_GROUPED: {
        // Few slots an expert (no more slots than experts: nearly every tile is one slot) and h on its way through f32 rows:
        // the per-slot gate . up launch is the faster one there (its one-column walk reads the activation operands a
        // super-block ahead: 83 against 102 us at the DeepSeek-V3 shape, 4 tokens) and the tile launch the faster down (54
        // against 84 us), so the step takes one of each; the down tiles then read their columns in slot order. The tokens'
        // columns are quantized once, beside the tables in their launch, not by every workgroup of the gate . up launch
        // (whose vector ALU is what bounds it at these types: 180 -> 172 us a step).
        if (down_q8k && act_form(s->gate_type) != 0 && n_slots <= n_experts && m <= bmk::kMaxDecodeTokens && per_slot_fits(s) &&
            n_experts <= bmk::kBucketExperts && n_slots <= bmk::kTileMaxSlots) {
            int rc = bm_tables_quantize(ctx, sel_dev, n_slots, n_experts, s->order, s->start, s->tiles, x_dev, m, s->act_x);
            if (!rc) rc = bm_gate_up(ctx, wg, wu, s->act_x, sel_dev, n_slots, ff, spt, rule, s->g, nullptr);
            if (!rc) // (a slot without an expert of the stack: its rows of h hold nothing, its column is left alone)
                rc = driver(ctx, what, bmk::quantize(launch_of(ctx), s->down_type, s->g, n_slots, ff, s->act_h->dev, nullptr, sel_dev,
                                                     (uint32_t)n_experts));
            if (!rc)
                rc = driver(ctx, what, bmk::gemv_tiles(launch_of(ctx), wd->wtype, wd->dev, n_experts, ff, s->act_h->dev, s->order, s->start,
                                                       s->tiles, n_slots, hidden, s->down, true));
            if (rc) return rc;
            break;
        }
        int rc = bm_tables_quantize(ctx, sel_dev, n_slots, n_experts, s->order, s->start, s->tiles, x_dev, m, s->act_x);
        if (!rc && !down_q8k)
            rc = bm_gate_up_tiles(ctx, wg, wu, s->act_x, s->order, s->start, s->tiles, n_slots, ff, spt, rule, nullptr, s->act_h);
        if (!rc && down_q8k) {
            rc = bm_gate_up_tiles(ctx, wg, wu, s->act_x, s->order, s->start, s->tiles, n_slots, ff, spt, rule, s->g, nullptr);
            if (!rc) rc = bm_quantize_ord(ctx, s->g, s->start, n_experts, n_slots, s->act_h);
        }
        if (!rc) rc = bm_gemv_tiles(ctx, wd, s->act_h, s->order, s->start, s->tiles, n_slots, hidden, s->down);
        if (rc) return rc;
        break;
    }
    default: {
        int rc = bm_route_fill_quantize(ctx, sel_dev, n_slots, s->route, x_dev, m, s->act_x);
        if (!rc) rc = bm_gemm(ctx, wg, ff, s->act_x, s->route, spt, s->g);
        if (!rc) rc = bm_gemm(ctx, wu, ff, s->act_x, s->route, spt, s->u);
        if (!rc) rc = bm_swiglu_quant_sel(ctx, s->g, s->u, sel_dev, n_experts, n_slots, rule, s->act_h);
        if (!rc) rc = bm_gemm(ctx, wd, hidden, s->act_h, s->route, 0, s->down);
        if (rc) return rc;
        break;
    }
    }
    // the slots' weighted sum; a slot that names no expert of the stack adds nothing, as in the per-slot path
    return driver(ctx, what, bmk::combine_tokens(launch_of(ctx), s->down, w_dev, nullptr, resid_dev, hidden, spt, m, y_dev, sel_dev,
                                                 (uint32_t)n_experts));
}

// crates/gpu/src/kquant/act.rs:71-125 Act::code: what the device rules can run, refused by name otherwise.
static int rule_checked(bm_ctx *ctx, const char *what, int rule, float limit, bmk::GateRule *out) {
    switch (rule) {
    case BM_ACT_SILU_MUL:
        limit = 0.0f;
        break;
    case BM_ACT_SWIGLU_CLAMP:
        if (!std::isfinite(limit)) return fail(ctx, BM_ESHAPE, "%s: the clamp limit must be finite, got %g", what, (double)limit);
        break;
    case BM_ACT_SWIGLU_OAI:
        if (!std::isfinite(limit) || limit < 0.0f)
            return fail(ctx, BM_ESHAPE, "%s: swigluoai runs at alpha 1.702 and a finite limit of at least 0, got limit %g", what,
                        (double)limit);
        break;
    case BM_ACT_SITU:
        if (!std::isfinite(limit) || !(limit > 0.0f))
            return fail(ctx, BM_ESHAPE, "%s: situ runs at linear beta 25 and a finite positive beta, got beta %g", what, (double)limit);
        break;
    case BM_ACT_SWIGLU_GCLAMP:
        if (!std::isfinite(limit) || !(limit > 0.0f))
            return fail(ctx, BM_ESHAPE, "%s: the gate-first clamp limit must be finite and positive, got %g; a caller that clamps "
                        "nothing runs BM_ACT_SWIGLU_CLAMP", what, (double)limit);
        break;
    default:
        return fail(ctx, BM_ETYPE, "%s: rule %d is not one of BM_ACT_SILU_MUL, BM_ACT_SWIGLU_CLAMP, BM_ACT_SWIGLU_OAI, BM_ACT_SITU, "
                    "BM_ACT_SWIGLU_GCLAMP", what, rule);
    }
    *out = bmk::GateRule{(uint32_t)rule, limit};
    return BM_OK;
}

int bm_set_gate_rule(bm_ctx *ctx, int rule, float limit) {
    const char *what = "bm_set_gate_rule";
    if (!ctx) return fail(nullptr, BM_EARG, "%s: ctx is NULL", what);
    return rule_checked(ctx, what, rule, limit, &ctx->rule);
}

int bm_set_gemm_mode(bm_ctx *ctx, int mode) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_set_gemm_mode: ctx is NULL");
    if (mode != BM_GEMM_EXACT && mode != BM_GEMM_FAST && mode != BM_GEMM_FAST_F16)
        return fail(ctx, BM_EARG, "bm_set_gemm_mode: mode %d is none of BM_GEMM_EXACT, BM_GEMM_FAST, BM_GEMM_FAST_F16", mode);
    ctx->gemm_mode = mode;
    return BM_OK;
}

int bm_set_down_form(bm_ctx *ctx, int form) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_set_down_form: ctx is NULL");
    if (form != BM_DOWN_RING && form != BM_DOWN_SPLIT)
        return fail(ctx, BM_EARG, "bm_set_down_form: form %d is neither BM_DOWN_RING nor BM_DOWN_SPLIT", form);
    ctx->down_form = form;
    return BM_OK;
}

int bm_swiglu_quant(bm_ctx *ctx, const float *g_dev, const float *u_dev, int n_cols, const bm_gate_act *rule, bm_act *act) {
    const char *what = "bm_swiglu_quant";
    if (!ctx || !g_dev || !u_dev || !act) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_cols < 1 || n_cols > act->m_cap)
        return fail(ctx, BM_ESHAPE, "%s: n_cols = %d columns, act holds %d", what, n_cols, act->m_cap);
    bmk::Launch L;
    if (int rc = launch_under(ctx, what, rule, &L)) return rc;
    return driver(ctx, what, bmk::swiglu_quant(L, g_dev, u_dev, n_cols, act->k, act->dev, act_form(act->wtype) != 0));
}

int bm_swiglu_quant_sel(bm_ctx *ctx, const float *g_dev, const float *u_dev, const uint32_t *sel_dev, int n_experts, int n_cols,
                        const bm_gate_act *rule, bm_act *act) {
    const char *what = "bm_swiglu_quant_sel";
    if (!ctx || !g_dev || !u_dev || !sel_dev || !act) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_experts < 1) return fail(ctx, BM_ESHAPE, "%s: n_experts = %d", what, n_experts);
    if (n_cols < 1 || n_cols > act->m_cap) return fail(ctx, BM_ESHAPE, "%s: %d columns, the activation holds %d", what, n_cols, act->m_cap);
    bmk::Launch L;
    int rc = launch_under(ctx, what, rule, &L);
    if (rc) return rc;
    return driver(ctx, what,
                  bmk::swiglu_quant(L, g_dev, u_dev, n_cols, act->k, act->dev, act_form(act->wtype) != 0, sel_dev, (uint32_t)n_experts));
}

int bm_weights_from_gguf(bm_ctx *ctx, const bm_gguf *g, const char *name, bm_weights **out, int *rows_per_expert, int *n_experts) {
    const char *what = "bm_weights_from_gguf";
    if (!ctx || !g || !name || !out) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    *out = nullptr;
    bm_gguf_tensor t;
    if (bm_gguf_find(g, name, &t) != BM_OK) return fail(ctx, BM_ESHAPE, "%s: %s", what, bm_gguf_last_error());
    if (!known_type(t.type))
        return fail(ctx, BM_ETYPE, "%s: %s is of ggml type %d; this library computes in Q3_K (11), Q4_K (12), Q5_K (13), Q6_K (14), IQ2_XXS (16), IQ3_XXS (18) and IQ4_XS (23)", what,
                    name, t.type);
    if (t.n_dims < 2 || t.n_dims > 3)
        return fail(ctx, BM_ESHAPE, "%s: %s has %d dimensions; a matrix has 2, an expert stack 3", what, name, t.n_dims);
    if (t.dims[0] > (1u << 30) || t.dims[1] > (1u << 30) || t.dims[2] > (1u << 20))
        return fail(ctx, BM_ESHAPE, "%s: %s is {%llu, %llu, %llu}: past what a stack holds", what, name, (unsigned long long)t.dims[0],
                    (unsigned long long)t.dims[1], (unsigned long long)t.dims[2]);
    const int k = (int)t.dims[0];
    const int64_t rows = (int64_t)t.dims[1] * (int64_t)t.dims[2];
    if ((uint64_t)rows * (uint64_t)bm_row_bytes(t.type, k) != t.nbytes)
        return fail(ctx, BM_ESHAPE, "%s: %s holds %llu bytes, %lld rows of %d values take %lld", what, name, (unsigned long long)t.nbytes,
                    (long long)rows, k, (long long)(rows * bm_row_bytes(t.type, k)));
    if (rows_per_expert) *rows_per_expert = (int)t.dims[1];
    if (n_experts) *n_experts = (int)t.dims[2];
    return bm_weights_create(ctx, t.type, rows, k, t.data, out);
}

int bm_route_softmax(bm_ctx *ctx, const float *logits_dev, int n_tokens, int n_experts, int top_k, int renorm, float *probs_dev,
                     uint32_t *ids_dev, float *weights_dev) {
    const char *what = "bm_route_softmax";
    if (!ctx || !logits_dev || !ids_dev || !weights_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_tokens < 1) return fail(ctx, BM_ESHAPE, "%s: n_tokens = %d must be positive", what, n_tokens);
    if (n_experts < 1 || n_experts > bmk::kRouteMaxExperts)
        return fail(ctx, BM_ESHAPE, "%s: n_experts = %d, the router takes 1 to %d", what, n_experts, bmk::kRouteMaxExperts);
    if (top_k < 1 || top_k > bmk::kRouteMaxPicks || top_k > n_experts)
        return fail(ctx, BM_ESHAPE, "%s: top_k = %d of %d experts, the router picks 1 to %d", what, top_k, n_experts,
                    bmk::kRouteMaxPicks);
    return driver(ctx, what, bmk::route_softmax(launch_of(ctx), logits_dev, n_tokens, n_experts, top_k, renorm != 0, probs_dev,
                                                ids_dev, weights_dev));
}

int bm_router_logits(bm_ctx *ctx, const float *router_dev, const float *x_dev, const float *gain_dev, float eps, int n_tokens,
                     int n_experts, int hidden, float *normed_dev, float *logits_dev) {
    const char *what = "bm_router_logits";
    if (!ctx || !router_dev || !x_dev || !logits_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_tokens < 1 || n_experts < 1) return fail(ctx, BM_ESHAPE, "%s: %d tokens, %d experts: both must be positive", what, n_tokens, n_experts);
    if (hidden < 8 || hidden % 8 != 0)
        return fail(ctx, BM_ESHAPE, "%s: hidden = %d is not a positive multiple of 8 (the f32 row dot's eight lanes)", what, hidden);
    if ((int64_t)n_tokens * n_experts > (1 << 30)) return fail(ctx, BM_ESHAPE, "%s: %d tokens x %d experts is past what a launch takes", what, n_tokens, n_experts);
    if (!bmk::router_logits_fits(hidden)) return fail(ctx, BM_ESHAPE, "%s: two rows of hidden = %d do not fit the workgroup's LDS", what, hidden);
    if ((((uintptr_t)router_dev | (uintptr_t)x_dev | (uintptr_t)gain_dev | (uintptr_t)normed_dev) & 15) != 0)
        return fail(ctx, BM_ESHAPE, "%s: router_dev %p, x_dev %p, gain_dev %p and normed_dev %p must be 16-byte aligned", what,
                    (const void *)router_dev, (const void *)x_dev, (const void *)gain_dev, (const void *)normed_dev);
    if (gain_dev && !(eps >= 0.0f)) return fail(ctx, BM_EARG, "%s: eps = %g is negative or not a number", what, (double)eps);
    return driver(ctx, what, bmk::router_logits(launch_of(ctx), router_dev, x_dev, gain_dev, eps, n_tokens, n_experts, hidden, normed_dev,
                                                logits_dev));
}

int bm_norm_route(bm_ctx *ctx, const float *router_dev, const float *x_dev, const float *gain_dev, float eps, int n_tokens,
                  int n_experts, int hidden, int top_k, int renorm, float *normed_dev, float *logits_dev, float *probs_dev,
                  uint32_t *ids_dev, float *weights_dev, bm_act *act_x) {
    const char *what = "bm_norm_route";
    if (!ctx || !router_dev || !x_dev || !logits_dev || !ids_dev || !weights_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (n_tokens < 1 || n_tokens > bmk::kNormRouteMaxTokens)
        return fail(ctx, BM_ESHAPE, "%s: n_tokens = %d, the fused launch takes 1 to %d (past that: bm_router_logits, then bm_route_softmax)",
                    what, n_tokens, bmk::kNormRouteMaxTokens);
    if (n_experts < 1 || n_experts > bmk::kRouteMaxExperts)
        return fail(ctx, BM_ESHAPE, "%s: n_experts = %d, the router takes 1 to %d", what, n_experts, bmk::kRouteMaxExperts);
    if (top_k < 1 || top_k > bmk::kRouteMaxPicks || top_k > n_experts)
        return fail(ctx, BM_ESHAPE, "%s: top_k = %d of %d experts, the router picks 1 to %d", what, top_k, n_experts,
                    bmk::kRouteMaxPicks);
    if (hidden < 8 || hidden % 8 != 0)
        return fail(ctx, BM_ESHAPE, "%s: hidden = %d is not a positive multiple of 8 (the f32 row dot's eight lanes)", what, hidden);
    if (!bmk::router_logits_fits(hidden)) return fail(ctx, BM_ESHAPE, "%s: two rows of hidden = %d do not fit the workgroup's LDS", what, hidden);
    if ((((uintptr_t)router_dev | (uintptr_t)x_dev | (uintptr_t)gain_dev | (uintptr_t)normed_dev) & 15) != 0)
        return fail(ctx, BM_ESHAPE, "%s: router_dev %p, x_dev %p, gain_dev %p and normed_dev %p must be 16-byte aligned", what,
                    (const void *)router_dev, (const void *)x_dev, (const void *)gain_dev, (const void *)normed_dev);
    if (gain_dev && !(eps >= 0.0f)) return fail(ctx, BM_EARG, "%s: eps = %g is negative or not a number", what, (double)eps);
    if (act_x && (act_x->k != hidden || act_x->m_cap < n_tokens))
        return fail(ctx, BM_ESHAPE, "%s: act_x must hold %d columns of k = %d; it holds %d of k = %d", what, n_tokens, hidden, act_x->m_cap,
                    act_x->k);
    return driver(ctx, what, bmk::norm_route(launch_of(ctx), router_dev, x_dev, gain_dev, eps, n_tokens, n_experts, hidden, normed_dev,
                                             logits_dev, top_k, renorm != 0, probs_dev, ids_dev, weights_dev, ctx->route_hand,
                                             act_x ? act_x->dev : nullptr, act_x && act_form(act_x->wtype) != 0, ctx->route_polls));
}

int bm_block_sums(bm_ctx *ctx, const bm_weights *w, int64_t row, const bm_act *act, int col, int32_t *out_dev) {
    const char *what = "bm_block_sums";
    if (!ctx || !w || !act || !out_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int rc = check_pair(ctx, what, w, act);
    if (rc) return rc;
    if (row < 0 || row >= w->rows) return fail(ctx, BM_ESHAPE, "%s: row %lld of %lld", what, (long long)row, (long long)w->rows);
    if (col < 0 || col >= act->m_cap) return fail(ctx, BM_ESHAPE, "%s: column %d of %d", what, col, act->m_cap);
    const uint8_t *wrow = w->dev + (size_t)row * (size_t)bm_row_bytes(w->wtype, w->k);
    const uint8_t *c = act->dev + (size_t)col * dev_col_bytes(act->wtype, act->k);
    return driver(ctx, what, bmk::block_sums(launch_of(ctx), w->wtype, wrow, w->k, c, out_dev));
}

// ------------------------------------------------------------------------------------ the card rule

static int check_card_planes(bm_ctx *ctx, const char *what, const void *codes, const void *d8, const void *s8) {
    if (((uintptr_t)codes & 15) != 0 || (((uintptr_t)d8 | (uintptr_t)s8) & 3) != 0)
        return fail(ctx, BM_ESHAPE, "%s: codes_dev %p must be 16-byte aligned, d8_dev %p and s8_dev %p 4-byte aligned", what, codes, d8, s8);
    return BM_OK;
}

int bm_card_quantize(bm_ctx *ctx, const float *x_dev, int m, int k, int8_t *codes_dev, float *d8_dev, int32_t *s8_dev) {
    const char *what = "bm_card_quantize";
    if (!ctx || !x_dev || !codes_dev || !d8_dev || !s8_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    if (k <= 0 || k % 256 != 0) return fail(ctx, BM_ESHAPE, "%s: card q8_1 columns are whole 256-value super-blocks, k = %d", what, k);
    if (m < 1) return fail(ctx, BM_ESHAPE, "%s: need m >= 1, got %d", what, m);
    if (((uintptr_t)x_dev & 15) != 0) return fail(ctx, BM_ESHAPE, "%s: x_dev %p must be 16-byte aligned", what, (const void *)x_dev);
    int rc = check_card_planes(ctx, what, codes_dev, d8_dev, s8_dev);
    if (rc) return rc;
    return driver(ctx, what, bmk::card_quantize(launch_of(ctx), x_dev, m, k, codes_dev, d8_dev, s8_dev));
}

static int check_card_weights(bm_ctx *ctx, const char *what, const bm_weights *w) {
    if (!bmk::card_type(w->wtype))
        return fail(ctx, BM_ETYPE, "%s: the card rule walks Q4_K (12) and Q3_K (11) rows; the weights are type %d", what, w->wtype);
    return BM_OK;
}

int bm_card_gemv(bm_ctx *ctx, const bm_weights *w, const int8_t *codes_dev, const float *d8_dev, const int32_t *s8_dev, int m,
                 float *y_dev) {
    const char *what = "bm_card_gemv";
    if (!ctx || !w || !codes_dev || !d8_dev || !s8_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int rc = check_card_weights(ctx, what, w);
    if (rc) return rc;
    if (m < 1 || m > 65535) return fail(ctx, BM_ESHAPE, "%s: m = %d columns (1 .. 65535)", what, m);
    rc = check_card_planes(ctx, what, codes_dev, d8_dev, s8_dev);
    if (rc) return rc;
    return driver(ctx, what, bmk::card_gemv(launch_of(ctx), w->wtype, w->dev, (long)w->rows, w->k, codes_dev, d8_dev, s8_dev, m, y_dev));
}

int bm_card_gemv_sel(bm_ctx *ctx, const bm_weights *w, const int8_t *codes_dev, const float *d8_dev, const int32_t *s8_dev,
                     const uint32_t *sel_dev, int n_slots, int rows_per_expert, float *y_dev) {
    const char *what = "bm_card_gemv_sel";
    if (!ctx || !w || !codes_dev || !d8_dev || !s8_dev || !sel_dev || !y_dev) return fail(ctx, BM_EARG, "%s: NULL argument", what);
    int rc = check_card_weights(ctx, what, w);
    if (rc) return rc;
    int n_experts = 0;
    rc = check_stack(ctx, what, w, rows_per_expert, &n_experts);
    if (rc) return rc;
    if (n_slots < 1) return fail(ctx, BM_ESHAPE, "%s: need n_slots >= 1, got %d", what, n_slots);
    if ((int64_t)n_slots * ((rows_per_expert + 7) / 8) > 0x7fffffff)
        return fail(ctx, BM_ESHAPE, "%s: %d slots of %d rows are past what a launch takes", what, n_slots, rows_per_expert);
    rc = check_card_planes(ctx, what, codes_dev, d8_dev, s8_dev);
    if (rc) return rc;
    return driver(ctx, what, bmk::card_gemv_sel(launch_of(ctx), w->wtype, w->dev, n_experts, w->k, codes_dev, d8_dev, s8_dev, sel_dev,
                                                n_slots, rows_per_expert, y_dev));
}

// ------------------------------------------------------------------------------------ graphs and events

struct bm_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

struct bm_event {
    hipEvent_t ev;
};

int bm_capture_begin(bm_ctx *ctx) {
    if (!ctx) return fail(nullptr, BM_EARG, "bm_capture_begin: ctx is NULL");
    return driver(ctx, "bm_capture_begin", hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
}

int bm_capture_end(bm_ctx *ctx, bm_graph **out) {
    if (!ctx || !out) return fail(ctx, BM_EARG, "bm_capture_end: NULL argument");
    *out = nullptr;
    hipGraph_t g = nullptr;
    int rc = driver(ctx, "bm_capture_end", hipStreamEndCapture(ctx->stream, &g));
    if (rc) return rc;
    hipGraphExec_t x = nullptr;
    rc = driver(ctx, "bm_capture_end: instantiate", hipGraphInstantiate(&x, g, nullptr, nullptr, 0));
    if (rc) {
        (void)hipGraphDestroy(g);
        return rc;
    }
    bm_graph *bg = new (std::nothrow) bm_graph{g, x};
    if (!bg) {
        (void)hipGraphExecDestroy(x);
        (void)hipGraphDestroy(g);
        return fail(ctx, BM_EDRIVER, "bm_capture_end: out of host memory");
    }
    *out = bg;
    return BM_OK;
}

int bm_graph_launch(bm_ctx *ctx, bm_graph *graph) {
    if (!ctx || !graph) return fail(ctx, BM_EARG, "bm_graph_launch: NULL argument");
    return driver(ctx, "bm_graph_launch", hipGraphLaunch(graph->exec, ctx->stream));
}

void bm_graph_destroy(bm_graph *graph) {
    if (!graph) return;
    (void)hipGraphExecDestroy(graph->exec);
    (void)hipGraphDestroy(graph->graph);
    delete graph;
}

int bm_event_create(bm_ctx *ctx, bm_event **out) {
    if (!ctx || !out) return fail(ctx, BM_EARG, "bm_event_create: NULL argument");
    *out = nullptr;
    hipEvent_t e;
    int rc = driver(ctx, "bm_event_create", hipEventCreate(&e));
    if (rc) return rc;
    *out = new (std::nothrow) bm_event{e};
    if (!*out) {
        (void)hipEventDestroy(e);
        return fail(ctx, BM_EDRIVER, "bm_event_create: out of host memory");
    }
    return BM_OK;
}

int bm_event_record(bm_ctx *ctx, bm_event *event) {
    if (!ctx || !event) return fail(ctx, BM_EARG, "bm_event_record: NULL argument");
    return driver(ctx, "bm_event_record", hipEventRecord(event->ev, ctx->stream));
}

int bm_event_wait(bm_ctx *ctx, bm_event *event) {
    if (!ctx || !event) return fail(ctx, BM_EARG, "bm_event_wait: NULL argument");
    return driver(ctx, "bm_event_wait", hipStreamWaitEvent(ctx->stream, event->ev, 0));
}

int bm_event_elapsed_ms(bm_ctx *ctx, bm_event *start, bm_event *stop, float *ms) {
    if (!ctx || !start || !stop || !ms) return fail(ctx, BM_EARG, "bm_event_elapsed_ms: NULL argument");
    int rc = driver(ctx, "bm_event_elapsed_ms: sync", hipEventSynchronize(stop->ev));
    if (rc) return rc;
    return driver(ctx, "bm_event_elapsed_ms", hipEventElapsedTime(ms, start->ev, stop->ev));
}

void bm_event_destroy(bm_event *event) {
    if (!event) return;
    (void)hipEventDestroy(event->ev);
    delete event;
}

} // extern "C"
