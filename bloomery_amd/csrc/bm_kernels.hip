// HIP kernels of the quantized MoE expert matmul for gfx950, decode side, and their launch functions: the
// activation quantizers, the dense gemv, the routed expert chain slot by slot (gate . up . SwiGLU, down, combine),
// its fused forms, and the block-sum verification kernel.
#include "bm_kernels.h"

#include <atomic>

#include "bm_stream.hpp"

namespace bmk {

// Timeline of the two decode launches, in measurement builds only (-DBM_TIMELINE: `make timeline` builds
// libbm_moe_hip_timeline.so, which bench.py --timeline loads; the library proper holds none of this). Thread 0 of
// workgroup b of k_gate_up_x leaves the device's constant-rate counter (100 MHz) in row b at marks 0 .. 4 (start, expert
// id known, token quantized, rows dotted, block of h stored); of k_down_combine in row kTimelineRows / 2 + b at marks
// 0 .. 3 (start, columns in LDS, rows dotted, sum stored) and, taken into registers and stored behind the barrier so that no
// store stands among the loads they time, 4 .. 6 (expert id known, the ring's first super-blocks asked for, columns arrived).
// The last launch of each kernel is what the table holds.
#ifdef BM_TIMELINE
__device__ __forceinline__ unsigned bm_block_linear() { return (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x; }
constexpr int kTimelineRows = 4096;
__device__ unsigned long long g_timeline[kTimelineRows * 8];
#define BM_MARK(base, mark)                                                                                            \
    do {                                                                                                               \
        if (threadIdx.x == 0 && (base) + bm_block_linear() < (unsigned)kTimelineRows)                                  \
            g_timeline[((base) + bm_block_linear()) * 8 + (mark)] = wall_clock64();                                           \
    } while (0)
// BM_TICK keeps the counter in a register once `dep` has arrived (no store among the loads it times); BM_TOCK stores it.
#define BM_TICK(var, dep)                                                                                              \
    unsigned long long var;                                                                                            \
    do {                                                                                                               \
        __asm__ volatile("" ::"v"(dep) : "memory");                                                                    \
        var = wall_clock64();                                                                                          \
    } while (0)
#define BM_TOCK(base, mark, var)                                                                                       \
    do {                                                                                                               \
        if (threadIdx.x == 0 && (base) + bm_block_linear() < (unsigned)kTimelineRows)                                  \
            g_timeline[((base) + bm_block_linear()) * 8 + (mark)] = var;                                                      \
    } while (0)
#else
#define BM_MARK(base, mark)                                                                                            \
    do {                                                                                                               \
    } while (0)
#define BM_TICK(var, dep)                                                                                              \
    do {                                                                                                               \
    } while (0)
#define BM_TOCK(base, mark, var)                                                                                       \
    do {                                                                                                               \
    } while (0)
#endif

// ----------------------------------------------------------------------------------------------- fill

__global__ void k_fill_u32(u32 *dst, u32 value, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = value;
}

hipError_t fill_u32(const Launch &L, uint32_t *dst, uint32_t value, size_t n) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, L.stream, dst, value, n);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------- quantizers

// x: m columns of k values -> Q8_2_X4 columns. One half wave a 32-value block.
__global__ __launch_bounds__(256) void k_quantize_q82x4(const float *x, int m, int k, uint8_t *act, const u32 *live,
                                                        u32 *fault, u32 layer) {
    const int bpc = k / 32; // blocks a column
    const long gblk = (long)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (gblk >= (long)m * bpc) return;
    const int col = (int)(gblk / bpc), blk = (int)(gblk % bpc), lane32 = threadIdx.x & 31;
    if (live && (u32)col >= *live) return; // a device-side column count: the columns past it keep what they held
    const float v = x[(size_t)col * k + 32 * blk + lane32];
    Q82Head hd;
    int s16;
    const int code = q82_block(v, &hd, &s16);
    if (hd.bad && lane32 == 0) bm_raise(fault, layer, kSiteQuantColumn);
    q82_store(act + (size_t)col * (k / 256) * BM_Q82_SB_EXT, k / 256, blk, lane32, code, hd, s16);
}

// x: m columns of k values -> Q8_K columns (crates/qdot/src/lib.rs:1787-1809). One workgroup a 256-value block.
// sel (optional): column c belongs to slot c; a slot whose id names no expert of the stack (served elsewhere, or refused) keeps
// its column as it stands and raises nothing here: its rows of x need not hold anything.
__global__ __launch_bounds__(256) void k_quantize_q8k(const float *x, int m, int k, uint8_t *act, const u32 *live,
                                                      const u32 *sel, u32 n_experts, u32 *fault, u32 layer) {
    const int bpc = k / 256;
    const int col = blockIdx.x / bpc, blk = blockIdx.x % bpc;
    if (live && (u32)col >= *live) return;
    if (sel && sel[col] >= n_experts) return;
    q8k_block_by_workgroup(x[(size_t)col * k + 256 * blk + threadIdx.x], act + ((size_t)col * bpc + blk) * BM_Q8K_STRIDE, fault, layer);
}

// The same columns with eight values a thread, a block a quad of lanes (two 16-byte loads a thread, fewer and fatter
// workgroups): the form for many columns at once, where the launch is bound by its traffic and not by its latency.
__global__ __launch_bounds__(256) void k_quantize_q82x4_wide(const float *x, int m, int k, uint8_t *act, const u32 *live,
                                                             u32 *fault, u32 layer) {
    const long at = ((long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (at >= (long)m * k) return;
    const int col = (int)(at / k), o = (int)(at % k);
    if (live && (u32)col >= *live) return;
    const float4 a = *reinterpret_cast<const float4 *>(x + at), b = *reinterpret_cast<const float4 *>(x + at + 4);
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    q82_quad8(v, act + (size_t)col * (k / 256) * BM_Q82_SB_EXT, k / 256, o >> 5, threadIdx.x & 3, fault, layer);
}

// Columns from which on the wide form is launched (and only for 16-byte aligned rows).
constexpr long kWideQuantValues = 1 << 18;

hipError_t quantize(const Launch &L, int wtype, const float *x, int m, int k, uint8_t *act, const uint32_t *live,
                    const uint32_t *sel, uint32_t n_experts) {
    if (sel && !bm_takes_q8k(wtype)) return hipErrorInvalidValue; // the slot-aware form is the Q8_K quantizer's
    if (!bm_takes_q8k(wtype) && (long)m * k >= kWideQuantValues && ((uintptr_t)x & 15) == 0) {
        const long threads = (long)m * k / 8;
        hipLaunchKernelGGL(k_quantize_q82x4_wide, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, L.stream, x, m, k, act,
                           live, L.fault, L.layer);
        return hipGetLastError();
    }
    if (bm_takes_q8k(wtype)) {
        hipLaunchKernelGGL(k_quantize_q8k, dim3((unsigned)(m * (k / 256))), dim3(256), 0, L.stream, x, m, k, act,
                           live, sel, n_experts, L.fault, L.layer);
    } else {
        const long blocks = (long)m * (k / 32);
        hipLaunchKernelGGL(k_quantize_q82x4, dim3((unsigned)((blocks + 7) / 8)), dim3(256), 0, L.stream, x, m, k, act,
                           live, L.fault, L.layer);
    }
    return hipGetLastError();
}

// Fills the two tables of `m` device Q8_2_X4 columns from their reference bytes (after an upload of those bytes).
__global__ __launch_bounds__(256) void k_q82_tables(uint8_t *act, int m, int nb) {
    const long g = (long)blockIdx.x * 256 + threadIdx.x; // one 16-value group a thread
    if (g >= (long)m * nb * 16) return;
    const int col = (int)(g / (nb * 16)), g16 = (int)(g % (nb * 16)), blk = g16 >> 1, half = g16 & 1;
    uint8_t *c = act + (size_t)col * nb * BM_Q82_SB_EXT;
    const uint8_t *group = c + (size_t)(blk >> 2) * BM_Q82X4_STRIDE;
    const signed char *codes = reinterpret_cast<const signed char *>(group + 16 + 32 * (blk & 3) + 16 * half);
    int s = 0;
    for (int n = 0; n < 16; n++) s += codes[n];
    *reinterpret_cast<int *>(c + (size_t)nb * (BM_Q82_SB_REF + 64) + 4 * g16) = s;
    if (half == 0) {
        const float d8 = bm_bf16_to_f32(*reinterpret_cast<const unsigned short *>(group + 2 * (blk & 3)));
        const int isum = *reinterpret_cast<const short *>(group + 8 + 2 * (blk & 3));
        *reinterpret_cast<float2 *>(c + (size_t)nb * BM_Q82_SB_REF + 8 * blk) = make_float2(d8, __fmul_rn(d8, (float)isum));
    }
}

hipError_t q82_tables(const Launch &L, uint8_t *act, int m, int k) {
    const int nb = k / 256;
    const long n = (long)m * nb * 16;
    hipLaunchKernelGGL(k_q82_tables, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, L.stream, act, m, nb);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------ gemv

// y[row * m_total + col0 + c] = row . column (col0 + c), c < m <= M. A quad a row, 64 rows a workgroup. M = 1 is the
// one-column form of the row dot, which reads a super-block's activation operands a super-block ahead.
// T: the workgroup's threads, T / 4 rows: 256, or 64 for a matrix of so few rows that workgroups of 64 rows would leave most of
// the card idle (768 rows are 12 of them, on 12 of 256 compute units, each streaming its 64 rows through one address unit).
template <int WT, int U, int NB, int M, int T = 256>
__global__ __launch_bounds__(T) void k_gemv(const uint8_t *w, long rows, int nb, const uint8_t *act, int m_total,
                                            int col0, int m, float *y) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3;
    const long row = (long)blockIdx.x * (T / 4) + (tid >> 2);
    const bool active = row < rows;
    const int n = NB > 0 ? NB : nb;
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const uint8_t *wrow = w + (size_t)(active ? row : 0) * row_bytes;
    // the columns' first bytes are asked for in front of the rows (vector loads come back in the order they were asked for:
    // behind the rows' requests the columns would wait for those as well); what a thread's few loads do not cover comes after
    Stage<(T == 64 ? 5 : 2), T> st;
    st.load(act + (size_t)col0 * col_bytes, m * col_bytes);
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT, T>(lds);
    uint8_t *cols = lds + tab_bytes<WT>();
    st.store(cols, act + (size_t)col0 * col_bytes, m * col_bytes);
    __syncthreads();
    float out[M];
    row_dot<WT, U, NB, M>(b, wrow, cols, col_bytes, m, n, q, tb, out, NoTap{});
    if (q == 0 && active) {
#pragma unroll
        for (int c = 0; c < M; c++)
            if (c < m) y[(size_t)row * m_total + col0 + c] = out[c];
    }
}

// --------------------------------------------------------------------------------- gate . up . SwiGLU

// One workgroup = 32 consecutive rows of one slot; eight lanes a row: a quad on the gate row, a quad on the up row.
// With act_h the 32 values are quantized to one q8_2 block of the slot's down activation in the same launch.
struct GateUpColLate { // the end of k_gate_up's arguments (see bm_kernarg_at)
    float *h;
    uint8_t *act_h;
    GateRule rule;
    u32 *fault;
    u32 layer;
};
struct GateUpColArgs { // k_gate_up's argument block
    const uint8_t *wg, *wu;
    u32 n_experts;
    int nb;
    const uint8_t *act;
    const u32 *sel;
    int rpe, spc_word;
    u32 n_slots;
    GateUpColLate late;
};
static_assert(offsetof(GateUpColArgs, late) == 56, "fourteen words in front of the late arguments");
constexpr unsigned kGateUpGridY = 32768; // slots along the grid's second dimension; the third counts the rest

// The grid: (blocks of 32 rows, slots, slots / kGateUpGridY): no division stands before the workgroup's first request.
// spc_word: slots_per_col, and above bit 24 one more than its log2 where it is a power of two.
template <int WT, int U, int NB>
__global__ __launch_bounds__(256) void k_gate_up(const uint8_t *wg, const uint8_t *wu, u32 n_experts, int nb,
                                                 const uint8_t *act, const u32 *sel, int rpe, int spc_word, u32 n_slots,
                                                 GateUpColLate) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3, which = (tid >> 2) & 1;
    const int slot = (int)(blockIdx.z * kGateUpGridY + blockIdx.y), rb = (int)blockIdx.x;
    if ((u32)slot >= n_slots) return;
    const int r = rb * 32 + (tid >> 3);
    const bool active = r < rpe;
    const u32 id = sel[slot];
    const int n = NB > 0 ? NB : nb;
    const int nb_h = rpe / 256;
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const int spc_shift = (spc_word >> 24) - 1;
    const int token = spc_shift >= 0 ? slot >> spc_shift : slot / (spc_word & 0xffffff);
    const uint8_t *act_col = act + (size_t)token * col_bytes;
    Stage<2> st;
    st.load(act_col, col_bytes);
    if (id >= n_experts) { // uniform over the workgroup: no weight is read (crates/gpu/src/kquant/sel.rs:22-28)
        if (id == 0xffffffffu) return; // a slot served elsewhere: nothing written, nothing raised (sel.rs:153-161)
        const GateUpColLate late = bm_kernarg_at<GateUpColLate>(offsetof(GateUpColArgs, late));
        float *const h = bm_global(late.h);
        uint8_t *const act_h = bm_global(late.act_h);
        if (tid == 0) bm_raise(bm_global(late.fault), late.layer, kSiteExpertId);
        if (h && active && (tid & 7) == 0) h[(size_t)slot * rpe + r] = bm_bits_f32(0x7fc00000u);
        if (act_h && tid < 32) q82_store(act_h + (size_t)slot * nb_h * BM_Q82_SB_EXT, nb_h, rb, tid, 0, Q82Head{0x7fc0u, 0, true}, 0);
        return;
    }
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const uint8_t *wrow = (which ? wu : wg) + ((size_t)id * rpe + (active ? r : 0)) * row_bytes;
    Blk<WT> b[U];
    // (behind the wait for the id; nothing reads them before the column stands in LDS)
    const GateUpColLate late = bm_kernarg_at<GateUpColLate>(offsetof(GateUpColArgs, late));
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *col = lds + tab_bytes<WT>();
    st.store(col, act_col, col_bytes);
    __syncthreads();
    float *const h = bm_global(late.h);
    uint8_t *const act_h = bm_global(late.act_h);
    u32 *const fault = bm_global(late.fault);
    const u32 layer = late.layer;
    uint8_t *hcol = act_h ? act_h + (size_t)slot * nb_h * BM_Q82_SB_EXT : nullptr;
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, col, col_bytes, 1, n, q, tb, v, NoTap{});
    const float hv = swiglu_of_pair(v[0], which, late.rule, fault, layer);
    if (h && active && (tid & 7) == 0) h[(size_t)slot * rpe + r] = hv;
    if (act_h) { // rpe is a multiple of 256 here, so every row of the block is live
        float *hbuf = reinterpret_cast<float *>(col + col_bytes);
        if ((tid & 7) == 0) hbuf[tid >> 3] = hv;
        __syncthreads();
        if (tid < 32) quantize_h_block(hbuf, hcol, nb_h, rb, tid, fault, layer);
    }
}

// ------------------------------------------------------------------------------------- down: gemv_sel

// Slot s: rows of expert sel[s] against column s. A quad a row, 64 rows a workgroup.
template <int WT, int U, int NB>
__global__ __launch_bounds__(256) void k_gemv_sel(const uint8_t *w, u32 n_experts, int nb, const uint8_t *act,
                                                  const u32 *sel, int rpe, float *y, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3;
    const int blocks_per_slot = (rpe + 63) / 64;
    const int slot = blockIdx.x / blocks_per_slot, rb = blockIdx.x % blocks_per_slot;
    const int r = rb * 64 + (tid >> 2);
    const bool active = r < rpe;
    const u32 id = sel[slot];
    const int n = NB > 0 ? NB : nb;
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const uint8_t *act_col = act + (size_t)slot * col_bytes;
    Stage<2> st;
    st.load(act_col, col_bytes);
    if (id >= n_experts) { // the slot's rows stay untouched; a host slot is skipped silently
        if (tid == 0 && rb == 0 && id != 0xffffffffu) bm_raise(fault, layer, kSiteExpertId);
        return;
    }
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const uint8_t *wrow = w + ((size_t)id * rpe + (active ? r : 0)) * row_bytes;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *col = lds + tab_bytes<WT>();
    st.store(col, act_col, col_bytes);
    __syncthreads();
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, col, col_bytes, 1, n, q, tb, v, NoTap{});
    if (q == 0 && active) y[(size_t)slot * rpe + r] = v[0];
}

// --------------------------------------------------------------------------------------------- combine

// crates/gpu/src/arch/qwen3moe/experts.rs:293-318 with crates/gpu/src/elem.rs:658-697: one thread a value.
// With a shared expert's rows: (sum + shexp) + resid, grouped as the reference groups its two adds
// (crates/gpu/src/moe_fused.rs:129-170 moe_combine).
// `sel` (optional): a slot whose id is at or past n_experts adds nothing, as in the fused down + combine launch.
__global__ __launch_bounds__(256) void k_combine(const float *down, const float *w, const float *shexp, const float *resid,
                                                 int rows, int n_slots, int m, float *y, const u32 *sel, u32 n_experts) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x; // (the launcher's 256 threads: blockDim.x is a load from memory)
    if (i >= (long)rows * m) return;
    const int t = (int)(i / rows), d = (int)(i % rows);
    float acc = 0.0f;
    for (int e = 0; e < n_slots; e++) {
        if (sel && sel[(size_t)t * n_slots + e] >= n_experts) continue;
        acc = fmaf(w[(size_t)t * n_slots + e], down[((size_t)t * n_slots + e) * rows + d], acc);
    }
    if (shexp) acc = __fadd_rn(acc, shexp[i]);
    y[i] = resid ? __fadd_rn(acc, resid[i]) : acc;
}

// The same with four consecutive values a thread (16-byte loads): the form for many tokens.
__global__ __launch_bounds__(256) void k_combine4(const float *down, const float *w, const float *shexp, const float *resid,
                                                  int rows, int n_slots, int m, float *y, const u32 *sel, u32 n_experts) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= (long)rows * m) return;
    const int t = (int)(i / rows), d = (int)(i % rows);
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int e = 0; e < n_slots; e++) {
        if (sel && sel[(size_t)t * n_slots + e] >= n_experts) continue;
        const float we = w[(size_t)t * n_slots + e];
        const float4 v = *reinterpret_cast<const float4 *>(down + ((size_t)t * n_slots + e) * rows + d);
        acc.x = fmaf(we, v.x, acc.x);
        acc.y = fmaf(we, v.y, acc.y);
        acc.z = fmaf(we, v.z, acc.z);
        acc.w = fmaf(we, v.w, acc.w);
    }
    if (shexp) {
        const float4 s4 = *reinterpret_cast<const float4 *>(shexp + i);
        acc = make_float4(__fadd_rn(acc.x, s4.x), __fadd_rn(acc.y, s4.y), __fadd_rn(acc.z, s4.z), __fadd_rn(acc.w, s4.w));
    }
    if (resid) {
        const float4 r4 = *reinterpret_cast<const float4 *>(resid + i);
        acc = make_float4(__fadd_rn(acc.x, r4.x), __fadd_rn(acc.y, r4.y), __fadd_rn(acc.z, r4.z), __fadd_rn(acc.w, r4.w));
    }
    *reinterpret_cast<float4 *>(y + i) = acc;
}

hipError_t combine_tokens(const Launch &L, const float *down, const float *w, const float *shexp, const float *resid,
                          int rows, int n_slots, int m, float *y, const uint32_t *sel, uint32_t n_experts) {
    const long n = (long)rows * m;
    const uintptr_t align = (uintptr_t)down | (uintptr_t)shexp | (uintptr_t)resid | (uintptr_t)y;
    if (n >= (1 << 18) && rows % 4 == 0 && (align & 15) == 0) {
        hipLaunchKernelGGL(k_combine4, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, L.stream, down, w, shexp, resid, rows,
                           n_slots, m, y, sel, n_experts);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(k_combine, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, L.stream, down, w, shexp, resid, rows,
                       n_slots, m, y, sel, n_experts);
    return hipGetLastError();
}

struct DownLate { // the end of k_down_combine's arguments
    float *y;
    u32 *fault;
    u32 layer;
};
struct DownArgs { // k_down_combine's argument block
    const uint8_t *w;
    u32 n_experts;
    int nb;
    const uint8_t *act;
    const u32 *sel;
    const float *wts, *resid;
    int spt_word, rpe;
    DownLate late;
};
struct GateUpLate { // the end of k_gate_up_x's arguments
    uint8_t *act_x, *act_h;
    float *h;
    GateRule rule;
    u32 *fault;
    u32 layer;
};
struct GateUpArgs { // k_gate_up_x's argument block
    const float *x;
    const uint8_t *wg, *wu;
    u32 n_experts;
    int nba, nh;
    const u32 *sel;
    int spt;
    GateUpLate late;
};
static_assert(offsetof(DownArgs, late) == 56 && offsetof(GateUpArgs, late) == 56, "fourteen words in front of the late arguments");

// --------------------------------------------------------------------------- down + combine in one launch

// A row's closing sum over its token's slots in slot order, acc = fma(w_s, v_s, acc) for the live slots, then the
// residual (crates/gpu/src/arch/qwen3moe/experts.rs:293-318). v, w and ids lie in LDS. With eight slots every operand is
// read before the first multiply-add (six 16-byte reads in flight at once); a loop that reads as it goes pays an LDS
// round trip a slot, 0.4 us at the end of the launch.
__device__ __forceinline__ float slot_sum(const float *v, const float *w, const u32 *ids, int spt, u32 n_experts,
                                          float resid_v, bool with_resid) {
    float acc = 0.0f;
    if (spt == 8) {
        const float4 v0 = *reinterpret_cast<const float4 *>(v), v1 = *reinterpret_cast<const float4 *>(v + 4);
        const float4 w0 = *reinterpret_cast<const float4 *>(w), w1 = *reinterpret_cast<const float4 *>(w + 4);
        const uint4 i0 = *reinterpret_cast<const uint4 *>(ids), i1 = *reinterpret_cast<const uint4 *>(ids + 4);
        acc = i0.x < n_experts ? fmaf(w0.x, v0.x, acc) : acc;
        acc = i0.y < n_experts ? fmaf(w0.y, v0.y, acc) : acc;
        acc = i0.z < n_experts ? fmaf(w0.z, v0.z, acc) : acc;
        acc = i0.w < n_experts ? fmaf(w0.w, v0.w, acc) : acc;
        acc = i1.x < n_experts ? fmaf(w1.x, v1.x, acc) : acc;
        acc = i1.y < n_experts ? fmaf(w1.y, v1.y, acc) : acc;
        acc = i1.z < n_experts ? fmaf(w1.z, v1.z, acc) : acc;
        acc = i1.w < n_experts ? fmaf(w1.w, v1.w, acc) : acc;
    } else {
        for (int s = 0; s < spt; s++)
            if (ids[s] < n_experts) acc = fmaf(w[s], v[s], acc);
    }
    return with_resid ? __fadd_rn(acc, resid_v) : acc;
}

// The shared body of the down + combine workgroup: token t, output rows rb * D .. + D with D = 64 / spt, a quad for
// every (row, slot).
template <int WT, int U, int NB, bool EIGHT = false>
__device__ __forceinline__ void down_combine_body(uint8_t *lds, const uint8_t *w, u32 n_experts, int nb,
                                                  const uint8_t *act, const u32 *sel, const float *wts,
                                                  const float *resid, int spt, int rpe, int t, int rb, int spt_shift = -1) {
    const int tid = threadIdx.x, q = tid & 3, quad = tid >> 2;
    BM_MARK(2048, 0);
    if constexpr (EIGHT) spt = 8, spt_shift = 3; // what the launcher has checked: constants from here on
    // (spt_shift: log2 of a power-of-two spt, else -1: the divisions by a count only known at run time are some eighty
    // instructions at the head of a workgroup whose first request waits for them)
    const int D = spt_shift >= 0 ? 64 >> spt_shift : 64 / spt;
    const int e = spt_shift >= 0 ? quad & (spt - 1) : quad % spt, dl = spt_shift >= 0 ? quad >> spt_shift : quad / spt;
    const int r = rb * D + dl;
    const int slot = t * spt + e;
    // eight slots a token: the token's ids through the scalar cache (one request a wave, a shorter way than a vector load's);
    // the lane picks its own out of the eight registers further down, behind the vector requests that do not wait for it
    constexpr bool eight = EIGHT; // (a variant of its own: a run-time choice leaves the id's register waiting for either way's load)
    u32 i8[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    u32 id = 0;
    if constexpr (eight) {
        const u32 *s8 = sel + (size_t)t * 8;
#pragma unroll
        for (int k = 0; k < 8; k++) i8[k] = s8[k];
    } else {
        id = sel[slot];
    }
    // the token's ids and weights for the closing sum, requested now and parked in LDS
    const int si = tid < spt ? tid : 0;
    const u32 my_sel = sel[t * spt + si];
    const float my_w = wts[t * spt + si];
    // the residual value of the row this thread closes, asked for now: at the end it would be a memory round trip
    const float resid_v = resid && tid < D && rb * D + tid < rpe ? resid[(size_t)t * rpe + rb * D + tid] : 0.0f;
    const int n = NB > 0 ? NB : nb;
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const uint8_t *act_cols = act + (size_t)t * spt * col_bytes;
    // the token's columns are asked for before anything waits for the expert id: they arrive with it
    Stage<5> st;
    st.load(act_cols, spt * col_bytes);
    if constexpr (eight) {
        __builtin_amdgcn_sched_barrier(0);
        const u32 a = (e & 1) ? i8[1] : i8[0], b2 = (e & 1) ? i8[3] : i8[2], c = (e & 1) ? i8[5] : i8[4], d = (e & 1) ? i8[7] : i8[6];
        const u32 ab = (e & 2) ? b2 : a, cd = (e & 2) ? d : c;
        id = (e & 4) ? cd : ab;
    }
    const bool live = id < n_experts;
    const bool active = dl < D && r < rpe && live;
    const uint8_t *wrow = w + ((size_t)(live ? id : 0) * rpe + (active ? r : 0)) * row_bytes;
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *cols = lds + tab_bytes<WT>();
    float *part = reinterpret_cast<float *>(cols + (size_t)spt * col_bytes); // [D][spt]
    float *s_w = part + D * spt;                                              // [spt]
    u32 *s_sel = reinterpret_cast<u32 *>(s_w + spt);                          // [spt]
    Blk<WT> b[U];
    BM_TICK(t_id, id);
    // behind the wait for the ids, and nothing reads them before the barrier: their way through memory runs under the columns'
    __builtin_amdgcn_sched_barrier(0);
    const DownLate late = bm_kernarg_at<DownLate>(offsetof(DownArgs, late));
    preload<WT, U>(b, wrow, q);
    BM_TICK(t_asked, tid);
    BM_TICK(t_cols, st.v[4].x);
    st.store(cols, act_cols, spt * col_bytes);
    if (tid < spt) {
        s_w[tid] = my_w;
        s_sel[tid] = my_sel;
    }
    __syncthreads();
    float *y = bm_global(late.y);
    if (!live && id != 0xffffffffu && rb == 0 && dl == 0 && q == 0) bm_raise(bm_global(late.fault), late.layer, kSiteExpertId);
    BM_MARK(2048, 1);
    BM_TOCK(2048, 4, t_id);
    BM_TOCK(2048, 5, t_asked);
    BM_TOCK(2048, 6, t_cols);
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, cols + (size_t)e * col_bytes, col_bytes, 1, n, q, tb, v, NoTap{});
    BM_MARK(2048, 2);
    if (q == 0 && dl < D) part[dl * spt + e] = v[0];
    __syncthreads();
    if (tid < D && rb * D + tid < rpe) y[(size_t)t * rpe + rb * D + tid] = slot_sum(part + tid * spt, s_w, s_sel, spt, n_experts, resid_v, resid != nullptr);
    BM_MARK(2048, 3);
}

template <int WT, int U, int NB, bool EIGHT>
__global__ __launch_bounds__(256) void k_down_combine(const uint8_t *w, u32 n_experts, int nb, const uint8_t *act,
                                                      const u32 *sel, const float *wts, const float *resid, int spt_word,
                                                      int rpe, DownLate) {
    extern __shared__ __align__(16) uint8_t lds[];
    // the grid: (row blocks of a token, tokens). spt_word: the slot count, and above bit 16 one more than its log2 where it is
    // a power of two - one word, so that both stand among the first fourteen argument words, which are in registers when the
    // wave starts (an argument behind them is a load from memory in front of the workgroup's first request)
    down_combine_body<WT, U, NB, EIGHT>(lds, w, n_experts, nb, act, sel, wts, resid, spt_word & 0xffff, rpe, (int)blockIdx.y, (int)blockIdx.x,
                                        (spt_word >> 16) - 1);
}

// k_down_combine for a Q6_K stack of NB super-blocks a row with the row's super-blocks dealt to the waves (BM_DOWN_SPLIT, the
// measured alternative: 5.6 us against the ring's 5.2 at the headline shape): a workgroup of 256 NB threads, the same 64
// (row, slot) pairs as k_down_combine's, wave w super-block w % NB of quads 16 (w / NB) .. + 16. Under the ring one wave a SIMD
// runs its loads, its wait and its arithmetic one after the other; here every super-block of every row is asked for at once by
// a wave of its own and NB waves a SIMD overlap. What it shows: the launch is bound by how fast a compute unit's address unit
// takes the quads' scattered 16-byte requests, not by waves to overlap - the twelve waves' requests queue for it, the first
// barrier (every wave's requests issued) comes 2.3 us after the start against 1.9, and the shorter arithmetic behind it (0.95
// us against 1.4) does not win that back. The numbers are the same:
// a wave leaves the operands of its super-block's multiply-adds (the f32 scale product and the integer sum as a float, two
// halves by two accumulators a lane) in LDS, and the wave of the last super-block runs the chain in the CPU path's order,
// super-block by super-block, then closes the quad as bm_quad_finish does.
template <int NB>
__global__ __launch_bounds__(256 * NB) void k_down_combine_q6k_split(const uint8_t *w, u32 n_experts, const uint8_t *act,
                                                                     const u32 *sel, const float *wts, const float *resid,
                                                                     int spt, int rpe, float *y, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int WT = BM_Q6K;
    const int tid = threadIdx.x, q = tid & 3, wave = tid >> 6;
    BM_MARK(2048, 0);
    const int i = wave % NB, quad = 16 * (wave / NB) + ((tid & 63) >> 2);
    const int D = 64 / spt;
    const int blocks_per_token = (rpe + D - 1) / D;
    const int t = blockIdx.x / blocks_per_token, rb = blockIdx.x % blocks_per_token;
    const int e = quad % spt, dl = quad / spt;
    const int r = rb * D + dl;
    const u32 id = sel[t * spt + e];
    const int si = tid < spt ? tid : 0;
    const u32 my_sel = sel[t * spt + si];
    const float my_w = wts[t * spt + si];
    const bool live = id < n_experts;
    const bool active = dl < D && r < rpe && live;
    const float resid_v = resid && tid < D && rb * D + tid < rpe ? resid[(size_t)t * rpe + rb * D + tid] : 0.0f;
    constexpr size_t row_bytes = (size_t)NB * BM_Q6K_BLOCK;
    constexpr int col_bytes = bm_act_col_bytes<WT>(NB);
    const uint8_t *act_cols = act + (size_t)t * spt * col_bytes;
    Stage<2, 256 * NB> st; // 16 bytes a thread of 768: the eight columns of 1248 bytes
    st.load(act_cols, spt * col_bytes);
    if (!live && id != 0xffffffffu && rb == 0 && dl == 0 && q == 0 && i == 0) bm_raise(fault, layer, kSiteExpertId);
    const uint8_t *wrow = w + ((size_t)(live ? id : 0) * rpe + (active ? r : 0)) * row_bytes;
    uint8_t *cols = lds;
    float *terms = reinterpret_cast<float *>(cols + (size_t)spt * col_bytes); // [64 quads][NB - 1][4 lanes][8]
    float *part = terms + 64 * (NB - 1) * 32;                                  // [D][spt]
    float *s_w = part + D * spt;                                               // [spt]
    u32 *s_sel = reinterpret_cast<u32 *>(s_w + spt);                           // [spt]
    BM_TICK(t_id, id);
    const Blk<WT> b = bm_load_blk<WT>(wrow, i, q);
    BM_TICK(t_asked, tid);
    st.store(cols, act_cols, spt * col_bytes);
    if (tid < spt) {
        s_w[tid] = my_w;
        s_sel[tid] = my_sel;
    }
    __syncthreads();
    BM_MARK(2048, 1);
    BM_TOCK(2048, 4, t_id);
    BM_TOCK(2048, 5, t_asked);
    const int c = q & 1, h = q >> 1;
    const Act<WT> a = bm_act_q6k(bm_act_view<WT>(cols + (size_t)e * col_bytes, NB), i, c, h);
    float p[4], s[4]; // (half 0: accumulator 0, accumulator 1), (half 1: ...)
    bm_q6k_terms(b, a, c, h, p, s);
    BM_TICK(t_terms, p[3]);
    float *mine = terms + ((size_t)(quad * (NB - 1) + i) * 4 + q) * 8;
    if (i < NB - 1) {
        *reinterpret_cast<float4 *>(mine) = make_float4(p[0], s[0], p[1], s[1]);
        *reinterpret_cast<float4 *>(mine + 4) = make_float4(p[2], s[2], p[3], s[3]);
    }
    __syncthreads();
    BM_MARK(2048, 2);
    BM_TOCK(2048, 6, t_terms);
    if (i == NB - 1) {
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int u = 0; u < NB - 1; u++) {
            const float *o = terms + ((size_t)(quad * (NB - 1) + u) * 4 + q) * 8;
            const float4 lo = *reinterpret_cast<const float4 *>(o), hi = *reinterpret_cast<const float4 *>(o + 4);
            a0 = fmaf(lo.x, lo.y, a0), a1 = fmaf(lo.z, lo.w, a1);
            a0 = fmaf(hi.x, hi.y, a0), a1 = fmaf(hi.z, hi.w, a1);
        }
        a0 = fmaf(p[0], s[0], a0), a1 = fmaf(p[1], s[1], a1);
        a0 = fmaf(p[2], s[2], a0), a1 = fmaf(p[3], s[3], a1);
        const float v = bm_quad_finish<WT>(a0, a1);
        if (q == 0 && dl < D) part[dl * spt + e] = v;
    }
    __syncthreads();
    if (tid < D && rb * D + tid < rpe) y[(size_t)t * rpe + rb * D + tid] = slot_sum(part + tid * spt, s_w, s_sel, spt, n_experts, resid_v, resid != nullptr);
    BM_MARK(2048, 3);
}

// The gate . up . SwiGLU workgroup of the fused step: as k_gate_up's, except that it quantizes its token's f32 row
// itself (into LDS; no quantizer launch, no activation column in memory) and always writes its q8_2 block of the
// slot's down activation.
template <int WA, int UA, int NBA>
__device__ __forceinline__ void gate_up_x_body(uint8_t *lds, const float *x, const uint8_t *wg, const uint8_t *wu,
                                               u32 n_experts, int na, int nh, const u32 *sel, int spt, int slot, int rb, int t) {
    const int tid = threadIdx.x, q = tid & 3, which = (tid >> 2) & 1;
    BM_MARK(0, 0);
    const int hidden = na * 256, ff = nh * 256;
    const int r = rb * 32 + (tid >> 3);
    const u32 id = sel[slot];
    const int col_bytes = bm_act_col_bytes<WA>(na);
    uint8_t *col = lds;
    // the token's row: eight consecutive values a lane, 2048 a pass. Asked for before anything reads an argument that is
    // not in a register when the wave starts (the first thirteen words are): scalar loads come back in any order, so the
    // first wait for one of them is a wait for the expert id as well, and the row's loads would stand behind it
    constexpr int kPasses = NBA > 0 ? (NBA * 256 + 2047) / 2048 : 1;
    float xv[kPasses][8];
#pragma unroll
    for (int p = 0; p < kPasses; p++) {
        int o = p * 2048 + tid * 8;
        o = o < hidden ? o : hidden - 8;
        const float4 lo = *reinterpret_cast<const float4 *>(x + (size_t)t * hidden + o);
        const float4 hi = *reinterpret_cast<const float4 *>(x + (size_t)t * hidden + o + 4);
        xv[p][0] = lo.x, xv[p][1] = lo.y, xv[p][2] = lo.z, xv[p][3] = lo.w;
        xv[p][4] = hi.x, xv[p][5] = hi.y, xv[p][6] = hi.z, xv[p][7] = hi.w;
    }
    __asm__ volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    if (id >= n_experts) { // uniform over the workgroup
        if (id == 0xffffffffu) return; // a slot served elsewhere: nothing written, nothing raised
        const GateUpLate late = bm_kernarg_at<GateUpLate>(offsetof(GateUpArgs, late));
        if (tid == 0) bm_raise(bm_global(late.fault), late.layer, kSiteExpertId);
        if (late.h && (tid & 7) == 0) bm_global(late.h)[(size_t)slot * ff + r] = bm_bits_f32(0x7fc00000u);
        if (late.act_h && tid < 32)
            q82_store(bm_global(late.act_h) + (size_t)slot * nh * BM_Q82_SB_EXT, nh, rb, tid, 0, Q82Head{0x7fc0u, 0, true}, 0);
        return;
    }
    BM_MARK(0, 1);
    const size_t row_bytes = (size_t)na * bm_block_bytes<WA>();
    const uint8_t *wrow = (which ? wu : wg) + ((size_t)id * ff + r) * row_bytes;
    Blk<WA> b[UA];
    // behind the wait for the id, and nothing reads them before the token's column stands in LDS: their way through memory runs
    // under the quantizer's work
    const GateUpLate late = bm_kernarg_at<GateUpLate>(offsetof(GateUpArgs, late));
    preload<WA, UA>(b, wrow, q);
    bool bad = false;
#pragma unroll
    for (int p = 0; p < kPasses; p++) {
        const int o = p * 2048 + tid * 8;
        if (o < hidden) bad |= q82_quad8<false>(xv[p], col, na, o >> 5, tid & 3, nullptr, 0);
    }
    if constexpr (NBA == 0) { // longer rows: the passes past the first, straight from memory
        for (int o = 2048 + tid * 8; o < hidden; o += 2048) {
            float v8[8];
            for (int k = 0; k < 8; k++) v8[k] = x[(size_t)t * hidden + o + k];
            bad |= q82_quad8<false>(v8, col, na, o >> 5, tid & 3, nullptr, 0);
        }
    }
    __syncthreads();
    uint8_t *const act_x = bm_global(late.act_x), *const act_h = bm_global(late.act_h);
    float *const h = bm_global(late.h);
    const GateRule rule = late.rule;
    u32 *const fault = bm_global(late.fault);
    const u32 layer = late.layer;
    uint8_t *hcol = act_h ? act_h + (size_t)slot * nh * BM_Q82_SB_EXT : nullptr; // none: the down stack takes Q8_K columns
    if (bad && (tid & 3) == 0) bm_raise(fault, layer, kSiteQuantColumn);
    if (act_x && rb == 0 && slot % spt == 0) stage_bytes(act_x + (size_t)t * col_bytes, col, col_bytes);
    BM_MARK(0, 2);
    float v[1];
    row_dot<WA, UA, NBA, 1>(b, wrow, col, col_bytes, 1, na, q, Iq2Tables{}, v, NoTap{});
    BM_MARK(0, 3);
    const float hv = swiglu_of_pair(v[0], which, rule, fault, layer);
    if (h && (tid & 7) == 0) h[(size_t)slot * ff + r] = hv;
    if (!hcol) return;
    float *hbuf = reinterpret_cast<float *>(col + col_bytes);
    if ((tid & 7) == 0) hbuf[tid >> 3] = hv;
    __syncthreads();
    if (tid < 32) quantize_h_block(hbuf, hcol, nh, rb, tid, fault, layer);
    BM_MARK(0, 4);
}

// The first half of the fused step as a launch of its own: x -> quantized h, slot by slot.
template <int WA, int UA, int NBA>
__global__ __launch_bounds__(256) void k_gate_up_x(const float *x, const uint8_t *wg, const uint8_t *wu, u32 n_experts,
                                                   int nba, int nh, const u32 *sel, int spt, GateUpLate) {
    extern __shared__ __align__(16) uint8_t lds[];
    // the grid: (blocks of 32 rows, slots of a token, tokens): no division stands before the workgroup's first request (and no
    // read of the grid's size, which comes from the dispatch packet in memory: spt is an argument, in a register at the start)
    gate_up_x_body<WA, UA, NBA>(lds, x, wg, wu, n_experts, NBA > 0 ? NBA : nba, nh, sel, spt,
                                (int)blockIdx.z * spt + (int)blockIdx.y, (int)blockIdx.x, (int)blockIdx.z);
}

// ------------------------------------------------------------- the fused step for the types that take Q8_K columns

// `cols` columns of nb blocks each, f32 rows at x (column c at x + c * nb * 256), into LDS at `dst` by the workgroup's
// waves, block by block.
__device__ __forceinline__ void q8k_stage_cols(const float *x, uint8_t *dst, int cols, int nb, u32 *fault, u32 layer,
                                               const u32 *ids = nullptr, u32 n_experts = 0) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = 4; // (256 threads: every caller's workgroup)
    const int total = cols * nb;
    constexpr int kAhead = 6; // blocks whose loads a wave has in flight
    for (int b0 = wave; b0 < total; b0 += kAhead * n_waves) {
        float4 x4[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; u++) {
            const int b = b0 + u * n_waves;
            x4[u] = *reinterpret_cast<const float4 *>(x + (size_t)(b < total ? b : b0) * 256 + 4 * lane);
        }
#pragma unroll
        for (int u = 0; u < kAhead; u++) {
            const int b = b0 + u * n_waves;
            // with ids: a column whose slot is not live is not encoded (its rows may hold anything)
            if (b < total && (!ids || ids[b / nb] < n_experts)) q8k_wave_block(x4[u], dst + (size_t)b * BM_Q8K_STRIDE, lane, fault, layer);
        }
    }
}

// `cols` columns of nb super-blocks each, f32 rows at x (column c at x + c * nb * 256), into LDS at `dst` as Q8_2_X4
// columns with their tables: a 32-value block is four consecutive lanes of eight values. In two steps, for a workgroup
// that has something else to request in between: the f32 values of the
// first R tasks a thread are requested at once (memory answers in order, so they are back before anything asked for
// after them), and encoded into LDS later, when those other requests are on their way; tasks past the first R a thread
// go through the plain loop afterwards.
// T: the workgroup's thread count, a constant here: the built-in is read from memory, and a read after the weight
// requests would wait for all of them.
template <int R, int T>
struct Q82Cols {
    float4 lo[R], hi[R];
    u32 id[R]; // the expert of a task's column: a column whose slot is not live is not encoded (its rows may hold anything)
    __device__ __forceinline__ void load(const float *x, int total, int per_col, const u32 *ids) {
#pragma unroll
        for (int u = 0; u < R; u++) {
            int task = (int)threadIdx.x + u * T;
            task = task < total ? task : total - 1; // a read that stays inside the token's rows; the value is not used
            const float *p = x + (size_t)task * 8;
            lo[u] = *reinterpret_cast<const float4 *>(p);
            hi[u] = *reinterpret_cast<const float4 *>(p + 4);
            id[u] = ids[task / per_col];
        }
        __asm__ volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    __device__ __forceinline__ void encode(const float *x, uint8_t *dst, int cols, int nb, const u32 *ids, u32 n_experts,
                                           u32 *fault, u32 layer) const {
        const int per_col = nb * 32, total = cols * per_col, col_bytes = nb * BM_Q82_SB_EXT;
#pragma unroll
        for (int u = 0; u < R; u++) {
            const int task = (int)threadIdx.x + u * T;
            if (task < total && id[u] < n_experts) { // whole quads: the tasks of a block are four neighbours
                const int c = task / per_col, at = task % per_col;
                const float v8[8] = {lo[u].x, lo[u].y, lo[u].z, lo[u].w, hi[u].x, hi[u].y, hi[u].z, hi[u].w};
                q82_quad8(v8, dst + (size_t)c * col_bytes, nb, at >> 2, task & 3, fault, layer);
            }
        }
        for (int task = (int)threadIdx.x + R * T; task < total; task += T) {
            const int c = task / per_col, at = task % per_col;
            if (ids[c] >= n_experts) continue;
            const float *p = x + (size_t)task * 8;
            const float4 l4 = *reinterpret_cast<const float4 *>(p), h4 = *reinterpret_cast<const float4 *>(p + 4);
            const float v8[8] = {l4.x, l4.y, l4.z, l4.w, h4.x, h4.y, h4.z, h4.w};
            q82_quad8(v8, dst + (size_t)c * col_bytes, nb, at >> 2, task & 3, fault, layer);
        }
    }
};

// k_gate_up_x for gate / up stacks that dot against Q8_K columns (Q3_K, IQ2_XXS, IQ3_XXS, IQ4_XS): the token's row is
// quantized by every workgroup into LDS, h is written as f32 rows, and where the down stack takes Q8_2_X4 columns
// (act_h given) the workgroup's 32 values also become their block of the slot's column.
template <int WA, int UA, int NBA>
__global__ __launch_bounds__(256) void k_gate_up_xq(const float *x, const uint8_t *wg, const uint8_t *wu, u32 n_experts,
                                                    int nba, int nh, const u32 *sel, int spt, uint8_t *act_x,
                                                    uint8_t *act_h, float *h, GateRule rule, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3, which = (tid >> 2) & 1;
    const int blocks_per_slot = nh * 8;
    const int slot = blockIdx.x / blocks_per_slot, rb = blockIdx.x % blocks_per_slot;
    const int na = NBA > 0 ? NBA : nba;
    const int hidden = na * 256, ff = nh * 256;
    const int t = slot / spt;
    const int r = rb * 32 + (tid >> 3);
    const u32 id = sel[slot];
    uint8_t *hcol = act_h ? act_h + (size_t)slot * nh * BM_Q82_SB_EXT : nullptr;
    if (id >= n_experts) { // uniform over the workgroup
        if (id == 0xffffffffu) return; // a slot served elsewhere: nothing written, nothing raised
        if (tid == 0) bm_raise(fault, layer, kSiteExpertId);
        if (h && (tid & 7) == 0) h[(size_t)slot * ff + r] = bm_bits_f32(0x7fc00000u);
        if (hcol && tid < 32) q82_store(hcol, nh, rb, tid, 0, Q82Head{0x7fc0u, 0, true}, 0);
        return;
    }
    const size_t row_bytes = (size_t)na * bm_block_bytes<WA>();
    const uint8_t *wrow = (which ? wu : wg) + ((size_t)id * ff + r) * row_bytes;
    Blk<WA> b[UA];
    preload<WA, UA>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WA>(lds);
    uint8_t *col = lds + tab_bytes<WA>();
    const int col_bytes = bm_act_col_bytes<WA>(na);
    q8k_stage_cols(x + (size_t)t * hidden, col, 1, na, fault, layer);
    __syncthreads();
    if (act_x && rb == 0 && slot % spt == 0) stage_bytes(act_x + (size_t)t * col_bytes, col, col_bytes);
    float v[1];
    row_dot<WA, UA, NBA, 1>(b, wrow, col, col_bytes, 1, na, q, tb, v, NoTap{});
    const float hv = swiglu_of_pair(v[0], which, rule, fault, layer);
    if (h && (tid & 7) == 0) h[(size_t)slot * ff + r] = hv;
    if (hcol) {
        float *hbuf = reinterpret_cast<float *>(col + col_bytes);
        if ((tid & 7) == 0) hbuf[tid >> 3] = hv;
        __syncthreads();
        if (tid < 32) quantize_h_block(hbuf, hcol, nh, rb, tid, fault, layer);
    }
}

// (Workgroups of 64 or 128 threads, as k_gemv takes for a matrix of few rows, measure slower here: 4.35 and 3.89 us against
// 3.55 at 768 x 2048 - a wave then quantizes four or two times as much of the column before its first product.)
// k_gemv with the activation quantizer folded in: grid row c is column c, an f32 row of k values that every workgroup
// quantizes into LDS for itself (the form its weight type dots against), so a matrix-vector product from f32 is one
// launch and no column passes through memory. With act_out the first workgroup of a column leaves its bytes there.
template <int WT, int U, int NB>
__global__ __launch_bounds__(256) void k_gemv_x(const float *x, const uint8_t *w, long rows, int nb, int m, uint8_t *act_out,
                                                float *y, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3, c = blockIdx.y;
    const long row = (long)blockIdx.x * 64 + (tid >> 2);
    const bool active = row < rows;
    const int n = NB > 0 ? NB : nb;
    const int k = n * 256;
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const uint8_t *wrow = w + (size_t)(active ? row : 0) * row_bytes;
    const float *xc = x + (size_t)c * k;
    // the column's first 2048 values are asked for in front of the rows: vector loads come back in the order they were asked
    // for, and behind the rows' requests the quantizer would wait for those as well
    float4 x_lo = make_float4(0, 0, 0, 0), x_hi = x_lo;
    if constexpr (!bm_takes_q8k(WT)) {
        const int o = tid * 8 < k ? tid * 8 : k - 8;
        x_lo = *reinterpret_cast<const float4 *>(xc + o), x_hi = *reinterpret_cast<const float4 *>(xc + o + 4);
        __asm__ volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *col = lds + tab_bytes<WT>();
    if constexpr (bm_takes_q8k(WT)) {
        q8k_stage_cols(xc, col, 1, n, fault, layer);
    } else { // a q8_2 block is four lanes of eight values; 2048 values a pass
        if (tid * 8 < k) {
            const float v8[8] = {x_lo.x, x_lo.y, x_lo.z, x_lo.w, x_hi.x, x_hi.y, x_hi.z, x_hi.w};
            q82_quad8(v8, col, n, tid >> 2, tid & 3, fault, layer);
        }
        for (int o = 2048 + tid * 8; o < k; o += 2048) {
            const float4 lo = *reinterpret_cast<const float4 *>(xc + o), hi = *reinterpret_cast<const float4 *>(xc + o + 4);
            float v8[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            q82_quad8(v8, col, n, o >> 5, tid & 3, fault, layer);
        }
    }
    __syncthreads();
    if (act_out && blockIdx.x == 0) stage_bytes(act_out + (size_t)c * col_bytes, col, col_bytes);
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, col, col_bytes, 1, n, q, tb, v, NoTap{});
    if (q == 0 && active) y[(size_t)row * m + c] = v[0];
}

// k_down_combine for down stacks that dot against Q8_K columns: the token's slot rows of h (f32) are quantized by
// every workgroup into LDS; the first workgroup of a token also leaves the columns in act_h.
template <int WT, int U, int NB>
__global__ __launch_bounds__(256) void k_down_combine_hq(const uint8_t *w, u32 n_experts, int nb, const float *h,
                                                         uint8_t *act_h, const u32 *sel, const float *wts,
                                                         const float *resid, int spt, int rpe, float *y, u32 *fault,
                                                         u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3, quad = tid >> 2;
    const int D = 64 / spt;
    const int blocks_per_token = (rpe + D - 1) / D;
    const int t = blockIdx.x / blocks_per_token, rb = blockIdx.x % blocks_per_token;
    const int e = quad % spt, dl = quad / spt;
    const int r = rb * D + dl;
    const int n = NB > 0 ? NB : nb;
    const u32 id = sel[t * spt + e];
    // Q8_2_X4 columns: the token's f32 rows of h are asked for before anything that waits for the expert id, so they
    // arrive with it and are encoded while the weight rows are on their way
    Q82Cols<4, 256> hrows;
    if constexpr (!bm_takes_q8k(WT)) hrows.load(h + (size_t)t * spt * n * 256, spt * n * 32, n * 32, sel + t * spt);
    const int si = tid < spt ? tid : 0;
    const u32 my_sel = sel[t * spt + si];
    const float my_w = wts[t * spt + si];
    const bool live = id < n_experts;
    const bool active = dl < D && r < rpe && live;
    const float resid_v = resid && tid < D && rb * D + tid < rpe ? resid[(size_t)t * rpe + rb * D + tid] : 0.0f;
    if (!live && id != 0xffffffffu && rb == 0 && dl == 0 && q == 0) bm_raise(fault, layer, kSiteExpertId);
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const uint8_t *wrow = w + ((size_t)(live ? id : 0) * rpe + (active ? r : 0)) * row_bytes;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *cols = lds + tab_bytes<WT>();
    float *part = reinterpret_cast<float *>(cols + (size_t)spt * col_bytes); // [D][spt]
    float *s_w = part + D * spt;                                              // [spt]
    u32 *s_sel = reinterpret_cast<u32 *>(s_w + spt);                          // [spt]
    if constexpr (bm_takes_q8k(WT)) q8k_stage_cols(h + (size_t)t * spt * n * 256, cols, spt, n, fault, layer, sel + t * spt, n_experts);
    else hrows.encode(h + (size_t)t * spt * n * 256, cols, spt, n, sel + t * spt, n_experts, fault, layer);
    if (tid < spt) {
        s_w[tid] = my_w;
        s_sel[tid] = my_sel;
    }
    __syncthreads();
    if (act_h && rb == 0) // the live slots' columns; the others keep what they held
        for (int c = 0; c < spt; c++)
            if (s_sel[c] < n_experts) stage_bytes(act_h + ((size_t)t * spt + c) * col_bytes, cols + (size_t)c * col_bytes, col_bytes);
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, cols + (size_t)e * col_bytes, col_bytes, 1, n, q, tb, v, NoTap{});
    if (q == 0 && dl < D) part[dl * spt + e] = v[0];
    __syncthreads();
    if (tid < D && rb * D + tid < rpe) y[(size_t)t * rpe + rb * D + tid] = slot_sum(part + tid * spt, s_w, s_sel, spt, n_experts, resid_v, resid != nullptr);
}

// ------------------------------------------------------------------------------------------ verification

struct StoreTap {
    static constexpr bool kActive = true;
    int *out; // 16 words a super-block, zeroed before the quad runs
    __device__ __forceinline__ void q4k(int i, int s, int, int v) const { atomicAdd(&out[16 * i + s], v); }
    __device__ __forceinline__ void q4k_isum(int i, int s, int v) const { out[16 * i + 8 + s] = v; }
    __device__ __forceinline__ void q6k(int i, int g, int v) const { out[16 * i + g] = v; }
    __device__ __forceinline__ void iq2(int i, int b, int q, int v) const {
        atomicAdd(&out[16 * i + b], v);
        (void)q;
    }
    __device__ __forceinline__ void iq4_sub(int i, int b, int v) const { out[16 * i + b] = v; }
    __device__ __forceinline__ void iq4_lane(int i, int l, int v) const { out[16 * i + 8 + l] = v; }
};

template <int WT, int U, int NB>
__global__ __launch_bounds__(64) void k_block_sums(const uint8_t *wrow, int nb, const uint8_t *act_col, int *out) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3;
    const int n = NB > 0 ? NB : nb;
    const int col_bytes = bm_act_col_bytes<WT>(n);
    for (int i = tid; i < 16 * n; i += 64) out[i] = 0;
    const Iq2Tables tb = stage_tables<WT, 64>(lds);
    uint8_t *col = lds + tab_bytes<WT>();
    stage_bytes<64>(col, act_col, col_bytes);
    __threadfence();
    __syncthreads();
    if (tid >= 4) return;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, col, col_bytes, 1, n, q, tb, v, StoreTap{out});
    if constexpr (WT == BM_IQ2XXS || WT == BM_IQ3XXS) {
        // the eight scales 2s + 1 of each super-block, as the dot reads them
        if (q == 0)
            for (int i = 0; i < n; i++)
                for (int s = 0; s < 8; s++) {
                    u32 aux;
                    if constexpr (WT == BM_IQ2XXS)
                        __builtin_memcpy(&aux, wrow + (size_t)i * BM_IQ2XXS_BLOCK + 6 + 8 * s, 4);
                    else
                        __builtin_memcpy(&aux, wrow + (size_t)i * BM_IQ3XXS_BLOCK + 66 + 4 * s, 4);
                    out[16 * i + 8 + s] = 2 * (int)(aux >> 28) + 1;
                }
    }
}

// ---------------------------------------------------------------------------------------- launch helpers

constexpr unsigned kCardUnits = 256; // compute units of the card these kernels are written for

int act_col_bytes(int wtype, int k) {
    const int nb = k / 256;
    return bm_takes_q8k(wtype) ? nb * BM_Q8K_STRIDE : nb * BM_Q82_SB_EXT;
}

int gemv_max_cols(int wtype, int k) {
    int m = (kMaxLds - tab_bytes_rt(wtype)) / act_col_bytes(wtype, k);
    return m > 8 ? 8 : m;
}

hipError_t gemv(const Launch &L, int wtype, const uint8_t *w, int64_t rows, int k, const uint8_t *act, int m_total,
                int col0, int m, float *y) {
    const int nb = k / 256;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)m * act_col_bytes(wtype, k);
    const bool few = m == 1 && (rows + 63) / 64 < (int64_t)kCardUnits; // one column of a matrix whose 64-row blocks do not fill the card
#define CALL_BODY                                                                                                      \
    if (few) {                                                                                                         \
        auto kern = k_gemv<WT, U, NB, 1, 64>;                                                                          \
        hipError_t e = allow_lds(kern, lds);                                                                           \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3((unsigned)((rows + 15) / 16)), dim3(64), lds, L.stream, w, (long)rows, nb, act,  \
                           m_total, col0, m, y);                                                                       \
    } else {                                                                                                           \
        auto kern = m == 1 ? k_gemv<WT, U, NB, 1> : k_gemv<WT, U, NB, 8>;                                              \
        hipError_t e = allow_lds(kern, lds);                                                                           \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3((unsigned)((rows + 63) / 64)), dim3(256), lds, L.stream, w, (long)rows, nb, act, \
                           m_total, col0, m, y);                                                                       \
    }
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

size_t gemv_x_lds(int wtype, int k) { return tab_bytes_rt(wtype) + (size_t)act_col_bytes(wtype, k); }

hipError_t gemv_x(const Launch &L, int wtype, const uint8_t *w, int64_t rows, int k, const float *x, int m, uint8_t *act_out,
                  float *y) {
    const int nb = k / 256;
    const size_t lds = gemv_x_lds(wtype, k);
#define CALL_BODY                                                                                                      \
    auto kern = k_gemv_x<WT, U, NB>;                                                                                   \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3((unsigned)((rows + 63) / 64), (unsigned)m), dim3(256), lds, L.stream, x, w,          \
                       (long)rows, nb, m, act_out, y, L.fault, L.layer);
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

hipError_t gate_up(const Launch &L, int wtype, const uint8_t *wg, const uint8_t *wu, int n_experts, int k,
                   const uint8_t *act, const uint32_t *sel, int n_slots, int rows_per_expert, int slots_per_col,
                   float *h, uint8_t *act_h) {
    const int nb = k / 256, rpe = rows_per_expert;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)act_col_bytes(wtype, k) + 32 * sizeof(float);
    if (n_slots <= 0 || slots_per_col <= 0) return hipErrorInvalidValue;
    if (slots_per_col > 0xffffff) { // (more slots a column than there are slots: column 0 either way)
        if (n_slots > 0xffffff) return hipErrorInvalidValue;
        slots_per_col = 0xffffff;
    }
    const unsigned grid_y = (unsigned)n_slots < kGateUpGridY ? (unsigned)n_slots : kGateUpGridY;
    const unsigned grid_z = ((unsigned)n_slots + kGateUpGridY - 1) / kGateUpGridY;
    const int spc_shift = (slots_per_col & (slots_per_col - 1)) == 0 ? __builtin_ctz((unsigned)slots_per_col) : -1;
#define CALL_BODY                                                                                                      \
    auto kern = k_gate_up<WT, U, NB>;                                                                                  \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3((unsigned)((rpe + 31) / 32), grid_y, grid_z), dim3(256), lds, L.stream, wg, wu, (u32)n_experts, nb, \
                       act, sel, rpe, slots_per_col | ((spc_shift + 1) << 24), (u32)n_slots,                           \
                       GateUpColLate{h, act_h, L.rule, L.fault, L.layer});
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

hipError_t gemv_sel(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                    const uint32_t *sel, int n_slots, int rows_per_expert, float *y) {
    const int nb = k / 256, rpe = rows_per_expert;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)act_col_bytes(wtype, k);
    const unsigned grid = (unsigned)n_slots * (unsigned)((rpe + 63) / 64);
#define CALL_BODY                                                                                                      \
    auto kern = k_gemv_sel<WT, U, NB>;                                                                                 \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, w, (u32)n_experts, nb, act, sel, rpe, y, L.fault,   \
                       L.layer);
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

size_t down_combine_lds(int wtype, int k, int spt) {
    const int D = 64 / spt;
    return tab_bytes_rt(wtype) + (size_t)spt * act_col_bytes(wtype, k) + ((size_t)D * spt + 2 * (size_t)spt) * sizeof(float);
}

hipError_t down_combine(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                        const uint32_t *sel, const float *wts, const float *resid, int slots_per_token, int m,
                        int rows_per_expert, float *y) {
    const int nb = k / 256, rpe = rows_per_expert, spt = slots_per_token;
    const int D = 64 / spt;
    const int spt_shift = (spt & (spt - 1)) == 0 ? __builtin_ctz((unsigned)spt) : -1;
    const size_t lds = down_combine_lds(wtype, k, spt);
    const unsigned grid = (unsigned)m * (unsigned)((rpe + D - 1) / D);
    if (L.down_form == 1 && wtype == BM_Q6K && nb == 3 && 64 % spt == 0) { // BM_DOWN_SPLIT where it is built: the super-blocks of a row dealt to the waves
        constexpr int NB = 3;
        const size_t lds_split = (size_t)spt * bm_act_col_bytes<BM_Q6K>(NB) + (64 * (NB - 1) * 32 + D * spt + 2 * spt) * sizeof(float);
        hipLaunchKernelGGL(k_down_combine_q6k_split<NB>, dim3(grid), dim3(256 * NB), lds_split, L.stream, w, (u32)n_experts, act, sel, wts,
                           resid, spt, rpe, y, L.fault, L.layer);
        return hipGetLastError();
    }
#define BM_DOWN_LAUNCH(EIGHT)                                                                                          \
    {                                                                                                                  \
        auto kern = k_down_combine<WT, U, NB, EIGHT>;                                                                  \
        hipError_t e = allow_lds(kern, lds);                                                                           \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3((unsigned)((rpe + D - 1) / D), (unsigned)m), dim3(256), lds, L.stream, w, (u32)n_experts, nb,    \
                           act, sel, wts, resid, spt | ((spt_shift + 1) << 16), rpe, DownLate{y, L.fault, L.layer});   \
    }
    // (eight slots a token: the form that takes the token's ids through the scalar cache)
#define CALL_BODY                                                                                                      \
    if (spt == 8) BM_DOWN_LAUNCH(true) else BM_DOWN_LAUNCH(false)
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
#undef BM_DOWN_LAUNCH
    return hipGetLastError();
}

static bool tab_known(int t) {
    return t == BM_Q3K || t == BM_Q4K || t == BM_Q5K || t == BM_Q6K || t == BM_IQ2XXS || t == BM_IQ3XXS || t == BM_IQ4XS;
}

// every type this library has a row dot for goes on either side of the fused step
bool moe_decode_supported(int gate_type, int down_type) { return tab_known(gate_type) && tab_known(down_type); }

hipError_t gate_up_x(const Launch &L, int gate_type, const float *x, const uint8_t *wg, const uint8_t *wu,
                     int n_experts, int hidden, int ff, const uint32_t *sel, int slots_per_token, int m,
                     uint8_t *act_x, uint8_t *act_h, float *h) {
    const int nba = hidden / 256, nbb = ff / 256, spt = slots_per_token;
    const size_t lds_a = (size_t)act_col_bytes(gate_type, hidden) + 32 * sizeof(float);
    const unsigned grid_a = (unsigned)m * (unsigned)spt * (unsigned)(ff / 32);
#define BM_GUX(WA, UA, NA)                                                                                             \
    {                                                                                                                  \
        auto kern = k_gate_up_x<WA, UA, NA>;                                                                           \
        hipError_t e = allow_lds(kern, lds_a);                                                                         \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3((unsigned)(ff / 32), (unsigned)spt, (unsigned)m), dim3(256), lds_a, L.stream, x, wg, wu,          \
                           (u32)n_experts, nba, nbb, sel, spt, GateUpLate{act_x, act_h, h, L.rule, L.fault, L.layer});                    \
    }
    if (gate_type == BM_Q4K) {
        if (nba == 8) BM_GUX(BM_Q4K, kRingQ4K, 8)
        else BM_GUX(BM_Q4K, 1, 0)
    } else if (gate_type == BM_Q5K) {
        if (nba == 8) BM_GUX(BM_Q5K, kRingQ5K, 8)
        else BM_GUX(BM_Q5K, 1, 0)
    } else if (gate_type == BM_Q6K) {
        if (nba % 2 == 0) BM_GUX(BM_Q6K, 2, 0)
        else BM_GUX(BM_Q6K, 1, 0)
    } else if (bm_takes_q8k(gate_type)) {
        const int nb = nba;
        const size_t lds_q = tab_bytes_rt(gate_type) + (size_t)act_col_bytes(gate_type, hidden) + 32 * sizeof(float);
#define CALL_BODY                                                                                                      \
    auto kern = k_gate_up_xq<WT, U, NB>;                                                                               \
    hipError_t e = allow_lds(kern, lds_q);                                                                             \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3(grid_a), dim3(256), lds_q, L.stream, x, wg, wu, (u32)n_experts, nba, nbb, sel, spt,  \
                       act_x, act_h, h, L.rule, L.fault, L.layer);
        BM_DISPATCH(gate_type, nb)
#undef CALL_BODY
    } else {
        return hipErrorInvalidValue;
    }
#undef BM_GUX
    return hipGetLastError();
}

// Down + combine from the f32 rows of h, for a down stack that takes Q8_K columns; act_h (optional) receives them.
hipError_t down_combine_hq(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const float *h,
                           uint8_t *act_h, const uint32_t *sel, const float *wts, const float *resid,
                           int slots_per_token, int m, int rows_per_expert, float *y) {
    const int nb = k / 256, rpe = rows_per_expert, spt = slots_per_token;
    const int D = 64 / spt;
    const size_t lds = down_combine_lds(wtype, k, spt);
    const unsigned grid = (unsigned)m * (unsigned)((rpe + D - 1) / D);
#define CALL_BODY                                                                                                      \
    auto kern = k_down_combine_hq<WT, U, NB>;                                                                          \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, w, (u32)n_experts, nb, h, act_h, sel, wts, resid,   \
                       spt, rpe, y, L.fault, L.layer);
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

hipError_t moe_decode(const Launch &L, int gate_type, int down_type, const float *x, const uint8_t *wg, const uint8_t *wu,
                      const uint8_t *wd, int n_experts, int hidden, int ff, const uint32_t *sel, const float *wts,
                      const float *resid, int slots_per_token, int m, uint8_t *act_x, uint8_t *act_h, float *h, float *y) {
    const int spt = slots_per_token;
    if (!moe_decode_supported(gate_type, down_type)) return hipErrorInvalidValue;
    // a down stack on Q8_K columns cannot get them from the gate . up launch (a column's block spans eight of
    // its workgroups): that launch leaves h as f32 rows and the down launch quantizes them itself
    // (for a down stack on Q8_2_X4 columns the same split measures slower, 12.2 us a token against 11.3 at the
    // Qwen3 shape: the gate . up launch loses its quantizer epilogue, 0.5 us, but every down workgroup then encodes
    // the token's 6144 values, 700 instructions a wave that do not hide behind its weight stream)
    const bool hq = bm_takes_q8k(down_type);
    hipError_t e = gate_up_x(L, gate_type, x, wg, wu, n_experts, hidden, ff, sel, spt, m, act_x, hq ? nullptr : act_h, h);
    if (e != hipSuccess) return e;
    if (hq) return down_combine_hq(L, down_type, wd, n_experts, ff, h, act_h, sel, wts, resid, spt, m, hidden, y);
    return down_combine(L, down_type, wd, n_experts, ff, act_h, sel, wts, resid, spt, m, hidden, y);
}

// --------------------------------------------------------------- the fused step on scratch the library holds

// What bm_moe_decode takes from its caller as act_h (and h, for a down stack on Q8_K columns), held here instead: one
// array a device for as long as the process lives, so the entry that uses it calls no allocator. Room for
// kStaticValues values of h (slots x ff): their activation columns in the wider of the two column forms first, their
// f32 rows after them.
constexpr size_t kStaticColBytes = kStaticValues / 256 * BM_Q82_SB_EXT; // Q8_K columns (296 a super-block) fit too
constexpr size_t kStaticBytes = kStaticColBytes + kStaticValues * sizeof(float);
static __device__ __align__(256) uint8_t scratch[kStaticBytes];

// The array's address on each device. Host code may not hand the symbol itself to a kernel (on the host it names a
// stand-in, not device memory): the address is asked for once a device, with that device current, and every launch
// takes it from here.
constexpr int kStaticMaxDevices = 64;
static std::atomic<uint8_t *> g_scratch_at[kStaticMaxDevices]; // contexts may be made from several threads at once

hipError_t static_scratch_init(int device) {
    if (device < 0 || device >= kStaticMaxDevices) return hipErrorInvalidDevice;
    if (g_scratch_at[device].load(std::memory_order_acquire)) return hipSuccess;
    void *at = nullptr;
    const hipError_t e = hipGetSymbolAddress(&at, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!at) return hipErrorInvalidSymbol;
    g_scratch_at[device].store(static_cast<uint8_t *>(at), std::memory_order_release); // every thread finds the same address
    return hipSuccess;
}

hipError_t moe_decode_static(const Launch &L, int device, int gate_type, int down_type, const float *x, const uint8_t *wg,
                             const uint8_t *wu, const uint8_t *wd, int n_experts, int hidden, int ff, const uint32_t *sel,
                             const float *wts, const float *resid, int slots_per_token, int m, float *y) {
    uint8_t *base = device < 0 || device >= kStaticMaxDevices ? nullptr : g_scratch_at[device].load(std::memory_order_acquire);
    if (!base) return hipErrorNotInitialized;
    if ((size_t)m * (size_t)slots_per_token * (size_t)ff > kStaticValues) return hipErrorInvalidValue;
    uint8_t *act_h = base;
    // the f32 rows of h are only read by a down stack on Q8_K columns: no other call writes them
    float *h = bm_takes_q8k(down_type) ? reinterpret_cast<float *>(base + kStaticColBytes) : nullptr;
    // every live slot's column (or f32 rows) is written whole by the first launch before the second reads it, and a
    // slot that is not live is never read into a sum: nothing here has to start at zero
    return moe_decode(L, gate_type, down_type, x, wg, wu, wd, n_experts, hidden, ff, sel, wts, resid,
                      slots_per_token, m, nullptr, act_h, h, y);
}

hipError_t block_sums(const Launch &L, int wtype, const uint8_t *wrow, int k, const uint8_t *col, int32_t *out) {
    const int nb = k / 256;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)act_col_bytes(wtype, k);
#define CALL_BODY                                                                                                      \
    auto kern = k_block_sums<WT, U, NB>;                                                                               \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3(1), dim3(64), lds, L.stream, wrow, nb, col, out);
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

} // namespace bmk

#ifdef BM_TIMELINE
// The table above, copied to the host: dst holds kTimelineRows * 8 words. Measurement builds only; not part of the C ABI.
extern "C" int bm_timeline_read(unsigned long long *dst) {
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(bmk::g_timeline), sizeof(unsigned long long) * bmk::kTimelineRows * 8);
}
#endif
