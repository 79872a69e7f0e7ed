// HIP kernels of the quantized MoE expert matmul for gfx950, and their launch functions.
//
// Every dot kernel follows one plan: a quad of lanes per weight row (bm_device.cuh); the token's quantized
// activation column requested first, then the row's first batch of super-blocks (128-bit loads), all from
// straight-line code so the hardware's in-order load counter lets the column be copied to LDS and the arithmetic
// start on the first super-block while the later ones are still in flight. Weights are read once, straight from
// the file's block bytes; the kernels are bound by HBM bandwidth.
//
// Variants: a kernel is instantiated per weight type and per (U, NB): U super-blocks a lane requests per batch,
// NB the row's super-block count when it is known at compile time (0: a run-time count that U divides). The hot
// shapes (Q4_K rows of 2048 values, Q6_K rows of 768) take NB = U = the whole row, one batch and no loop.
#include "bm_kernels.h"

#define BM_TABLE_QUAL __device__ const
#include "iq2xxs_tables.h"

#include "bm_device.cuh"

namespace bmk {

constexpr u32 kSiteQuantColumn = 1; // crates/device/src/fault.rs:73-76
constexpr u32 kSiteExpertId = 7;    // crates/device/src/fault.rs:89

// LDS bytes of the IQ2_XXS tables: 2048 grid + 128 signs + 64 nibble masks, padded to a 16-byte multiple.
constexpr int kTabBytes = 2048 + 128 + 64 + 64;

template <int WT>
__host__ __device__ constexpr int tab_bytes() {
    return WT == BM_IQ2XXS ? kTabBytes : 0;
}

template <int WT>
__device__ __forceinline__ Iq2Tables stage_tables(uint8_t *lds) {
    Iq2Tables tb{nullptr, nullptr, nullptr};
    if constexpr (WT == BM_IQ2XXS) {
        uint2 *grid = reinterpret_cast<uint2 *>(lds);
        uint8_t *ks = lds + 2048;
        u32 *nm = reinterpret_cast<u32 *>(lds + 2048 + 128);
        for (int t = threadIdx.x; t < 256; t += blockDim.x) {
            const uint64_t g = BM_IQ2XXS_GRID[t];
            grid[t] = make_uint2((u32)g, (u32)(g >> 32));
        }
        for (int t = threadIdx.x; t < 128; t += blockDim.x) ks[t] = BM_KSIGNS_IQ2XS[t];
        for (int t = threadIdx.x; t < 16; t += blockDim.x)
            nm[t] = ((t & 1) ? 0xffu : 0u) | ((t & 2) ? 0xff00u : 0u) | ((t & 4) ? 0xff0000u : 0u) |
                    ((t & 8) ? 0xff000000u : 0u);
        tb.grid = grid;
        tb.ksigns = ks;
        tb.nibmask = nm;
    }
    return tb;
}

// `bytes` (a multiple of 8) from 8-byte aligned global memory to 8-byte aligned LDS, by the whole workgroup.
__device__ __forceinline__ void stage_bytes(uint8_t *dst, const uint8_t *src, int bytes) {
    for (int o = threadIdx.x * 8; o < bytes; o += blockDim.x * 8)
        *reinterpret_cast<uint2 *>(dst + o) = *reinterpret_cast<const uint2 *>(src + o);
}

// The same copy in two halves: R unconditional loads a thread (offsets past the end are clamped onto the last
// word, so no branch stands between them and the weight loads that follow), then the LDS stores. Memory returns
// in order, so the stores wait for these loads only. Bytes past R * 8 * blockDim are copied afterwards by
// stage_bytes' loop (that part waits for everything in flight).
template <int R>
struct Stage {
    uint2 v[R];
    __device__ __forceinline__ void load(const uint8_t *src, int bytes) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            int o = (r * (int)blockDim.x + (int)threadIdx.x) * 8;
            o = o < bytes ? o : bytes - 8;
            v[r] = *reinterpret_cast<const uint2 *>(src + o);
        }
        // keep these loads ahead of whatever is requested next: the in-order wait depends on it
        __asm__ volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    __device__ __forceinline__ void store(uint8_t *dst, const uint8_t *src, int bytes) const {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int o = (r * (int)blockDim.x + (int)threadIdx.x) * 8;
            if (o < bytes) *reinterpret_cast<uint2 *>(dst + o) = v[r];
        }
        for (int o = (R * (int)blockDim.x + (int)threadIdx.x) * 8; o < bytes; o += (int)blockDim.x * 8)
            *reinterpret_cast<uint2 *>(dst + o) = *reinterpret_cast<const uint2 *>(src + o);
    }
};

// Super-blocks 0..U of the row, requested unconditionally (the launch functions pick U to divide the row).
template <int WT, int U>
__device__ __forceinline__ void preload(Blk<WT> (&b)[U], const uint8_t *wrow, int q) {
#pragma unroll
    for (int u = 0; u < U; u++) b[u] = bm_load_blk<WT>(wrow, u, q);
}

// Row `wrow` against `m` <= M columns (LDS, `col_stride` apart); b holds the first batch already.
// NB > 0: the row has NB super-blocks (a multiple of U); NB == 0: it has nb, a multiple of U.
template <int WT, int U, int NB, int M, class Tap>
__device__ __forceinline__ void row_dot(Blk<WT> (&b)[U], const uint8_t *wrow, const uint8_t *cols, int col_stride,
                                        int m, int nb, int q, const Iq2Tables &tb, float (&out)[M], const Tap &tap) {
    float a0[M], a1[M];
#pragma unroll
    for (int c = 0; c < M; c++) a0[c] = a1[c] = 0.0f;
    if constexpr (NB == U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int c = 0; c < M; c++)
                if (M == 1 || c < m) bm_dot_blk<WT>(b[u], cols + (size_t)c * col_stride, u, q, tb, a0[c], a1[c], tap);
        }
    } else {
        const int n = NB > 0 ? NB : nb;
        for (int i0 = 0;;) {
#pragma unroll
            for (int u = 0; u < U; u++) {
#pragma unroll
                for (int c = 0; c < M; c++)
                    if (M == 1 || c < m)
                        bm_dot_blk<WT>(b[u], cols + (size_t)c * col_stride, i0 + u, q, tb, a0[c], a1[c], tap);
            }
            i0 += U;
            if (i0 >= n) break;
#pragma unroll
            for (int u = 0; u < U; u++) b[u] = bm_load_blk<WT>(wrow, i0 + u, q);
        }
    }
#pragma unroll
    for (int c = 0; c < M; c++) out[c] = bm_quad_finish<WT>(a0[c], a1[c]);
}

// ----------------------------------------------------------------------------------------------- fill

__global__ void k_fill_u32(u32 *dst, u32 value, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = value;
}

hipError_t fill_u32(const Launch &L, uint32_t *dst, uint32_t value, size_t n) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, L.stream, dst, value, n);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------- quantizers

// One 32-value q8_2 block on the 32 lanes of a half wave (crates/qdot/src/lib.rs:3883-3904).
// Returns the code; *t_out / *isum_out are valid on every lane. `bad` reports a value that is not finite.
__device__ __forceinline__ int q82_block(float v, u32 *t_out, int *isum_out, bool *bad) {
    u32 ab = bm_f32_bits(v) & 0x7fffffffu;
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1) {
        u32 o = (u32)__shfl_xor((int)ab, s, 32);
        ab = o > ab ? o : ab;
    }
    if (ab > 0x7f7fffffu) {
        *bad = true;
        *t_out = 0x7fc0u; // a NaN scale, zero codes (crates/gpu/src/lib.rs:925-933)
        *isum_out = 0;
        return 0;
    }
    *bad = false;
    const float amax = bm_bits_f32(ab);
    const u32 t = bm_fp32_to_bf16_bits(__fdiv_rn(amax, 127.0f));
    const float id = bm_q82_inverse(t);
    const int q = bm_nearest_int(__fmul_rn(v, id));
    int isum = q;
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1) isum += __shfl_xor(isum, s, 32);
    *t_out = t;
    *isum_out = isum;
    return q < -128 ? -128 : (q > 127 ? 127 : q);
}

// Stores one q8_2 block (its 32 codes, scale and sum) into a column's Q8_2_X4 bytes.
__device__ __forceinline__ void q82_store(uint8_t *col, int blk, int lane32, int code, u32 t, int isum) {
    uint8_t *group = col + (size_t)(blk >> 2) * BM_Q82X4_STRIDE;
    const int ir = blk & 3;
    // four codes a lane-quad -> one dword store from its first lane
    u32 c = (u32)(code & 0xff);
    c |= (u32)(__shfl_down((int)c, 1, 32) & 0xff) << 8;
    c |= (u32)(__shfl_down((int)c, 2, 32) & 0xffff) << 16;
    if ((lane32 & 3) == 0) *reinterpret_cast<u32 *>(group + 16 + 32 * ir + lane32) = c;
    if (lane32 == 0) {
        *reinterpret_cast<unsigned short *>(group + 2 * ir) = (unsigned short)t;
        *reinterpret_cast<unsigned short *>(group + 8 + 2 * ir) = (unsigned short)(short)isum;
    }
}

// x: m columns of k values -> Q8_2_X4 columns. One half wave a 32-value block.
__global__ __launch_bounds__(256) void k_quantize_q82x4(const float *x, int m, int k, uint8_t *act, u32 *fault,
                                                        u32 layer) {
    const int bpc = k / 32; // blocks a column
    const long gblk = (long)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (gblk >= (long)m * bpc) return;
    const int col = (int)(gblk / bpc), blk = (int)(gblk % bpc), lane32 = threadIdx.x & 31;
    const float v = x[(size_t)col * k + 32 * blk + lane32];
    u32 t;
    int isum;
    bool bad;
    const int code = q82_block(v, &t, &isum, &bad);
    if (bad && lane32 == 0) bm_raise(fault, layer, kSiteQuantColumn);
    q82_store(act + (size_t)col * (k / 128) * BM_Q82X4_STRIDE, blk, lane32, code, t, isum);
}

// x: m columns of k values -> Q8_K columns (crates/qdot/src/lib.rs:1787-1809). One workgroup a 256-value block.
__global__ __launch_bounds__(256) void k_quantize_q8k(const float *x, int m, int k, uint8_t *act, u32 *fault,
                                                      u32 layer) {
    __shared__ unsigned long long s_key[4];
    __shared__ int s_codes[256];
    const int bpc = k / 256;
    const int col = blockIdx.x / bpc, blk = blockIdx.x % bpc, tid = threadIdx.x;
    const float *xb = x + (size_t)col * k + 256 * blk;
    uint8_t *o = act + ((size_t)col * bpc + blk) * BM_Q8K_STRIDE;
    const float v = xb[tid];
    // the largest magnitude, first on ties: maximise (|bits|, 255 - index)
    unsigned long long key = ((unsigned long long)(bm_f32_bits(v) & 0x7fffffffu) << 32) | (u32)(255 - tid);
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        unsigned long long other = __shfl_xor(key, s, 64);
        key = other > key ? other : key;
    }
    if ((tid & 63) == 0) s_key[tid >> 6] = key;
    __syncthreads();
    key = s_key[0];
    for (int w = 1; w < 4; w++) key = s_key[w] > key ? s_key[w] : key;
    const u32 ab = (u32)(key >> 32);
    const int first = 255 - (int)(key & 0xffffffffu);
    float d;
    int code = 0;
    if (ab > 0x7f7fffffu) {
        if (tid == 0) bm_raise(fault, layer, kSiteQuantColumn);
        d = bm_bits_f32(0x7fc00000u);
    } else if (ab == 0) {
        d = 0.0f;
    } else {
        const float max = xb[first];
        const float iscale = __fdiv_rn(-127.0f, max);
        int q = bm_nearest_int(__fmul_rn(iscale, v));
        q = q > 127 ? 127 : q;
        code = (int)(signed char)(q & 0xff); // `as i8`: the low byte
        d = __fdiv_rn(1.0f, iscale);
    }
    s_codes[tid] = code;
    __syncthreads();
    if ((tid & 3) == 0) {
        const u32 c = (u32)(s_codes[tid] & 0xff) | ((u32)(s_codes[tid + 1] & 0xff) << 8) |
                      ((u32)(s_codes[tid + 2] & 0xff) << 16) | ((u32)(s_codes[tid + 3] & 0xff) << 24);
        *reinterpret_cast<u32 *>(o + 8 + tid) = c;
    }
    if (tid < 16) {
        int sum = 0;
        for (int ii = 0; ii < 16; ii++) sum += s_codes[16 * tid + ii];
        *reinterpret_cast<unsigned short *>(o + 264 + 2 * tid) = (unsigned short)(short)sum;
    }
    if (tid == 0) {
        *reinterpret_cast<float *>(o) = d;
        *reinterpret_cast<u32 *>(o + 4) = 0u;
    }
}

hipError_t quantize(const Launch &L, int wtype, const float *x, int m, int k, uint8_t *act) {
    if (wtype == BM_IQ2XXS) {
        hipLaunchKernelGGL(k_quantize_q8k, dim3((unsigned)(m * (k / 256))), dim3(256), 0, L.stream, x, m, k, act,
                           L.fault, L.layer);
    } else {
        const long blocks = (long)m * (k / 32);
        hipLaunchKernelGGL(k_quantize_q82x4, dim3((unsigned)((blocks + 7) / 8)), dim3(256), 0, L.stream, x, m, k, act,
                           L.fault, L.layer);
    }
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------ gemv

// y[row * m_total + col0 + c] = row . column (col0 + c), c < m <= 8. A quad a row, 64 rows a workgroup.
template <int WT, int U, int NB>
__global__ __launch_bounds__(256) void k_gemv(const uint8_t *w, long rows, int nb, const uint8_t *act, int m_total,
                                              int col0, int m, float *y) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3;
    const long row = (long)blockIdx.x * 64 + (tid >> 2);
    const bool active = row < rows;
    const int n = NB > 0 ? NB : nb;
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const int col_bytes = n * bm_act_sb_bytes<WT>();
    const uint8_t *wrow = w + (size_t)(active ? row : 0) * row_bytes;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *cols = lds + tab_bytes<WT>();
    stage_bytes(cols, act + (size_t)col0 * col_bytes, m * col_bytes);
    __syncthreads();
    float out[8];
    row_dot<WT, U, NB, 8>(b, wrow, cols, col_bytes, m, n, q, tb, out, NoTap{});
    if (q == 0 && active) {
#pragma unroll
        for (int c = 0; c < 8; c++)
            if (c < m) y[(size_t)row * m_total + col0 + c] = out[c];
    }
}

// --------------------------------------------------------------------------------- gate . up . SwiGLU

// One workgroup = 32 consecutive rows of one slot; eight lanes a row: a quad on the gate row, a quad on the up row.
// With act_h the 32 values are quantized to one q8_2 block of the slot's down activation in the same launch.
template <int WT, int U, int NB>
__global__ __launch_bounds__(256) void k_gate_up(const uint8_t *wg, const uint8_t *wu, u32 n_experts, int nb,
                                                 const uint8_t *act, const u32 *sel, int rpe, int slots_per_col,
                                                 float *h, uint8_t *act_h, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3, which = (tid >> 2) & 1;
    const int blocks_per_slot = (rpe + 31) / 32;
    const int slot = blockIdx.x / blocks_per_slot, rb = blockIdx.x % blocks_per_slot;
    const int r = rb * 32 + (tid >> 3);
    const bool active = r < rpe;
    const u32 id = sel[slot];
    const int n = NB > 0 ? NB : nb;
    const int h_col_bytes = (rpe / 128) * BM_Q82X4_STRIDE;
    const int col_bytes = n * bm_act_sb_bytes<WT>();
    const uint8_t *act_col = act + (size_t)(slot / slots_per_col) * col_bytes;
    Stage<2> st;
    st.load(act_col, col_bytes);
    if (id >= n_experts) { // uniform over the workgroup: no weight is read (crates/gpu/src/kquant/sel.rs:22-28)
        if (tid == 0) bm_raise(fault, layer, kSiteExpertId);
        if (h && active && (tid & 7) == 0) h[(size_t)slot * rpe + r] = bm_bits_f32(0x7fc00000u);
        if (act_h && tid < 32) q82_store(act_h + (size_t)slot * h_col_bytes, rb, tid, 0, 0x7fc0u, 0);
        return;
    }
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const uint8_t *wrow = (which ? wu : wg) + ((size_t)id * rpe + (active ? r : 0)) * row_bytes;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *col = lds + tab_bytes<WT>();
    st.store(col, act_col, col_bytes);
    __syncthreads();
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, col, col_bytes, 1, n, q, tb, v, NoTap{});
    const float other = __shfl_xor(v[0], 4, 64);
    const float hv = bm_swiglu(which ? other : v[0], which ? v[0] : other);
    if (h && active && (tid & 7) == 0) h[(size_t)slot * rpe + r] = hv;
    if (act_h) { // rpe is a multiple of 256 here, so every row of the block is live
        float *hbuf = reinterpret_cast<float *>(col + col_bytes);
        if ((tid & 7) == 0) hbuf[tid >> 3] = hv;
        __syncthreads();
        if (tid < 32) {
            u32 t;
            int isum;
            bool bad;
            const int code = q82_block(hbuf[tid], &t, &isum, &bad);
            if (bad && tid == 0) bm_raise(fault, layer, kSiteQuantColumn);
            q82_store(act_h + (size_t)slot * h_col_bytes, rb, tid, code, t, isum);
        }
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
    const int col_bytes = n * bm_act_sb_bytes<WT>();
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
__global__ __launch_bounds__(256) void k_combine(const float *down, const float *w, const float *resid, int rows,
                                                 int n_slots, int m, float *y) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long)rows * m) return;
    const int t = (int)(i / rows), d = (int)(i % rows);
    float acc = 0.0f;
    for (int e = 0; e < n_slots; e++)
        acc = fmaf(w[(size_t)t * n_slots + e], down[((size_t)t * n_slots + e) * rows + d], acc);
    y[i] = resid ? __fadd_rn(acc, resid[i]) : acc;
}

hipError_t combine_tokens(const Launch &L, const float *down, const float *w, const float *resid, int rows,
                          int n_slots, int m, float *y) {
    const long n = (long)rows * m;
    hipLaunchKernelGGL(k_combine, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, L.stream, down, w, resid, rows,
                       n_slots, m, y);
    return hipGetLastError();
}

// --------------------------------------------------------------------------- down + combine in one launch

// One workgroup = one token and D = 64 / slots_per_token output rows: a quad for every (row, slot). The slot values
// meet in LDS and one thread a row folds them in slot order, then adds the residual.
template <int WT, int U, int NB>
__global__ __launch_bounds__(256) void k_down_combine(const uint8_t *w, u32 n_experts, int nb, const uint8_t *act,
                                                      const u32 *sel, const float *wts, const float *resid, int spt,
                                                      int rpe, float *y, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3, quad = tid >> 2;
    const int D = 64 / spt;
    const int blocks_per_token = (rpe + D - 1) / D;
    const int t = blockIdx.x / blocks_per_token, rb = blockIdx.x % blocks_per_token;
    const int e = quad % spt, dl = quad / spt;
    const int r = rb * D + dl;
    const int slot = t * spt + e;
    const u32 id = sel[slot];
    // the token's ids and weights for the closing sum, requested now and parked in LDS
    const int si = tid < spt ? tid : 0;
    const u32 my_sel = sel[t * spt + si];
    const float my_w = wts[t * spt + si];
    const bool live = id < n_experts;
    const bool active = dl < D && r < rpe && live;
    if (!live && id != 0xffffffffu && rb == 0 && dl == 0 && q == 0) bm_raise(fault, layer, kSiteExpertId);
    const int n = NB > 0 ? NB : nb;
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const int col_bytes = n * bm_act_sb_bytes<WT>();
    const uint8_t *act_cols = act + (size_t)t * spt * col_bytes;
    Stage<4> st;
    st.load(act_cols, spt * col_bytes);
    const uint8_t *wrow = w + ((size_t)(live ? id : 0) * rpe + (active ? r : 0)) * row_bytes;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *cols = lds + tab_bytes<WT>();
    st.store(cols, act_cols, spt * col_bytes);
    float *part = reinterpret_cast<float *>(cols + (size_t)spt * col_bytes); // [D][spt]
    float *s_w = part + D * spt;                                              // [spt]
    u32 *s_sel = reinterpret_cast<u32 *>(s_w + spt);                          // [spt]
    if (tid < spt) {
        s_w[tid] = my_w;
        s_sel[tid] = my_sel;
    }
    __syncthreads();
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, cols + (size_t)e * col_bytes, col_bytes, 1, n, q, tb, v, NoTap{});
    if (q == 0 && dl < D) part[dl * spt + e] = v[0];
    __syncthreads();
    if (tid < D && rb * D + tid < rpe) {
        float acc = 0.0f;
        for (int s = 0; s < spt; s++)
            if (s_sel[s] < n_experts) acc = fmaf(s_w[s], part[tid * spt + s], acc);
        const size_t o = (size_t)t * rpe + rb * D + tid;
        y[o] = resid ? __fadd_rn(acc, resid[o]) : acc;
    }
}

// ------------------------------------------------------------------------------------------ verification

struct StoreTap {
    int *out; // 16 words a super-block, zeroed before the quad runs
    __device__ __forceinline__ void q4k(int i, int s, int, int v) const { atomicAdd(&out[16 * i + s], v); }
    __device__ __forceinline__ void q4k_isum(int i, int s, int v) const { out[16 * i + 8 + s] = v; }
    __device__ __forceinline__ void q6k(int i, int g, int v) const { out[16 * i + g] = v; }
    __device__ __forceinline__ void iq2(int i, int b, int q, int v) const {
        atomicAdd(&out[16 * i + b], v);
        (void)q;
    }
};

template <int WT, int U, int NB>
__global__ __launch_bounds__(64) void k_block_sums(const uint8_t *wrow, int nb, const uint8_t *act_col, int *out) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3;
    const int n = NB > 0 ? NB : nb;
    const int col_bytes = n * bm_act_sb_bytes<WT>();
    for (int i = tid; i < 16 * n; i += blockDim.x) out[i] = 0;
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *col = lds + tab_bytes<WT>();
    stage_bytes(col, act_col, col_bytes);
    __threadfence();
    __syncthreads();
    if (tid >= 4) return;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    float v[1];
    row_dot<WT, U, NB, 1>(b, wrow, col, col_bytes, 1, n, q, tb, v, StoreTap{out});
    if constexpr (WT == BM_IQ2XXS) {
        // the eight scales 2s + 1 of each super-block, as the dot reads them
        if (q == 0)
            for (int i = 0; i < n; i++)
                for (int s = 0; s < 8; s++) {
                    u32 aux;
                    __builtin_memcpy(&aux, wrow + (size_t)i * BM_IQ2XXS_BLOCK + 6 + 8 * s, 4);
                    out[16 * i + 8 + s] = 2 * (int)(aux >> 28) + 1;
                }
    }
}

// ---------------------------------------------------------------------------------------- launch helpers

template <typename K>
static hipError_t allow_lds(K kernel, size_t lds) {
    if (lds <= 64 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)lds);
}

// Picks the kernel variant for a row of nb super-blocks and runs CALL with WT, U and NB as constants. Each type
// lists its whole-row variant first (the hot shape), then a batch of four, then one super-block at a time, which
// divides every row.
#define BM_VARIANT(T, UU, NN)                                                                                          \
    {                                                                                                                  \
        constexpr int WT = T, U = UU, NB = NN;                                                                         \
        CALL_BODY;                                                                                                     \
    }
#define BM_DISPATCH(wtype, nb)                                                                                         \
    switch (wtype) {                                                                                                   \
    case BM_Q4K:                                                                                                       \
        if ((nb) == 8) BM_VARIANT(BM_Q4K, 8, 8)                                                                        \
        else if ((nb) % 4 == 0) BM_VARIANT(BM_Q4K, 4, 0)                                                               \
        else BM_VARIANT(BM_Q4K, 1, 0)                                                                                  \
        break;                                                                                                         \
    case BM_Q6K:                                                                                                       \
        if ((nb) == 3) BM_VARIANT(BM_Q6K, 3, 3)                                                                        \
        else if ((nb) % 4 == 0) BM_VARIANT(BM_Q6K, 4, 0)                                                               \
        else BM_VARIANT(BM_Q6K, 1, 0)                                                                                  \
        break;                                                                                                         \
    case BM_IQ2XXS:                                                                                                    \
        if ((nb) % 4 == 0) BM_VARIANT(BM_IQ2XXS, 4, 0)                                                                 \
        else BM_VARIANT(BM_IQ2XXS, 1, 0)                                                                               \
        break;                                                                                                         \
    default:                                                                                                           \
        return hipErrorInvalidValue;                                                                                   \
    }

static int act_sb_bytes(int wtype) { return wtype == BM_IQ2XXS ? BM_Q8K_STRIDE : 2 * BM_Q82X4_STRIDE; }
static int tab_bytes_rt(int wtype) { return wtype == BM_IQ2XXS ? kTabBytes : 0; }

int gemv_max_cols(int wtype, int k) {
    const int col_bytes = (k / 256) * act_sb_bytes(wtype);
    int m = (kMaxLds - tab_bytes_rt(wtype)) / col_bytes;
    return m > 8 ? 8 : m;
}

hipError_t gemv(const Launch &L, int wtype, const uint8_t *w, int64_t rows, int k, const uint8_t *act, int m_total,
                int col0, int m, float *y) {
    const int nb = k / 256;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)m * nb * act_sb_bytes(wtype);
#define CALL_BODY                                                                                                      \
    auto kern = k_gemv<WT, U, NB>;                                                                                     \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3((unsigned)((rows + 63) / 64)), dim3(256), lds, L.stream, w, (long)rows, nb, act,     \
                       m_total, col0, m, y);
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

hipError_t gate_up(const Launch &L, int wtype, const uint8_t *wg, const uint8_t *wu, int n_experts, int k,
                   const uint8_t *act, const uint32_t *sel, int n_slots, int rows_per_expert, int slots_per_col,
                   float *h, uint8_t *act_h) {
    const int nb = k / 256, rpe = rows_per_expert;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)nb * act_sb_bytes(wtype) + 32 * sizeof(float);
    const unsigned grid = (unsigned)n_slots * (unsigned)((rpe + 31) / 32);
#define CALL_BODY                                                                                                      \
    auto kern = k_gate_up<WT, U, NB>;                                                                                  \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, wg, wu, (u32)n_experts, nb, act, sel, rpe,          \
                       slots_per_col, h, act_h, L.fault, L.layer);
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

hipError_t gemv_sel(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                    const uint32_t *sel, int n_slots, int rows_per_expert, float *y) {
    const int nb = k / 256, rpe = rows_per_expert;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)nb * act_sb_bytes(wtype);
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

hipError_t down_combine(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                        const uint32_t *sel, const float *wts, const float *resid, int slots_per_token, int m,
                        int rows_per_expert, float *y) {
    const int nb = k / 256, rpe = rows_per_expert, spt = slots_per_token;
    const int D = 64 / spt;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)spt * nb * act_sb_bytes(wtype) +
                       ((size_t)D * spt + 2 * (size_t)spt) * sizeof(float);
    const unsigned grid = (unsigned)m * (unsigned)((rpe + D - 1) / D);
#define CALL_BODY                                                                                                      \
    auto kern = k_down_combine<WT, U, NB>;                                                                             \
    hipError_t e = allow_lds(kern, lds);                                                                               \
    if (e != hipSuccess) return e;                                                                                     \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, w, (u32)n_experts, nb, act, sel, wts, resid, spt,   \
                       rpe, y, L.fault, L.layer);
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
    return hipGetLastError();
}

hipError_t block_sums(const Launch &L, int wtype, const uint8_t *wrow, int k, const uint8_t *col, int32_t *out) {
    const int nb = k / 256;
    const size_t lds = tab_bytes_rt(wtype) + (size_t)nb * act_sb_bytes(wtype);
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
