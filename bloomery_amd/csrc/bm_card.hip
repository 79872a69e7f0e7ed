// The card rule: the reference's GPU tier has activations and row walks of its own (its q8_1 form: 128-value blocks,
// an f32 scale amax / 127, codes rounded half away from zero, a code sum per 32 values; a Q4_K or Q3_K row walked by 32
// lanes whose accumulators meet in a butterfly), and the reference restates both on the CPU so the two tiers can be
// compared bit for bit (crates/qdot/src/lib.rs:2885-3620 card_q8_1, card_q4k_dot_row, card_q3k_dot_row). These kernels
// give the same values on this GPU: a 64-lane wave carries two of the rule's 32-lane walks, one row each, with every
// lane's integer chain, f32 operations and the butterfly's order kept as the rule states them. The column planes lie
// in value order: codes i8 [m][k], d8 f32 [m][k / 128], s8 i32 [m][k / 32].
#include "bm_stream.hpp"

namespace bmk {

// ------------------------------------------------------------------------------------------------ quantizer

// crates/gpu/src/lib.rs:944-1026 q8_1_quant_vals with crates/gpu/src/cores.rs:159-168 q8_quad, as
// crates/qdot/src/lib.rs:2917-2948 states their values: 32 lanes a 128-value block, four values a lane.
__global__ __launch_bounds__(256) void k_card_quantize(const float *x, long n_blocks, u32 *codes, float *d8, int *s8, u32 *fault,
                                                       u32 layer) {
    const int lane = threadIdx.x & 31;
    const long b = (long)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (b >= n_blocks) return; // whole half-waves leave together: the exchanges below stay inside a half
    const float4 v = *reinterpret_cast<const float4 *>(x + b * 128 + 4 * lane);
    const u32 a0 = __float_as_uint(v.x) & 0x7fffffffu, a1 = __float_as_uint(v.y) & 0x7fffffffu;
    const u32 a2 = __float_as_uint(v.z) & 0x7fffffffu, a3 = __float_as_uint(v.w) & 0x7fffffffu;
    u32 am = a0 > a1 ? a0 : a1;
    am = a2 > am ? a2 : am;
    am = a3 > am ? a3 : am;
    am = bm_max32(am); // magnitudes order as their bits do; anything not finite sorts at or above 0x7f800000
    const bool bad = am >= 0x7f800000u;
    const float amax = __uint_as_float(am);
    const float d = bad ? __uint_as_float(0x7fc00000u) : amax > 0.0f ? amax / 127.0f : 1.0f;
    auto code = [&](float val) -> int {
        if (bad) return 0;
        const float r = roundf(val / d); // half away from zero
        // a NaN (0 / 0 under a scale that underflowed to zero) is code 0, an infinity the clamp's end
        return r != r ? 0 : r < -127.0f ? -127 : r > 127.0f ? 127 : (int)r;
    };
    const int q0 = code(v.x), q1 = code(v.y), q2 = code(v.z), q3 = code(v.w);
    codes[b * 32 + lane] = (u32)(q0 & 0xff) | ((u32)(q1 & 0xff) << 8) | ((u32)(q2 & 0xff) << 16) | ((u32)(q3 & 0xff) << 24);
    int g = q0 + q1 + q2 + q3; // a 32-value group is eight lanes
    g += (int)bm_dpp<kDppXor1>((u32)g);
    g += (int)bm_dpp<kDppXor2>((u32)g);
    g += (int)bm_dpp<kDppHalfMirror>((u32)g);
    if ((lane & 7) == 0) s8[b * 4 + (lane >> 3)] = g;
    if (lane == 0) {
        d8[b] = d;
        if (bad) bm_raise(fault, layer, kSiteQuantColumn);
    }
}

hipError_t card_quantize(const Launch &L, const float *x, int m, int k, int8_t *codes, float *d8, int32_t *s8) {
    const long n_blocks = (long)m * (k / 128);
    hipLaunchKernelGGL(k_card_quantize, dim3((unsigned)((n_blocks + 7) / 8)), dim3(256), 0, L.stream, x, n_blocks,
                       reinterpret_cast<u32 *>(codes), d8, s8, L.fault, L.layer);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------ row walks

__device__ __forceinline__ u32 card_rd32(const uint8_t *p) { // a word at a two-byte boundary
    return (u32) * reinterpret_cast<const unsigned short *>(p) | ((u32) * reinterpret_cast<const unsigned short *>(p + 2) << 16);
}

// crates/qdot/src/lib.rs:3331-3341 card_warp_sum_scalar: strides 16, 8, 4, 2, 1; lane 0 of each 32 holds the tree's value.
__device__ __forceinline__ float card_warp_sum(float v) {
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 8);
    v += __shfl_xor(v, 4);
    v += __shfl_xor(v, 2);
    v += __shfl_xor(v, 1);
    return v;
}

// crates/qdot/src/lib.rs:3184 card_q4k_nibble
__device__ __forceinline__ u32 card_q4k_nibble(u32 qsw, u32 nib_sh) {
    return ((((qsw >> nib_sh) & 0x0f0f0f0fu) | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

struct CardTerm {
    float x, e;
};

// One lane's term of iteration `it` (crates/gpu/src/cores.rs q4k_iter_term; crates/qdot/src/lib.rs:3297-3322): lane
// (grp, s) takes sub-block s of super-block 4 it + grp.
__device__ __forceinline__ CardTerm card_q4k_term(const uint8_t *wrow, const uint8_t *codes, const float *d8, const int *s8, int it,
                                                  int lane) {
    const int s = lane & 7, grp = lane >> 3, sbp = 4 * it + grp;
    const uint8_t *sb = wrow + (size_t)sbp * BM_Q4K_BLOCK;
    const uint4 hd = *reinterpret_cast<const uint4 *>(sb);
    const uint4 qa = *reinterpret_cast<const uint4 *>(sb + 16 + 32 * (s >> 1));
    const uint4 qb = *reinterpret_cast<const uint4 *>(sb + 32 + 32 * (s >> 1));
    const uint8_t *cw = codes + 1024 * (size_t)it + 256 * grp + 32 * s;
    const uint4 ca = *reinterpret_cast<const uint4 *>(cw), cb = *reinterpret_cast<const uint4 *>(cw + 16);
    const float d = bm_half_to_f32(hd.x & 0xffffu), dmin = bm_half_to_f32(hd.x >> 16);
    int sc, mi; // crates/qdot/src/lib.rs:3165-3180 card_q4k_scale_min
    if (s < 4) {
        sc = (int)((hd.y >> (8 * s)) & 63);
        mi = (int)((hd.z >> (8 * s)) & 63);
    } else {
        const int sh = 8 * (s - 4);
        const u32 qs = (hd.z >> sh) & 0xff, qs4 = (hd.w >> sh) & 0xff, qsm = (hd.y >> sh) & 0xff;
        sc = (int)(qs4 & 0x0f) | ((int)(qsm >> 6) << 4);
        mi = (int)(qs4 >> 4) | ((int)(qs >> 6) << 4);
    }
    const float cda = d * (float)sc;
    const float cdb = fmaf(8.0f * d, (float)sc, -(dmin * (float)mi));
    const u32 nib_sh = (u32)(s & 1) * 4;
    int a = bm_sdot4(card_q4k_nibble(qa.x, nib_sh), ca.x, 0);
    a = bm_sdot4(card_q4k_nibble(qa.y, nib_sh), ca.y, a);
    a = bm_sdot4(card_q4k_nibble(qa.z, nib_sh), ca.z, a);
    a = bm_sdot4(card_q4k_nibble(qa.w, nib_sh), ca.w, a);
    a = bm_sdot4(card_q4k_nibble(qb.x, nib_sh), cb.x, a);
    a = bm_sdot4(card_q4k_nibble(qb.y, nib_sh), cb.y, a);
    a = bm_sdot4(card_q4k_nibble(qb.z, nib_sh), cb.z, a);
    a = bm_sdot4(card_q4k_nibble(qb.w, nib_sh), cb.w, a);
    const int b = s8[32 * it + lane];
    CardTerm t;
    t.x = fmaf(cda, (float)a, cdb * (float)b); // crates/gpu/src/cores.rs:270 q4k_sub_value
    t.e = d8[2 * sbp + (s >> 2)];
    return t;
}

// crates/gpu/src/cores.rs:536-620 q4k_row_dot_1col, crates/qdot/src/lib.rs:3288-3327 card_q4k_lane_walk: the
// iterations whose four super-blocks all exist go two at a time, the first term's product rounded before it is added,
// the second fused; what is left goes one at a time behind the guard, fused.
__device__ __forceinline__ float card_q4k_walk(const uint8_t *wrow, const uint8_t *codes, const float *d8, const int *s8, int n_sb,
                                               int lane) {
    const int iters = (n_sb + 3) / 4, full = n_sb / 4, grp = lane >> 3;
    float f = 0.0f;
    int it = 0;
    for (; it + 2 <= full; it += 2) {
        const CardTerm t0 = card_q4k_term(wrow, codes, d8, s8, it, lane);
        const CardTerm t1 = card_q4k_term(wrow, codes, d8, s8, it + 1, lane);
        f = f + t0.e * t0.x;
        f = fmaf(t1.e, t1.x, f);
    }
    for (; it < iters; it++) {
        if (4 * it + grp < n_sb) {
            const CardTerm t = card_q4k_term(wrow, codes, d8, s8, it, lane);
            f = fmaf(t.e, t.x, f);
        }
    }
    return f;
}

// crates/qdot/src/lib.rs:3135-3144 card_q3k_field
__device__ __forceinline__ u32 card_q3k_field(u32 vl, u32 vh1, u32 f) {
    return ((((vl >> (2 * f)) & 0x03030303u) | 0x80808080u) - (((vh1 >> f) << 2) & 0x04040404u)) ^ 0x80808080u;
}

// crates/qdot/src/lib.rs:3239-3276 card_q3k_lane_walk: lane (half, w16) takes, of super-block 2 it + half, the four
// values 4 (w16 & 7) .. + 3 of every 32-value quarter of the 128-value half w16 >> 3.
__device__ __forceinline__ float card_q3k_walk(const uint8_t *wrow, const uint8_t *codes, const float *d8, int n_sb, int lane) {
    const int iters = (n_sb + 1) / 2;
    const int w16 = lane & 15, half = lane >> 4;
    const int s0 = 8 * (w16 >> 3) + ((w16 & 7) >> 2), d8_base = w16 >> 3;
    const u32 sh = (u32)(((s0 & 1) << 3) | ((s0 >> 3) << 2));
    float f = 0.0f;
    for (int it = 0; it < iters; it++) {
        const int sbp = 2 * it + half;
        if (sbp >= n_sb) continue;
        const uint8_t *sb = wrow + (size_t)sbp * BM_Q3K_BLOCK;
        const u32 vl = card_rd32(sb + 32 + 4 * w16);
        const u32 hm = card_rd32(sb + 4 * (w16 & 7));
        const u32 vh1 = (~hm) >> (4 * (w16 >> 3));
        const u32 a0w = card_rd32(sb + 96), a1w = card_rd32(sb + 100), a2w = card_rd32(sb + 104);
        // crates/qdot/src/lib.rs:3150-3160 card_q3k_sub_scales
        const u32 p0 = ((a0w >> sh) & 0x000f000fu) | (((a2w >> sh) & 0x00030003u) << 4);
        const u32 p1 = ((a1w >> sh) & 0x000f000fu) | (((a2w >> (sh + 2)) & 0x00030003u) << 4);
        const int sc0 = (int)(p0 & 0xff) - 32, sc1 = (int)(p0 >> 16) - 32, sc2 = (int)(p1 & 0xff) - 32, sc3 = (int)(p1 >> 16) - 32;
        const float drow = bm_half_to_f32(*reinterpret_cast<const unsigned short *>(sb + 108));
        const u32 *cw = reinterpret_cast<const u32 *>(codes) + 128 * it + 64 * half + 32 * d8_base + (lane & 7);
        int a = bm_sdot4(card_q3k_field(vl, vh1, 0), cw[0], 0) * sc0;
        a += bm_sdot4(card_q3k_field(vl, vh1, 1), cw[8], 0) * sc1;
        a += bm_sdot4(card_q3k_field(vl, vh1, 2), cw[16], 0) * sc2;
        a += bm_sdot4(card_q3k_field(vl, vh1, 3), cw[24], 0) * sc3;
        const float e0 = d8[2 * sbp + d8_base];
        f = fmaf(e0 * drow, (float)a, f);
    }
    return f;
}

template <int WT>
__device__ __forceinline__ float card_row_dot(const uint8_t *wrow, const uint8_t *codes, const float *d8, const int *s8, int n_sb,
                                              int lane) {
    const float f = WT == BM_Q4K ? card_q4k_walk(wrow, codes, d8, s8, n_sb, lane) : card_q3k_walk(wrow, codes, d8, n_sb, lane);
    return card_warp_sum(f);
}

// y[r * m + c] (crates/gpu/src/lib.rs:1617 q4k_gemv): 32 lanes a row, eight rows a workgroup, a column a grid row.
template <int WT>
__global__ __launch_bounds__(256) void k_card_gemv(const uint8_t *w, long rows, int n_sb, const uint8_t *codes, const float *d8,
                                                   const int *s8, int m, float *y) {
    const int lane = threadIdx.x & 31, c = blockIdx.y;
    const long r = (long)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (r >= rows) return;
    const size_t k = (size_t)n_sb * 256;
    const float v = card_row_dot<WT>(w + (size_t)r * n_sb * bm_block_bytes<WT>(), codes + c * k, d8 + c * (k / 128), s8 + c * (k / 32),
                                     n_sb, lane);
    if (lane == 0) y[r * m + c] = v;
}

// y[s * rpe + r]: slot s's column against the rows of expert sel[s] (crates/gpu/src/q4k_sel.rs:358 q4k_gemv_sel). An id
// past the stack raises ExpertId and leaves the slot's rows untouched; 0xffffffff (a host slot) is skipped silently.
template <int WT>
__global__ __launch_bounds__(256) void k_card_gemv_sel(const uint8_t *w, u32 n_experts, int rpe, int n_sb, const uint8_t *codes,
                                                       const float *d8, const int *s8, const u32 *sel, float *y, u32 *fault,
                                                       u32 layer) {
    const int lane = threadIdx.x & 31;
    const int blocks_per_slot = (rpe + 7) / 8;
    const int slot = blockIdx.x / blocks_per_slot, rb = blockIdx.x % blocks_per_slot;
    const int r = rb * 8 + (threadIdx.x >> 5);
    const u32 id = sel[slot];
    if (id >= n_experts) {
        if (threadIdx.x == 0 && rb == 0 && id != 0xffffffffu) bm_raise(fault, layer, kSiteExpertId);
        return;
    }
    if (r >= rpe) return;
    const size_t k = (size_t)n_sb * 256;
    const float v = card_row_dot<WT>(w + ((size_t)id * rpe + r) * n_sb * bm_block_bytes<WT>(), codes + slot * k, d8 + slot * (k / 128),
                                     s8 + slot * (k / 32), n_sb, lane);
    if (lane == 0) y[(size_t)slot * rpe + r] = v;
}

bool card_type(int wtype) { return wtype == BM_Q4K || wtype == BM_Q3K; }

hipError_t card_gemv(const Launch &L, int wtype, const uint8_t *w, long rows, int k, const int8_t *codes, const float *d8,
                     const int32_t *s8, int m, float *y) {
    if (!card_type(wtype)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((rows + 7) / 8), (unsigned)m);
    const uint8_t *c = reinterpret_cast<const uint8_t *>(codes);
    if (wtype == BM_Q4K) hipLaunchKernelGGL(k_card_gemv<BM_Q4K>, grid, dim3(256), 0, L.stream, w, rows, k / 256, c, d8, s8, m, y);
    else hipLaunchKernelGGL(k_card_gemv<BM_Q3K>, grid, dim3(256), 0, L.stream, w, rows, k / 256, c, d8, s8, m, y);
    return hipGetLastError();
}

hipError_t card_gemv_sel(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const int8_t *codes, const float *d8,
                         const int32_t *s8, const uint32_t *sel, int n_slots, int rows_per_expert, float *y) {
    if (!card_type(wtype)) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)n_slots * (unsigned)((rows_per_expert + 7) / 8);
    const uint8_t *c = reinterpret_cast<const uint8_t *>(codes);
    if (wtype == BM_Q4K)
        hipLaunchKernelGGL(k_card_gemv_sel<BM_Q4K>, dim3(grid), dim3(256), 0, L.stream, w, (u32)n_experts, rows_per_expert, k / 256, c,
                           d8, s8, sel, y, L.fault, L.layer);
    else
        hipLaunchKernelGGL(k_card_gemv_sel<BM_Q3K>, dim3(grid), dim3(256), 0, L.stream, w, (u32)n_experts, rows_per_expert, k / 256, c,
                           d8, s8, sel, y, L.fault, L.layer);
    return hipGetLastError();
}

} // namespace bmk
