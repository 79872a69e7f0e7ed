// Shared device pieces of the dot kernels: staging of activation columns and IQ2_XXS tables into LDS, the register
// ring a weight row streams through, the Q8_2 block quantizer, and the host-side variant dispatch.
//
// Every dot kernel follows one plan: a quad of lanes per weight row (bm_device.hpp); the token's quantized
// activation column requested first, then the row's super-blocks (128-bit loads) through a small ring of
// registers, a few super-blocks ahead of the arithmetic, all from straight-line code so the hardware's in-order
// load counter lets the arithmetic of one super-block run while the later ones are still in flight. Weights are
// read once, straight from the file's block bytes.
//
// Variants: a kernel is instantiated per weight type and per (U, NB): U the ring's size in super-blocks, NB the
// row's super-block count when it is known at compile time (0: a run-time count that U divides). The hot shapes
// (Q4_K rows of 2048 values, Q6_K rows of 768) have NB set and their stages unrolled.
#ifndef BM_STREAM_HPP
#define BM_STREAM_HPP

#include "bm_kernels.h"

#define BM_TABLE_QUAL static __device__ const
#include "iq2xxs_tables.h"

#include "bm_device.hpp"

namespace bmk {

constexpr u32 kSiteQuantColumn = 1; // crates/device/src/fault.rs:73-76
constexpr u32 kSiteExpertId = 7;    // crates/device/src/fault.rs:89
constexpr u32 kSiteF32Product = 21; // crates/device/src/fault.rs:151-155: a gate or up sum that is not finite under a clamp

// LDS bytes of the IQ2_XXS tables: 256 grid entries of 8 + 128 sign entries of 8.
constexpr int kTabBytes = 256 * 8 + 128 * 8;

constexpr int kTabBytes3 = 256 * 8 + 128 * 8; // IQ3_XXS: 256 grid entries of 8 + 128 sign entries of 8

template <int WT>
__host__ __device__ constexpr int tab_bytes() {
    return WT == BM_IQ2XXS ? kTabBytes : WT == BM_IQ3XXS ? kTabBytes3 : 0;
}

// A sign index's eight signs as two words of byte masks: 0xff where the value is negative.
__device__ __forceinline__ uint2 iq_sign_masks(int t) {
    const u32 sg = BM_KSIGNS_IQ2XS[t];
    u32 m[2];
    for (int half = 0; half < 2; half++) {
        const u32 nib = (sg >> (4 * half)) & 15u;
        m[half] = ((nib & 1) ? 0xffu : 0u) | ((nib & 2) ? 0xff00u : 0u) | ((nib & 4) ? 0xff0000u : 0u) |
                  ((nib & 8) ? 0xff000000u : 0u);
    }
    return make_uint2(m[0], m[1]);
}

// (T: the workgroup's thread count, a constant: blockDim.x is a load from the dispatch packet, in front of whatever comes next)
template <int WT, int T = 256>
__device__ __forceinline__ Iq2Tables stage_tables(uint8_t *lds) {
    Iq2Tables tb{nullptr, nullptr, nullptr};
    if constexpr (WT == BM_IQ2XXS) {
        // a grid point as eight byte selectors over the three magnitudes (8, 25, 43 -> 0, 1, 2), a sign index as eight bytes
        // of 4 where the value is negative: their sum picks a value's code byte 43 +- magnitude out of six (bm_iq2_codes)
        uint2 *grid = reinterpret_cast<uint2 *>(lds);
        uint2 *signs = reinterpret_cast<uint2 *>(lds + 256 * 8);
        for (int t = threadIdx.x; t < 256; t += T) {
            const uint64_t g = BM_IQ2XXS_GRID[t];
            const u32 lo = (u32)g, hi = (u32)(g >> 32);
            // 0x08 -> 0, 0x19 -> 1, 0x2b -> 2: bit 0 of the byte is 1 for 0x19 and 0x2b, bit 1 for 0x2b only
            grid[t] = make_uint2(((lo & 0x01010101u) + ((lo >> 1) & 0x01010101u)), ((hi & 0x01010101u) + ((hi >> 1) & 0x01010101u)));
        }
        for (int t = threadIdx.x; t < 128; t += T) {
            const uint2 m = iq_sign_masks(t);
            signs[t] = make_uint2(m.x & 0x04040404u, m.y & 0x04040404u);
        }
        tb.grid = grid;
        tb.signs = signs;
    }
    if constexpr (WT == BM_IQ3XXS) {
        uint2 *grid = reinterpret_cast<uint2 *>(lds);
        uint2 *signs = reinterpret_cast<uint2 *>(lds + 256 * 8);
        for (int t = threadIdx.x; t < 256; t += T) {
            const u32 g = BM_IQ3XXS_GRID[t]; // bytes 4 .. 62: 64 + and 64 - stay inside a byte
            grid[t] = make_uint2(0x40404040u + g, 0x40404040u - g);
        }
        for (int t = threadIdx.x; t < 128; t += T) signs[t] = iq_sign_masks(t);
        tb.grid3 = grid;
        tb.signs = signs;
    }
    return tb;
}

// `bytes` (a multiple of 8) from 8-byte aligned global memory to 8-byte aligned LDS, by the whole workgroup of T threads.
template <int T = 256>
__device__ __forceinline__ void stage_bytes(uint8_t *dst, const uint8_t *src, int bytes) {
    for (int o = threadIdx.x * 8; o < bytes; o += T * 8)
        *reinterpret_cast<uint2 *>(dst + o) = *reinterpret_cast<const uint2 *>(src + o);
}

// The same copy in two halves: R unconditional loads a thread (offsets past the end are clamped onto the last
// word, so no branch stands between them and the weight loads that follow), then the LDS stores. Memory returns
// in order, so the stores wait for these loads only. Bytes past R * 8 * T are copied afterwards by
// stage_bytes' loop (that part waits for everything in flight). T: the workgroup's thread count, a constant here: the
// built-in is read from memory, a round trip in front of the workgroup's first requests.
template <int R, int T = 256>
struct Stage {
    uint2 v[R];
    __device__ __forceinline__ void load(const uint8_t *src, int bytes) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            int o = (r * T + (int)threadIdx.x) * 8;
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
            const int o = (r * T + (int)threadIdx.x) * 8;
            if (o < bytes) *reinterpret_cast<uint2 *>(dst + o) = v[r];
        }
        for (int o = (R * T + (int)threadIdx.x) * 8; o < bytes; o += T * 8)
            *reinterpret_cast<uint2 *>(dst + o) = *reinterpret_cast<const uint2 *>(src + o);
    }
};

// The weight stream of a row is a ring of U super-blocks in registers: the first U - 1 are requested up front
// (preload), and each stage requests the super-block U - 1 ahead of the one it is about to use before it starts its
// arithmetic. A wave that asks for a whole row at once sits in the memory pipeline's queue until most of it has
// arrived and only then starts to compute; with the ring the requests trickle out between the stages and the
// arithmetic runs under the stream.
template <int WT, int U>
__device__ __forceinline__ void preload(Blk<WT> (&b)[U], const uint8_t *wrow, int q) {
#pragma unroll
    for (int u = 0; u + 1 < U; u++) b[u] = bm_load_blk<WT>(wrow, u, q);
}

// One stage: request super-block `ahead` into its ring slot, read the next stage's activation operands from LDS,
// then the arithmetic of super-block i (ring slot `slot`). The asm statements pin that order: the compiler may
// neither hoist the reads of later stages nor sink this stage's sums past them.
template <int WT, int U, class Tap>
__device__ __forceinline__ void stage_one(Blk<WT> (&b)[U], int slot, int fill, const uint8_t *wrow, int ahead,
                                          const ActView &av, int i, int act_next, int q, const Iq2Tables &tb,
                                          Act<WT> &cur, float &a0, float &a1, const Tap &tap, bool fetch = true) {
    __asm__ volatile("" ::: "memory");
    if (U > 1 && fetch) b[fill] = bm_load_blk<WT>(wrow, ahead, q);
    const Act<WT> next = bm_load_act<WT, Tap::kActive>(av, act_next, q);
    __asm__ volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    if (U == 1) b[0] = bm_load_blk<WT>(wrow, i, q);
    bm_dot_blk<WT>(b[slot], cur, i, q, tb, a0, a1, tap);
    __asm__ volatile("" : "+v"(a0), "+v"(a1)::"memory");
    __builtin_amdgcn_sched_barrier(0);
    cur = next;
}

// Row `wrow` against `m` <= M columns (LDS, `col_stride` apart); b holds the ring, preloaded.
// NB > 0: the row has NB super-blocks, the stages are unrolled; NB == 0: it has nb, a multiple of U.
// Indices past the row's end are clamped onto its last super-block: a redundant read, no branch in the stream.
template <int WT, int U, int NB, int M, class Tap>
__device__ __forceinline__ void row_dot(Blk<WT> (&b)[U], const uint8_t *wrow, const uint8_t *cols, int col_stride,
                                        int m, int nb, int q, const Iq2Tables &tb, float (&out)[M], const Tap &tap) {
    float a0[M], a1[M];
    ActView av[M];
    const int n = NB > 0 ? NB : nb;
#pragma unroll
    for (int c = 0; c < M; c++) {
        a0[c] = a1[c] = 0.0f;
        av[c] = bm_act_view<WT>(cols + (size_t)c * col_stride, n);
    }
    if constexpr (M == 1) {
        Act<WT> cur = bm_load_act<WT, Tap::kActive>(av[0], 0, q);
        if constexpr (NB > 0) {
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int ahead = i + U - 1 < NB ? i + U - 1 : NB - 1;
                stage_one<WT, U>(b, i % U, (i + U - 1) % U, wrow, ahead, av[0], i, i + 1 < NB ? i + 1 : i, q, tb, cur,
                                 a0[0], a1[0], tap, i + U - 1 < NB); // the count is known here: nothing is asked for past the end
            }
        } else {
            for (int i0 = 0; i0 < n; i0 += U) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int i = i0 + u;
                    const int ahead = i + U - 1 < n ? i + U - 1 : n - 1;
                    stage_one<WT, U>(b, u, (u + U - 1) % U, wrow, ahead, av[0], i, i + 1 < n ? i + 1 : i, q, tb, cur,
                                     a0[0], a1[0], tap);
                }
            }
        }
    } else {
        // several columns: the same ring for the weights, the activation operands read where they are used
        auto stage = [&](int slot, int fill, int i) {
            const int ahead = i + U - 1 < n ? i + U - 1 : n - 1;
            if (NB == 0 || U == 1 || i + U - 1 < NB) b[fill] = bm_load_blk<WT>(wrow, U > 1 ? ahead : i, q);
            if constexpr (WT == BM_IQ2XXS) { // the table lookups once, not once a column
                const Iq2Dec dec = bm_decode_iq2xxs(b[slot], q, tb);
#pragma unroll
                for (int c = 0; c < M; c++)
                    if (c < m) {
                        const Act<WT> a = bm_load_act<WT, Tap::kActive>(av[c], i, q);
                        bm_dot_iq2xxs_dec(b[slot], dec, a, i, q, a0[c], a1[c], tap);
                    }
            } else if constexpr (WT == BM_IQ3XXS) {
                const Iq2Dec dec = bm_decode_iq3xxs(b[slot], q, tb);
#pragma unroll
                for (int c = 0; c < M; c++)
                    if (c < m) {
                        const Act<WT> a = bm_load_act<WT, Tap::kActive>(av[c], i, q);
                        bm_dot_iq3xxs_dec(b[slot], dec, a, i, q, a0[c], a1[c], tap);
                    }
            } else if constexpr (WT == BM_IQ4XS) { // likewise the level permutes
                const Iq4Dec dec = bm_decode_iq4xs(b[slot], q);
#pragma unroll
                for (int c = 0; c < M; c++)
                    if (c < m) {
                        const Act<WT> a = bm_load_act<WT, Tap::kActive>(av[c], i, q);
                        bm_dot_iq4xs_dec(b[slot], dec, a, i, q, a0[c], a1[c], tap);
                    }
            } else if constexpr (WT == BM_Q4K || WT == BM_Q5K) { // the nibble words and the scale products
                Q45Dec dec;
                if constexpr (WT == BM_Q5K) dec = bm_decode_q45k<true>(b[slot].hdr, b[slot].qa, b[slot].qb, b[slot].qh, q & 1, q >> 1);
                else dec = bm_decode_q45k<false>(b[slot].hdr, b[slot].qa, b[slot].qb, b[slot].hdr, q & 1, q >> 1);
#pragma unroll
                for (int c = 0; c < M; c++)
                    if (c < m) {
                        const Act<WT> a = bm_load_act<WT, Tap::kActive>(av[c], i, q);
                        bm_dot_q45k_dec(dec, a, i, q & 1, q >> 1, a0[c], a1[c], tap);
                    }
            } else if constexpr (WT == BM_Q6K) {
                const Q6Dec dec = bm_decode_q6k(b[slot], q & 1, q >> 1);
#pragma unroll
                for (int c = 0; c < M; c++)
                    if (c < m) {
                        const Act<WT> a = bm_load_act<WT, Tap::kActive>(av[c], i, q);
                        bm_dot_q6k_dec(dec, a, i, q & 1, q >> 1, a0[c], a1[c], tap);
                    }
            } else {
#pragma unroll
                for (int c = 0; c < M; c++)
                    if (c < m) {
                        const Act<WT> a = bm_load_act<WT, Tap::kActive>(av[c], i, q);
                        bm_dot_blk<WT>(b[slot], a, i, q, tb, a0[c], a1[c], tap);
                    }
            }
        };
        if constexpr (NB > 0) {
#pragma unroll
            for (int i = 0; i < NB; i++) stage(i % U, (i + U - 1) % U, i);
        } else {
            for (int i0 = 0; i0 < n; i0 += U) {
#pragma unroll
                for (int u = 0; u < U; u++) stage(u, (u + U - 1) % U, i0 + u);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < M; c++) out[c] = bm_quad_finish<WT>(a0[c], a1[c]);
}

// What one q8_2 block's header needs beside its codes.
struct Q82Head {
    u32 t;    // bf16 scale bits
    int isum; // sum of the unsaturated codes
    bool bad; // a value that is not finite: NaN scale, zero codes (crates/gpu/src/lib.rs:925-933)
};

// One 32-value q8_2 block on an aligned group of 32 lanes, a value a lane (crates/qdot/src/lib.rs:3883-3904).
// Returns the stored code; *s16 is the sum of the stored codes over the lane's aligned group of 16.
__device__ __forceinline__ int q82_block(float v, Q82Head *hd, int *s16) {
    const u32 ab = bm_max32(bm_f32_bits(v) & 0x7fffffffu);
    if (ab > 0x7f7fffffu) {
        hd->t = 0x7fc0u;
        hd->isum = 0;
        hd->bad = true;
        *s16 = 0;
        return 0;
    }
    const u32 t = bm_fp32_to_bf16_bits(__fdiv_rn(bm_bits_f32(ab), 127.0f));
    const float id = bm_q82_inverse(t);
    const int q = bm_nearest_int(__fmul_rn(v, id));
    const int code = q < -128 ? -128 : (q > 127 ? 127 : q);
    const int s = bm_sum16(q);
    hd->t = t;
    hd->isum = s + (int)bm_swap16((u32)s);
    hd->bad = false;
    *s16 = bm_sum16(code);
    return code;
}

// Stores block `blk` of a device Q8_2_X4 column of nb super-blocks: codes, scale, sum and the two table entries.
// Called by the block's 32 lanes with their `lane32`.
__device__ __forceinline__ void q82_store(uint8_t *col, int nb, int blk, int lane32, int code, const Q82Head &hd,
                                          int s16) {
    uint8_t *group = col + (size_t)(blk >> 2) * BM_Q82X4_STRIDE;
    const int ir = blk & 3;
    // four codes a lane-quad -> one dword store from its first lane
    u32 c = (u32)(code & 0xff);
    c |= (bm_dpp<kDppShl1>(c) & 0xffu) << 8;
    c |= (bm_dpp<kDppShl2>(c) & 0xffffu) << 16;
    if ((lane32 & 3) == 0) *reinterpret_cast<u32 *>(group + 16 + 32 * ir + lane32) = c;
    if ((lane32 & 15) == 0)
        *reinterpret_cast<int *>(col + (size_t)nb * (BM_Q82_SB_REF + 64) + 4 * (2 * blk + (lane32 >> 4))) = s16;
    if (lane32 == 0) {
        *reinterpret_cast<unsigned short *>(group + 2 * ir) = (unsigned short)hd.t;
        *reinterpret_cast<unsigned short *>(group + 8 + 2 * ir) = (unsigned short)(short)hd.isum;
        const float d8 = bm_bf16_to_f32(hd.t);
        *reinterpret_cast<float2 *>(col + (size_t)nb * BM_Q82_SB_REF + 8 * blk) =
            make_float2(d8, __fmul_rn(d8, (float)(short)hd.isum));
    }
}

// One 32-value q8_2 block held eight values a lane by four consecutive lanes (the in-kernel token quantizer). Returns whether
// the block holds a value that is not finite; RAISE: raises QuantColumn for it as well (without: the caller does, where the
// fault word's address has come in).
template <bool RAISE = true>
__device__ __forceinline__ bool q82_quad8(const float (&v)[8], uint8_t *col, int nb, int blk, int lane4, u32 *fault,
                                          u32 layer) {
    u32 ab = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const u32 a = bm_f32_bits(v[k]) & 0x7fffffffu;
        ab = a > ab ? a : ab;
    }
    u32 o;
    o = bm_dpp<kDppXor1>(ab), ab = o > ab ? o : ab;
    o = bm_dpp<kDppXor2>(ab), ab = o > ab ? o : ab;
    uint8_t *group = col + (size_t)(blk >> 2) * BM_Q82X4_STRIDE;
    const int ir = blk & 3;
    u32 t;
    int isum = 0, csum = 0;
    u32 c0 = 0, c1 = 0;
    const bool bad = ab > 0x7f7fffffu;
    if (bad) {
        t = 0x7fc0u;
        if constexpr (RAISE)
            if (lane4 == 0) bm_raise(fault, layer, kSiteQuantColumn);
    } else {
        t = bm_fp32_to_bf16_bits(__fdiv_rn(bm_bits_f32(ab), 127.0f));
        const float id = bm_q82_inverse(t);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int qv = bm_nearest_int(__fmul_rn(v[k], id));
            const int code = qv < -128 ? -128 : (qv > 127 ? 127 : qv);
            isum += qv;
            csum += code;
            if (k < 4)
                c0 |= (u32)(code & 0xff) << (8 * k);
            else
                c1 |= (u32)(code & 0xff) << (8 * (k - 4));
        }
    }
    isum += (int)bm_dpp<kDppXor1>((u32)isum);
    isum += (int)bm_dpp<kDppXor2>((u32)isum);
    csum += (int)bm_dpp<kDppXor1>((u32)csum); // lanes (0,1): first 16 values, lanes (2,3): second
    *reinterpret_cast<uint2 *>(group + 16 + 32 * ir + 8 * lane4) = make_uint2(c0, c1);
    if ((lane4 & 1) == 0)
        *reinterpret_cast<int *>(col + (size_t)nb * (BM_Q82_SB_REF + 64) + 4 * (2 * blk + (lane4 >> 1))) = csum;
    if (lane4 == 0) {
        *reinterpret_cast<unsigned short *>(group + 2 * ir) = (unsigned short)t;
        *reinterpret_cast<unsigned short *>(group + 8 + 2 * ir) = (unsigned short)(short)isum;
        const float d8 = bm_bf16_to_f32(t);
        *reinterpret_cast<float2 *>(col + (size_t)nb * BM_Q82_SB_REF + 8 * blk) =
            make_float2(d8, __fmul_rn(d8, (float)(short)isum));
    }
    return bad;
}

// One 256-value block of a Q8_K column by one wave, four consecutive values a lane: k_quantize_q8k's operations on the
// same operands (crates/qdot/src/lib.rs:1787-1809), the block's maximum and the sums met through lane exchanges.
// `o` is the block's 296 bytes (LDS or global memory).
__device__ __forceinline__ void q8k_wave_block(const float4 x4, uint8_t *o, int lane, u32 *fault, u32 layer) {
    const float v[4] = {x4.x, x4.y, x4.z, x4.w};
    // the largest magnitude: a maximum of the sign-less bit patterns over the wave
    u32 mine_ab = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const u32 a = bm_f32_bits(v[k]) & 0x7fffffffu;
        mine_ab = a > mine_ab ? a : mine_ab;
    }
    const u32 half_ab = bm_max32(mine_ab); // over each half of the wave
    const u32 lo_ab = (u32)__builtin_amdgcn_readlane((int)half_ab, 0), hi_ab = (u32)__builtin_amdgcn_readlane((int)half_ab, 32);
    const u32 ab = lo_ab > hi_ab ? lo_ab : hi_ab;
    // its first holder (value 4 * lane + k): the lowest lane among those that hold it at k, the lowest such value
    int first = 1 << 20;
    float max = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const unsigned long long holders = __ballot((bm_f32_bits(v[k]) & 0x7fffffffu) == ab);
        if (holders) { // uniform over the wave
            const int at = __builtin_ctzll(holders);
            const float val = bm_bits_f32((u32)__builtin_amdgcn_readlane((int)bm_f32_bits(v[k]), at));
            if (4 * at + k < first) first = 4 * at + k, max = val;
        }
    }
    float d;
    int code[4] = {0, 0, 0, 0};
    if (ab > 0x7f7fffffu) {
        if (lane == 0) bm_raise(fault, layer, kSiteQuantColumn);
        d = bm_bits_f32(0x7fc00000u);
    } else if (ab == 0) {
        d = 0.0f;
    } else {
        const float iscale = __fdiv_rn(-127.0f, max);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int qv = bm_nearest_int(__fmul_rn(iscale, v[k]));
            qv = qv > 127 ? 127 : qv;
            code[k] = (int)(signed char)(qv & 0xff); // `as i8`: the low byte
        }
        d = __fdiv_rn(1.0f, iscale);
    }
    *reinterpret_cast<u32 *>(o + 8 + 4 * lane) = (u32)(code[0] & 0xff) | ((u32)(code[1] & 0xff) << 8) |
                                                 ((u32)(code[2] & 0xff) << 16) | ((u32)(code[3] & 0xff) << 24);
    int sum = code[0] + code[1] + code[2] + code[3]; // sixteen codes a sum: four lanes
    sum += (int)bm_dpp<kDppXor1>((u32)sum);
    sum += (int)bm_dpp<kDppXor2>((u32)sum);
    if ((lane & 3) == 0) *reinterpret_cast<unsigned short *>(o + 264 + 2 * (lane >> 2)) = (unsigned short)(short)sum;
    if (lane == 0) {
        *reinterpret_cast<float *>(o) = d;
        *reinterpret_cast<u32 *>(o + 4) = 0u;
    }
}

// The gate/up exchange of the eight lanes of an output: lanes 0..3 hold the gate dot, 4..7 the up dot.
__device__ __forceinline__ float swiglu_of_pair(float v, int which, GateRule rule, u32 *fault, u32 layer) {
    // both moves run on every lane: a lane-crossing move under a divergent branch reads switched-off lanes as 0
    const float from_above = bm_dppf<kDppShl4>(v), from_below = bm_dppf<kDppShr4>(v);
    bool odd;
    const float hv = bm_gate_rule(rule.act, rule.limit, which ? from_below : v, which ? v : from_above, odd);
    if (odd) bm_raise(fault, layer, kSiteF32Product);
    return hv;
}

// An argument read from the launch's argument block at the place in the code where this call stands. The first fourteen
// words of the block are in registers when a wave starts; an argument behind them is a scalar load, and the compiler asks
// for it at the top of the kernel: scalar loads come back in any order, so the first wait for one of them - the expert id's -
// would be a wait for those words as well. The arguments the head of a decode launch does not need stand at the end of its
// list as one struct, which the kernel does not touch, and are read through this behind the launch's first requests.
template <class T>
__device__ __forceinline__ T bm_kernarg_at(unsigned offset) {
    static_assert(sizeof(T) % 4 == 0, "whole words");
    typedef __attribute__((address_space(4))) const uint8_t *Block;
    typedef __attribute__((address_space(4))) const u32 *Words;
    const Words from = (Words)((Block)__builtin_amdgcn_kernarg_segment_ptr() + offset);
    struct Raw {
        u32 w[sizeof(T) / 4];
    } raw;
#pragma unroll
    for (unsigned i = 0; i < sizeof(T) / 4; i++) raw.w[i] = from[i];
    return __builtin_bit_cast(T, raw);
}

// A pointer that came out of bm_kernarg_at's words, as what a pointer argument is: an address in global memory (without this
// the compiler takes it for one that may also lie in LDS or scratch, and every wait for a vector load behind its first use is
// a wait for all of them).
template <class P>
__device__ __forceinline__ P *bm_global(P *p) {
    return (P *)(__attribute__((address_space(1))) P *)(uintptr_t)p;
}

// The 32 values a workgroup produced (hbuf, LDS) as block `rb` of column `hcol`, by the first 32 threads.
__device__ __forceinline__ void quantize_h_block(const float *hbuf, uint8_t *hcol, int nb_h, int rb, int tid,
                                                 u32 *fault, u32 layer) {
    Q82Head hd;
    int s16;
    const int code = q82_block(hbuf[tid], &hd, &s16);
    if (hd.bad && tid == 0) bm_raise(fault, layer, kSiteQuantColumn);
    q82_store(hcol, nb_h, rb, tid, code, hd, s16);
}

// ------------------------------------------------------------------------------------- grouping by expert

// Exclusive prefix sum over the 1024 threads of a workgroup (value v of thread tid); *total gets the sum.
// `scratch` holds 17 words of LDS. Every thread calls it.
__device__ __forceinline__ u32 block_scan_1024(u32 v, u32 *scratch, u32 *total) {
    const u32 tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    u32 inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const u32 o = (u32)__shfl_up((int)inc, d, 64);
        if (lane >= (u32)d) inc += o;
    }
    if (lane == 63) scratch[wave] = inc;
    __syncthreads();
    if (tid == 0) {
        u32 at = 0;
        for (int w = 0; w < 16; w++) {
            const u32 c = scratch[w];
            scratch[w] = at;
            at += c;
        }
        scratch[16] = at;
    }
    __syncthreads();
    *total = scratch[16];
    return scratch[wave] + inc - v;
}


// The slots 0 .. n of a workgroup of 1024 threads listed by bucket (an expert, or one more bucket a caller adds),
// ascending slot order inside a bucket - the stable counting sort both slot tables are. The slots are cut into up
// to 16 chunks, a wave a chunk: counts per (chunk, bucket) give every chunk its place inside every bucket's run, so
// the waves place their slots independently; inside a wave 64 consecutive slots are placed at a time, each lane's
// rank among the lanes of its bucket read off the ballots of the bucket's bits.
constexpr u32 kNoBucket = 0xffffffffu;
constexpr int kGroupHist = 8192, kGroupWaves = 16, kGroupBuckets = 1025;
constexpr u32 kGroupThreads = 1024; // the workgroups these routines run in (a constant: blockDim.x is a load from the dispatch packet)
struct GroupLds {
    u32 hist[kGroupHist + kGroupWaves]; // [chunk][bucket]: the chunk's next place inside the bucket's run
    u32 base[kGroupBuckets + 1];        // bucket b's run is list[base[b] .. base[b + 1]]
    u32 scan[17];
};

// The lanes of the wave whose bucket is this lane's (a lane that is not live: the lanes that are not), read off the
// ballots of the bucket's bits.
__device__ __forceinline__ unsigned long long lanes_of_my_bucket(u32 b, bool live, int bits) {
    const unsigned long long all_live = __ballot(live);
    unsigned long long same = live ? all_live : ~all_live;
    for (int k = 0; k < bits; k++) {
        const unsigned long long set = __ballot(live && ((b >> k) & 1u));
        same &= (live && ((b >> k) & 1u)) ? set : ~set;
    }
    return same;
}

// bucket_of(s): slot s's bucket below n_buckets, or kNoBucket for a slot that joins no run. Called twice a slot.
// Every thread of the workgroup calls group_slots; afterwards g.base holds the runs' bounds.
template <class BucketOf>
__device__ __forceinline__ void group_slots(GroupLds &g, u32 n, u32 n_buckets, u32 *list, const BucketOf &bucket_of) {
    const u32 tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    u32 chunks = (u32)kGroupHist / n_buckets;
    chunks = chunks < (u32)kGroupWaves ? chunks : (u32)kGroupWaves;
    const u32 per = ((n + chunks - 1) / chunks + 63) & ~63u; // whole batches of 64 a chunk
    const u32 lo = wave * per, hi = lo + per < n ? lo + per : n;
    for (u32 i = tid; i < chunks * n_buckets; i += kGroupThreads) g.hist[i] = 0;
    __syncthreads();
    if (wave < chunks)
        for (u32 s = lo + lane; s < hi; s += 64) {
            const u32 b = bucket_of(s);
            if (b != kNoBucket) atomicAdd(&g.hist[wave * n_buckets + b], 1u);
        }
    __syncthreads();
    u32 count = 0;
    for (u32 b = tid; b < n_buckets; b += kGroupThreads) { // a chunk's count -> its offset inside the bucket's run
        u32 sum = 0;
        for (u32 c = 0; c < chunks; c++) {
            const u32 v = g.hist[c * n_buckets + b];
            g.hist[c * n_buckets + b] = sum;
            sum += v;
        }
        if (b < 1024) count = sum;
        else g.base[kGroupBuckets] = sum; // bucket 1024's count, parked
    }
    u32 total;
    const u32 at = block_scan_1024(count, g.scan, &total);
    if (tid < n_buckets) g.base[tid] = at;
    if (tid == 0) {
        if (n_buckets == (u32)kGroupBuckets) {
            const u32 last = g.base[kGroupBuckets];
            g.base[1024] = total;
            g.base[kGroupBuckets] = total + last;
        } else {
            g.base[n_buckets] = total;
        }
    }
    __syncthreads();
    if (wave < chunks) {
        const int bits = 32 - __builtin_clz(n_buckets | 1u);
        for (u32 s0 = lo; s0 < hi; s0 += 64) {
            const u32 s = s0 + lane;
            const u32 b = s < hi ? bucket_of(s) : kNoBucket;
            const bool live = b != kNoBucket;
            unsigned long long same = __ballot(live);
            for (int k = 0; k < bits; k++) {
                const unsigned long long set = __ballot((b >> k) & 1u);
                same &= ((b >> k) & 1u) ? set : ~set;
            }
            const int leader = live ? __builtin_ctzll(same) : (int)lane;
            u32 first = 0;
            if (live && lane == (u32)leader) first = atomicAdd(&g.hist[wave * n_buckets + b], (u32)__builtin_popcountll(same));
            first = (u32)__shfl((int)first, leader, 64);
            if (live) list[g.base[b] + first + (u32)__builtin_popcountll(same & ((1ull << lane) - 1ull))] = s;
        }
    }
    __syncthreads();
}

// The same list made by several workgroups of 1024 threads, none waiting for another: the slots are cut into
// group_parts(n, n_buckets) parts and workgroup `part` places the slots of its part. Every workgroup counts all the slots
// (light work: two counters a bucket, the ids come from the cache after the first reader), so each knows every run's start
// and how many of a bucket's slots lie in the parts before its own; it then counts its own part once more, a sub-part a
// wave, and its waves place their sub-parts as group_slots' waves place their chunks. `off` holds n_buckets words of LDS.
// Afterwards g.base holds the runs' bounds in every workgroup; a workgroup whose `part` is group_parts(..) or more places
// nothing and has the bounds sooner than the others are done (for what a caller makes of the bounds alone).
__host__ __device__ inline u32 group_chunks(u32 n_buckets) {
    const u32 chunks = (u32)kGroupHist / n_buckets;
    return chunks < (u32)kGroupWaves ? chunks : (u32)kGroupWaves;
}
__host__ __device__ inline u32 group_chunk_len(u32 n, u32 chunks) { return ((n + chunks - 1) / chunks + 63) & ~63u; }
__host__ __device__ inline u32 group_parts(u32 n, u32 n_buckets) {
    const u32 per = group_chunk_len(n, group_chunks(n_buckets));
    return n ? (n + per - 1) / per : 1;
}

template <class BucketOf>
__device__ __forceinline__ void group_slots_part(GroupLds &g, u32 *off, u32 n, u32 n_buckets, u32 part, u32 *list,
                                                 const BucketOf &bucket_of) {
    const u32 tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const u32 chunks = group_chunks(n_buckets);
    const u32 per = group_chunk_len(n, chunks);
    const u32 p_lo = part * per < n ? part * per : n, p_hi = p_lo + per < n ? p_lo + per : n;
    const int bits = 32 - __builtin_clz(n_buckets | 1u);
    // All the slots, thread by thread, four loads at a time: a bucket's count in the parts before this one, and its count
    // from this part on. A lane adds to one of up to 16 copies of the counters, picked by its number, on banks of their
    // own (an odd stride): with a popular expert a quarter of a wave's lanes would otherwise queue up on one word.
    const u32 rstride = 2 * n_buckets + 1;
    u32 reps = 16;
    while (reps > 1 && reps * rstride > (u32)kGroupHist) reps >>= 1;
    u32 *mine = g.hist + (lane & (reps - 1)) * rstride;
    for (u32 i = tid; i < reps * rstride; i += kGroupThreads) g.hist[i] = 0;
    __syncthreads();
    for (u32 s0 = tid; s0 < n; s0 += 4 * kGroupThreads) {
        u32 b[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const u32 s = s0 + (u32)j * kGroupThreads;
            b[j] = s < n ? bucket_of(s) : kNoBucket;
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (b[j] != kNoBucket) atomicAdd(&mine[(s0 + (u32)j * kGroupThreads < p_lo ? 0u : n_buckets) + b[j]], 1u);
    }
    __syncthreads();
    u32 count = 0;
    for (u32 b = tid; b < n_buckets; b += kGroupThreads) {
        u32 bef = 0, aft = 0;
        for (u32 r = 0; r < reps; r++) {
            bef += g.hist[r * rstride + b];
            aft += g.hist[r * rstride + n_buckets + b];
        }
        off[b] = bef;
        if (b < 1024) count = bef + aft;
        else g.base[kGroupBuckets] = bef + aft; // bucket 1024's count, parked
    }
    u32 total;
    const u32 at = block_scan_1024(count, g.scan, &total);
    if (tid < n_buckets) g.base[tid] = at;
    if (tid == 0) {
        if (n_buckets == (u32)kGroupBuckets) {
            const u32 last = g.base[kGroupBuckets];
            g.base[1024] = total;
            g.base[kGroupBuckets] = total + last;
        } else {
            g.base[n_buckets] = total;
        }
    }
    for (u32 i = tid; i < chunks * n_buckets; i += kGroupThreads) g.hist[i] = 0; // (its readers passed the scan's barriers)
    __syncthreads();
    if (p_lo >= n) return; // a workgroup past the last part: the bounds only
    // this part once more, a sub-part a wave
    const u32 sub = group_chunk_len(p_hi - p_lo, chunks);
    const u32 lo = p_lo + wave * sub < p_hi ? p_lo + wave * sub : p_hi, hi = lo + sub < p_hi ? lo + sub : p_hi;
    if (wave < chunks)
        for (u32 s0 = lo; s0 < hi; s0 += 64) {
            const u32 s = s0 + lane;
            const u32 b = s < hi ? bucket_of(s) : kNoBucket;
            const unsigned long long same = lanes_of_my_bucket(b, b != kNoBucket, bits);
            if (b != kNoBucket && lane == (u32)__builtin_ctzll(same)) atomicAdd(&g.hist[wave * n_buckets + b], (u32)__builtin_popcountll(same));
        }
    __syncthreads();
    for (u32 b = tid; b < n_buckets; b += kGroupThreads) { // a sub-part's count -> its first place in the list
        u32 sum = g.base[b] + off[b];
        for (u32 c = 0; c < chunks; c++) {
            const u32 v = g.hist[c * n_buckets + b];
            g.hist[c * n_buckets + b] = sum;
            sum += v;
        }
    }
    __syncthreads();
    if (wave < chunks) {
        for (u32 s0 = lo; s0 < hi; s0 += 64) {
            const u32 s = s0 + lane;
            const u32 b = s < hi ? bucket_of(s) : kNoBucket;
            const bool live = b != kNoBucket;
            const unsigned long long same = lanes_of_my_bucket(b, live, bits);
            const int leader = live ? __builtin_ctzll(same) : (int)lane;
            u32 first = 0;
            if (live && lane == (u32)leader) first = atomicAdd(&g.hist[wave * n_buckets + b], (u32)__builtin_popcountll(same));
            first = (u32)__shfl((int)first, leader, 64);
            if (live) list[first + (u32)__builtin_popcountll(same & ((1ull << lane) - 1ull))] = s;
        }
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------------------- launch helpers

template <typename K>
static hipError_t allow_lds(K kernel, size_t lds) {
    if (lds <= 64 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)lds);
}

// Picks the kernel variant for a row of nb super-blocks and runs CALL_BODY with WT, U and NB as constants. Each
// type lists the hot shape first (its count known at compile time, stages unrolled), then a ring of two for even
// counts, then one super-block at a time, which divides every row.
constexpr int kRingQ4K = 4, kRingQ5K = 4, kRingQ6K = 3;
#define BM_VARIANT(T, UU, NN)                                                                                          \
    {                                                                                                                  \
        constexpr int WT = T, U = UU, NB = NN;                                                                         \
        CALL_BODY;                                                                                                     \
    }
#define BM_DISPATCH(wtype, nb)                                                                                         \
    switch (wtype) {                                                                                                   \
    case BM_Q3K:                                                                                                       \
        if ((nb) % 2 == 0) BM_VARIANT(BM_Q3K, 2, 0)                                                                    \
        else BM_VARIANT(BM_Q3K, 1, 0)                                                                                  \
        break;                                                                                                         \
    case BM_Q4K:                                                                                                       \
        if ((nb) == 8) BM_VARIANT(BM_Q4K, kRingQ4K, 8)                                                                 \
        else if ((nb) % 2 == 0) BM_VARIANT(BM_Q4K, 2, 0)                                                               \
        else BM_VARIANT(BM_Q4K, 1, 0)                                                                                  \
        break;                                                                                                         \
    case BM_Q5K:                                                                                                       \
        if ((nb) == 8) BM_VARIANT(BM_Q5K, kRingQ5K, 8)                                                                 \
        else if ((nb) % 2 == 0) BM_VARIANT(BM_Q5K, 2, 0)                                                                    \
        else BM_VARIANT(BM_Q5K, 1, 0)                                                                                  \
        break;                                                                                                         \
    case BM_Q6K:                                                                                                       \
        if ((nb) == 3) BM_VARIANT(BM_Q6K, kRingQ6K, 3)                                                                 \
        else if ((nb) % 2 == 0) BM_VARIANT(BM_Q6K, 2, 0)                                                               \
        else BM_VARIANT(BM_Q6K, 1, 0)                                                                                  \
        break;                                                                                                         \
    case BM_IQ2XXS:                                                                                                    \
        if ((nb) % 2 == 0) BM_VARIANT(BM_IQ2XXS, 2, 0)                                                                 \
        else BM_VARIANT(BM_IQ2XXS, 1, 0)                                                                               \
        break;                                                                                                         \
    case BM_IQ3XXS:                                                                                                    \
        if ((nb) % 2 == 0) BM_VARIANT(BM_IQ3XXS, 2, 0)                                                                 \
        else BM_VARIANT(BM_IQ3XXS, 1, 0)                                                                               \
        break;                                                                                                         \
    case BM_IQ4XS:                                                                                                     \
        if ((nb) % 2 == 0) BM_VARIANT(BM_IQ4XS, 2, 0)                                                                  \
        else BM_VARIANT(BM_IQ4XS, 1, 0)                                                                                \
        break;                                                                                                         \
    default:                                                                                                           \
        return hipErrorInvalidValue;                                                                                   \
    }

// One 256-value block of a Q8_K column by a workgroup of 256 threads, thread t holding value t (crates/qdot/src/lib.rs:
// 1787-1809): the scale from the largest magnitude, the first on ties; codes nearest(iscale v) capped at 127; the sixteen
// 16-value sums. `o`: the block's 296 bytes.
__device__ __forceinline__ void q8k_block_by_workgroup(float v, uint8_t *o, u32 *fault, u32 layer) {
    __shared__ unsigned long long s_key[4];
    __shared__ int s_codes[256];
    __shared__ float s_vals[256];
    const int tid = threadIdx.x;
    s_vals[tid] = v;
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
        const float max = s_vals[first];
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

static inline int tab_bytes_rt(int wtype) { return wtype == BM_IQ2XXS ? kTabBytes : wtype == BM_IQ3XXS ? kTabBytes3 : 0; }

} // namespace bmk

#endif // BM_STREAM_HPP
