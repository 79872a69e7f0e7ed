// Device-side building blocks of the quantized row dots on gfx950 (wave64).
//
// Lane map ("quad"): one weight row is dotted by four consecutive lanes. The CPU path this library reproduces
// (crates/qdot/src/lib.rs:4363-4447 Q4_K, :4991-5090 Q5_K, :4776-4874 Q6_K, :8677-8724 IQ2_XXS) keeps eight f32 accumulators per
// row and walks the super-blocks in order; here each lane of the quad owns two of the eight and walks every
// super-block of the row itself, so each accumulator sees the reference's fused multiply-adds in the reference's
// order and the final butterfly over the quad is the reference's closing sum ((t0+t2)+(t1+t3), t_l = acc_l +
// acc_{l+4}). The integer sums are formed with v_dot4_i32_i8 over the same 16-value (Q4_K, Q5_K, Q6_K) or 4-value
// (IQ2_XXS) spans the reference's i32 lanes cover; they are exact, so their inner order is free.
//
// Activation columns on the device. A Q8_K column (IQ2_XXS weights) is the CPU path's bytes, 296 a super-block.
// A Q8_2_X4 column (Q4_K, Q5_K, Q6_K weights) is the CPU path's bytes (288 a super-block) followed by two tables the
// quantizers write beside them so the dots need no per-block unpacking: for each 32-value block the pair
// (d8 as f32, d8 * (f32)isum) - the second is the product the reference forms first in its min term - and for each
// 16 values the i32 sum of the stored codes (Q6_K's -32 offset comes out through it). nb super-blocks give
// nb * 288 bytes, then nb * 64 table bytes, then nb * 64 sum bytes: 416 * nb in all.
//
// Build: -ffp-contract=off (a product meets a sum in one rounding only where fmaf is written), f32 denormals
// kept, correctly rounded f32 divide (hipcc's defaults for gfx950).
#ifndef BM_DEVICE_HPP
#define BM_DEVICE_HPP

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32;

#define BM_Q3K 11
#define BM_Q4K 12
#define BM_Q5K 13
#define BM_Q6K 14
#define BM_IQ2XXS 16
#define BM_IQ3XXS 18
#define BM_IQ4XS 23

#define BM_Q3K_BLOCK 110
#define BM_Q4K_BLOCK 144
#define BM_Q5K_BLOCK 176
#define BM_Q6K_BLOCK 210
#define BM_IQ2XXS_BLOCK 66
#define BM_IQ3XXS_BLOCK 98
#define BM_IQ4XS_BLOCK 136
#define BM_Q82X4_STRIDE 144
#define BM_Q8K_STRIDE 296
#define BM_Q82_SB_REF 288 // reference bytes of one super-block of a Q8_2_X4 column
#define BM_Q82_SB_EXT 416 // with the two tables

// ------------------------------------------------------------------------------------------------ scalars

__device__ __forceinline__ float bm_bits_f32(u32 u) { return __uint_as_float(u); }
__device__ __forceinline__ u32 bm_f32_bits(float f) { return __float_as_uint(f); }

// f16 bits -> f32: v_cvt_f32_f16, exact for every f16 (subnormals included; f16 denormals are on).
__device__ __forceinline__ float bm_half_to_f32(u32 h16) { return __half2float(__ushort_as_half((unsigned short)h16)); }

__device__ __forceinline__ float bm_bf16_to_f32(u32 b16) { return bm_bits_f32(b16 << 16); }

// crates/gguf/src/quant.rs:544-551.
__device__ __forceinline__ u32 bm_fp32_to_bf16_bits(float s) {
    u32 u = bm_f32_bits(s);
    if ((u & 0x7fffffffu) > 0x7f800000u) return ((u >> 16) | 64u) & 0xffffu;
    return ((u + (0x7fffu + ((u >> 16) & 1u))) >> 16) & 0xffffu;
}

// Round to nearest even through one f32 add (crates/gguf/src/quant.rs:2222-2226). __fadd_rn keeps the add from
// being folded or fused whatever the caller's surrounding arithmetic.
__device__ __forceinline__ int bm_nearest_int(float v) {
    float val = __fadd_rn(v, 12582912.0f);
    return (int)(bm_f32_bits(val) & 0x007fffffu) - 0x00400000;
}

// crates/gguf/src/quant.rs:2237-2241.
__device__ __forceinline__ float bm_q82_inverse(u32 t) {
    float d = bm_bf16_to_f32(t);
    float id = d > 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
    return (bm_f32_bits(id) & 0x7fffffffu) < 0x7f800000u ? id : 0.0f;
}

// The correctly rounded square root of a positive normal f32. The hardware's is within a unit in the last place (and
// the runtime's "rn" form compiles to it as it stands), so the two neighbours are tried against the exact residuals:
// x <= s_down * s puts sqrt(x) below the midpoint of s_down and s, x > s_up * s above that of s and s_up.
__device__ __forceinline__ float bm_sqrt_rn(float x) {
    float s = __builtin_amdgcn_sqrtf(x);
    if (!(x > 0.0f) || bm_f32_bits(x) >= 0x7f800000u) return s; // zero, negative, infinite, NaN: the instruction's own result
    const float s_dn = bm_bits_f32(bm_f32_bits(s) - 1u), s_up = bm_bits_f32(bm_f32_bits(s) + 1u);
    const float vp = fmaf(-s_dn, s, x), vs = fmaf(-s_up, s, x);
    s = vp <= 0.0f ? s_dn : s;
    s = vs > 0.0f ? s_up : s;
    return s;
}

__device__ __forceinline__ int bm_sdot4(u32 a, u32 b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

// a * b + c for factors inside 24 signed bits (every integer the IQ cores scale is): one full-rate instruction where
// the 32-bit multiply takes four times as long.
__device__ __forceinline__ int bm_mad24(int a, int b, int c) { return __mul24(a, b) + c; }
__device__ __forceinline__ int bm_mul24(int a, int b) { return __mul24(a, b); }

// 16 bytes from an address of any alignment (global memory takes unaligned vector loads on this target).
__device__ __forceinline__ uint4 bm_ld16u(const uint8_t *p) {
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}

__device__ __forceinline__ uint4 bm_ld16(const uint8_t *p) { return *reinterpret_cast<const uint4 *>(p); }

__device__ __forceinline__ u32 bm_ld2u(const uint8_t *p) {
    unsigned short v;
    __builtin_memcpy(&v, p, 2);
    return v;
}

// ------------------------------------------------------------------------------------------ lane exchange

// Data-parallel-primitive moves: no LDS traffic, a few cycles each. CTRL is the DPP control word.
template <int CTRL>
__device__ __forceinline__ u32 bm_dpp(u32 v) {
    return (u32)__builtin_amdgcn_mov_dpp((int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float bm_dppf(float v) {
    return bm_bits_f32(bm_dpp<CTRL>(bm_f32_bits(v)));
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7 - i inside each 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15 - i inside each 16
constexpr int kDppShl1 = 0x101, kDppShl2 = 0x102, kDppShl4 = 0x104; // lane i reads lane i + n of its row of 16
constexpr int kDppShr4 = 0x114;                                     // lane i reads lane i - 4

__device__ __forceinline__ float bm_quad_xor1(float v) { return bm_dppf<kDppXor1>(v); }
__device__ __forceinline__ float bm_quad_xor2(float v) { return bm_dppf<kDppXor2>(v); }
__device__ __forceinline__ u32 bm_quad_bcast(u32 v, int k) {
    switch (k) {
    case 0:
        return bm_dpp<0x00>(v);
    case 1:
        return bm_dpp<0x55>(v);
    case 2:
        return bm_dpp<0xAA>(v);
    default:
        return bm_dpp<0xFF>(v);
    }
}

// Lanes 16..31 <-> 0..15 of each half wave (ds_swizzle bit mode: xor 0x10; goes through the LDS crossbar only).
__device__ __forceinline__ u32 bm_swap16(u32 v) { return (u32)__builtin_amdgcn_ds_swizzle((int)v, 0x401F); }

// All-reduce over each aligned group of 32 lanes: every lane ends with the group's maximum / sum.
__device__ __forceinline__ u32 bm_max32(u32 v) {
    u32 o;
    o = bm_dpp<kDppXor1>(v), v = o > v ? o : v;
    o = bm_dpp<kDppXor2>(v), v = o > v ? o : v;
    o = bm_dpp<kDppHalfMirror>(v), v = o > v ? o : v;
    o = bm_dpp<kDppMirror>(v), v = o > v ? o : v;
    o = bm_swap16(v), v = o > v ? o : v;
    return v;
}
__device__ __forceinline__ int bm_sum16(int v) { // over each aligned group of 16 lanes
    v += (int)bm_dpp<kDppXor1>((u32)v);
    v += (int)bm_dpp<kDppXor2>((u32)v);
    v += (int)bm_dpp<kDppHalfMirror>((u32)v);
    v += (int)bm_dpp<kDppMirror>((u32)v);
    return v;
}

// ------------------------------------------------------------------------------------------ fault raising

// crates/device/src/fault.rs:9-60: word 0 takes (layer << 8) | site by atomic minimum, word 1 + layer the site bit.
__device__ __forceinline__ void bm_raise(u32 *fault, u32 layer, u32 site) {
    atomicMin(&fault[0], (layer << 8) | site);
    atomicOr(&fault[1 + layer], 1u << site);
}

// -------------------------------------------------------------------------------------------------- taps

// A tap sees the exact integers a core forms. The launchers pass NoTap (everything folds away); the
// verification kernel passes one that stores them, so it checks the code the launchers run.
struct NoTap {
    static constexpr bool kActive = false;
    __device__ __forceinline__ void q4k(int, int, int, int) const {}
    __device__ __forceinline__ void q4k_isum(int, int, int) const {}
    __device__ __forceinline__ void q6k(int, int, int) const {}
    __device__ __forceinline__ void iq2(int, int, int, int) const {}
    __device__ __forceinline__ void iq4_sub(int, int, int) const {}
    __device__ __forceinline__ void iq4_lane(int, int, int) const {}
};

// ------------------------------------------------------------------------------------------ activation view

// One activation column in LDS (or global memory): its reference bytes and, for the Q8_2_X4 form, the tables.
struct ActView {
    const uint8_t *col;
    const uint8_t *tbl; // nb * 8 pairs (f32 d8, f32 d8 * isum)
    const uint8_t *s16; // nb * 16 i32 sums of 16 stored codes
};

// The types that dot against a Q8_K column (crates/gguf/src/qtype.rs host_act); the others take Q8_2_X4.
__host__ __device__ constexpr bool bm_takes_q8k(int wt) {
    return wt == BM_Q3K || wt == BM_IQ2XXS || wt == BM_IQ3XXS || wt == BM_IQ4XS;
}

// Bytes of one column of nb super-blocks on the device, in the form type WT dots against.
template <int WT>
__host__ __device__ constexpr int bm_act_col_bytes(int nb) {
    return bm_takes_q8k(WT) ? nb * BM_Q8K_STRIDE : nb * BM_Q82_SB_EXT;
}

template <int WT>
__device__ __forceinline__ ActView bm_act_view(const uint8_t *col, int nb) {
    if (bm_takes_q8k(WT)) return ActView{col, nullptr, nullptr};
    return ActView{col, col + (size_t)nb * BM_Q82_SB_REF, col + (size_t)nb * (BM_Q82_SB_REF + 64)};
}

// ------------------------------------------------------------------------------------------------- cores

template <int WT>
struct Blk;

// ---- Q4_K: lane (c = q & 1, h = q >> 1) owns accumulators l = 4h + 2c and 4h + 2c + 1 of the reference's eight.
// It reads bytes [32c + 16h, +16) of the first and of the second 64 code bytes: low nibbles are the 16 values of
// half h of sub-block 2c (resp. 4 + 2c), high nibbles those of sub-block 2c + 1 (resp. 5 + 2c).
template <>
struct Blk<BM_Q4K> {
    uint4 hdr, qa, qb;
};

__device__ __forceinline__ Blk<BM_Q4K> bm_load_q4k(const uint8_t *wrow, int i, int c, int h) {
    const uint8_t *wb = wrow + (size_t)i * BM_Q4K_BLOCK;
    Blk<BM_Q4K> b;
    b.hdr = bm_ld16(wb);
    b.qa = bm_ld16(wb + 16 + 32 * c + 16 * h);
    b.qb = bm_ld16(wb + 16 + 64 + 32 * c + 16 * h);
    return b;
}

__device__ __forceinline__ void bm_q4_dot16(uint4 q, uint4 alo, uint4 ahi, int &lo, int &hi) {
    const u32 m = 0x0f0f0f0fu;
    lo = bm_sdot4(q.x & m, alo.x, 0);
    lo = bm_sdot4(q.y & m, alo.y, lo);
    lo = bm_sdot4(q.z & m, alo.z, lo);
    lo = bm_sdot4(q.w & m, alo.w, lo);
    hi = bm_sdot4((q.x >> 4) & m, ahi.x, 0);
    hi = bm_sdot4((q.y >> 4) & m, ahi.y, hi);
    hi = bm_sdot4((q.z >> 4) & m, ahi.z, hi);
    hi = bm_sdot4((q.w >> 4) & m, ahi.w, hi);
}

// What the Q4_K core reads of one column for one super-block: read a super-block ahead of its use, the LDS
// latency hides behind the previous super-block's arithmetic.
template <int WT>
struct Act;
template <>
struct Act<BM_Q4K> {
    uint4 lo0, hi0, lo1, hi1; // codes against the low / high nibbles of the first and second 64 code bytes
    float4 e0, e1, em;        // (d8, d8 * isum) of sub-blocks (2c, 2c + 1), (4 + 2c, 5 + 2c), (4h + 2c, 4h + 2c + 1)
    u32 sw;                   // the two stored isums (taps only)
};

template <>
struct Act<BM_Q5K> : Act<BM_Q4K> {};

template <bool WithSums>
__device__ __forceinline__ Act<BM_Q4K> bm_act_q4k(const ActView &av, int i, int c, int h) {
    const uint8_t *g0 = av.col + (size_t)(2 * i) * BM_Q82X4_STRIDE + 16 + 64 * c + 16 * h;
    const uint8_t *g1 = g0 + BM_Q82X4_STRIDE;
    const uint8_t *te = av.tbl + (size_t)i * 64 + 16 * c;
    Act<BM_Q4K> a;
    a.lo0 = *reinterpret_cast<const uint4 *>(g0);
    a.hi0 = *reinterpret_cast<const uint4 *>(g0 + 32);
    a.lo1 = *reinterpret_cast<const uint4 *>(g1);
    a.hi1 = *reinterpret_cast<const uint4 *>(g1 + 32);
    a.e0 = *reinterpret_cast<const float4 *>(te);
    a.e1 = *reinterpret_cast<const float4 *>(te + 32);
    a.em = *reinterpret_cast<const float4 *>(te + 32 * h);
    a.sw = 0;
    if constexpr (WithSums)
        a.sw = *reinterpret_cast<const u32 *>(av.col + (size_t)(2 * i + h) * BM_Q82X4_STRIDE + 8 + 4 * c);
    return a;
}

// One super-block `i` of one column, from the header word, the two code words and the column's reads. `Bits` adds
// a code's fifth bit (Q5_K) before the integer dots; Q4_K passes none.
template <class Bits, class Tap>
__device__ __forceinline__ void bm_dot_q45k(uint4 hdr, uint4 qa, uint4 qb, const Bits &bits, const Act<BM_Q4K> &a, int i,
                                            int c, int h, float &acc0, float &acc1, const Tap &tap) {
    const float d = bm_half_to_f32(hdr.x & 0xffffu), dmin = bm_half_to_f32(hdr.x >> 16);
    const u32 a0 = hdr.y, a1 = hdr.z, a2 = hdr.w; // crates/qdot/src/lib.rs:3868-3878
    const int sh = 16 * c;                         // this lane's two sub-blocks sit in bytes 2c, 2c + 1
    const u32 s0 = (a0 & 0x3f3f3f3fu) >> sh;       // scales of sub-blocks 2c, 2c + 1
    const u32 s1 = ((a2 & 0x0f0f0f0fu) | ((a0 >> 2) & 0x30303030u)) >> sh; // 4 + 2c, 5 + 2c
    // both forms and a bitwise pick: a conditional here compiles to a branch a super-block, which also fences the
    // scheduling of the loads around it
    const u32 hm = 0u - (u32)h;
    const u32 mw = ((((a2 >> 4) & 0x0f0f0f0fu) | ((a1 >> 2) & 0x30303030u)) & hm) | ((a1 & 0x3f3f3f3fu) & ~hm);
    const u32 mm = mw >> sh; // mins of sub-blocks 4h + 2c, 4h + 2c + 1
    // Min term of accumulators l = 4h + t (lib.rs:4389-4394): fma(d8 * isum, -(dmin * m), acc).
    acc0 = fmaf(a.em.y, -(dmin * (float)(mm & 0xffu)), acc0);
    acc1 = fmaf(a.em.w, -(dmin * (float)((mm >> 8) & 0xffu)), acc1);
    if constexpr (Tap::kActive) {
        tap.q4k_isum(i, 4 * h + 2 * c, (int)(short)(a.sw & 0xffffu));
        tap.q4k_isum(i, 4 * h + 2 * c + 1, (int)(short)(a.sw >> 16));
    }
    // j = 0: sub-blocks 2c, 2c + 1 (group 0); j = 1: 4 + 2c, 5 + 2c (group 1) (lib.rs:4402-4436).
    {
        int lo, hi;
        bits.dot16(qa, 2 * c, a.lo0, a.hi0, lo, hi);
        acc0 = fmaf((d * (float)(s0 & 0xffu)) * a.e0.x, (float)lo, acc0);
        acc1 = fmaf((d * (float)((s0 >> 8) & 0xffu)) * a.e0.z, (float)hi, acc1);
        tap.q4k(i, 2 * c, h, lo);
        tap.q4k(i, 2 * c + 1, h, hi);
    }
    {
        int lo, hi;
        bits.dot16(qb, 4 + 2 * c, a.lo1, a.hi1, lo, hi);
        acc0 = fmaf((d * (float)(s1 & 0xffu)) * a.e1.x, (float)lo, acc0);
        acc1 = fmaf((d * (float)((s1 >> 8) & 0xffu)) * a.e1.z, (float)hi, acc1);
        tap.q4k(i, 4 + 2 * c, h, lo);
        tap.q4k(i, 5 + 2 * c, h, hi);
    }
}

struct NoFifthBit {
    __device__ __forceinline__ void dot16(uint4 q, int, uint4 alo, uint4 ahi, int &lo, int &hi) const {
        bm_q4_dot16(q, alo, ahi, lo, hi);
    }
};

template <class Tap>
__device__ __forceinline__ void bm_dot_q4k(const Blk<BM_Q4K> &b, const Act<BM_Q4K> &a, int i, int c, int h,
                                           float &acc0, float &acc1, const Tap &tap) {
    bm_dot_q45k(b.hdr, b.qa, b.qb, NoFifthBit{}, a, i, c, h, acc0, acc1, tap);
}

// ---- Q5_K (crates/qdot/src/lib.rs:4876-4893): Q4_K's lane map over the 176-byte block. The lane also reads high
// bytes [16h, +16): value 32s + 16h + t takes bit s of high byte 16h + t as its fifth bit, so the low nibbles of the
// first code word (sub-block 2c) take bit 2c, its high nibbles bit 2c + 1, the second word's bits 4 + 2c and 5 + 2c.
template <>
struct Blk<BM_Q5K> {
    uint4 hdr, qh, qa, qb;
};

__device__ __forceinline__ Blk<BM_Q5K> bm_load_q5k(const uint8_t *wrow, int i, int c, int h) {
    const uint8_t *wb = wrow + (size_t)i * BM_Q5K_BLOCK;
    Blk<BM_Q5K> b;
    b.hdr = bm_ld16(wb);
    b.qh = bm_ld16(wb + 16 + 16 * h);
    b.qa = bm_ld16(wb + 48 + 32 * c + 16 * h);
    b.qb = bm_ld16(wb + 48 + 64 + 32 * c + 16 * h);
    return b;
}

struct FifthBit {
    uint4 qh;
    // `s`: the sub-block of q's low nibbles; its high nibbles are sub-block s + 1
    __device__ __forceinline__ void dot16(uint4 q, int s, uint4 alo, uint4 ahi, int &lo, int &hi) const {
        const u32 m = 0x0f0f0f0fu, one = 0x01010101u;
        lo = bm_sdot4((q.x & m) | (((qh.x >> s) & one) << 4), alo.x, 0);
        lo = bm_sdot4((q.y & m) | (((qh.y >> s) & one) << 4), alo.y, lo);
        lo = bm_sdot4((q.z & m) | (((qh.z >> s) & one) << 4), alo.z, lo);
        lo = bm_sdot4((q.w & m) | (((qh.w >> s) & one) << 4), alo.w, lo);
        hi = bm_sdot4(((q.x >> 4) & m) | (((qh.x >> (s + 1)) & one) << 4), ahi.x, 0);
        hi = bm_sdot4(((q.y >> 4) & m) | (((qh.y >> (s + 1)) & one) << 4), ahi.y, hi);
        hi = bm_sdot4(((q.z >> 4) & m) | (((qh.z >> (s + 1)) & one) << 4), ahi.z, hi);
        hi = bm_sdot4(((q.w >> 4) & m) | (((qh.w >> (s + 1)) & one) << 4), ahi.w, hi);
    }
};

template <class Tap>
__device__ __forceinline__ void bm_dot_q5k(const Blk<BM_Q5K> &b, const Act<BM_Q5K> &a, int i, int c, int h,
                                           float &acc0, float &acc1, const Tap &tap) {
    bm_dot_q45k(b.hdr, b.qa, b.qb, FifthBit{b.qh}, a, i, c, h, acc0, acc1, tap);
}

// A Q4_K / Q5_K super-block's weight side, formed once and dotted against several columns: the code words as the dot
// takes them (the fifth bit joined), the four scale products d * sc and the two min products -(dmin * m), each the
// value bm_dot_q45k forms for every column anew.
struct Q45Dec {
    u32 lo0[4], hi0[4], lo1[4], hi1[4];
    float w00, w01, w10, w11, n0, n1;
};

template <bool Fifth>
__device__ __forceinline__ Q45Dec bm_decode_q45k(uint4 hdr, uint4 qa, uint4 qb, uint4 qh, int c, int h) {
    const float d = bm_half_to_f32(hdr.x & 0xffffu), dmin = bm_half_to_f32(hdr.x >> 16);
    const u32 a0 = hdr.y, a1 = hdr.z, a2 = hdr.w;
    const int sh = 16 * c;
    const u32 s0 = (a0 & 0x3f3f3f3fu) >> sh;
    const u32 s1 = ((a2 & 0x0f0f0f0fu) | ((a0 >> 2) & 0x30303030u)) >> sh;
    const u32 hm = 0u - (u32)h;
    const u32 mw = ((((a2 >> 4) & 0x0f0f0f0fu) | ((a1 >> 2) & 0x30303030u)) & hm) | ((a1 & 0x3f3f3f3fu) & ~hm);
    const u32 mm = mw >> sh;
    Q45Dec x;
    x.n0 = -(dmin * (float)(mm & 0xffu));
    x.n1 = -(dmin * (float)((mm >> 8) & 0xffu));
    x.w00 = d * (float)(s0 & 0xffu);
    x.w01 = d * (float)((s0 >> 8) & 0xffu);
    x.w10 = d * (float)(s1 & 0xffu);
    x.w11 = d * (float)((s1 >> 8) & 0xffu);
    const u32 m = 0x0f0f0f0fu, one = 0x01010101u;
    const u32 wa[4] = {qa.x, qa.y, qa.z, qa.w}, wb[4] = {qb.x, qb.y, qb.z, qb.w}, wh[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
    for (int t = 0; t < 4; t++) {
        x.lo0[t] = wa[t] & m;
        x.hi0[t] = (wa[t] >> 4) & m;
        x.lo1[t] = wb[t] & m;
        x.hi1[t] = (wb[t] >> 4) & m;
        if constexpr (Fifth) { // sub-blocks 2c, 2c + 1 of the first word, 4 + 2c, 5 + 2c of the second
            x.lo0[t] |= ((wh[t] >> (2 * c)) & one) << 4;
            x.hi0[t] |= ((wh[t] >> (2 * c + 1)) & one) << 4;
            x.lo1[t] |= ((wh[t] >> (4 + 2 * c)) & one) << 4;
            x.hi1[t] |= ((wh[t] >> (5 + 2 * c)) & one) << 4;
        }
    }
    return x;
}

__device__ __forceinline__ int bm_dot16_words(const u32 (&w)[4], uint4 a) {
    int s = bm_sdot4(w[0], a.x, 0);
    s = bm_sdot4(w[1], a.y, s);
    s = bm_sdot4(w[2], a.z, s);
    return bm_sdot4(w[3], a.w, s);
}

// bm_dot_q45k's column side over a decoded super-block: the same products and sums in the same order.
template <class Tap>
__device__ __forceinline__ void bm_dot_q45k_dec(const Q45Dec &x, const Act<BM_Q4K> &a, int i, int c, int h, float &acc0,
                                                float &acc1, const Tap &tap) {
    acc0 = fmaf(a.em.y, x.n0, acc0);
    acc1 = fmaf(a.em.w, x.n1, acc1);
    if constexpr (Tap::kActive) {
        tap.q4k_isum(i, 4 * h + 2 * c, (int)(short)(a.sw & 0xffffu));
        tap.q4k_isum(i, 4 * h + 2 * c + 1, (int)(short)(a.sw >> 16));
    }
    {
        const int lo = bm_dot16_words(x.lo0, a.lo0), hi = bm_dot16_words(x.hi0, a.hi0);
        acc0 = fmaf(x.w00 * a.e0.x, (float)lo, acc0);
        acc1 = fmaf(x.w01 * a.e0.z, (float)hi, acc1);
        tap.q4k(i, 2 * c, h, lo);
        tap.q4k(i, 2 * c + 1, h, hi);
    }
    {
        const int lo = bm_dot16_words(x.lo1, a.lo1), hi = bm_dot16_words(x.hi1, a.hi1);
        acc0 = fmaf(x.w10 * a.e1.x, (float)lo, acc0);
        acc1 = fmaf(x.w11 * a.e1.z, (float)hi, acc1);
        tap.q4k(i, 4 + 2 * c, h, lo);
        tap.q4k(i, 5 + 2 * c, h, hi);
    }
}

// ---- Q6_K: lane (c, h) owns accumulators l = 4h + c and 4h + c + 2. Per 128-value half j it reads ql bytes
// [64j + 32c + 16h, +16) (low nibbles: quarter c, high nibbles: quarter c + 2, both half h) and qh bytes
// [32j + 16h, +16) (bits 2a of quarter a).
// Four loads a lane and super-block, nothing fetched twice by a quad: the two ql pieces; one of the two qh pieces (lane c
// of a pair takes half c's, its neighbour the other, and they exchange on use); and for the scales and d, lane 0 of the quad
// takes the 16 scale bytes, lane 1 the 16 bytes that end with d (the address unit works through a load 64 bytes at a time
// whether the lanes ask for different bytes or the same: with every lane asking for qh twice, the scales and d, a quad's
// 210 bytes cost six passes instead of four; measured on the headline layer's down stack, 16 tokens slot by slot: 66.2 -> 64.1 us).
template <>
struct Blk<BM_Q6K> {
    uint4 ql0, ql1, qhx, scd;
};

__device__ __forceinline__ Blk<BM_Q6K> bm_load_q6k(const uint8_t *wrow, int i, int c, int h) {
    const uint8_t *wb = wrow + (size_t)i * BM_Q6K_BLOCK;
    Blk<BM_Q6K> b;
    b.ql0 = bm_ld16u(wb + 32 * c + 16 * h);
    b.ql1 = bm_ld16u(wb + 64 + 32 * c + 16 * h);
    b.qhx = bm_ld16u(wb + 128 + 32 * c + 16 * h);
    b.scd = bm_ld16u(wb + 192 + ((c & ~h & 1) ? 2 : 0)); // lane (c, h) = (1, 0): bytes 194 .. 210, d the last two
    return b;
}

// What the lane computes with, exchanged inside the quad once the loads are back: qh of both halves, the scales, d.
struct Q6Parts {
    uint4 qh0, qh1, sc;
    u32 d;
};
template <int CTRL>
__device__ __forceinline__ uint4 bm_dpp4(uint4 v) {
    return make_uint4(bm_dpp<CTRL>(v.x), bm_dpp<CTRL>(v.y), bm_dpp<CTRL>(v.z), bm_dpp<CTRL>(v.w));
}
__device__ __forceinline__ Q6Parts bm_q6k_parts(const Blk<BM_Q6K> &b) {
    Q6Parts p;
    p.qh0 = bm_dpp4<0xA0>(b.qhx); // quad_perm [0,0,2,2]: the pair's lane c = 0 holds half 0's piece
    p.qh1 = bm_dpp4<0xF5>(b.qhx); // quad_perm [1,1,3,3]
    p.sc = bm_dpp4<0x00>(b.scd);  // quad lane 0
    p.d = bm_dpp<0x55>(b.scd.w) >> 16; // quad lane 1: bytes 208, 209
    return p;
}

// The two 16-value dots of one half: quarter c (low nibbles, high bits 2c) against aa and quarter c + 2 (high
// nibbles, high bits 2c + 4) against ab, each sum q6 * a with the 6-bit code taken as it is (it fits a signed byte).
__device__ __forceinline__ void bm_q6_dot16x2(uint4 ql, uint4 qh, int hs, uint4 aa, uint4 ab, int &s0, int &s1) {
    const u32 ml = 0x0f0f0f0fu, mh = 0x30303030u;
    const u32 hx = qh.x >> hs, hy = qh.y >> hs, hz = qh.z >> hs, hw = qh.w >> hs; // this lane's bits at 0..1, 4..5
    s0 = bm_sdot4((ql.x & ml) | ((hx << 4) & mh), aa.x, 0);
    s0 = bm_sdot4((ql.y & ml) | ((hy << 4) & mh), aa.y, s0);
    s0 = bm_sdot4((ql.z & ml) | ((hz << 4) & mh), aa.z, s0);
    s0 = bm_sdot4((ql.w & ml) | ((hw << 4) & mh), aa.w, s0);
    s1 = bm_sdot4(((ql.x >> 4) & ml) | (hx & mh), ab.x, 0);
    s1 = bm_sdot4(((ql.y >> 4) & ml) | (hy & mh), ab.y, s1);
    s1 = bm_sdot4(((ql.z >> 4) & ml) | (hz & mh), ab.z, s1);
    s1 = bm_sdot4(((ql.w >> 4) & ml) | (hw & mh), ab.w, s1);
}

template <>
struct Act<BM_Q6K> {
    uint4 aa[2], ab[2]; // per 128-value half j: the 16 codes of 32-block c and of 32-block c + 2, half h
    float d8a[2], d8b[2];
    int sa[2], sb[2]; // sums of those 16 codes
};

__device__ __forceinline__ Act<BM_Q6K> bm_act_q6k(const ActView &av, int i, int c, int h) {
    const uint8_t *g0 = av.col + (size_t)(2 * i) * BM_Q82X4_STRIDE + 16 + 32 * c + 16 * h;
    const uint8_t *te = av.tbl + (size_t)i * 64 + 8 * c;
    const int *s16 = reinterpret_cast<const int *>(av.s16 + (size_t)i * 64) + 2 * c + h;
    Act<BM_Q6K> a;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        a.aa[j] = *reinterpret_cast<const uint4 *>(g0 + j * BM_Q82X4_STRIDE);
        a.ab[j] = *reinterpret_cast<const uint4 *>(g0 + j * BM_Q82X4_STRIDE + 64);
        a.d8a[j] = *reinterpret_cast<const float *>(te + 32 * j);
        a.d8b[j] = *reinterpret_cast<const float *>(te + 32 * j + 16);
        a.sa[j] = s16[8 * j];
        a.sb[j] = s16[8 * j + 4];
    }
    return a;
}

template <class Tap>
__device__ __forceinline__ void bm_dot_q6k(const Blk<BM_Q6K> &b, const Act<BM_Q6K> &a, int i, int c, int h,
                                           float &acc0, float &acc1, const Tap &tap) {
    const Q6Parts p = bm_q6k_parts(b);
    const float d = bm_half_to_f32(p.d);
    const int bi = 8 * (2 * c + h); // this lane's scale byte inside each word of four
#pragma unroll
    for (int j = 0; j < 2; j++) {
        int s0, s1;
        bm_q6_dot16x2(j ? b.ql1 : b.ql0, j ? p.qh1 : p.qh0, 2 * c, a.aa[j], a.ab[j], s0, s1);
        s0 -= 32 * a.sa[j]; // sum (q6 - 32) * a
        s1 -= 32 * a.sb[j];
        // scale bytes 8j + 2c + h and 8j + 4 + 2c + h (crates/qdot/src/lib.rs:4455 K_SHUFFLE_Q6K, :4794-4809)
        const int sc0 = __builtin_amdgcn_sbfe((int)(j ? p.sc.z : p.sc.x), bi, 8);
        const int sc1 = __builtin_amdgcn_sbfe((int)(j ? p.sc.w : p.sc.y), bi, 8);
        acc0 = fmaf((d * (float)sc0) * a.d8a[j], (float)s0, acc0);
        acc1 = fmaf((d * (float)sc1) * a.d8b[j], (float)s1, acc1);
        tap.q6k(i, 8 * j + 2 * c + h, s0);
        tap.q6k(i, 8 * j + 4 + 2 * c + h, s1);
    }
}

// The operands of bm_dot_q6k's four multiply-adds, in its order: (half 0: accumulator 0, accumulator 1), (half 1: the same);
// acc = fmaf(p, s, acc) over them is bm_dot_q6k.
__device__ __forceinline__ void bm_q6k_terms(const Blk<BM_Q6K> &b, const Act<BM_Q6K> &a, int c, int h, float (&p)[4], float (&s)[4]) {
    const Q6Parts parts = bm_q6k_parts(b);
    const float d = bm_half_to_f32(parts.d);
    const int bi = 8 * (2 * c + h);
#pragma unroll
    for (int j = 0; j < 2; j++) {
        int s0, s1;
        bm_q6_dot16x2(j ? b.ql1 : b.ql0, j ? parts.qh1 : parts.qh0, 2 * c, a.aa[j], a.ab[j], s0, s1);
        s0 -= 32 * a.sa[j];
        s1 -= 32 * a.sb[j];
        const int sc0 = __builtin_amdgcn_sbfe((int)(j ? parts.sc.z : parts.sc.x), bi, 8);
        const int sc1 = __builtin_amdgcn_sbfe((int)(j ? parts.sc.w : parts.sc.y), bi, 8);
        p[2 * j] = (d * (float)sc0) * a.d8a[j];
        s[2 * j] = (float)s0;
        p[2 * j + 1] = (d * (float)sc1) * a.d8b[j];
        s[2 * j + 1] = (float)s1;
    }
}

// A Q6_K super-block's weight side, formed once for several columns: the 6-bit code words of the lane's four
// 16-value groups and the four products d * scale.
struct Q6Dec {
    u32 wa[2][4], wb[2][4];
    float fa[2], fb[2];
};

__device__ __forceinline__ Q6Dec bm_decode_q6k(const Blk<BM_Q6K> &b, int c, int h) {
    const Q6Parts p = bm_q6k_parts(b);
    const float d = bm_half_to_f32(p.d);
    const int bi = 8 * (2 * c + h), hs = 2 * c;
    const u32 ml = 0x0f0f0f0fu, mh = 0x30303030u;
    Q6Dec x;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint4 ql = j ? b.ql1 : b.ql0, qh = j ? p.qh1 : p.qh0;
        const u32 l[4] = {ql.x, ql.y, ql.z, ql.w}, hh[4] = {qh.x >> hs, qh.y >> hs, qh.z >> hs, qh.w >> hs};
#pragma unroll
        for (int t = 0; t < 4; t++) {
            x.wa[j][t] = (l[t] & ml) | ((hh[t] << 4) & mh);
            x.wb[j][t] = ((l[t] >> 4) & ml) | (hh[t] & mh);
        }
        const int sc0 = __builtin_amdgcn_sbfe((int)(j ? p.sc.z : p.sc.x), bi, 8); // the builtin's type is unsigned
        const int sc1 = __builtin_amdgcn_sbfe((int)(j ? p.sc.w : p.sc.y), bi, 8);
        x.fa[j] = d * (float)sc0;
        x.fb[j] = d * (float)sc1;
    }
    return x;
}

template <class Tap>
__device__ __forceinline__ void bm_dot_q6k_dec(const Q6Dec &x, const Act<BM_Q6K> &a, int i, int c, int h, float &acc0,
                                               float &acc1, const Tap &tap) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int s0 = bm_dot16_words(x.wa[j], a.aa[j]) - 32 * a.sa[j];
        const int s1 = bm_dot16_words(x.wb[j], a.ab[j]) - 32 * a.sb[j];
        acc0 = fmaf(x.fa[j] * a.d8a[j], (float)s0, acc0);
        acc1 = fmaf(x.fb[j] * a.d8b[j], (float)s1, acc1);
        tap.q6k(i, 8 * j + 2 * c + h, s0);
        tap.q6k(i, 8 * j + 4 + 2 * c + h, s1);
    }
}

// ---- IQ2_XXS: lane q owns accumulators l = 2q and 2q + 1: values 8q .. 8q + 8 (grid group q) of every
// sub-block. The quad loads the block's 64 code bytes once (16 each) and shares them through DPP.
template <>
struct Blk<BM_IQ2XXS> {
    uint4 q; // sub-blocks 2q' and 2q' + 1 of this lane's quarter q': (idx, aux, idx, aux)
    u32 d;
};

__device__ __forceinline__ Blk<BM_IQ2XXS> bm_load_iq2xxs(const uint8_t *wrow, int i, int q) {
    const uint8_t *blk = wrow + (size_t)i * BM_IQ2XXS_BLOCK;
    Blk<BM_IQ2XXS> b;
    b.q = bm_ld16u(blk + 2 + 16 * q);
    b.d = bm_ld2u(blk);
    return b;
}

// LDS tables of the IQ decodes. The CPU path dots the unsigned bytes u = +-mag + off (IQ2_XXS: off 43, IQ3_XXS: 64) and
// takes the offsets back out through the column's sums. IQ2_XXS: selector tables and a byte permute (bm_iq2_codes below).
// IQ3_XXS: a grid point of four magnitudes is kept as its four bytes 64 + mag and its four bytes 64 - mag, a sign index as
// eight byte masks (0xff where the value is negative), and u is a bitwise pick between the two by the mask (one operation a
// word).
__device__ __forceinline__ u32 bm_iq_pick(u32 plus, u32 minus, u32 mask) { return (minus & mask) | (plus & ~mask); }

// a * b + c over 24-bit factors as one multiply-add: the empty statement pins the running sum, so the compiler cannot
// regroup a chain of these into multiplies and three-operand adds (three instructions for two products where two do).
// (The instruction itself is not written by hand: the compiler places the wait states a dot product's result needs
// before another kind of instruction reads it, and cannot see into a hand-written one.)
__device__ __forceinline__ int bm_mad24_chain(int a, int b, int c) {
    int r = __mul24(a, b) + c;
    asm volatile("" : "+v"(r));
    return r;
}
struct Iq2Tables {
    const uint2 *grid;  // IQ2_XXS: a grid point's eight magnitude selectors (0, 1, 2), a byte each
    const uint2 *grid3; // IQ3_XXS: (64 + magnitudes, 64 - magnitudes) of a four-value grid point
    const uint2 *signs; // IQ2_XXS: 4 in the bytes of the negative values; IQ3_XXS: 0xff there
};

// The eight code bytes 43 +- magnitude of an IQ2_XXS group (what the CPU path dots, crates/qdot/src/lib.rs:8677-8724): two
// 8-byte table reads, a grid point's magnitude selectors and a sign index's bytes of 4, whose sum is a byte selector into the
// six possible codes: 0 .. 2 pick 43 + {8, 25, 43}, 4 .. 6 pick 43 - {8, 25, 43} (the reference's card kernels decode the same
// way, crates/gpu/src/iq.rs:473-512). A third less LDS traffic than ready-made code bytes of both signs and half the banks
// an entry, for two more vector instructions a group.
constexpr u32 kIq2Plus = 0x00564433u, kIq2Minus = 0x00001223u;
__device__ __forceinline__ void bm_iq2_codes(const Iq2Tables &tb, u32 grid_idx, u32 sign_idx, u32 &lo, u32 &hi) {
    const uint2 g = tb.grid[grid_idx], sg = tb.signs[sign_idx];
    lo = __builtin_amdgcn_perm(kIq2Minus, kIq2Plus, g.x | sg.x);
    hi = __builtin_amdgcn_perm(kIq2Minus, kIq2Plus, g.y | sg.y);
}

template <>
struct Act<BM_IQ2XXS> {
    float dy;
    uint2 bs;   // bsums 4q .. 4q + 3
    uint2 a[8]; // values 8q .. 8q + 8 of each of the eight sub-blocks
};

__device__ __forceinline__ Act<BM_IQ2XXS> bm_act_iq2xxs(const ActView &av, int i, int q) {
    const uint8_t *blk = av.col + (size_t)i * BM_Q8K_STRIDE;
    Act<BM_IQ2XXS> a;
    a.dy = *reinterpret_cast<const float *>(blk);
    a.bs = *reinterpret_cast<const uint2 *>(blk + 264 + 8 * q);
#pragma unroll
    for (int sb = 0; sb < 8; sb++) a.a[sb] = *reinterpret_cast<const uint2 *>(blk + 8 + 32 * sb + 8 * q);
    return a;
}

// The block's codes as this lane dots them: per sub-block the eight signed grid values (two words) and the
// scale 2s + 1. Decoded once a super-block, whatever the number of columns.
struct Iq2Dec {
    u32 u_lo[8], u_hi[8]; // the bytes +-mag + 43
    int sc[8];
};

__device__ __forceinline__ Iq2Dec bm_decode_iq2xxs(const Blk<BM_IQ2XXS> &b, int q, const Iq2Tables &tb) {
    Iq2Dec dec;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        // Quarter k of the block (sub-blocks 2k, 2k + 1) sits in lane k of the quad.
        const u32 idx_a = bm_quad_bcast(b.q.x, k), aux_a = bm_quad_bcast(b.q.y, k);
        const u32 idx_b = bm_quad_bcast(b.q.z, k), aux_b = bm_quad_bcast(b.q.w, k);
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int sb = 2 * k + e;
            const u32 idx = e ? idx_b : idx_a, aux = e ? aux_b : aux_a;
            dec.sc[sb] = 2 * (int)(aux >> 28) + 1;
            bm_iq2_codes(tb, (idx >> (8 * q)) & 0xffu, (aux >> (7 * q)) & 127u, dec.u_lo[sb], dec.u_hi[sb]);
        }
    }
    return dec;
}

// The float and integer steps IQ2_XXS and IQ3_XXS share (crates/qdot/src/lib.rs:8677-8724, :7494-7541): the fold of
// the offset through the column's 16-value sums first, then the scaled sums of offset byte x code. `off`: 43 / 64;
// d: f16 / 8 or f16 / 4; sca, scb: the scales 2s + 1 of the lane's own sub-blocks 2q and 2q + 1.
template <int OFF, class Tap>
__device__ __forceinline__ void bm_dot_iqx_dec(float d, int sca, int scb, const Iq2Dec &dec, const Act<BM_IQ2XXS> &act,
                                               int i, int q, float &acc0, float &acc1, const Tap &tap) {
    const float dy = act.dy;
    const float dmin = -d * (float)OFF;
    // Fold first (crates/qdot/src/lib.rs:8691-8694): accumulator l takes sub-block l's scale on its two bsums.
    {
        const uint2 bs = act.bs;
        const int b0 = (int)(short)(bs.x & 0xffffu), b1 = (int)(short)(bs.x >> 16);
        const int b2 = (int)(short)(bs.y & 0xffffu), b3 = (int)(short)(bs.y >> 16);
        const int ma = bm_mad24(sca, b0, bm_mul24(sca, b1)), mb = bm_mad24(scb, b2, bm_mul24(scb, b3)); // bsums: 16 bits
        const float f = dmin * dy;
        acc0 = fmaf(f, (float)ma, acc0);
        acc1 = fmaf(f, (float)mb, acc1);
    }
    int sumi0 = 0, sumi1 = 0;
#pragma unroll
    for (int sb = 0; sb < 8; sb++) {
        const uint2 a = act.a[sb];
        // the reference sums sc * u * a (the offsets come back out through the fold above); sums within 4 * 126 * 128
        // and sc <= 31 lie inside 24 bits
        const int d_lo = bm_sdot4(dec.u_lo[sb], a.x, 0), d_hi = bm_sdot4(dec.u_hi[sb], a.y, 0);
        sumi0 = bm_mad24_chain(dec.sc[sb], d_lo, sumi0);
        sumi1 = bm_mad24_chain(dec.sc[sb], d_hi, sumi1);
        if constexpr (Tap::kActive) // the signed sum: less the offset times the eight codes
            tap.iq2(i, sb, q, d_lo + d_hi - OFF * (bm_sdot4(0x01010101u, a.x, 0) + bm_sdot4(0x01010101u, a.y, 0)));
    }
    const float f = d * dy;
    acc0 = fmaf(f, (float)sumi0, acc0);
    acc1 = fmaf(f, (float)sumi1, acc1);
}

template <class Tap>
__device__ __forceinline__ void bm_dot_iq2xxs_dec(const Blk<BM_IQ2XXS> &b, const Iq2Dec &dec, const Act<BM_IQ2XXS> &act,
                                                  int i, int q, float &acc0, float &acc1, const Tap &tap) {
    bm_dot_iqx_dec<43>(0.125f * bm_half_to_f32(b.d), 2 * (int)(b.q.y >> 28) + 1, 2 * (int)(b.q.w >> 28) + 1, dec, act, i, q,
                       acc0, acc1, tap);
}

template <class Tap>
__device__ __forceinline__ void bm_dot_iq2xxs(const Blk<BM_IQ2XXS> &b, const Act<BM_IQ2XXS> &act, int i, int q,
                                              const Iq2Tables &tb, float &acc0, float &acc1, const Tap &tap) {
    const Iq2Dec dec = bm_decode_iq2xxs(b, q, tb);
    bm_dot_iq2xxs_dec(b, dec, act, i, q, acc0, acc1, tap);
}

// ---- IQ3_XXS (crates/qdot/src/lib.rs:7494-7541): IQ2_XXS's lane map. Lane q owns accumulators 2q and 2q + 1: the
// values 8q .. 8q + 7 of every sub-block, i.e. the two four-magnitude grid words its index bytes 2q and 2q + 1 name
// and the sub-block's sign group q. The quad loads the block's 64 index bytes and eight sign/scale words once
// (16 + 8 bytes a lane: sub-blocks 2q and 2q + 1) and shares them through DPP.
template <>
struct Blk<BM_IQ3XXS> {
    uint4 qi;  // the index bytes of sub-blocks 2q (x, y) and 2q + 1 (z, w)
    uint2 aux; // their sign/scale words
    u32 d;
};

__device__ __forceinline__ Blk<BM_IQ3XXS> bm_load_iq3xxs(const uint8_t *wrow, int i, int q) {
    const uint8_t *blk = wrow + (size_t)i * BM_IQ3XXS_BLOCK;
    Blk<BM_IQ3XXS> b;
    b.qi = bm_ld16u(blk + 2 + 16 * q);
    __builtin_memcpy(&b.aux, blk + 66 + 8 * q, 8);
    b.d = bm_ld2u(blk);
    return b;
}

template <>
struct Act<BM_IQ3XXS> : Act<BM_IQ2XXS> {};

__device__ __forceinline__ Iq2Dec bm_decode_iq3xxs(const Blk<BM_IQ3XXS> &b, int q, const Iq2Tables &tb) {
    Iq2Dec dec;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        // sub-blocks 2k and 2k + 1 sit in lane k of the quad; this lane's two index bytes are bytes 2q, 2q + 1 of a
        // sub-block's eight: the first word's for q < 2, the second's otherwise
        const u32 ia0 = bm_quad_bcast(b.qi.x, k), ia1 = bm_quad_bcast(b.qi.y, k);
        const u32 ib0 = bm_quad_bcast(b.qi.z, k), ib1 = bm_quad_bcast(b.qi.w, k);
        const u32 aux_a = bm_quad_bcast(b.aux.x, k), aux_b = bm_quad_bcast(b.aux.y, k);
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int sb = 2 * k + e;
            const u32 word = (q & 2) ? (e ? ib1 : ia1) : (e ? ib0 : ia0), aux = e ? aux_b : aux_a;
            const u32 pair = word >> (16 * (q & 1));
            dec.sc[sb] = 2 * (int)(aux >> 28) + 1;
            const uint2 g0 = tb.grid3[pair & 0xffu], g1 = tb.grid3[(pair >> 8) & 0xffu];
            const uint2 sg = tb.signs[(aux >> (7 * q)) & 127u];
            dec.u_lo[sb] = bm_iq_pick(g0.x, g0.y, sg.x);
            dec.u_hi[sb] = bm_iq_pick(g1.x, g1.y, sg.y);
        }
    }
    return dec;
}

template <class Tap>
__device__ __forceinline__ void bm_dot_iq3xxs_dec(const Blk<BM_IQ3XXS> &b, const Iq2Dec &dec, const Act<BM_IQ3XXS> &act,
                                                  int i, int q, float &acc0, float &acc1, const Tap &tap) {
    bm_dot_iqx_dec<64>(0.25f * bm_half_to_f32(b.d), 2 * (int)(b.aux.x >> 28) + 1, 2 * (int)(b.aux.y >> 28) + 1, dec, act, i,
                       q, acc0, acc1, tap);
}

template <class Tap>
__device__ __forceinline__ void bm_dot_iq3xxs(const Blk<BM_IQ3XXS> &b, const Act<BM_IQ3XXS> &act, int i, int q,
                                              const Iq2Tables &tb, float &acc0, float &acc1, const Tap &tap) {
    const Iq2Dec dec = bm_decode_iq3xxs(b, q, tb);
    bm_dot_iq3xxs_dec(b, dec, act, i, q, acc0, acc1, tap);
}

// ---- Q3_K (crates/qdot/src/lib.rs:2223-2245, layout crates/gguf/src/quant.rs:671-678): one integer a super-block
// and one f32 accumulator a row. Lane q takes the 16 field bytes 16q .. of qs: half j = q / 2, cells 16 (q % 2) .. + 15,
// whose four two-bit fields are the 16-value groups 8j + 2f + q % 2, with the high bits of hmask bytes 16 (q % 2) ..
// (bit 4j + f). A code u = low | high << 2 becomes the signed byte u - 4 through a byte permute of the eight levels;
// the lane scales its four group sums, the quad adds the four shares, and every lane applies the same float step,
// acc + (dcol * d) * sum with each operation rounded on its own.
template <>
struct Blk<BM_Q3K> {
    uint4 qs, hm; // the lane's field bytes and the high-bit bytes of their cells
    uint4 tail;   // block bytes 94 .. 109: the twelve scale bytes at 2 .., d at 14
};

__device__ __forceinline__ Blk<BM_Q3K> bm_load_q3k(const uint8_t *wrow, int i, int q) {
    const uint8_t *blk = wrow + (size_t)i * BM_Q3K_BLOCK;
    Blk<BM_Q3K> b;
    b.qs = bm_ld16u(blk + 32 + 16 * q);
    b.hm = bm_ld16u(blk + 16 * (q & 1));
    b.tail = bm_ld16u(blk + 94);
    return b;
}

template <>
struct Act<BM_Q3K> {
    float dcol;
    uint2 a[8]; // field f's 16 codes: a[2f], a[2f + 1]
};

__device__ __forceinline__ Act<BM_Q3K> bm_act_q3k(const ActView &av, int i, int q) {
    const uint8_t *blk = av.col + (size_t)i * BM_Q8K_STRIDE;
    Act<BM_Q3K> a;
    a.dcol = *reinterpret_cast<const float *>(blk);
    const uint8_t *at = blk + 8 + 128 * (q >> 1) + 16 * (q & 1);
#pragma unroll
    for (int f = 0; f < 4; f++) {
        a.a[2 * f] = *reinterpret_cast<const uint2 *>(at + 32 * f);
        a.a[2 * f + 1] = *reinterpret_cast<const uint2 *>(at + 32 * f + 8);
    }
    return a;
}

template <class Tap>
__device__ __forceinline__ void bm_dot_q3k(const Blk<BM_Q3K> &b, const Act<BM_Q3K> &act, int i, int q, float &acc0,
                                           const Tap &tap) {
    const int j = q >> 1, odd = q & 1;
    // the sixteen six-bit scales (crates/qdot/src/lib.rs:2162-2174); this lane's are bytes 2 (f % 2) + q % 2 of words
    // 2j + f / 2
    const u32 a0 = (b.tail.x >> 16) | (b.tail.y << 16), a1 = (b.tail.y >> 16) | (b.tail.z << 16);
    const u32 a2 = (b.tail.z >> 16) | (b.tail.w << 16);
    const u32 lo = j ? (a0 >> 4) : a0, lo1 = j ? (a1 >> 4) : a1, hi = a2 >> (4 * j);
    const u32 w0 = (lo & 0x0f0f0f0fu) | ((hi & 0x03030303u) << 4);
    const u32 w1 = (lo1 & 0x0f0f0f0fu) | (((hi >> 2) & 0x03030303u) << 4);
    const u32 qw[4] = {b.qs.x, b.qs.y, b.qs.z, b.qs.w}, hw[4] = {b.hm.x, b.hm.y, b.hm.z, b.hm.w};
    int sum = 0;
#pragma unroll
    for (int f = 0; f < 4; f++) {
        int g = 0;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const u32 low = (qw[t] >> (2 * f)) & 0x03030303u;
            const u32 high = (hw[t] >> (4 * j + f)) & 0x01010101u;
            // u = low | high << 2 picks its level: bytes -4, -3, -2, -1 then 0, 1, 2, 3
            const u32 v = __builtin_amdgcn_perm(0x03020100u, 0xfffefdfcu, (high << 2) | low);
            const uint2 a = act.a[2 * f + (t >> 1)];
            g = bm_sdot4(v, (t & 1) ? a.y : a.x, g);
        }
        tap.q6k(i, 8 * j + 2 * f + odd, g);
        const u32 word = (f >> 1) ? w1 : w0;
        const int sc = (int)((word >> (8 * (2 * (f & 1) + odd))) & 0xffu) - 32;
        sum = bm_mad24(sc, g, sum); // |g| <= 16 * 4 * 128, |sc| <= 32
    }
    sum += (int)bm_dpp<kDppXor1>((u32)sum);
    sum += (int)bm_dpp<kDppXor2>((u32)sum);
    const float d = bm_half_to_f32(b.tail.w >> 16);
    acc0 = __fadd_rn(acc0, __fmul_rn(__fmul_rn(act.dcol, d), (float)sum));
}

// ---- IQ4_XS (crates/qdot/src/lib.rs:11033-11180): lane q reads sub-blocks 2q and 2q + 1 whole (32 consecutive code
// bytes) and their 64 activation codes, turns the nibbles into levels with byte permutes of the sixteen-entry table,
// and forms its share of the CPU path's eight i32 lanes: lane l of those sums, scale by scale, the values 4l .. 4l + 3
// of every sub-block (low nibbles of code bytes 4l .., then for l >= 4 the high nibbles of bytes 4 (l - 4) ..). The
// quad adds the shares up (integers: any order) and lane q applies the f32 step to accumulators 2q and 2q + 1.
template <>
struct Blk<BM_IQ4XS> {
    uint4 qa, qb; // the code bytes of sub-blocks 2q and 2q + 1
    uint2 hd;     // d | scales_h << 16, scales_l
};

__device__ __forceinline__ Blk<BM_IQ4XS> bm_load_iq4xs(const uint8_t *wrow, int i, int q) {
    const uint8_t *blk = wrow + (size_t)i * BM_IQ4XS_BLOCK;
    Blk<BM_IQ4XS> b;
    b.hd = *reinterpret_cast<const uint2 *>(blk);
    b.qa = bm_ld16u(blk + 8 + 32 * q);
    b.qb = bm_ld16u(blk + 24 + 32 * q);
    return b;
}

template <>
struct Act<BM_IQ4XS> {
    float dy;
    uint2 a[8]; // the 64 codes of sub-blocks 2q and 2q + 1
};

__device__ __forceinline__ Act<BM_IQ4XS> bm_act_iq4xs(const ActView &av, int i, int q) {
    const uint8_t *blk = av.col + (size_t)i * BM_Q8K_STRIDE;
    Act<BM_IQ4XS> a;
    a.dy = *reinterpret_cast<const float *>(blk);
#pragma unroll
    for (int k = 0; k < 8; k++) a.a[k] = *reinterpret_cast<const uint2 *>(blk + 8 + 64 * q + 8 * k);
    return a;
}

// Four 4-bit codes, one in the low nibble of each byte of x >> shift, as four levels: the table's low and high halves
// through one byte permute each (selector: the code's low three bits), then a third that takes byte k from the high
// half where code k has its top bit set.
template <int SHIFT>
__device__ __forceinline__ u32 bm_iq4_levels(u32 x) {
    constexpr u32 t0 = bm_iq4_levels_word(0), t1 = bm_iq4_levels_word(1), t2 = bm_iq4_levels_word(2), t3 = bm_iq4_levels_word(3);
    const u32 s = (x >> SHIFT) & 0x07070707u;
    const u32 lo = __builtin_amdgcn_perm(t1, t0, s), hi = __builtin_amdgcn_perm(t3, t2, s);
    const u32 pick = ((x >> (SHIFT + 1)) & 0x04040404u) | 0x03020100u;
    return __builtin_amdgcn_perm(hi, lo, pick);
}

// The block's levels as this lane dots them, decoded once a super-block whatever the number of columns.
struct Iq4Dec {
    u32 lo[2][4], hi[2][4]; // sub-block 2q + e: levels of values 4j .. (low nibbles) and 16 + 4j .. (high nibbles)
    int sc[2];
};

__device__ __forceinline__ Iq4Dec bm_decode_iq4xs(const Blk<BM_IQ4XS> &b, int q) {
    Iq4Dec dec;
    const u32 qw[2][4] = {{b.qa.x, b.qa.y, b.qa.z, b.qa.w}, {b.qb.x, b.qb.y, b.qb.z, b.qb.w}};
#pragma unroll
    for (int e = 0; e < 2; e++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            dec.lo[e][j] = bm_iq4_levels<0>(qw[e][j]);
            dec.hi[e][j] = bm_iq4_levels<4>(qw[e][j]);
        }
        // crates/gguf/src/quant.rs:1989-1991: nibble b % 2 of scales_l[b / 2] under bits 2b .. of scales_h, less 32;
        // sub-blocks 2q, 2q + 1 are the two nibbles of scales_l[q]
        const u32 sl = (b.hd.y >> (8 * q + 4 * e)) & 15u, sh = (b.hd.x >> (16 + 4 * q + 2 * e)) & 3u;
        dec.sc[e] = (int)(sl | (sh << 4)) - 32;
    }
    return dec;
}

template <class Tap>
__device__ __forceinline__ void bm_dot_iq4xs_dec(const Blk<BM_IQ4XS> &b, const Iq4Dec &dec, const Act<BM_IQ4XS> &act, int i,
                                                 int q, float &acc0, float &acc1, const Tap &tap) {
    int lanes[8];
#pragma unroll
    for (int e = 0; e < 2; e++) {
        int sub = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // values 4j .. 4j + 3 of the sub-block are word j % 2 of its code group j / 2; 16 + 4j .. of group 2 + j / 2
            const uint2 alo = act.a[4 * e + (j >> 1)], ahi = act.a[4 * e + 2 + (j >> 1)];
            const int p_lo = bm_sdot4(dec.lo[e][j], (j & 1) ? alo.y : alo.x, 0);
            const int p_hi = bm_sdot4(dec.hi[e][j], (j & 1) ? ahi.y : ahi.x, 0);
            // |p| <= 4 * 127 * 128 and |scale| <= 32: inside 24 bits
            lanes[j] = e ? bm_mad24(dec.sc[1], p_lo, lanes[j]) : bm_mul24(dec.sc[0], p_lo);
            lanes[4 + j] = e ? bm_mad24(dec.sc[1], p_hi, lanes[4 + j]) : bm_mul24(dec.sc[0], p_hi);
            sub += p_lo + p_hi;
        }
        tap.iq4_sub(i, 2 * q + e, sub);
    }
    // the quad's four shares of each lane sum
#pragma unroll
    for (int l = 0; l < 8; l++) {
        lanes[l] += (int)bm_dpp<kDppXor1>((u32)lanes[l]);
        lanes[l] += (int)bm_dpp<kDppXor2>((u32)lanes[l]);
        if (q == 0) tap.iq4_lane(i, l, lanes[l]);
    }
    const int s0 = q == 0 ? lanes[0] : (q == 1 ? lanes[2] : (q == 2 ? lanes[4] : lanes[6]));
    const int s1 = q == 0 ? lanes[1] : (q == 1 ? lanes[3] : (q == 2 ? lanes[5] : lanes[7]));
    // one fused multiply-add a super-block and lane (crates/qdot/src/lib.rs:11171-11173)
    const float f = bm_half_to_f32(b.hd.x & 0xffffu) * act.dy;
    acc0 = fmaf(f, (float)s0, acc0);
    acc1 = fmaf(f, (float)s1, acc1);
}

template <class Tap>
__device__ __forceinline__ void bm_dot_iq4xs(const Blk<BM_IQ4XS> &b, const Act<BM_IQ4XS> &act, int i, int q, float &acc0,
                                             float &acc1, const Tap &tap) {
    const Iq4Dec dec = bm_decode_iq4xs(b, q);
    bm_dot_iq4xs_dec(b, dec, act, i, q, acc0, acc1, tap);
}

// ---- closing sums: (t0 + t2) + (t1 + t3) with t_l = acc_l + acc_{l+4}; every lane of the quad gets the value.
template <int WT>
__device__ __forceinline__ float bm_quad_finish(float acc0, float acc1) {
    // lane ^ 2 holds acc_{l+4} (Q4_K, Q5_K, Q6_K: the other half h; IQ2_XXS, IQ4_XS: lane q + 2 owns l + 4)
    if (WT == BM_Q3K) return acc0; // one accumulator a row, the same in the four lanes
    const float x = acc0 + bm_quad_xor2(acc0), y = acc1 + bm_quad_xor2(acc1);
    if (WT == BM_Q6K) {
        // lane c holds t_c and t_{c+2}
        const float z = x + y;
        return z + bm_quad_xor1(z);
    }
    // lane c holds t_{2c} and t_{2c+1}
    const float X = x + bm_quad_xor1(x), Y = y + bm_quad_xor1(y);
    return X + Y;
}

// Uniform front over the types.
template <int WT>
__device__ __forceinline__ Blk<WT> bm_load_blk(const uint8_t *wrow, int i, int q);
template <>
__device__ __forceinline__ Blk<BM_Q3K> bm_load_blk<BM_Q3K>(const uint8_t *wrow, int i, int q) {
    return bm_load_q3k(wrow, i, q);
}
template <>
__device__ __forceinline__ Blk<BM_Q4K> bm_load_blk<BM_Q4K>(const uint8_t *wrow, int i, int q) {
    return bm_load_q4k(wrow, i, q & 1, q >> 1);
}
template <>
__device__ __forceinline__ Blk<BM_Q5K> bm_load_blk<BM_Q5K>(const uint8_t *wrow, int i, int q) {
    return bm_load_q5k(wrow, i, q & 1, q >> 1);
}
template <>
__device__ __forceinline__ Blk<BM_Q6K> bm_load_blk<BM_Q6K>(const uint8_t *wrow, int i, int q) {
    return bm_load_q6k(wrow, i, q & 1, q >> 1);
}
template <>
__device__ __forceinline__ Blk<BM_IQ2XXS> bm_load_blk<BM_IQ2XXS>(const uint8_t *wrow, int i, int q) {
    return bm_load_iq2xxs(wrow, i, q);
}
template <>
__device__ __forceinline__ Blk<BM_IQ3XXS> bm_load_blk<BM_IQ3XXS>(const uint8_t *wrow, int i, int q) {
    return bm_load_iq3xxs(wrow, i, q);
}
template <>
__device__ __forceinline__ Blk<BM_IQ4XS> bm_load_blk<BM_IQ4XS>(const uint8_t *wrow, int i, int q) {
    return bm_load_iq4xs(wrow, i, q);
}

template <int WT, bool WithSums>
__device__ __forceinline__ Act<WT> bm_load_act(const ActView &av, int i, int q) {
    if constexpr (WT == BM_Q4K)
        return bm_act_q4k<WithSums>(av, i, q & 1, q >> 1);
    else if constexpr (WT == BM_Q5K) {
        Act<BM_Q5K> a;
        static_cast<Act<BM_Q4K> &>(a) = bm_act_q4k<WithSums>(av, i, q & 1, q >> 1);
        return a;
    } else if constexpr (WT == BM_Q6K)
        return bm_act_q6k(av, i, q & 1, q >> 1);
    else if constexpr (WT == BM_IQ4XS)
        return bm_act_iq4xs(av, i, q);
    else if constexpr (WT == BM_Q3K)
        return bm_act_q3k(av, i, q);
    else if constexpr (WT == BM_IQ3XXS) {
        Act<BM_IQ3XXS> a;
        static_cast<Act<BM_IQ2XXS> &>(a) = bm_act_iq2xxs(av, i, q);
        return a;
    } else
        return bm_act_iq2xxs(av, i, q);
}

template <int WT, class Tap>
__device__ __forceinline__ void bm_dot_blk(const Blk<WT> &b, const Act<WT> &a, int i, int q, const Iq2Tables &tb,
                                           float &acc0, float &acc1, const Tap &tap) {
    if constexpr (WT == BM_Q4K)
        bm_dot_q4k(b, a, i, q & 1, q >> 1, acc0, acc1, tap);
    else if constexpr (WT == BM_Q5K)
        bm_dot_q5k(b, a, i, q & 1, q >> 1, acc0, acc1, tap);
    else if constexpr (WT == BM_Q6K)
        bm_dot_q6k(b, a, i, q & 1, q >> 1, acc0, acc1, tap);
    else if constexpr (WT == BM_IQ4XS)
        bm_dot_iq4xs(b, a, i, q, acc0, acc1, tap);
    else if constexpr (WT == BM_Q3K)
        bm_dot_q3k(b, a, i, q, acc0, tap);
    else if constexpr (WT == BM_IQ3XXS)
        bm_dot_iq3xxs(b, a, i, q, tb, acc0, acc1, tap);
    else
        bm_dot_iq2xxs(b, a, i, q, tb, acc0, acc1, tap);
}

template <int WT>
__host__ __device__ constexpr int bm_block_bytes() {
    return WT == BM_Q3K ? BM_Q3K_BLOCK : WT == BM_Q4K ? BM_Q4K_BLOCK : WT == BM_Q5K ? BM_Q5K_BLOCK : WT == BM_Q6K ? BM_Q6K_BLOCK : WT == BM_IQ4XS ? BM_IQ4XS_BLOCK : WT == BM_IQ3XXS ? BM_IQ3XXS_BLOCK : BM_IQ2XXS_BLOCK;
}

// ---- SwiGLU: crates/qdot/src/lib.rs:3741-3773 (expf) and :11467-11478 (divide, then multiply).
__device__ __forceinline__ float bm_expf_ik(float x) {
    const float SHIFT = bm_bits_f32(0x4b400000u), LOG2E = bm_bits_f32(0x3fb8aa3bu);
    const float LN2_HI = bm_bits_f32(0x3f317200u), LN2_LO = bm_bits_f32(0x35bfbe8eu);
    const float C0 = bm_bits_f32(0x3f7ffff6u), C1 = bm_bits_f32(0x3efffedbu), C2 = bm_bits_f32(0x3e2aaf33u);
    const float C3 = bm_bits_f32(0x3d2b9f17u), C4 = bm_bits_f32(0x3c072010u);
    const float z = fmaf(x, LOG2E, SHIFT);
    const float n = __fsub_rn(z, SHIFT);
    const float b = fmaf(-n, LN2_LO, fmaf(-n, LN2_HI, x));
    const u32 e = bm_f32_bits(z) << 23;
    const float k = bm_bits_f32(e + 0x3f800000u);
    const float u = __fmul_rn(b, b);
    const float j = fmaf(fmaf(fmaf(C4, b, C3), u, fmaf(C2, b, C1)), u, __fmul_rn(C0, b));
    if (fabsf(n) > 126.0f) {
        const u32 g = (n <= 0.0f) ? 0x82000000u : 0u;
        const float s1 = bm_bits_f32(g + 0x7f000000u);
        const float s2 = bm_bits_f32(e - g);
        if (fabsf(n) > 192.0f) return __fmul_rn(s1, s1);
        return __fmul_rn(fmaf(s2, j, s2), s1);
    }
    return fmaf(j, k, k);
}

__device__ __forceinline__ float bm_silu(float g) {
    const float e = bm_expf_ik(__fsub_rn(0.0f, g));
    return __fdiv_rn(g, __fadd_rn(1.0f, e));
}

__device__ __forceinline__ float bm_swiglu(float g, float u) { return __fmul_rn(bm_silu(g), u); }

// The clamped rules, comparison for comparison as the CPU path spells them (a NaN falls through each the same way).
// ik's: min(silu(g), limit) * clamp(u, -limit, limit), nothing clamped at limit <= 1e-6
// (crates/qdot/src/lib.rs:11492-11523 swiglu_clamp).
__device__ __forceinline__ float bm_swiglu_clamp(float g, float u, float limit) {
    float s = bm_silu(g), c = u;
    if (limit > 1e-6f) {
        s = limit < s ? limit : s;
        c = u < limit ? u : limit;
        c = -limit < c ? c : -limit;
    }
    return __fmul_rn(c, s);
}
// gpt-oss / MiniMax: x = min(g, limit), y = clamp(u, -limit, limit), x / (1 + e^(-alpha x)) * (y + 1), alpha 1.702
// (crates/qdot/src/lib.rs swiglu_oai_1, crates/gpu/src/kquant/act.rs:213-223).
__device__ __forceinline__ float bm_swiglu_oai(float g, float u, float limit) {
    const float x = limit < g ? limit : g;
    const float y = u < -limit ? -limit : (limit < u ? limit : u);
    const float e = bm_expf_ik(__fmul_rn(1.702f, __fsub_rn(0.0f, x)));
    return __fmul_rn(__fdiv_rn(x, __fadd_rn(1.0f, e)), __fadd_rn(y, 1.0f));
}
// ggml's gate-first clamp: silu(min(g, limit)) * clamp(u, -limit, limit), nothing clamped at limit <= 1e-6
// (crates/qdot/src/lib.rs:11617-11660 swiglu_gclamp, swiglu_gclamp_1).
__device__ __forceinline__ float bm_swiglu_gclamp(float g, float u, float limit) {
    float x = g, y = u;
    if (limit > 1e-6f) {
        x = limit < g ? limit : g;
        y = u < -limit ? -limit : (limit < u ? limit : u);
    }
    return __fmul_rn(bm_silu(x), y);
}

// SiTU-GLU: (beta tanh(g / beta) * sigmoid(g)) * (25 tanh(u / 25)), each scale by the f32 reciprocal, the tanh, the
// scale back, then the products (crates/gpu/src/kquant/act.rs:152-163 situ; crates/model/src/ops.rs:2345-2360 on the
// host). The sigmoid is ik's; the tanh is the device library's f32 one, which can differ from the host libm's in the
// last bits, as the reference's own card and host do.
__device__ __forceinline__ float bm_situ(float g, float u, float beta) {
    const float a = __fmul_rn(tanhf(__fmul_rn(g, __fdiv_rn(1.0f, beta))), beta);
    const float s = __fdiv_rn(1.0f, __fadd_rn(1.0f, bm_expf_ik(__fsub_rn(0.0f, g))));
    const float v = __fmul_rn(tanhf(__fmul_rn(u, __fdiv_rn(1.0f, 25.0f))), 25.0f);
    return __fmul_rn(__fmul_rn(a, s), v);
}

// A row's value under rule `act` (crates/gpu/src/kquant/act.rs:136-149 apply). Under the clamped rules and SiTU a sum that is
// not finite would come out finite: `odd` reports it and the value is NaN (:166-175 apply_checked; the CPU path's
// rules return false for such a block). The plain rule lets it through as it is, as the CPU path's swiglu does.
__device__ __forceinline__ float bm_gate_rule(u32 act, float limit, float g, float u, bool &odd) {
    odd = false;
    if (act == 0u) return bm_swiglu(g, u);
    if (!(fabsf(g) <= 3.402823466e38f && fabsf(u) <= 3.402823466e38f)) {
        odd = true;
        return bm_bits_f32(0x7fc00000u);
    }
    if (act == 1u) return bm_swiglu_clamp(g, u, limit);
    if (act == 2u) return bm_swiglu_oai(g, u, limit);
    if (act == 3u) return bm_situ(g, u, limit);
    return bm_swiglu_gclamp(g, u, limit);
}

#endif // BM_DEVICE_HPP
