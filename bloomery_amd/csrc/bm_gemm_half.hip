// Prefill, tolerance mode in its f16 form (BM_GEMM_FAST_F16): the grouped expert GEMM with both scales folded into the
// matrix operands.
//
// The CPU path's form of a Q4_K row against a Q8_2_X4 column (crates/qdot/src/lib.rs:4363-4447) scales every 32-value
// block's integer sum by the product of the row's sub-scale and the column's block scale: on int8 matrix instructions
// that leaves a conversion and a multiply-add on the vector ALU for every (row, slot, block), and the vector ALU, not
// the matrix cores, bounds the kernel (k_gemm_fast in bm_prefill.hip, the int8 form). Here the scales ride in the
// operands instead, as exact f16 values, and the products come out of v_mfma_f32_32x32x16_f16 already scaled:
//   weight side   sc q: the 6-bit sub-scale times the 4-bit code, an integer below 1024, exact in f16;
//   column side   d8 a: the block's bf16 scale (8 significant bits) times the int8 code, 15 significant bits: the f16
//                 nearest to it (hi) and what is left (lo, exact), two matrix instructions a 16-value step. The column is
//                 first brought to the f16 range by a power of two of its own (the largest block scale to [1, 2)), taken
//                 out again at the end; a block more than 2^17 below the column's largest loses low bits of lo.
// A super-block's sum P = sum (sc q)(d8 a) is exact up to the f32 accumulation of the matrix cores; on the vector ALU
// are left, a super-block, y += d P and y += -dmin P2, where P2 = sum over the eight blocks of m[row] x (d8 isum)[slot]
// is one more matrix instruction (K = 16: the eight blocks against hi and against lo). So the vector ALU's share is two
// multiply-adds a (row, slot, super-block) plus the operand conversions (about 7 vector instructions a matrix instruction,
// against 19 in the int8 form), and the matrix cores carry four times the int8 form's cycles a value (two pieces at half
// the rate). Differs from the exact mode by f32 rounding only (order of the sums); the quantized activations are the CPU
// path's bytes. Measured on MI355X it is the slower of the two forms (gate GEMM of the 2048-token step 167 us against 125):
// matrix pipe 39 %, vector ALU 35 %, LDS 40 % busy, and the three do not overlap as the counts would allow; it is kept as
// the measured alternative, not taken by default.
//
// A workgroup of eight waves takes 256 rows of an expert and a tile's 64 slots, a wave 32 rows x 64 slots. LDS holds, in
// two buffers, half a super-block: the rows' code bytes as they lie in the file (converted to f16 in registers by the
// wave that owns the rows: nothing is converted twice) and the columns' two f16 planes (converted once a workgroup while
// they are staged); the tables of a super-block (sub-scales as f16 pairs, mins, d, dmin, the columns' d8 isum) in two more.
#include <type_traits>

#include "bm_gemm.hpp"

namespace bmk {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kHRows = 256, kHThreads = 512;
constexpr int kHARow = 64 + 8;               // Q4_K: a row's 64 code bytes of half a super-block, padded off the bank period
constexpr int kHBPlane = 256;                // a column's 128 values of one piece, f16
constexpr int kHBCol = 2 * kHBPlane + 16;    // hi plane, lo plane, pad
constexpr int kHScRow = 48;                  // a row's eight (sc, sc) f16 pairs of a super-block, padded
constexpr int kHMinCol = 32 + 16;            // a column's (d8 isum) hi[8], lo[8] f16 of a super-block, padded

struct HalfTabs {                      // a super-block's tables
    uint8_t sc2[kHRows * kHScRow];     // [row][block] (sc, sc)
    uint8_t mins[kHRows * 16];         // [row][block] m as f16
    float d[kHRows], ndmin[kHRows];    // d, -dmin
    uint8_t bmin[kGemmBN * kHMinCol];  // [slot][piece][block]
};
struct HalfBuf {
    uint8_t a[kHRows * kHARow];
    uint8_t b[kGemmBN * kHBCol];
};
struct HalfLds {
    GemmLds tab;
    float scale[kGemmBN], unscale[kGemmBN]; // the column's power of two and its inverse
    HalfTabs tabs[2];
    HalfBuf buf[2];
};

__device__ __forceinline__ v2h h2_of(u32 x) { return __builtin_bit_cast(v2h, x); }
__device__ __forceinline__ u32 u32_of(v2h x) { return __builtin_bit_cast(u32, x); }
// Eight codes (the bytes of w0, w1, each below 64) times a scale: 0x6400 | q is the f16 1024 + q, and
// (1024 + q) sc - 1024 sc leaves q sc in one rounding, which is exact below 2048.
__device__ __forceinline__ v8h codes_times(u32 w0, u32 w1, v2h sc2, v2h nsc2) {
    const u32 K = 0x64646464u;
    const u32 p0 = __builtin_amdgcn_perm(K, w0, 0x04010400u), p1 = __builtin_amdgcn_perm(K, w0, 0x04030402u);
    const u32 p2 = __builtin_amdgcn_perm(K, w1, 0x04010400u), p3 = __builtin_amdgcn_perm(K, w1, 0x04030402u);
    struct {
        u32 a, b, c, d;
    } s{u32_of(__builtin_elementwise_fma(h2_of(p0), sc2, nsc2)), u32_of(__builtin_elementwise_fma(h2_of(p1), sc2, nsc2)),
        u32_of(__builtin_elementwise_fma(h2_of(p2), sc2, nsc2)), u32_of(__builtin_elementwise_fma(h2_of(p3), sc2, nsc2))};
    return __builtin_bit_cast(v8h, s);
}

// Sixteen int8 codes (four words) times the block's scale as the f16 nearest to each product (hi) and the rest (lo).
__device__ __forceinline__ void column_pieces(const uint4 c, v2h d2, u32 (&hi)[8], u32 (&lo)[8]) {
    const u32 K = 0x64646464u;
    const v2h off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
    const u32 w[4] = {c.x ^ 0x80808080u, c.y ^ 0x80808080u, c.z ^ 0x80808080u, c.w ^ 0x80808080u}; // code + 128, a byte
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const u32 p = __builtin_amdgcn_perm(K, w[i], j ? 0x04030402u : 0x04010400u); // (1024 + 128 + code) pairs
            const v2h a = h2_of(p) + off;                                                // the codes, exact
            const v2h h = a * d2;
            hi[2 * i + j] = u32_of(h);
            lo[2 * i + j] = u32_of(__builtin_elementwise_fma(a, d2, -h));
        }
    }
}

template <int WT>
__global__ __launch_bounds__(kHThreads, 2) void k_gemm_half(const uint8_t *w, int rpe, int nb, const uint8_t *act, const u32 *cols,
                                                            const u32 *tiles, const u32 *n_tiles, u32 n_slabs, u32 slot_div,
                                                            u32 n_slots, float *y) {
    static_assert(WT == BM_Q4K, "the Q4_K walk");
    extern __shared__ __align__(16) uint8_t lds_raw[];
    HalfLds &L = *reinterpret_cast<HalfLds *>(lds_raw);
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, l32 = lane & 31, kh = lane >> 5;
    const u32 g = tile_of_block(blockIdx.x, n_slabs);
    const int row0 = (int)slab_of_block(blockIdx.x, n_slabs) * kHRows;
    const u32 count = n_tiles[0];
    if (g > count) return;
    if (g == count) { // the refused slots' rows: NaN (crates/gpu/src/gemm/grouped.rs:2283-2287)
        const u32 refused = n_tiles[1];
        for (u32 i = tid; i < refused * kHRows; i += kHThreads) {
            const u32 s = cols[n_slots - n_tiles[2] - refused + i / kHRows];
            const int r = row0 + (int)(i % kHRows);
            if (r < rpe) y[(size_t)s * rpe + r] = bm_bits_f32(0x7fc00000u);
        }
        return;
    }
    const u32 e = tiles[2 * g], word = tiles[2 * g + 1];
    const int start = (int)(word & 0xffffu), len = (int)(word >> 16);
    if (tid < kGemmBN) {
        const u32 s = cols[start + (tid < len ? tid : 0)];
        L.tab.slot[tid] = s;
        L.tab.col[tid] = s / slot_div;
    }
    __syncthreads();
    constexpr int kBlock = BM_Q4K_BLOCK;
    const u32 row_bytes = (u32)nb * kBlock, col_bytes = (u32)nb * BM_Q82_SB_EXT;

    // the columns' powers of two: eight lanes a column over its nb * 8 block scales
    {
        const int c = tid >> 3, part = tid & 7;
        const float *pairs = reinterpret_cast<const float *>(act + (size_t)L.tab.col[c] * col_bytes + (size_t)nb * BM_Q82_SB_REF);
        u32 top = 0;
        for (int b = part; b < nb * 8; b += 8) {
            const u32 v = bm_f32_bits(pairs[2 * b]) & 0x7fffffffu;
            top = v > top ? v : top;
        }
        u32 o;
        o = bm_dpp<kDppXor1>(top), top = o > top ? o : top;
        o = bm_dpp<kDppXor2>(top), top = o > top ? o : top;
        o = bm_dpp<kDppHalfMirror>(top), top = o > top ? o : top;
        if (part == 0) {
            const u32 ex = top >> 23; // the largest scale's biased exponent; a zero, huge or non-finite one is left as it is
            const bool plain = ex == 0 || ex >= 254;
            L.scale[c] = plain ? 1.0f : bm_bits_f32((254u - ex) << 23);
            L.unscale[c] = plain ? 1.0f : bm_bits_f32(ex << 23);
        }
    }
    __syncthreads();

    // What a thread stages of every half super-block: two 16-byte pieces of row codes (rows tid / 4 and 128 + tid / 4,
    // piece tid % 4 of the half's four), one 16-byte piece of column codes (column tid / 8, piece tid % 8 of the half's
    // eight) with its block's scale; of every super-block the header of row tid (threads below 256) and one (d8 isum) pair
    // (column tid / 8, block tid % 8).
    const uint8_t *we = w + (size_t)e * rpe * row_bytes;
    const int ar = tid >> 2, ap = tid & 3;
    u32 src_a[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
        src_a[j] = (u32)(row0 + ar + 128 * j < rpe ? row0 + ar + 128 * j : rpe - 1) * row_bytes + 16u + 16u * (u32)ap;
    const u32 src_h = (u32)(row0 + (tid & 255) < rpe ? row0 + (tid & 255) : rpe - 1) * row_bytes;
    const int bc = tid >> 3, bp = tid & 7;
    const u32 colp = L.tab.col[bc] * col_bytes;
    const float my_scale = L.scale[bc];
    uint4 ra[2], rb, rh;
    float rd8;
    float2 rpair;
    auto fetch = [&](int i, int half) {
#pragma unroll
        for (int j = 0; j < 2; j++) ra[j] = *reinterpret_cast<const uint4 *>(we + (src_a[j] + (u32)i * kBlock + 64u * (u32)half));
        // the half's 128 codes: group 2 i + half of the column (144 bytes: 16 of scales and sums, 128 codes)
        rb = *reinterpret_cast<const uint4 *>(act + (colp + (u32)(2 * i + half) * BM_Q82X4_STRIDE + 16u + 16u * (u32)bp));
        rd8 = *reinterpret_cast<const float *>(act + (colp + (u32)nb * BM_Q82_SB_REF + 8u * (u32)(8 * i + 4 * half + (bp >> 1))));
        if (half == 0) {
            if (tid < kHRows) rh = *reinterpret_cast<const uint4 *>(we + (src_h + (u32)i * kBlock));
            rpair = *reinterpret_cast<const float2 *>(act + (colp + (u32)nb * BM_Q82_SB_REF + 8u * (u32)(8 * i + bp)));
        }
    };
    // Storing what fetch() brought, in pieces that compute() places between its products (the buffer they go to is the other
    // one: nothing reads it in this stage). Pieces 0: the rows' code bytes; 1, 2: the column's two f16 planes, eight values a
    // piece; 3, 4 (a super-block's first half only): its tables.
    u32 hi[8], lo[8];
    auto stash_piece = [&](int piece, int i, int half) {
        HalfBuf &B = L.buf[half];
        HalfTabs &T = L.tabs[i & 1];
        if (piece == 0) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint8_t *dst = B.a + (ar + 128 * j) * kHARow + 16 * ap;
                *reinterpret_cast<uint2 *>(dst) = make_uint2(ra[j].x, ra[j].y); // rows are 8 bytes apart modulo 16
                *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(ra[j].z, ra[j].w);
            }
        } else if (piece == 1) {
            const float d8s = __fmul_rn(rd8, my_scale);
            const v2h d2 = {(_Float16)d8s, (_Float16)d8s};
            column_pieces(rb, d2, hi, lo);
            uint8_t *dst = B.b + bc * kHBCol + 32 * bp;
            *reinterpret_cast<uint4 *>(dst) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            *reinterpret_cast<uint4 *>(dst + 16) = make_uint4(hi[4], hi[5], hi[6], hi[7]);
        } else if (piece == 2) {
            uint8_t *dst = B.b + bc * kHBCol + 32 * bp + kHBPlane;
            *reinterpret_cast<uint4 *>(dst) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            *reinterpret_cast<uint4 *>(dst + 16) = make_uint4(lo[4], lo[5], lo[6], lo[7]);
        } else if (piece == 3 && half == 0) {
            if (tid < kHRows) {
                // the eight 6-bit scales and mins as bytes of four words (crates/gguf/src/quant.rs:620-628 get_scale_min_k4, four
                // sub-blocks a word), then each byte b as the f16 1024 + b (0x6400 | b) less 1024
                const u32 sc_lo = rh.y & 0x3f3f3f3fu, mn_lo = rh.z & 0x3f3f3f3fu;
                const u32 sc_hi = (rh.w & 0x0f0f0f0fu) | ((rh.y >> 2) & 0x30303030u);
                const u32 mn_hi = ((rh.w >> 4) & 0x0f0f0f0fu) | ((rh.z >> 2) & 0x30303030u);
                const u32 K = 0x64646464u;
                const v2h off = {(_Float16)-1024.0f, (_Float16)-1024.0f};
                auto twice = [&](u32 wd, int byte) { // (b, b)
                    const u32 sel = 0x04000400u | ((u32)byte << 16) | (u32)byte;
                    return u32_of(h2_of(__builtin_amdgcn_perm(K, wd, sel)) + off);
                };
                auto pair = [&](u32 wd, int byte) { // (b[byte], b[byte + 1])
                    const u32 sel = 0x04000400u | ((u32)(byte + 1) << 16) | (u32)byte;
                    return u32_of(h2_of(__builtin_amdgcn_perm(K, wd, sel)) + off);
                };
                uint4 *d = reinterpret_cast<uint4 *>(T.sc2 + tid * kHScRow);
                d[0] = make_uint4(twice(sc_lo, 0), twice(sc_lo, 1), twice(sc_lo, 2), twice(sc_lo, 3));
                d[1] = make_uint4(twice(sc_hi, 0), twice(sc_hi, 1), twice(sc_hi, 2), twice(sc_hi, 3));
                *reinterpret_cast<uint4 *>(T.mins + tid * 16) = make_uint4(pair(mn_lo, 0), pair(mn_lo, 2), pair(mn_hi, 0), pair(mn_hi, 2));
                T.d[tid] = bm_half_to_f32(rh.x & 0xffffu);
                T.ndmin[tid] = -bm_half_to_f32(rh.x >> 16);
            }
        } else if (piece == 4 && half == 0) {
            // (d8 isum) of block bp of column bc under the column's power of two, as hi + lo
            const float v = __fmul_rn(rpair.y, my_scale);
            const _Float16 h = (_Float16)v;
            const _Float16 l = (_Float16)(v - (float)h);
            reinterpret_cast<_Float16 *>(T.bmin + bc * kHMinCol)[bp] = h;
            reinterpret_cast<_Float16 *>(T.bmin + bc * kHMinCol + 16)[bp] = l;
        }
    };
    auto stash = [&](int i, int half) {
#pragma unroll
        for (int piece = 0; piece < 5; piece++) stash_piece(piece, i, half);
    };

    // this wave's rows 32 wv .. and all 64 slots; this lane: operand row / slot lane % 32, values 8 (lane / 32) .. of a
    // 16-value step; result v of a product is row 8 (v / 4) + 4 (lane / 32) + v % 4 of slot lane % 32
    const int my_row = 32 * wv + l32;
    v16f Y[2], P[2];
#pragma unroll
    for (int ct = 0; ct < 2; ct++)
#pragma unroll
        for (int v = 0; v < 16; v++) Y[ct][v] = 0.0f, P[ct][v] = 0.0f;
    const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    // next_i, next_half: the stage fetch() has just asked for, stored here among the products (next_i < 0: none)
    auto compute = [&](int i, auto half_c, auto wide_c, int next_i) __attribute__((always_inline)) {
        constexpr int half = decltype(half_c)::value;
        constexpr bool wide = decltype(wide_c)::value; // else slots 32 .. 63 are all padding: their products are left out
        constexpr int next_half = 1 - half;
        const HalfBuf &B = L.buf[half];
        const HalfTabs &T = L.tabs[i & 1];
        const uint8_t *my_a = B.a + my_row * kHARow + 8 * kh;
        const uint8_t *my_b[2] = {B.b + l32 * kHBCol + 16 * kh, B.b + (32 + l32) * kHBCol + 16 * kh};
        if (half == 0) {
            // the min terms: y += -dmin sum over the blocks of m x (d8 isum); then the block sums start from zero
            const v8h am = *reinterpret_cast<const v8h *>(T.mins + my_row * 16);
            float nd[16];
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const float4 d4 = *reinterpret_cast<const float4 *>(T.ndmin + 32 * wv + 8 * q4 + 4 * kh);
                nd[4 * q4] = d4.x, nd[4 * q4 + 1] = d4.y, nd[4 * q4 + 2] = d4.z, nd[4 * q4 + 3] = d4.w;
            }
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
                if (ct == 0 || wide) {
                    const v8h bm = *reinterpret_cast<const v8h *>(T.bmin + (32 * ct + l32) * kHMinCol + 16 * kh);
                    P[ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bm, zero, 0, 0, 0);
                }
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
                if (ct == 0 || wide)
#pragma unroll
                    for (int v = 0; v < 16; v++) Y[ct][v] = fmaf(nd[v], P[ct][v], Y[ct][v]);
        }
        // The half's four blocks in eight 16-value steps; a pair of blocks (2 p, 2 p + 1) comes from the same code bytes (low
        // and high nibbles), eight of them a lane a 16-value half: a unit of two steps. The columns' operands of a step are
        // read from LDS a step ahead of their products, the code bytes of a unit a unit ahead, and the unit's conversion runs
        // among the products of the unit before (the fences keep the compiler from folding that order back).
        const uint4 s2a = *reinterpret_cast<const uint4 *>(T.sc2 + my_row * kHScRow + 16 * half);
        const u32 s2[4] = {s2a.x, s2a.y, s2a.z, s2a.w};
        const v2h m1024 = {(_Float16)-1024.0f, (_Float16)-1024.0f};
        v8h Bf[2][2][2]; // [step parity][column tile][piece]
        v8h A[2][2];     // [unit parity][block of the pair]
        uint2 raw[2];
        auto read_b = [&](int step) { // step = 4 p + 2 h16 + j
            const int pp = step >> 2, hh = (step >> 1) & 1, jj = step & 1;
            const int k0 = 2 * (32 * (2 * pp + jj) + 16 * hh);
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
#pragma unroll
                for (int pc = 0; pc < 2; pc++)
                    if (ct == 0 || wide) Bf[step & 1][ct][pc] = *reinterpret_cast<const v8h *>(my_b[ct] + pc * kHBPlane + k0);
        };
        auto read_raw = [&](int unit) { raw[unit & 1] = *reinterpret_cast<const uint2 *>(my_a + 32 * (unit >> 1) + 16 * (unit & 1)); };
        auto convert = [&](int unit) {
            const int pp = unit >> 1;
            const v2h sc_lo = h2_of(s2[2 * pp]), sc_hi = h2_of(s2[2 * pp + 1]);
            const uint2 r = raw[unit & 1];
            A[unit & 1][0] = codes_times(r.x & 0x0f0f0f0fu, r.y & 0x0f0f0f0fu, sc_lo, sc_lo * m1024);
            A[unit & 1][1] = codes_times((r.x >> 4) & 0x0f0f0f0fu, (r.y >> 4) & 0x0f0f0f0fu, sc_hi, sc_hi * m1024);
        };
        read_raw(0);
        read_b(0);
        read_raw(1);
        convert(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int step = 0; step < 8; step++) {
            const int unit = step >> 1, jj = step & 1;
            if (step + 1 < 8) read_b(step + 1);
            if (jj == 1 && unit + 2 < 4) read_raw(unit + 2);
            __builtin_amdgcn_sched_barrier(0);
            if (jj == 1 && unit + 1 < 4) convert(unit + 1);
            // the loads of the next stage have had three steps to arrive
            if (next_i >= 0 && step >= 3) stash_piece(step - 3, next_i, next_half);
            const bool first = half == 0 && step == 0;
#pragma unroll
            for (int pc = 0; pc < 2; pc++)
#pragma unroll
                for (int ct = 0; ct < 2; ct++)
                    if (ct == 0 || wide)
                        P[ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[unit & 1][jj], Bf[step & 1][ct][pc], first && pc == 0 ? zero : P[ct], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (half == 1) { // the super-block's sums into the outputs under the rows' d
            float dv[16];
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const float4 d4 = *reinterpret_cast<const float4 *>(T.d + 32 * wv + 8 * q4 + 4 * kh);
                dv[4 * q4] = d4.x, dv[4 * q4 + 1] = d4.y, dv[4 * q4 + 2] = d4.z, dv[4 * q4 + 3] = d4.w;
            }
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
                if (ct == 0 || wide)
#pragma unroll
                    for (int v = 0; v < 16; v++) Y[ct][v] = fmaf(dv[v], P[ct][v], Y[ct][v]);
        }
    };

    // Two stages a super-block, a buffer a half: the next half is fetched to registers before the arithmetic on the present
    // one and stored behind it; the buffer it goes to was last read a stage ago, before the barrier that ended that stage.
    fetch(0, 0);
    stash(0, 0);
    __syncthreads();
    auto stages = [&](auto wide_c) __attribute__((always_inline)) {
        for (int i = 0; i < nb; i++) {
            fetch(i, 1);
            compute(i, std::integral_constant<int, 0>{}, wide_c, i);
            __syncthreads();
            const bool more = i + 1 < nb;
            if (more) fetch(i + 1, 0);
            compute(i, std::integral_constant<int, 1>{}, wide_c, more ? i + 1 : -1);
            __syncthreads();
        }
    };
    if (len > 32) stages(std::true_type{});
    else stages(std::false_type{});
#pragma unroll
    for (int ct = 0; ct < 2; ct++) {
        const int n = 32 * ct + l32;
        if (n < len) {
            const float us = L.unscale[n];
            float *out = y + (size_t)L.tab.slot[n] * rpe + row0 + 32 * wv + 4 * kh;
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                // rows_per_expert is a multiple of 16 and these four rows start at a multiple of 4: all inside or all outside
                if (row0 + 32 * wv + 4 * kh + 8 * q4 < rpe)
                    *reinterpret_cast<float4 *>(out + 8 * q4) = make_float4(Y[ct][4 * q4 + 0] * us, Y[ct][4 * q4 + 1] * us,
                                                                           Y[ct][4 * q4 + 2] * us, Y[ct][4 * q4 + 3] * us);
            }
        }
    }
}

bool gemm_half_supported(int wtype) { return wtype == BM_Q4K; }

hipError_t gemm_half(const Launch &L, int wtype, const uint8_t *w, int n_experts, int rows_per_expert, int k, const uint8_t *act,
                     const uint32_t *cols, const uint32_t *tiles_dev, const uint32_t *n_tiles, int n_slots, int slot_div, float *y) {
    const int nb = k / 256;
    const u32 max_tiles = (u32)gemm_max_tiles(n_slots, n_experts) + 1; // one more: the block that fills refused slots
    const u32 n_slabs = (u32)((rows_per_expert + kHRows - 1) / kHRows);
    const unsigned grid = ((max_tiles + 7) / 8) * 8 * n_slabs;
    const size_t lds = sizeof(HalfLds);
    if (wtype != BM_Q4K) return hipErrorInvalidValue;
    auto kern = k_gemm_half<BM_Q4K>;
    hipError_t e = allow_lds(kern, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kHThreads), lds, L.stream, w, rows_per_expert, nb, act, cols, tiles_dev, n_tiles, n_slabs,
                       (u32)slot_div, (u32)n_slots, y);
    return hipGetLastError();
}

} // namespace bmk
