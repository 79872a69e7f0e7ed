// TEST INFRASTRUCTURE ONLY. The card rule: the reference's GPU tier quantizes activations to its own q8_1 form
// (128-value blocks, an f32 scale amax / 127, codes rounded half away from zero, an exact code sum per 32 values)
// and walks a Q4_K or Q3_K row with 32 lanes whose partial sums meet in a butterfly. The reference restates that
// tier on the CPU (crates/qdot/src/lib.rs:2885-3620 card_q8_1, card_q4k_dot_row, card_q3k_dot_row) so the two can
// be compared bit for bit; this file restates those scalar mirrors in C, each function citing the lines it follows.
//
// What pins it: the quantizer by the worked cases of the reference's own test
// (crates/qdot/tests/qdot.rs:7942-8040: ties at every magnitude, near ties, the zero block, subnormal and
// underflowed scales, refused blocks, the sums) and an independent numpy restatement; the dots by an f64 band
// around the dequantized row against the decoded column (qdot.rs:8043-8098), by one-lane rows whose value is a
// three-operation f32 chain worked by hand in the tests, and by a second spelling of the walk written from the
// device's loop (crates/gpu/src/cores.rs:536-620: a pair loop over the guard-free prefix, then the guarded tail).
#include <math.h>
#include <string.h>

#include "bm_oracle.h"
#include "ora_common.h"

// crates/qdot/src/lib.rs:2917-2948 card_q8_1_fill_scalar. refused may be NULL. Returns the number of refused
// blocks, or ORA_EUNALIGNED (card_q8_1_check :2951: whole 256-value super-blocks, at least one).
int ora_card_q8_1(const float *x, int k, int8_t *codes, float *d8, int32_t *s8, uint8_t *refused) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    int n_bad = 0;
    for (int b = 0; b < k / 128; b++) {
        const float *blk = x + 128 * b;
        int bad = 0;
        float amax = 0.0f;
        for (int j = 0; j < 128; j++) {
            if (!isfinite(blk[j])) bad = 1;
            const float a = fabsf(blk[j]);
            if (a > amax) amax = a; // f32::max keeps the number when the other side is NaN
        }
        const float d = bad ? NAN : amax > 0.0f ? amax / 127.0f : 1.0f;
        for (int g = 0; g < 4; g++) {
            int32_t sum = 0;
            for (int j = 0; j < 32; j++) {
                int q = 0;
                if (!bad) {
                    // (v / d).round().clamp(-127, 127) as i32: round is half away from zero, a NaN (0 / 0) stays
                    // NaN through the clamp and converts to 0, an infinity clamps to +-127
                    const float r = roundf(blk[32 * g + j] / d);
                    q = r != r ? 0 : r < -127.0f ? -127 : r > 127.0f ? 127 : (int)r;
                }
                codes[128 * b + 32 * g + j] = (int8_t)q;
                sum += q;
            }
            s8[4 * b + g] = sum;
        }
        d8[b] = d;
        if (refused) refused[b] = (uint8_t)bad;
        n_bad += bad;
    }
    return n_bad;
}

// crates/qdot/src/lib.rs:3118 card_dp4a, :3126 card_word
static int32_t dp4a(uint32_t vi, uint32_t w) {
    int32_t a = 0;
    for (int b = 0; b < 4; b++) a += (int32_t)(int8_t)(vi >> (8 * b)) * (int32_t)(int8_t)(w >> (8 * b));
    return a;
}
static uint32_t code_word(const int8_t *codes, int v4) { return ora_rd32((const uint8_t *)codes + 4 * v4); }

// crates/qdot/src/lib.rs:3331-3341 card_warp_sum_scalar
static float warp_sum(float *v) {
    static const int strides[5] = {16, 8, 4, 2, 1};
    for (int i = 0; i < 5; i++)
        for (int l = 0; l < 32; l++)
            if ((l & strides[i]) == 0) v[l] += v[l | strides[i]];
    return v[0];
}

// crates/qdot/src/lib.rs:3165-3180 card_q4k_scale_min
static void q4k_scale_min(int s, uint32_t w1, uint32_t w2, uint32_t w3, int *sc, int *mi) {
    if (s < 4) {
        *sc = (int)((w1 >> (8 * s)) & 63);
        *mi = (int)((w2 >> (8 * s)) & 63);
    } else {
        const int sh = 8 * (s - 4);
        const uint32_t qs = (w2 >> sh) & 0xff, qs4 = (w3 >> sh) & 0xff, qsm = (w1 >> sh) & 0xff;
        *sc = (int)(qs4 & 0x0f) | ((int)(qsm >> 6) << 4);
        *mi = (int)(qs4 >> 4) | ((int)(qs >> 6) << 4);
    }
}

// crates/qdot/src/lib.rs:3184-3186 card_q4k_nibble: the nibble field's nib - 8 as four signed bytes
static uint32_t q4k_nibble(uint32_t qsw, uint32_t nib_sh) {
    return ((((qsw >> nib_sh) & 0x0f0f0f0fu) | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

// crates/qdot/src/lib.rs:3288-3327 card_q4k_lane_walk
static float q4k_lane_walk(const uint8_t *wrow, const int8_t *codes, const float *d8, const int32_t *s8, int n_sb, int lane) {
    const int iters = (n_sb + 3) / 4, full = n_sb / 4;
    const int s = lane & 7, grp = lane >> 3;
    float f = 0.0f;
    for (int it = 0; it < iters; it++) {
        const int sbp = 4 * it + grp;
        if (sbp >= n_sb) continue;
        const uint8_t *sb = wrow + (size_t)sbp * ORA_Q4K_BLOCK;
        const float d = ora_half_to_f32(ora_rd16(sb)), dmin = ora_half_to_f32(ora_rd16(sb + 2));
        int sc, mi;
        q4k_scale_min(s, ora_rd32(sb + 4), ora_rd32(sb + 8), ora_rd32(sb + 12), &sc, &mi);
        const float cda = d * (float)sc;
        const float cdb = fmaf(8.0f * d, (float)sc, -dmin * (float)mi);
        const uint32_t nib_sh = (uint32_t)(s & 1) * 4;
        const uint8_t *qs = sb + 16 + 32 * (s >> 1);
        int32_t a = 0;
        for (int i = 0; i < 8; i++) a += dp4a(q4k_nibble(ora_rd32(qs + 4 * i), nib_sh), code_word(codes, 256 * it + 64 * grp + 8 * s + i));
        const int32_t b = s8[32 * it + lane];
        const float e0 = d8[2 * sbp + (s >> 2)];
        const float x = fmaf(cda, (float)a, cdb * (float)b);
        const int split = (it & 1) == 0 && it + 2 <= full;
        f = split ? f + e0 * x : fmaf(e0, x, f);
    }
    return f;
}

// crates/qdot/src/lib.rs:3135-3144 card_q3k_field: field f's nib - 4 * hbit as four signed bytes
static uint32_t q3k_field(uint32_t vl, uint32_t vh1, uint32_t f) {
    const uint32_t hb = (vh1 >> f) << 2;
    return ((((vl >> (2 * f)) & 0x03030303u) | 0x80808080u) - (hb & 0x04040404u)) ^ 0x80808080u;
}

// crates/qdot/src/lib.rs:3150-3160 card_q3k_sub_scales
static void q3k_sub_scales(uint32_t a0w, uint32_t a1w, uint32_t a2w, int s0, int32_t *sc) {
    const uint32_t sh = (uint32_t)(((s0 & 1) << 3) | ((s0 >> 3) << 2));
    const uint32_t p0 = ((a0w >> sh) & 0x000f000fu) | (((a2w >> sh) & 0x00030003u) << 4);
    const uint32_t p1 = ((a1w >> sh) & 0x000f000fu) | (((a2w >> (sh + 2)) & 0x00030003u) << 4);
    sc[0] = (int32_t)(p0 & 0xff) - 32;
    sc[1] = (int32_t)(p0 >> 16) - 32;
    sc[2] = (int32_t)(p1 & 0xff) - 32;
    sc[3] = (int32_t)(p1 >> 16) - 32;
}

// crates/qdot/src/lib.rs:3239-3276 card_q3k_lane_walk
static float q3k_lane_walk(const uint8_t *wrow, const int8_t *codes, const float *d8, int n_sb, int lane) {
    const int iters = (n_sb + 1) / 2;
    const int w16 = lane & 15, half = lane >> 4;
    const int s0 = 8 * (w16 >> 3) + ((w16 & 7) >> 2), d8_base = w16 >> 3;
    float f = 0.0f;
    for (int it = 0; it < iters; it++) {
        const int sbp = 2 * it + half;
        if (sbp >= n_sb) continue;
        const uint8_t *sb = wrow + (size_t)sbp * ORA_Q3K_BLOCK;
        const uint32_t vl = ora_rd32(sb + 32 + 4 * w16);
        const uint32_t hm = ora_rd32(sb + 4 * (w16 & 7));
        const uint32_t vh1 = (~hm) >> (4 * (w16 >> 3));
        int32_t sc[4];
        q3k_sub_scales(ora_rd32(sb + 96), ora_rd32(sb + 100), ora_rd32(sb + 104), s0, sc);
        const float drow = ora_half_to_f32(ora_rd16(sb + 108));
        const int v4 = 128 * it + 64 * half + 32 * d8_base + (lane & 7);
        int32_t a = 0;
        for (int fld = 0; fld < 4; fld++)
            a += dp4a(q3k_field(vl, vh1, (uint32_t)fld), code_word(codes, v4 + 16 * (fld >> 1) + 8 * (fld & 1))) * sc[fld];
        const float e0 = d8[2 * sbp + d8_base];
        f = fmaf(e0 * drow, (float)a, f);
    }
    return f;
}

// crates/qdot/src/lib.rs:3361-3372, 3604-3614 card_q3k/q4k_dot_row_scalar_into: every lane's walk, then the
// butterfly. wtype is ORA_TYPE_Q4_K or ORA_TYPE_Q3_K (the two types the reference mirrors); s8 is read by Q4_K only.
int ora_card_dot_row(int wtype, const uint8_t *wrow, int k, const int8_t *codes, const float *d8, const int32_t *s8, float *out) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    if (wtype != ORA_TYPE_Q4_K && wtype != ORA_TYPE_Q3_K) return ORA_ETYPE;
    float v[32];
    for (int lane = 0; lane < 32; lane++)
        v[lane] = wtype == ORA_TYPE_Q4_K ? q4k_lane_walk(wrow, codes, d8, s8, k / 256, lane) : q3k_lane_walk(wrow, codes, d8, k / 256, lane);
    *out = warp_sum(v);
    return 0;
}

// y[r * m + c] = row r . column c (the card gemv's output order, crates/gpu/src/lib.rs q4k_gemv); column c's planes
// start at codes + c * k, d8 + c * k / 128, s8 + c * k / 32.
int ora_card_gemv(int wtype, const uint8_t *w, int rows, int k, const int8_t *codes, const float *d8, const int32_t *s8, int m, float *y) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    if (wtype != ORA_TYPE_Q4_K && wtype != ORA_TYPE_Q3_K) return ORA_ETYPE;
    const size_t rb = (size_t)(wtype == ORA_TYPE_Q4_K ? ORA_Q4K_BLOCK : ORA_Q3K_BLOCK) * (size_t)(k / 256);
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < m; c++) {
            const int rc = ora_card_dot_row(wtype, w + rb * r, k, codes + (size_t)c * k, d8 + (size_t)c * (k / 128), s8 + (size_t)c * (k / 32),
                                            &y[(size_t)r * m + c]);
            if (rc) return rc;
        }
    return 0;
}

// The MoE down step of the card tier (crates/gpu/src/q4k_sel.rs:358 q4k_gemv_sel): slot s's column against the rows
// of expert sel[s]: y[s * rows_per_expert + r]. An id >= n_experts is ORA_ESHAPE.
int ora_card_gemv_sel(int wtype, const uint8_t *w, int n_experts, int rows_per_expert, int k, const int8_t *codes, const float *d8,
                      const int32_t *s8, const uint32_t *sel, int n_slots, float *y) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    if (wtype != ORA_TYPE_Q4_K && wtype != ORA_TYPE_Q3_K) return ORA_ETYPE;
    const size_t rb = (size_t)(wtype == ORA_TYPE_Q4_K ? ORA_Q4K_BLOCK : ORA_Q3K_BLOCK) * (size_t)(k / 256);
    for (int s = 0; s < n_slots; s++) {
        if (sel[s] >= (uint32_t)n_experts) return ORA_ESHAPE;
        const uint8_t *we = w + rb * (size_t)rows_per_expert * sel[s];
        for (int r = 0; r < rows_per_expert; r++) {
            const int rc = ora_card_dot_row(wtype, we + rb * r, k, codes + (size_t)s * k, d8 + (size_t)s * (k / 128), s8 + (size_t)s * (k / 32),
                                            &y[(size_t)s * rows_per_expert + r]);
            if (rc) return rc;
        }
    }
    return 0;
}
