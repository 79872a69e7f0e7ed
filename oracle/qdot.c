// TEST INFRASTRUCTURE ONLY (see ora_common.h). Scalar restatement of the reference's quantized row dots:
// the activation encoders, the three weight-type dots in the scalar mirrors' float order, the exact per-block
// integer sums, the dequantizers and SwiGLU.
#include "bm_oracle.h"
#include "iq_tables.h"
#include "ora_common.h"

// ------------------------------------------------------------------------------------------- activation encoders

// Q8_2_X4: crates/qdot/src/lib.rs:3883-3904 (whole 128-value groups; K-quant columns have no 32-value tail).
int ora_quantize_q82x4(const float *x, int k, uint8_t *out) {
    if (k <= 0 || k % 128 != 0) return ORA_EUNALIGNED;
    int bad = 0;
    for (int gi = 0; gi < k / 128; gi++) {
        uint8_t *group = out + (size_t)gi * ORA_Q82X4_STRIDE;
        memset(group, 0, ORA_Q82X4_STRIDE);
        for (int ir = 0; ir < 4; ir++) {
            const float *xb = x + 128 * gi + 32 * ir;
            float amax = fabsf(ora_activation_max(xb, 32, &bad));
            if (bad) return ORA_ENONFINITE;
            uint16_t t = ora_fp32_to_bf16_bits(amax / 127.0f);
            ora_wr16(group + 2 * ir, t);
            float id = ora_q82_inverse(t);
            uint8_t *qs = group + 16 + 32 * ir;
            int32_t isum = 0;
            for (int m = 0; m < 32; m++) {
                int32_t q = ora_nearest_int(xb[m] * id);
                int32_t c = q < -128 ? -128 : (q > 127 ? 127 : q);
                qs[m] = (uint8_t)(int8_t)c;
                isum += q;
            }
            ora_wr16(group + 8 + 2 * ir, (uint16_t)(int16_t)isum);
        }
    }
    return 0;
}

// Q8_K (ik's 296-byte block): crates/qdot/src/lib.rs:1787-1809.
int ora_quantize_q8k(const float *x, int k, uint8_t *out) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    int bad = 0;
    for (int b = 0; b < k / 256; b++) {
        const float *xb = x + 256 * b;
        uint8_t *o = out + (size_t)b * ORA_Q8K_STRIDE;
        float max = ora_activation_max(xb, 256, &bad);
        if (bad) return ORA_ENONFINITE;
        memset(o + 4, 0, 4);
        if (max == 0.0f) {
            memset(o, 0, ORA_Q8K_STRIDE);
            continue;
        }
        float iscale = -127.0f / max;
        for (int j = 0; j < 256; j++) {
            int32_t q = ora_nearest_int(iscale * xb[j]);
            if (q > 127) q = 127;
            o[8 + j] = (uint8_t)(q & 0xff); // `as i8`: the low byte
        }
        for (int j = 0; j < 16; j++) {
            int32_t sum = 0;
            for (int ii = 0; ii < 16; ii++) sum += (int8_t)o[8 + 16 * j + ii];
            ora_wr16(o + 264 + 2 * j, (uint16_t)(int16_t)sum);
        }
        float d = 1.0f / iscale;
        uint32_t db = ora_f32_bits(d);
        o[0] = (uint8_t)db;
        o[1] = (uint8_t)(db >> 8);
        o[2] = (uint8_t)(db >> 16);
        o[3] = (uint8_t)(db >> 24);
    }
    return 0;
}

int ora_col_bytes(int wtype, int k) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED; // crates/qdot/src/lib.rs:381-422
    switch (wtype) {
    case ORA_TYPE_Q4_K:
    case ORA_TYPE_Q5_K:
    case ORA_TYPE_Q6_K:
        return k / 128 * ORA_Q82X4_STRIDE;
    case ORA_TYPE_Q3_K:
    case ORA_TYPE_IQ2_XXS:
    case ORA_TYPE_IQ3_XXS:
    case ORA_TYPE_IQ4_XS:
        return k / 256 * ORA_Q8K_STRIDE;
    default:
        return ORA_ETYPE;
    }
}

int ora_row_bytes(int wtype, int k) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED; // crates/qdot/src/lib.rs:1727-1762
    switch (wtype) {
    case ORA_TYPE_Q3_K:
        return k / 256 * ORA_Q3K_BLOCK;
    case ORA_TYPE_Q4_K:
        return k / 256 * ORA_Q4K_BLOCK;
    case ORA_TYPE_Q5_K:
        return k / 256 * ORA_Q5K_BLOCK;
    case ORA_TYPE_Q6_K:
        return k / 256 * ORA_Q6K_BLOCK;
    case ORA_TYPE_IQ2_XXS:
        return k / 256 * ORA_IQ2XXS_BLOCK;
    case ORA_TYPE_IQ3_XXS:
        return k / 256 * ORA_IQ3XXS_BLOCK;
    case ORA_TYPE_IQ4_XS:
        return k / 256 * ORA_IQ4XS_BLOCK;
    default:
        return ORA_ETYPE;
    }
}

int ora_quantize_col(int wtype, const float *x, int k, uint8_t *out) {
    switch (wtype) { // crates/qdot/src/lib.rs:500-534
    case ORA_TYPE_Q4_K:
    case ORA_TYPE_Q5_K:
    case ORA_TYPE_Q6_K:
        return ora_quantize_q82x4(x, k, out);
    case ORA_TYPE_Q3_K:
    case ORA_TYPE_IQ2_XXS:
    case ORA_TYPE_IQ3_XXS:
    case ORA_TYPE_IQ4_XS:
        return ora_quantize_q8k(x, k, out);
    default:
        return ORA_ETYPE;
    }
}

// ------------------------------------------------------------------------------------------------------ Q3_K dot

// A super-block's sixteen scales as stored, six bits each, s + 32 (crates/qdot/src/lib.rs:2162-2174).
static void q3k_scales6(const uint8_t *blk, uint8_t sc[16]) {
    uint32_t a0 = ora_rd32(blk + 96), a1 = ora_rd32(blk + 100), a2 = ora_rd32(blk + 104);
    uint32_t w[4] = {(a0 & 0x0f0f0f0fu) | ((a2 & 0x03030303u) << 4), (a1 & 0x0f0f0f0fu) | (((a2 >> 2) & 0x03030303u) << 4),
                     ((a0 >> 4) & 0x0f0f0f0fu) | (((a2 >> 4) & 0x03030303u) << 4),
                     ((a1 >> 4) & 0x0f0f0f0fu) | (((a2 >> 6) & 0x03030303u) << 4)};
    for (int j = 0; j < 16; j++) sc[j] = (uint8_t)(w[j / 4] >> (8 * (j % 4)));
}

// Value n of a super-block less its offset: u - 4 with u = two low bits of qs | the hmask bit << 2
// (crates/qdot/src/lib.rs:2176-2185, crates/gguf/src/quant.rs:671-727).
static inline int q3k_value(const uint8_t *blk, int n) {
    int half = n / 128, field = (n / 32) % 4, cell = n % 32;
    int low = (blk[32 + 32 * half + cell] >> (2 * field)) & 3;
    int high = (blk[cell] >> (4 * half + field)) & 1;
    return (low | (high << 2)) - 4;
}

// Q3_K x Q8_K (crates/qdot/src/lib.rs:2223-2245): one exact integer a super-block, one f32 accumulator a row, a
// product and a sum each rounded on its own.
float ora_dot_q3k_q8k(const uint8_t *wrow, const uint8_t *acol, int nb) {
    float acc = 0.0f;
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_Q3K_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        uint8_t sc[16];
        q3k_scales6(blk, sc);
        float d = ora_half_to_f32(ora_rd16(blk + 108));
        float dcol = ora_bits_f32(ora_rd32(col));
        int32_t sumi = 0;
        for (int n = 0; n < 256; n++) sumi += ((int32_t)sc[n / 16] - 32) * q3k_value(blk, n) * (int32_t)(int8_t)col[8 + n];
        float t = dcol * d;
        t = t * (float)sumi;
        acc = acc + t;
    }
    return acc;
}

// Per super-block the sixteen sums S[g] = sum over 16-value group g of (u - 4) * a.
void ora_q3k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *s_out) {
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_Q3K_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        for (int g = 0; g < 16; g++) {
            int32_t sum = 0;
            for (int n = 16 * g; n < 16 * g + 16; n++) sum += q3k_value(blk, n) * (int32_t)(int8_t)col[8 + n];
            s_out[16 * i + g] = sum;
        }
    }
}

// ------------------------------------------------------------------------------------------------------ Q4_K dot

// The 12 packed bytes as eight 6-bit scales then eight 6-bit mins (crates/qdot/src/lib.rs:3868-3878,
// the same values as get_scale_min_k4, crates/gguf/src/quant.rs:620).
static void q4k_scales_mins(const uint8_t *s12, uint8_t sc[8], uint8_t mn[8]) {
    uint32_t a0 = ora_rd32(s12), a1 = ora_rd32(s12 + 4), a2 = ora_rd32(s12 + 8);
    uint32_t u[4] = {a0 & 0x3f3f3f3fu, (a2 & 0x0f0f0f0fu) | ((a0 >> 2) & 0x30303030u), a1 & 0x3f3f3f3fu,
                     ((a2 >> 4) & 0x0f0f0f0fu) | ((a1 >> 2) & 0x30303030u)};
    for (int l = 0; l < 8; l++) {
        sc[l] = (uint8_t)(u[l / 4] >> (8 * (l % 4)));
        mn[l] = (uint8_t)(u[2 + l / 4] >> (8 * (l % 4)));
    }
}

// Value n (0..256) of a Q4_K super-block's 4-bit codes (crates/gguf/src/quant.rs:738-767).
static inline int q4k_code(const uint8_t *qs, int n) {
    int p = n / 64, r = n % 64;
    uint8_t b = qs[32 * p + (r & 31)];
    return r < 32 ? (b & 0xf) : (b >> 4);
}

// Value n of a Q5_K super-block's 5-bit codes: the Q4_K nibble of its code bytes (at 48) and bit n / 32 of high byte
// n % 32 (at 16) on top (crates/gguf/src/quant.rs dequant_q5_k; crates/qdot/src/lib.rs:4882-4893: "value 128 j + 32 b +
// l takes bit 4 j + b of qh[l]").
static inline int q5k_code(const uint8_t *wb, int n) {
    return q4k_code(wb + 48, n) | (((wb[16 + (n & 31)] >> (n >> 5)) & 1) << 4);
}

// The exact integers of super-block `i`: halves[s][h] = sum over the 16 values 32s+16h.. of q * a, the two i32
// lanes `s & 3` and `4 + (s & 3)` of the reference's sumi for j = s / 4 (crates/qdot/src/lib.rs:4402-4430: with
// codes <= 15 (Q5_K: <= 31, :4889-4891) and |a| <= 128 neither maddubs nor the i16 adds saturate or wrap, so the
// lanes are plain sums). Q5_K is the same walk over 5-bit codes (:4882-4893).
static void q45k_halves(const uint8_t *wb, const uint8_t *acol, int i, int q5, int32_t halves[8][2]) {
    for (int s = 0; s < 8; s++) {
        const uint8_t *g = acol + (size_t)(2 * i + s / 4) * ORA_Q82X4_STRIDE;
        const int8_t *a = (const int8_t *)(g + 16 + 32 * (s & 3));
        for (int h = 0; h < 2; h++) {
            int32_t sum = 0;
            for (int n = 0; n < 16; n++) {
                int at = 32 * s + 16 * h + n;
                sum += (q5 ? q5k_code(wb, at) : q4k_code(wb + 16, at)) * a[16 * h + n];
            }
            halves[s][h] = sum;
        }
    }
}
static void q4k_halves(const uint8_t *wb, const uint8_t *acol, int i, int32_t halves[8][2]) {
    q45k_halves(wb, acol, i, 0, halves);
}

static float dot_q45k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb, int q5);

// Q4_K x Q8_2_X4, the scalar mirror's float steps in its order (crates/qdot/src/lib.rs:4363-4447).
float ora_dot_q4k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb) { return dot_q45k_q82x4(wrow, acol, nb, 0); }

// Q5_K x Q8_2_X4 (crates/qdot/src/lib.rs:4991-5090 dot_q5k_q82x4_emul): the Q4_K walk, block for block and lane for
// lane, over the wider block and its 5-bit codes.
float ora_dot_q5k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb) { return dot_q45k_q82x4(wrow, acol, nb, 1); }

static float dot_q45k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb, int q5) {
    float accd[8] = {0};
    for (int i = 0; i < nb; i++) {
        const uint8_t *wb = wrow + (size_t)i * (q5 ? ORA_Q5K_BLOCK : ORA_Q4K_BLOCK);
        const uint8_t *g0 = acol + (size_t)(2 * i) * ORA_Q82X4_STRIDE;
        const uint8_t *g1 = g0 + ORA_Q82X4_STRIDE;
        float d = ora_half_to_f32(ora_rd16(wb));
        float dmin = ora_half_to_f32(ora_rd16(wb + 2));
        uint8_t sc[8], mn[8];
        q4k_scales_mins(wb + 4, sc, mn);
        float mins[8], d8[8], all_scales[8];
        for (int l = 0; l < 8; l++) mins[l] = -(dmin * (float)mn[l]);
        for (int l = 0; l < 4; l++) {
            d8[l] = ora_bf16_to_f32(ora_rd16(g0 + 2 * l));
            d8[4 + l] = ora_bf16_to_f32(ora_rd16(g1 + 2 * l));
        }
        for (int l = 0; l < 4; l++) {
            float s0 = (float)(int16_t)ora_rd16(g0 + 8 + 2 * l);
            float s1 = (float)(int16_t)ora_rd16(g1 + 8 + 2 * l);
            accd[l] = fmaf(d8[l] * s0, mins[l], accd[l]);
            accd[4 + l] = fmaf(d8[4 + l] * s1, mins[4 + l], accd[4 + l]);
        }
        for (int l = 0; l < 8; l++) all_scales[l] = d * (float)sc[l];
        int32_t halves[8][2];
        q45k_halves(wb, acol, i, q5, halves);
        for (int j = 0; j < 2; j++) {
            for (int l = 0; l < 8; l++) {
                int idx = 4 * j + (l & 3);
                float d4d8 = all_scales[idx] * d8[idx];
                accd[l] = fmaf(d4d8, (float)halves[idx][l >> 2], accd[l]);
            }
        }
    }
    float t[4] = {accd[0] + accd[4], accd[1] + accd[5], accd[2] + accd[6], accd[3] + accd[7]};
    return (t[0] + t[2]) + (t[1] + t[3]);
}

// Per super-block, per 32-value sub-block: A = sum q4 * a (= lane s&3 + lane 4+(s&3) of the reference's sumi)
// and the column's isum as the dot reads it.
void ora_q4k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *a_out, int32_t *isum_out) {
    for (int i = 0; i < nb; i++) {
        int32_t halves[8][2];
        q4k_halves(wrow + (size_t)i * ORA_Q4K_BLOCK, acol, i, halves);
        for (int s = 0; s < 8; s++) {
            const uint8_t *g = acol + (size_t)(2 * i + s / 4) * ORA_Q82X4_STRIDE;
            a_out[8 * i + s] = halves[s][0] + halves[s][1];
            isum_out[8 * i + s] = (int16_t)ora_rd16(g + 8 + 2 * (s & 3));
        }
    }
}

void ora_q5k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *a_out, int32_t *isum_out) {
    for (int i = 0; i < nb; i++) {
        int32_t halves[8][2];
        q45k_halves(wrow + (size_t)i * ORA_Q5K_BLOCK, acol, i, 1, halves);
        for (int s = 0; s < 8; s++) {
            const uint8_t *g = acol + (size_t)(2 * i + s / 4) * ORA_Q82X4_STRIDE;
            a_out[8 * i + s] = halves[s][0] + halves[s][1];
            isum_out[8 * i + s] = (int16_t)ora_rd16(g + 8 + 2 * (s & 3));
        }
    }
}

// ------------------------------------------------------------------------------------------------------ Q6_K dot

// Value n (0..256) of a Q6_K super-block, already less 32 (crates/gguf/src/quant.rs:826-859).
static inline int q6k_code(const uint8_t *wb, int n) {
    int c = n / 128, r = n % 128, a = r / 32, l = r % 32;
    uint8_t lb = wb[64 * c + 32 * (a & 1) + l];
    int lo = (a < 2) ? (lb & 0xf) : (lb >> 4);
    int hi = (wb[128 + 32 * c + l] >> (2 * a)) & 3;
    return (lo | (hi << 4)) - 32;
}

// `_mm256_sign_epi8(a, b)` on one byte.
static inline int8_t sign_epi8(int8_t a, int8_t b) { return b < 0 ? (int8_t)(uint8_t)(-(int)a) : (b == 0 ? 0 : a); }

// One i32 lane of the reference's Q6_K sumi: the 16 values n0.. of the super-block against codes a[0..16].
// `fold` takes the kernel's own route, |w| on maddubs' unsigned side and the weight's sign folded into the
// activation byte (crates/qdot/src/lib.rs:4827-4859), which differs from the plain sum only where an activation
// code of -128 meets a negative weight: -(-128) wraps to -128. A maddubs pair peaks at 2*32*128 = 8192 and four
// of them at 32768 - 4*... stays inside i16 for every reachable input, so no saturation is modelled beyond it.
static int32_t q6k_lane(const uint8_t *wb, int n0, const int8_t *a, int fold) {
    int32_t sum = 0;
    for (int n = 0; n < 16; n++) {
        int w = q6k_code(wb, n0 + n);
        if (fold) {
            int uw = w < 0 ? -w : w;
            sum += uw * (int)sign_epi8(a[n], (int8_t)w);
        } else {
            sum += w * (int)a[n];
        }
    }
    return sum;
}

// Q6_K x Q8_2_X4, the scalar mirror's float steps in its order (crates/qdot/src/lib.rs:4776-4874).
float ora_dot_q6k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb) {
    float accd[8] = {0};
    for (int i = 0; i < nb; i++) {
        const uint8_t *wb = wrow + (size_t)i * ORA_Q6K_BLOCK;
        const uint8_t *g0 = acol + (size_t)(2 * i) * ORA_Q82X4_STRIDE;
        const uint8_t *g1 = g0 + ORA_Q82X4_STRIDE;
        float d = ora_half_to_f32(ora_rd16(wb + 208));
        float d8[8];
        for (int l = 0; l < 4; l++) {
            d8[l] = ora_bf16_to_f32(ora_rd16(g0 + 2 * l));
            d8[4 + l] = ora_bf16_to_f32(ora_rd16(g1 + 2 * l));
        }
        for (int j = 0; j < 2; j++) {
            const uint8_t *g = j ? g1 : g0;
            for (int l = 0; l < 8; l++) {
                // Lane l < 4 reads scale 8j + 2l, lane 4 + l scale 8j + 2l + 1 (K_SHUFFLE_Q6K, :4455).
                int blk = l & 3, half = l >> 2;
                float sc = (float)(int8_t)wb[192 + 8 * j + 2 * blk + half];
                float scale = (d * sc) * d8[4 * j + blk];
                const int8_t *a = (const int8_t *)(g + 16 + 32 * blk + 16 * half);
                int32_t sumi = q6k_lane(wb, 128 * j + 32 * blk + 16 * half, a, 1);
                accd[l] = fmaf(scale, (float)sumi, accd[l]);
            }
        }
    }
    float t[4] = {accd[0] + accd[4], accd[1] + accd[5], accd[2] + accd[6], accd[3] + accd[7]};
    return (t[0] + t[2]) + (t[1] + t[3]);
}

// Per super-block, per 16-value group g: S = sum (q6 - 32) * a. `fold` != 0 gives the reference kernel's lanes.
void ora_q6k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int fold, int32_t *s_out) {
    for (int i = 0; i < nb; i++) {
        const uint8_t *wb = wrow + (size_t)i * ORA_Q6K_BLOCK;
        for (int g = 0; g < 16; g++) {
            const uint8_t *grp = acol + (size_t)(2 * i + g / 8) * ORA_Q82X4_STRIDE;
            const int8_t *a = (const int8_t *)(grp + 16 + 16 * (g & 7));
            s_out[16 * i + g] = q6k_lane(wb, 16 * g, a, fold);
        }
    }
}

// --------------------------------------------------------------------------------------------------- IQ2_XXS dot

// Signed grid value n (0..32) of sub-block b (crates/qdot/src/lib.rs:8699-8707).
static inline int iq2xxs_value(const uint8_t *blk, int b, int n) {
    const uint8_t *idx = blk + 2 + 8 * b;
    uint32_t word = ora_rd32(blk + 6 + 8 * b);
    int mag = (int)((ORA_IQ2XXS_GRID[idx[n / 8]] >> (8 * (n % 8))) & 0xff);
    uint8_t signs = ORA_KSIGNS_IQ2XS[(word >> (7 * (n / 8))) & 127];
    return ((signs >> (n % 8)) & 1) ? -mag : mag;
}

// IQ2_XXS x Q8_K, the scalar mirror's float steps in its order (crates/qdot/src/lib.rs:8677-8724).
float ora_dot_iq2xxs_q8k(const uint8_t *wrow, const uint8_t *acol, int nb) {
    float accd[8] = {0};
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ2XXS_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        float d = 0.125f * ora_half_to_f32(ora_rd16(blk));
        int32_t sc[8];
        for (int b = 0; b < 8; b++) sc[b] = 2 * (int32_t)(ora_rd32(blk + 6 + 8 * b) >> 28) + 1;
        float dmin = -d * 43.0f;
        float dy = ora_bits_f32(ora_rd32(col));
        for (int l = 0; l < 8; l++) {
            int32_t b0 = (int16_t)ora_rd16(col + 264 + 4 * l);
            int32_t b1 = (int16_t)ora_rd16(col + 266 + 4 * l);
            int32_t m = sc[l] * b0 + sc[l] * b1;
            accd[l] = fmaf(dmin * dy, (float)m, accd[l]);
        }
        int32_t sumi[8] = {0};
        for (int b = 0; b < 8; b++) {
            for (int n = 0; n < 32; n++) {
                int v = iq2xxs_value(blk, b, n);
                int32_t u = (uint8_t)(int8_t)(v + 43);
                int32_t a = (int8_t)col[8 + 32 * b + n];
                sumi[n / 4] += sc[b] * u * a;
            }
        }
        for (int l = 0; l < 8; l++) accd[l] = fmaf(d * dy, (float)sumi[l], accd[l]);
    }
    float t[4] = {accd[0] + accd[4], accd[1] + accd[5], accd[2] + accd[6], accd[3] + accd[7]};
    return (t[0] + t[2]) + (t[1] + t[3]);
}

// Per super-block: I[b] = sum over sub-block b of (+-grid) * a (no +43), sc[b] = 2s + 1, and the two aggregates
// the reference's lanes add up to: codes = sum_b sc_b * (I_b + 43 * (bsum[2b] + bsum[2b+1])) and
// fold = sum_b sc_b * (bsum[2b] + bsum[2b+1]).
void ora_iq2xxs_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *i_out, int32_t *sc_out,
                           int32_t *codes_out, int32_t *fold_out) {
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ2XXS_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        int32_t codes = 0, fold = 0;
        for (int b = 0; b < 8; b++) {
            int32_t s = 2 * (int32_t)(ora_rd32(blk + 6 + 8 * b) >> 28) + 1;
            int32_t sum = 0;
            for (int n = 0; n < 32; n++) sum += iq2xxs_value(blk, b, n) * (int32_t)(int8_t)col[8 + 32 * b + n];
            int32_t bs = (int16_t)ora_rd16(col + 264 + 4 * b) + (int16_t)ora_rd16(col + 266 + 4 * b);
            i_out[8 * i + b] = sum;
            sc_out[8 * i + b] = s;
            codes += s * (sum + 43 * bs);
            fold += s * bs;
        }
        codes_out[i] = codes;
        fold_out[i] = fold;
    }
}

// --------------------------------------------------------------------------------------------------- IQ3_XXS dot

// Signed grid value n (0..32) of sub-block b: group n / 8 takes grid words qs[8b + 2 (n / 8)] (its values 0..3) and the
// next (4..7), four magnitudes a word, and bit n % 8 of the group's sign byte (crates/gguf/src/quant.rs:1739-1772).
static inline int iq3xxs_value(const uint8_t *blk, int b, int n) {
    uint32_t word = ora_rd32(blk + 66 + 4 * b);
    int mag = (int)((ORA_IQ3XXS_GRID[blk[2 + 8 * b + n / 4]] >> (8 * (n % 4))) & 0xff);
    uint8_t signs = ORA_KSIGNS_IQ2XS[(word >> (7 * (n / 8))) & 127];
    return ((signs >> (n % 8)) & 1) ? -mag : mag;
}

// IQ3_XXS x Q8_K, the scalar mirror's float steps in its order (crates/qdot/src/lib.rs:7494-7541): IQ2_XXS's walk with
// d = f16 / 4, the offset 64 and four-magnitude grid words.
float ora_dot_iq3xxs_q8k(const uint8_t *wrow, const uint8_t *acol, int nb) {
    float accd[8] = {0};
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ3XXS_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        float d = 0.25f * ora_half_to_f32(ora_rd16(blk));
        int32_t sc[8];
        for (int b = 0; b < 8; b++) sc[b] = 2 * (int32_t)(ora_rd32(blk + 66 + 4 * b) >> 28) + 1;
        float dmin = -d * 64.0f;
        float dy = ora_bits_f32(ora_rd32(col));
        for (int l = 0; l < 8; l++) {
            int32_t b0 = (int16_t)ora_rd16(col + 264 + 4 * l);
            int32_t b1 = (int16_t)ora_rd16(col + 266 + 4 * l);
            int32_t m = sc[l] * b0 + sc[l] * b1;
            accd[l] = fmaf(dmin * dy, (float)m, accd[l]);
        }
        int32_t sumi[8] = {0};
        for (int b = 0; b < 8; b++) {
            for (int n = 0; n < 32; n++) {
                int v = iq3xxs_value(blk, b, n);
                int32_t u = (uint8_t)(int8_t)(v + 64);
                int32_t a = (int8_t)col[8 + 32 * b + n];
                sumi[n / 4] += sc[b] * u * a;
            }
        }
        for (int l = 0; l < 8; l++) accd[l] = fmaf(d * dy, (float)sumi[l], accd[l]);
    }
    float t[4] = {accd[0] + accd[4], accd[1] + accd[5], accd[2] + accd[6], accd[3] + accd[7]};
    return (t[0] + t[2]) + (t[1] + t[3]);
}

// As ora_iq2xxs_block_sums, with the offset 64.
void ora_iq3xxs_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *i_out, int32_t *sc_out,
                           int32_t *codes_out, int32_t *fold_out) {
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ3XXS_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        int32_t codes = 0, fold = 0;
        for (int b = 0; b < 8; b++) {
            int32_t s = 2 * (int32_t)(ora_rd32(blk + 66 + 4 * b) >> 28) + 1;
            int32_t sum = 0;
            for (int n = 0; n < 32; n++) sum += iq3xxs_value(blk, b, n) * (int32_t)(int8_t)col[8 + 32 * b + n];
            int32_t bs = (int16_t)ora_rd16(col + 264 + 4 * b) + (int16_t)ora_rd16(col + 266 + 4 * b);
            i_out[8 * i + b] = sum;
            sc_out[8 * i + b] = s;
            codes += s * (sum + 64 * bs);
            fold += s * bs;
        }
        codes_out[i] = codes;
        fold_out[i] = fold;
    }
}

// ---------------------------------------------------------------------------------------------------- IQ4_XS dot

// Sub-block b's 6-bit scale less 32: nibble b % 2 of scales_l[b / 2] under bits 2b.. of scales_h
// (crates/gguf/src/quant.rs:1989-1991, crates/qdot/src/lib.rs:11158-11160).
static inline int iq4xs_scale(const uint8_t *blk, int b) {
    int lo = (blk[4 + b / 2] >> (4 * (b % 2))) & 0x0f, hi = (ora_rd16(blk + 2) >> (2 * b)) & 3;
    return (lo | (hi << 4)) - 32;
}

// Level n (0..32) of sub-block b: values 0..15 are the low nibbles of its sixteen bytes, 16..31 the high ones.
static inline int iq4xs_value(const uint8_t *blk, int b, int n) {
    uint8_t byte = blk[8 + 16 * b + (n % 16)];
    return ORA_KVALUES_IQ4NL[n < 16 ? (byte & 0x0f) : (byte >> 4)];
}

// IQ4_XS x Q8_K, the scalar mirror's steps in its order (crates/qdot/src/lib.rs:11147-11180). The vector kernel puts
// a level's magnitude on the unsigned side and folds its sign into the activation byte; -(-128) wraps there, so a
// -128 code under a negative level counts as -128 (ik's Q8_K encoder never writes one).
float ora_dot_iq4xs_q8k(const uint8_t *wrow, const uint8_t *acol, int nb) {
    float accd[8] = {0};
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ4XS_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        float d = ora_half_to_f32(ora_rd16(blk));
        float dy = ora_bits_f32(ora_rd32(col));
        int32_t sumi[8] = {0};
        for (int b = 0; b < 8; b++) {
            int scale = iq4xs_scale(blk, b);
            for (int n = 0; n < 32; n++) {
                int w = iq4xs_value(blk, b, n);
                int8_t a = (int8_t)col[8 + 32 * b + n];
                int8_t q = w < 0 ? (int8_t)(uint8_t)(0u - (uint8_t)a) : (w == 0 ? 0 : a);
                sumi[n / 4] += scale * (w < 0 ? -w : w) * (int32_t)q;
            }
        }
        for (int l = 0; l < 8; l++) accd[l] = fmaf(d * dy, (float)sumi[l], accd[l]);
    }
    float t[4] = {accd[0] + accd[4], accd[1] + accd[5], accd[2] + accd[6], accd[3] + accd[7]};
    return (t[0] + t[2]) + (t[1] + t[3]);
}

// Per super-block: I[b] = sum over sub-block b of level * a, and the eight lane sums L[l] = sum_b scale_b * (sum over
// values 4l .. 4l + 3 of sub-block b of level * a) the reference's i32 lanes hold. `fold` counts a -128 code under a
// negative level as the vector kernel's sign fold does (see the dot above); without it the products are plain.
void ora_iq4xs_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int fold, int32_t *i_out,
                          int32_t *lanes_out) {
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ4XS_BLOCK;
        const uint8_t *col = acol + (size_t)i * ORA_Q8K_STRIDE;
        for (int l = 0; l < 8; l++) lanes_out[8 * i + l] = 0;
        for (int b = 0; b < 8; b++) {
            int32_t sum = 0;
            for (int n = 0; n < 32; n++) {
                int32_t w = iq4xs_value(blk, b, n), a = (int8_t)col[8 + 32 * b + n];
                int32_t p = (fold && w < 0 && a == -128) ? w * 128 : w * a;
                sum += p;
                lanes_out[8 * i + n / 4] += iq4xs_scale(blk, b) * p;
            }
            i_out[8 * i + b] = sum;
        }
    }
}

// ----------------------------------------------------------------------------------------------------- dispatch

// crates/qdot/src/lib.rs:691-723 with check_row's refusals (:1727-1779) as return codes.
int ora_dot_row(int wtype, const uint8_t *wrow, size_t wrow_len, const uint8_t *acol, size_t acol_len, int k,
                float *out) {
    int need_w = ora_row_bytes(wtype, k);
    if (need_w < 0) return need_w;
    int need_a = ora_col_bytes(wtype, k);
    if (wrow_len < (size_t)need_w) return ORA_ESHORTROW;
    if (acol_len < (size_t)need_a) return ORA_ESHORTCOL;
    int nb = k / 256;
    switch (wtype) {
    case ORA_TYPE_Q3_K:
        *out = ora_dot_q3k_q8k(wrow, acol, nb);
        return 0;
    case ORA_TYPE_Q4_K:
        *out = ora_dot_q4k_q82x4(wrow, acol, nb);
        return 0;
    case ORA_TYPE_Q5_K:
        *out = ora_dot_q5k_q82x4(wrow, acol, nb);
        return 0;
    case ORA_TYPE_Q6_K:
        *out = ora_dot_q6k_q82x4(wrow, acol, nb);
        return 0;
    case ORA_TYPE_IQ2_XXS:
        *out = ora_dot_iq2xxs_q8k(wrow, acol, nb);
        return 0;
    case ORA_TYPE_IQ3_XXS:
        *out = ora_dot_iq3xxs_q8k(wrow, acol, nb);
        return 0;
    case ORA_TYPE_IQ4_XS:
        *out = ora_dot_iq4xs_q8k(wrow, acol, nb);
        return 0;
    default:
        return ORA_ETYPE;
    }
}

// y[r * m + c] = row r . column c for r < rows, c < m: the shape of the reference's gemv
// (crates/gpu/src/lib.rs:1617), every value dot_row's (the multi-column forms are per-column bit-identical,
// crates/qdot/src/lib.rs:892-904).
int ora_gemv(int wtype, const uint8_t *w, int rows, int k, const uint8_t *act, int m, float *y) {
    int rb = ora_row_bytes(wtype, k), cb = ora_col_bytes(wtype, k);
    if (rb < 0) return rb;
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < m; c++) {
            int rc = ora_dot_row(wtype, w + (size_t)r * rb, rb, act + (size_t)c * cb, cb, k, &y[(size_t)r * m + c]);
            if (rc) return rc;
        }
    return 0;
}

// --------------------------------------------------------------------------------------------------- dequantize

int ora_dequant_row(int wtype, const uint8_t *src, int k, float *dst) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    for (int i = 0; i < k / 256; i++) {
        float *out = dst + 256 * i;
        if (wtype == ORA_TYPE_Q3_K) { // crates/gguf/src/quant.rs:679-727
            const uint8_t *blk = src + (size_t)i * ORA_Q3K_BLOCK;
            float d = ora_half_to_f32(ora_rd16(blk + 108));
            uint8_t sc[16];
            q3k_scales6(blk, sc);
            for (int n = 0; n < 256; n++) out[n] = (d * (float)((int)sc[n / 16] - 32)) * (float)q3k_value(blk, n);
        } else if (wtype == ORA_TYPE_Q4_K) { // crates/gguf/src/quant.rs:738-767
            const uint8_t *blk = src + (size_t)i * ORA_Q4K_BLOCK;
            float d = ora_half_to_f32(ora_rd16(blk)), dmin = ora_half_to_f32(ora_rd16(blk + 2));
            uint8_t sc[8], mn[8];
            q4k_scales_mins(blk + 4, sc, mn);
            for (int n = 0; n < 256; n++) {
                float d1 = d * (float)sc[n / 32], m1 = dmin * (float)mn[n / 32];
                out[n] = fmaf((float)q4k_code(blk + 16, n), d1, -m1);
            }
        } else if (wtype == ORA_TYPE_Q5_K) { // crates/gguf/src/quant.rs:780-816
            const uint8_t *blk = src + (size_t)i * ORA_Q5K_BLOCK;
            float d = ora_half_to_f32(ora_rd16(blk)), dmin = ora_half_to_f32(ora_rd16(blk + 2));
            uint8_t sc[8], mn[8];
            q4k_scales_mins(blk + 4, sc, mn);
            for (int n = 0; n < 256; n++) {
                float d1 = d * (float)sc[n / 32], m1 = dmin * (float)mn[n / 32];
                out[n] = fmaf((float)q5k_code(blk, n), d1, -m1);
            }
        } else if (wtype == ORA_TYPE_Q6_K) { // crates/gguf/src/quant.rs:826-859
            const uint8_t *blk = src + (size_t)i * ORA_Q6K_BLOCK;
            float d = ora_half_to_f32(ora_rd16(blk + 208));
            for (int n = 0; n < 256; n++) out[n] = (d * (float)(int8_t)blk[192 + n / 16]) * (float)q6k_code(blk, n);
        } else if (wtype == ORA_TYPE_IQ2_XXS) { // crates/gguf/src/quant.rs:1679-1700
            const uint8_t *blk = src + (size_t)i * ORA_IQ2XXS_BLOCK;
            float d = ora_half_to_f32(ora_rd16(blk));
            for (int b = 0; b < 8; b++) {
                uint32_t aux = ora_rd32(blk + 6 + 8 * b);
                float db = d * (0.5f + (float)(aux >> 28)) * 0.25f;
                for (int n = 0; n < 32; n++) {
                    int v = iq2xxs_value(blk, b, n);
                    float mag = (float)(v < 0 ? -v : v);
                    out[32 * b + n] = db * mag * (v < 0 ? -1.0f : 1.0f);
                }
            }
        } else if (wtype == ORA_TYPE_IQ3_XXS) { // crates/gguf/src/quant.rs:1748-1772
            const uint8_t *blk = src + (size_t)i * ORA_IQ3XXS_BLOCK;
            float d = ora_half_to_f32(ora_rd16(blk));
            for (int b = 0; b < 8; b++) {
                uint32_t aux = ora_rd32(blk + 66 + 4 * b);
                float db = d * (0.5f + (float)(aux >> 28)) * 0.5f;
                for (int n = 0; n < 32; n++) {
                    int v = iq3xxs_value(blk, b, n);
                    float mag = (float)(v < 0 ? -v : v);
                    out[32 * b + n] = db * mag * (v < 0 ? -1.0f : 1.0f);
                }
            }
        } else if (wtype == ORA_TYPE_IQ4_XS) { // crates/gguf/src/quant.rs:1977-1999
            const uint8_t *blk = src + (size_t)i * ORA_IQ4XS_BLOCK;
            float d = ora_half_to_f32(ora_rd16(blk));
            for (int b = 0; b < 8; b++) {
                float dl = d * (float)iq4xs_scale(blk, b);
                for (int n = 0; n < 32; n++) out[32 * b + n] = dl * (float)iq4xs_value(blk, b, n);
            }
        } else {
            return ORA_ETYPE;
        }
    }
    return 0;
}

// Decoded value of one activation column (code times its block scale), for the f64 band checks.
int ora_dequant_col(int wtype, const uint8_t *acol, int k, float *dst) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    if (ora_takes_q8k(wtype)) {
        for (int b = 0; b < k / 256; b++) {
            const uint8_t *o = acol + (size_t)b * ORA_Q8K_STRIDE;
            float d = ora_bits_f32(ora_rd32(o));
            for (int j = 0; j < 256; j++) dst[256 * b + j] = d * (float)(int8_t)o[8 + j];
        }
        return 0;
    }
    if (wtype != ORA_TYPE_Q4_K && wtype != ORA_TYPE_Q5_K && wtype != ORA_TYPE_Q6_K) return ORA_ETYPE;
    for (int g = 0; g < k / 128; g++) {
        const uint8_t *grp = acol + (size_t)g * ORA_Q82X4_STRIDE;
        for (int ir = 0; ir < 4; ir++) {
            float d = ora_bf16_to_f32(ora_rd16(grp + 2 * ir));
            for (int m = 0; m < 32; m++) dst[128 * g + 32 * ir + m] = d * (float)(int8_t)grp[16 + 32 * ir + m];
        }
    }
    return 0;
}

// ------------------------------------------------------------------------------------------------------- SwiGLU

// crates/qdot/src/lib.rs:3741-3773.
float ora_expf_ik(float x) {
    const float SHIFT = ora_bits_f32(0x4b400000u), LOG2E = ora_bits_f32(0x3fb8aa3bu);
    const float LN2_HI = ora_bits_f32(0x3f317200u), LN2_LO = ora_bits_f32(0x35bfbe8eu);
    const float C0 = ora_bits_f32(0x3f7ffff6u), C1 = ora_bits_f32(0x3efffedbu), C2 = ora_bits_f32(0x3e2aaf33u);
    const float C3 = ora_bits_f32(0x3d2b9f17u), C4 = ora_bits_f32(0x3c072010u);
    float z = fmaf(x, LOG2E, SHIFT);
    float n = z - SHIFT;
    float b = fmaf(-n, LN2_LO, fmaf(-n, LN2_HI, x));
    uint32_t e = ora_f32_bits(z) << 23;
    float k = ora_bits_f32(e + 0x3f800000u);
    float u = b * b;
    float j = fmaf(fmaf(fmaf(C4, b, C3), u, fmaf(C2, b, C1)), u, C0 * b);
    if (fabsf(n) > 126.0f) {
        uint32_t g = (n <= 0.0f) ? 0x82000000u : 0u;
        float s1 = ora_bits_f32(g + 0x7f000000u);
        float s2 = ora_bits_f32(e - g);
        if (fabsf(n) > 192.0f) return s1 * s1;
        return fmaf(s2, j, s2) * s1;
    }
    return fmaf(j, k, k);
}

// crates/qdot/src/lib.rs:11467-11478: divide, then multiply.
void ora_swiglu(const float *gate, const float *up, int n, float *out) {
    for (int i = 0; i < n; i++) out[i] = gate[i] / (1.0f + ora_expf_ik(0.0f - gate[i])) * up[i];
}

// The other gate . up rules of the CPU path, each comparison spelled as the reference spells it (so a NaN falls
// through the same way), the exponential ik's. rule 1: swiglu_clamp (crates/qdot/src/lib.rs:11492-11523): min(silu(g),
// limit) * clamp(u), nothing clamped at limit <= 1e-6. rule 2: swiglu_oai / swiglu_oai_1 at alpha 1.702 (the value the
// launchers run, crates/gpu/src/kquant/act.rs:58-60): x = min(g, limit), y = clamp(u), x / (1 + e^(alpha (0 - x))) *
// (y + 1). rule 4: swiglu_gclamp / swiglu_gclamp_1 (:11617-11660): silu(min(g, limit)) * clamp(u), nothing clamped at
// limit <= 1e-6. rule 3: SiTU-GLU at linear beta 25, limit = the gate's beta (crates/model/src/ops.rs:2345-2360
// situ_into: each scale by the f32 reciprocal, the host libm's tanhf, the scale back, 1 / (1 + e^(0 - g)), (a * s) * v);
// its tanh is whatever libm this file is linked with, so the rule is pinned to the closed form in f64 at the
// reference's own bound (1e-5 relative, ops.rs:7124-7160), not to bits. rule 0: ora_swiglu. Returns what the reference's functions return: 0 when a clamping rule met a gate
// or up value that is not finite (the caller refuses the block), else 1; -1 for a rule this file does not hold.
int ora_gate_rule(int rule, float limit, const float *gate, const float *up, int n, float *out) {
    if (rule == 0) {
        ora_swiglu(gate, up, n, out);
        return 1;
    }
    if (rule < 1 || rule > 4) return -1;
    if ((rule == 1 || rule == 4) && !(limit > 1e-6f)) { // a NaN limit clamps nothing either
        ora_swiglu(gate, up, n, out);
        return 1;
    }
    int finite = 1;
    for (int i = 0; i < n; i++) {
        const float g = gate[i], u = up[i];
        if (!isfinite(g) || !isfinite(u)) finite = 0;
        if (rule == 3) {
            const float a = tanhf(g * (1.0f / limit)) * limit;
            const float sg = 1.0f / (1.0f + ora_expf_ik(0.0f - g));
            const float v = tanhf(u * (1.0f / 25.0f)) * 25.0f;
            out[i] = (a * sg) * v;
        } else if (rule == 1) {
            float s = g / (1.0f + ora_expf_ik(0.0f - g));
            s = limit < s ? limit : s;
            float c = u < limit ? u : limit;
            c = -limit < c ? c : -limit;
            out[i] = c * s;
        } else {
            const float x = limit < g ? limit : g;
            const float y = u < -limit ? -limit : (limit < u ? limit : u);
            if (rule == 2)
                out[i] = x / (1.0f + ora_expf_ik(1.702f * (0.0f - x))) * (y + 1.0f);
            else
                out[i] = x / (1.0f + ora_expf_ik(0.0f - x)) * y;
        }
    }
    return finite;
}
