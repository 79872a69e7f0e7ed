// TEST INFRASTRUCTURE ONLY (see ora_common.h). AVX2+FMA+F16C restatement of the reference's vector kernels, in
// their instruction order: the two activation encoders and the Q4_K / Q5_K / Q6_K / IQ2_XXS / IQ4_XS row dots, one column or a
// tile of up to eight columns that unpacks each weight block once. It has two uses: the test suite holds it
// bit-equal to the scalar restatement in qdot.c (two independently written paths through the same arithmetic,
// the reference's own first gate, crates/qdot/tests/qdot.rs:346,738,818,2664), and the benchmark times it as the
// CPU baseline. Build with -mavx2 -mfma -mf16c -ffp-contract=off.
#define _GNU_SOURCE
#include <sched.h>
#include <immintrin.h>
#include <pthread.h>
#include <stdlib.h>

#include "bm_oracle.h"
#include "bm_oracle_avx2.h"
#include "iq_tables.h"
#include "ora_common.h"

int ora_avx2_supported(void) {
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") && __builtin_cpu_supports("f16c");
}

// ------------------------------------------------------------------------------------------------- small helpers

// crates/qdot/src/lib.rs:1822-1832.
static inline __m256i v_nearest_int(__m256 y) {
    __m256 z = _mm256_add_ps(y, _mm256_set1_ps(12582912.0f));
    __m256i b = _mm256_castps_si256(z);
    return _mm256_sub_epi32(_mm256_and_si256(b, _mm256_set1_epi32(0x007fffff)), _mm256_set1_epi32(0x00400000));
}

// crates/qdot/src/lib.rs:1844-1851.
static inline __m256i v_wrap_i8(__m256i q) {
    __m256i t = _mm256_and_si256(q, _mm256_set1_epi32(0xFF));
    __m256i ge = _mm256_cmpgt_epi32(t, _mm256_set1_epi32(127));
    return _mm256_sub_epi32(t, _mm256_and_si256(ge, _mm256_set1_epi32(256)));
}

// crates/qdot/src/lib.rs:1862-1871.
static inline float hmax_ps(__m256 v) {
    __m128 lo = _mm256_castps256_ps128(v), hi = _mm256_extractf128_ps(v, 1);
    __m128 m = _mm_max_ps(lo, hi);
    m = _mm_max_ps(m, _mm_movehl_ps(m, m));
    return _mm_cvtss_f32(_mm_max_ss(m, _mm_movehdup_ps(m)));
}

// crates/qdot/src/lib.rs:1978-1986.
static inline int32_t hsum_i32(__m256i v) {
    __m128i lo = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    lo = _mm_add_epi32(lo, _mm_shuffle_epi32(lo, 0x4E));
    lo = _mm_add_epi32(lo, _mm_shuffle_epi32(lo, 0x8D));
    return _mm_cvtsi128_si32(lo);
}

// crates/qdot/src/lib.rs:4128-4137. The order is load-bearing.
static inline float hsum_float_8(__m256 x) {
    __m128 res = _mm256_extractf128_ps(x, 1);
    res = _mm_add_ps(res, _mm256_castps256_ps128(x));
    res = _mm_add_ps(res, _mm_movehl_ps(res, res));
    res = _mm_add_ss(res, _mm_movehdup_ps(res));
    return _mm_cvtss_f32(res);
}

static inline float f16c_to_f32(uint16_t h) { return _mm_cvtss_f32(_mm_cvtph_ps(_mm_cvtsi32_si128(h))); }

// ------------------------------------------------------------------------------------------- activation encoders

// One 32-value q8_2 block (crates/qdot/src/lib.rs:3953-4002 under the bf16 rule, :3930-3939).
static int q82_block_avx2(const float *x, uint8_t *codes, uint16_t *t_out, int16_t *isum_out) {
    const __m256 sgn = _mm256_set1_ps(-0.0f);
    __m256 m = _mm256_setzero_ps(), unord = _mm256_setzero_ps();
    for (int j = 0; j < 4; j++) {
        __m256 v = _mm256_loadu_ps(x + 8 * j);
        m = _mm256_max_ps(_mm256_andnot_ps(sgn, v), m);
        unord = _mm256_or_ps(unord, _mm256_cmp_ps(v, v, _CMP_UNORD_Q));
    }
    float amax = hmax_ps(m);
    if (_mm256_movemask_ps(unord) != 0 || !isfinite(amax)) return ORA_ENONFINITE;
    uint16_t t = ora_fp32_to_bf16_bits(amax / 127.0f);
    __m256 idv = _mm256_set1_ps(ora_q82_inverse(t));
    __m256i qi[4];
    for (int j = 0; j < 4; j++) qi[j] = v_nearest_int(_mm256_mul_ps(_mm256_loadu_ps(x + 8 * j), idv));
    __m256i p0 = _mm256_packs_epi32(qi[0], qi[1]), p1 = _mm256_packs_epi32(qi[2], qi[3]);
    __m256i c = _mm256_packs_epi16(p0, p1);
    c = _mm256_permutevar8x32_epi32(c, _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7));
    _mm256_storeu_si256((__m256i *)codes, c);
    *t_out = t;
    *isum_out =
        (int16_t)hsum_i32(_mm256_add_epi32(_mm256_add_epi32(qi[0], qi[1]), _mm256_add_epi32(qi[2], qi[3])));
    return 0;
}

// crates/qdot/src/lib.rs:4014-4036 (whole groups).
int ora_avx2_quantize_q82x4(const float *x, int k, uint8_t *out) {
    if (k <= 0 || k % 128 != 0) return ORA_EUNALIGNED;
    for (int gi = 0; gi < k / 128; gi++) {
        uint8_t *group = out + (size_t)gi * ORA_Q82X4_STRIDE;
        memset(group, 0, ORA_Q82X4_STRIDE);
        for (int ir = 0; ir < 4; ir++) {
            uint16_t d;
            int16_t isum;
            int rc = q82_block_avx2(x + 128 * gi + 32 * ir, group + 16 + 32 * ir, &d, &isum);
            if (rc) return rc;
            ora_wr16(group + 2 * ir, d);
            ora_wr16(group + 8 + 2 * ir, (uint16_t)isum);
        }
    }
    return 0;
}

// crates/qdot/src/lib.rs:1885-1955.
int ora_avx2_quantize_q8k(const float *x, int k, uint8_t *out) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    const __m256 sgn = _mm256_set1_ps(-0.0f);
    for (int b = 0; b < k / 256; b++) {
        const float *xb = x + 256 * b;
        uint8_t *o = out + (size_t)b * ORA_Q8K_STRIDE;
        __m256 m = _mm256_setzero_ps(), unord = _mm256_setzero_ps();
        for (int i = 0; i < 32; i++) {
            __m256 v = _mm256_loadu_ps(xb + 8 * i);
            m = _mm256_max_ps(_mm256_andnot_ps(sgn, v), m);
            unord = _mm256_or_ps(unord, _mm256_cmp_ps(v, v, _CMP_UNORD_Q));
        }
        float amax = hmax_ps(m);
        if (_mm256_movemask_ps(unord) != 0 || !isfinite(amax)) return ORA_ENONFINITE;
        if (amax == 0.0f) {
            memset(o, 0, ORA_Q8K_STRIDE);
            continue;
        }
        __m256 amax_v = _mm256_set1_ps(amax);
        int first = 256;
        for (int i = 0; i < 32 && first == 256; i++) {
            __m256 v = _mm256_loadu_ps(xb + 8 * i);
            unsigned mask = (unsigned)_mm256_movemask_ps(_mm256_cmp_ps(_mm256_andnot_ps(sgn, v), amax_v, _CMP_EQ_OQ));
            if (mask) first = 8 * i + __builtin_ctz(mask);
        }
        float max = xb[first];
        float iscale = -127.0f / max;
        __m256 iscale_v = _mm256_set1_ps(iscale);
        __m256i clamp = _mm256_set1_epi32(127);
        for (int g = 0; g < 8; g++) {
            __m256i qi[4];
            for (int j = 0; j < 4; j++) {
                __m256 y = _mm256_mul_ps(_mm256_loadu_ps(xb + 32 * g + 8 * j), iscale_v);
                qi[j] = v_wrap_i8(_mm256_min_epi32(v_nearest_int(y), clamp));
            }
            __m256i p0 = _mm256_packs_epi32(qi[0], qi[1]), p1 = _mm256_packs_epi32(qi[2], qi[3]);
            __m256i c = _mm256_packs_epi16(p0, p1);
            c = _mm256_permutevar8x32_epi32(c, _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7));
            _mm256_storeu_si256((__m256i *)(o + 8 + 32 * g), c);
            ora_wr16(o + 264 + 4 * g, (uint16_t)(int16_t)hsum_i32(_mm256_add_epi32(qi[0], qi[1])));
            ora_wr16(o + 266 + 4 * g, (uint16_t)(int16_t)hsum_i32(_mm256_add_epi32(qi[2], qi[3])));
        }
        float d = 1.0f / iscale;
        memcpy(o, &d, 4);
        memset(o + 4, 0, 4);
    }
    return 0;
}

int ora_avx2_quantize_col(int wtype, const float *x, int k, uint8_t *out) {
    if (wtype == ORA_TYPE_Q4_K || wtype == ORA_TYPE_Q5_K || wtype == ORA_TYPE_Q6_K) return ora_avx2_quantize_q82x4(x, k, out);
    if (ora_takes_q8k(wtype)) return ora_avx2_quantize_q8k(x, k, out);
    return ORA_ETYPE;
}

// --------------------------------------------------------------------------------------------- shared dot pieces

// The eight bf16 block scales of super-block i's two groups as f32 (crates/qdot/src/lib.rs:4149-4158).
static inline __m256 q82x4_dy(const uint8_t *col, int i) {
    const uint8_t *g0 = col + (size_t)(2 * i) * ORA_Q82X4_STRIDE, *g1 = g0 + ORA_Q82X4_STRIDE;
    __m128i d4_1 = _mm_cvtepu16_epi32(_mm_loadl_epi64((const __m128i *)g0));
    __m128i d4_2 = _mm_cvtepu16_epi32(_mm_loadl_epi64((const __m128i *)g1));
    return _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_set_m128i(d4_2, d4_1), 16));
}

// dy times the blocks' i16 sums (crates/qdot/src/lib.rs:4160-4168).
static inline __m256 q82x4_my(const uint8_t *col, int i, __m256 dy) {
    const uint8_t *g0 = col + (size_t)(2 * i) * ORA_Q82X4_STRIDE, *g1 = g0 + ORA_Q82X4_STRIDE;
    __m128i m4_1 = _mm_cvtepi16_epi32(_mm_loadl_epi64((const __m128i *)(g0 + 8)));
    __m128i m4_2 = _mm_cvtepi16_epi32(_mm_loadl_epi64((const __m128i *)(g1 + 8)));
    return _mm256_mul_ps(dy, _mm256_cvtepi32_ps(_mm256_set_m128i(m4_2, m4_1)));
}

// Four maddubs results of a 128-value half reduced to eight i32 lanes: lane t the first 16 values of 32-block t,
// lane 4 + t the second 16 (crates/qdot/src/lib.rs:4251-4261).
static inline __m256i reduce4(__m256i s1, __m256i s2, __m256i s3, __m256i s4) {
    __m256i t1 = _mm256_add_epi16(_mm256_unpacklo_epi32(s1, s2), _mm256_unpackhi_epi32(s1, s2));
    __m256i t3 = _mm256_add_epi16(_mm256_unpacklo_epi32(s3, s4), _mm256_unpackhi_epi32(s3, s4));
    __m256i t = _mm256_add_epi16(_mm256_unpacklo_epi64(t1, t3), _mm256_unpackhi_epi64(t1, t3));
    return _mm256_madd_epi16(_mm256_set1_epi16(1), t);
}

static inline void q4_unpack_scales(const uint8_t *s12, uint32_t utmp[4]) {
    uint32_t a0, a1, a2;
    memcpy(&a0, s12, 4);
    memcpy(&a1, s12 + 4, 4);
    memcpy(&a2, s12 + 8, 4);
    utmp[0] = a0 & 0x3f3f3f3fu;
    utmp[1] = (a2 & 0x0f0f0f0fu) | ((a0 >> 2) & 0x30303030u);
    utmp[2] = a1 & 0x3f3f3f3fu;
    utmp[3] = ((a2 >> 4) & 0x0f0f0f0fu) | ((a1 >> 2) & 0x30303030u);
}

// -------------------------------------------------------------------------------------------------- Q4_K tile

// One Q4_K row against C <= 8 columns, each column the one-column kernel's steps
// (crates/qdot/src/lib.rs:4203-4272): weights unpacked once per block. With `q5` a Q5_K row, the twin kernel
// (:4895-4990): the wider block, the codes at 48, and bit 4 of each code folded in from the 32 high bytes at 16 (in
// half j, value 128 j + 32 b + l takes bit 4 j + b of qh[l]: qh at j = 0, qh >> 4 in 16-bit lanes at j = 1, shifted
// left by 4 - b onto bit 4).
static void dot_q45k_tile(const uint8_t *wrow, const uint8_t *const *acols, int C, int nb, int q5, float *out) {
    const __m256i ml = _mm256_set1_epi8(0xF), mh = _mm256_set1_epi8(0x10);
    const int block = q5 ? ORA_Q5K_BLOCK : ORA_Q4K_BLOCK, codes_at = q5 ? 48 : 16;
    __m256 accd[8];
    for (int c = 0; c < C; c++) accd[c] = _mm256_setzero_ps();
    for (int i = 0; i < nb; i++) {
        const uint8_t *wb = wrow + (size_t)i * block;
        uint16_t dh, mnh;
        memcpy(&dh, wb, 2);
        memcpy(&mnh, wb + 2, 2);
        float d = f16c_to_f32(dh), dmin = f16c_to_f32(mnh);
        uint32_t utmp[4];
        q4_unpack_scales(wb + 4, utmp);
        __m256 mins_v = _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i *)(utmp + 2))));
        __m256 mins = _mm256_mul_ps(_mm256_set1_ps(-dmin), mins_v);
        __m256 all_scales = _mm256_mul_ps(
            _mm256_set1_ps(d), _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i *)utmp))));
        __m128 lo = _mm256_castps256_ps128(all_scales), hi = _mm256_extractf128_ps(all_scales, 1);
        __m256 scales[2] = {_mm256_set_m128(lo, lo), _mm256_set_m128(hi, hi)};
        __m256i values[2][4];
        for (int j = 0; j < 2; j++) {
            __m256i bits0 = _mm256_loadu_si256((const __m256i *)(wb + codes_at + 64 * j));
            __m256i bits1 = _mm256_loadu_si256((const __m256i *)(wb + codes_at + 64 * j + 32));
            values[j][0] = _mm256_and_si256(bits0, ml);
            values[j][1] = _mm256_and_si256(_mm256_srli_epi16(bits0, 4), ml);
            values[j][2] = _mm256_and_si256(bits1, ml);
            values[j][3] = _mm256_and_si256(_mm256_srli_epi16(bits1, 4), ml);
            if (q5) {
                __m256i qh = _mm256_loadu_si256((const __m256i *)(wb + 16));
                __m256i hbits = j == 0 ? qh : _mm256_srli_epi16(qh, 4);
                values[j][0] = _mm256_or_si256(values[j][0], _mm256_and_si256(_mm256_slli_epi16(hbits, 4), mh));
                values[j][1] = _mm256_or_si256(values[j][1], _mm256_and_si256(_mm256_slli_epi16(hbits, 3), mh));
                values[j][2] = _mm256_or_si256(values[j][2], _mm256_and_si256(_mm256_slli_epi16(hbits, 2), mh));
                values[j][3] = _mm256_or_si256(values[j][3], _mm256_and_si256(_mm256_slli_epi16(hbits, 1), mh));
            }
        }
        for (int c = 0; c < C; c++) {
            const uint8_t *acol = acols[c];
            __m256 dy = q82x4_dy(acol, i);
            __m256 my = q82x4_my(acol, i, dy);
            __m128 dy4[2] = {_mm256_castps256_ps128(dy), _mm256_extractf128_ps(dy, 1)};
            __m256 sumi_f[2], d4d8[2];
            for (int j = 0; j < 2; j++) {
                d4d8[j] = _mm256_mul_ps(scales[j], _mm256_set_m128(dy4[j], dy4[j]));
                const uint8_t *qs = acol + (size_t)(2 * i + j) * ORA_Q82X4_STRIDE + 16;
                __m256i s1 = _mm256_maddubs_epi16(values[j][0], _mm256_loadu_si256((const __m256i *)qs));
                __m256i s2 = _mm256_maddubs_epi16(values[j][1], _mm256_loadu_si256((const __m256i *)(qs + 32)));
                __m256i s3 = _mm256_maddubs_epi16(values[j][2], _mm256_loadu_si256((const __m256i *)(qs + 64)));
                __m256i s4 = _mm256_maddubs_epi16(values[j][3], _mm256_loadu_si256((const __m256i *)(qs + 96)));
                sumi_f[j] = _mm256_cvtepi32_ps(reduce4(s1, s2, s3, s4));
            }
            accd[c] = _mm256_fmadd_ps(my, mins, accd[c]);
            accd[c] = _mm256_fmadd_ps(d4d8[0], sumi_f[0], accd[c]);
            accd[c] = _mm256_fmadd_ps(d4d8[1], sumi_f[1], accd[c]);
        }
    }
    for (int c = 0; c < C; c++) out[c] = hsum_float_8(accd[c]);
}

// -------------------------------------------------------------------------------------------------- Q6_K tile

static const uint8_t K_SHUFFLE_Q6K[32] = {0, 1, 4, 5, 8, 9, 12, 13, 2, 3, 6, 7, 10, 11, 14, 15,
                                          0, 1, 4, 5, 8, 9, 12, 13, 2, 3, 6, 7, 10, 11, 14, 15};

// One Q6_K row against C <= 8 columns (crates/qdot/src/lib.rs:4469-4579).
static void dot_q6k_tile(const uint8_t *wrow, const uint8_t *const *acols, int C, int nb, float *out) {
    const __m256i ml = _mm256_set1_epi8(0xF), mh = _mm256_set1_epi8(0x30), m32n = _mm256_set1_epi8(-32);
    const __m256i shuff = _mm256_loadu_si256((const __m256i *)K_SHUFFLE_Q6K);
    __m256 accd[8];
    for (int c = 0; c < C; c++) accd[c] = _mm256_setzero_ps();
    for (int i = 0; i < nb; i++) {
        const uint8_t *wb = wrow + (size_t)i * ORA_Q6K_BLOCK;
        uint16_t dh;
        memcpy(&dh, wb + 208, 2);
        __m256 vd = _mm256_set1_ps(f16c_to_f32(dh));
        __m256i sc16 =
            _mm256_shuffle_epi8(_mm256_cvtepi8_epi16(_mm_loadu_si128((const __m128i *)(wb + 192))), shuff);
        __m256 wscales[2] = {
            _mm256_mul_ps(vd, _mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_castsi256_si128(sc16)))),
            _mm256_mul_ps(vd, _mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_extracti128_si256(sc16, 1))))};
        __m256i values[2][4], us[2][4];
        for (int j = 0; j < 2; j++) {
            __m256i lbits1 = _mm256_loadu_si256((const __m256i *)(wb + 64 * j));
            __m256i lbits2 = _mm256_loadu_si256((const __m256i *)(wb + 64 * j + 32));
            __m256i hbits = _mm256_loadu_si256((const __m256i *)(wb + 128 + 32 * j));
            values[j][0] = _mm256_or_si256(_mm256_and_si256(lbits1, ml), _mm256_and_si256(_mm256_slli_epi16(hbits, 4), mh));
            values[j][1] = _mm256_or_si256(_mm256_and_si256(lbits2, ml), _mm256_and_si256(_mm256_slli_epi16(hbits, 2), mh));
            values[j][2] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(lbits1, 4), ml), _mm256_and_si256(hbits, mh));
            values[j][3] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(lbits2, 4), ml),
                                           _mm256_and_si256(_mm256_srli_epi16(hbits, 2), mh));
            for (int q = 0; q < 4; q++) {
                values[j][q] = _mm256_add_epi8(values[j][q], m32n);
                us[j][q] = _mm256_sign_epi8(values[j][q], values[j][q]);
            }
        }
        for (int c = 0; c < C; c++) {
            const uint8_t *acol = acols[c];
            __m256 dy = q82x4_dy(acol, i);
            __m128 dyl = _mm256_castps256_ps128(dy), dyh = _mm256_extractf128_ps(dy, 1);
            __m256 scales[2] = {_mm256_mul_ps(wscales[0], _mm256_set_m128(dyl, dyl)),
                                _mm256_mul_ps(wscales[1], _mm256_set_m128(dyh, dyh))};
            __m256i sumis[2];
            for (int j = 0; j < 2; j++) {
                const uint8_t *qs = acol + (size_t)(2 * i + j) * ORA_Q82X4_STRIDE + 16;
                __m256i s[4];
                for (int q = 0; q < 4; q++)
                    s[q] = _mm256_maddubs_epi16(
                        us[j][q], _mm256_sign_epi8(_mm256_loadu_si256((const __m256i *)(qs + 32 * q)), values[j][q]));
                sumis[j] = reduce4(s[0], s[1], s[2], s[3]);
            }
            accd[c] = _mm256_fmadd_ps(scales[0], _mm256_cvtepi32_ps(sumis[0]), accd[c]);
            accd[c] = _mm256_fmadd_ps(scales[1], _mm256_cvtepi32_ps(sumis[1]), accd[c]);
        }
    }
    for (int c = 0; c < C; c++) out[c] = hsum_float_8(accd[c]);
}

// ------------------------------------------------------------------------------------------------ IQ2_XXS tile

static uint64_t KEVEN_SIGNS[128]; // crates/qdot/src/lib.rs:7201-7218: 0xff where the sign bit is set, 0x01 where clear
static pthread_once_t keven_once = PTHREAD_ONCE_INIT;

static void keven_init(void) {
    for (int i = 0; i < 128; i++) {
        uint64_t t = 0;
        for (int b = 0; b < 8; b++) t |= (uint64_t)(((ORA_KSIGNS_IQ2XS[i] >> b) & 1) ? 0xff : 0x01) << (8 * b);
        KEVEN_SIGNS[i] = t;
    }
}

// One IQ2_XXS row against C <= 8 columns (crates/qdot/src/lib.rs:8328-8354 per column; new_block :8494, prepare
// :8558, half step :8599, group :8636).
static void dot_iq2xxs_tile(const uint8_t *wrow, const uint8_t *const *acols, int C, int nb, float *out) {
    const __m256i min_value = _mm256_set1_epi8(43);
    __m256 accd[8];
    for (int c = 0; c < C; c++) accd[c] = _mm256_setzero_ps();
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ2XXS_BLOCK;
        size_t at = (size_t)i * ORA_Q8K_STRIDE;
        uint16_t dh;
        memcpy(&dh, blk, 2);
        float d = 0.125f * f16c_to_f32(dh);
        float dmin = -d * 43.0f;
        __m256 lo = _mm256_castsi256_ps(_mm256_loadu_si256((const __m256i *)(blk + 2)));
        __m256 hi = _mm256_castsi256_ps(_mm256_loadu_si256((const __m256i *)(blk + 34)));
        __m256i words = _mm256_permute4x64_epi64(_mm256_castps_si256(_mm256_shuffle_ps(lo, hi, 0xDD)), 0xD8);
        __m256i sc32 = _mm256_or_si256(_mm256_slli_epi32(_mm256_srli_epi32(words, 28), 1), _mm256_set1_epi32(1));
        __m128i sc16 = _mm_packs_epi32(_mm256_castsi256_si128(sc32), _mm256_extracti128_si256(sc32, 1));
        __m256i mins = _mm256_set_m128i(
            _mm_shuffle_epi8(sc16, _mm_set_epi32(0x0f0e0f0e, 0x0d0c0d0c, 0x0b0a0b0a, 0x09080908)),
            _mm_shuffle_epi8(sc16, _mm_set_epi32(0x07060706, 0x05040504, 0x03020302, 0x01000100)));
        __m256i all_scales = _mm256_set_m128i(sc16, sc16);
        __m256i sumi[8];
        for (int c = 0; c < C; c++) {
            const uint8_t *col = acols[c] + at;
            float dy;
            memcpy(&dy, col, 4);
            __m256i bsums = _mm256_loadu_si256((const __m256i *)(col + 264));
            accd[c] = _mm256_fmadd_ps(_mm256_set1_ps(dmin * dy), _mm256_cvtepi32_ps(_mm256_madd_epi16(mins, bsums)),
                                      accd[c]);
        }
        for (int j = 0; j < 2; j++) {
            __m256i values[4], scales[4];
            for (int q = 0; q < 4; q++) {
                const uint8_t *qs = blk + 2 + 8 * (4 * j + q);
                uint32_t aux;
                memcpy(&aux, qs + 4, 4);
                __m256i q2 = _mm256_set_epi64x((long long)ORA_IQ2XXS_GRID[qs[3]], (long long)ORA_IQ2XXS_GRID[qs[2]],
                                               (long long)ORA_IQ2XXS_GRID[qs[1]], (long long)ORA_IQ2XXS_GRID[qs[0]]);
                __m256i sg = _mm256_set_epi64x((long long)KEVEN_SIGNS[(aux >> 21) & 127], (long long)KEVEN_SIGNS[(aux >> 14) & 127],
                                               (long long)KEVEN_SIGNS[(aux >> 7) & 127], (long long)KEVEN_SIGNS[aux & 127]);
                values[q] = _mm256_add_epi8(_mm256_sign_epi8(q2, sg), min_value);
                int b = 8 * j + 2 * q;
                scales[q] = _mm256_shuffle_epi8(all_scales, _mm256_set1_epi16((short)(b | ((b + 1) << 8))));
            }
            for (int c = 0; c < C; c++) {
                const uint8_t *col = acols[c] + at;
                __m256i p[4];
                for (int q = 0; q < 4; q++) {
                    __m256i q8 = _mm256_loadu_si256((const __m256i *)(col + 8 + 32 * (4 * j + q)));
                    p[q] = _mm256_madd_epi16(scales[q], _mm256_maddubs_epi16(values[q], q8));
                }
                if (j == 0) {
                    sumi[c] = _mm256_add_epi32(_mm256_add_epi32(p[0], p[2]), _mm256_add_epi32(p[1], p[3]));
                } else {
                    sumi[c] = _mm256_add_epi32(sumi[c], _mm256_add_epi32(p[0], p[2]));
                    sumi[c] = _mm256_add_epi32(sumi[c], _mm256_add_epi32(p[1], p[3]));
                }
            }
        }
        for (int c = 0; c < C; c++) {
            float dy;
            memcpy(&dy, acols[c] + at, 4);
            accd[c] = _mm256_fmadd_ps(_mm256_set1_ps(d * dy), _mm256_cvtepi32_ps(sumi[c]), accd[c]);
        }
    }
    for (int c = 0; c < C; c++) out[c] = hsum_float_8(accd[c]);
}

// --------------------------------------------------------------------------------------------------- Q3_K tile

static inline int hsum_i32_8(__m256i v) {
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x4e));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xb1));
    return _mm_cvtsi128_si32(s);
}

// One Q3_K row against C <= 8 columns, each column by the one-column kernel's steps (crates/qdot/src/lib.rs:2036-2157,
// field_dot :1997-2030): a field's two low bits on maddubs' unsigned side, the 4 of a clear high bit likewise and
// subtracted, the pairs scaled per 16 values in madd; one integer a super-block, then acc += (dcol * d) * sum, each
// operation rounded on its own.
static void dot_q3k_tile(const uint8_t *wrow, const uint8_t *const *acols, int C, int nb, float *out) {
    const __m256i m3 = _mm256_set1_epi8(3), mone = _mm256_set1_epi8(1);
    float acc[8] = {0};
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_Q3K_BLOCK;
        __m256i hbits = _mm256_loadu_si256((const __m256i *)blk);
        uint32_t a0 = ora_rd32(blk + 96), a1 = ora_rd32(blk + 100), a2 = ora_rd32(blk + 104);
        uint32_t w[4] = {(a0 & 0x0f0f0f0fu) | ((a2 & 0x03030303u) << 4), (a1 & 0x0f0f0f0fu) | (((a2 >> 2) & 0x03030303u) << 4),
                         ((a0 >> 4) & 0x0f0f0f0fu) | (((a2 >> 4) & 0x03030303u) << 4),
                         ((a1 >> 4) & 0x0f0f0f0fu) | (((a2 >> 6) & 0x03030303u) << 4)};
        short sc[16];
        for (int j = 0; j < 16; j++) sc[j] = (short)((int)((w[j / 4] >> (8 * (j % 4))) & 0xff) - 32);
        uint16_t dh;
        memcpy(&dh, blk + 108, 2);
        float d = f16c_to_f32(dh);
        __m256i sumi[8];
        for (int c = 0; c < C; c++) sumi[c] = _mm256_setzero_si256();
        for (int j = 0; j < 2; j++) {
            __m256i q3bits = _mm256_loadu_si256((const __m256i *)(blk + 32 + 32 * j));
            for (int f = 0; f < 4; f++) {
                int bit = 4 * j + f, g = 8 * j + 2 * f;
                __m256i q3l = _mm256_and_si256(_mm256_srl_epi16(q3bits, _mm_cvtsi32_si128(2 * f)), m3);
                __m256i clear = _mm256_andnot_si256(hbits, _mm256_sll_epi16(mone, _mm_cvtsi32_si128(bit)));
                __m256i q3h = _mm256_slli_epi16(_mm256_srl_epi16(clear, _mm_cvtsi32_si128(bit)), 2);
                __m256i scv = _mm256_set_m128i(_mm_set1_epi16(sc[g + 1]), _mm_set1_epi16(sc[g]));
                for (int c = 0; c < C; c++) {
                    __m256i q8 = _mm256_loadu_si256((const __m256i *)(acols[c] + (size_t)i * ORA_Q8K_STRIDE + 8 + 128 * j + 32 * f));
                    __m256i p = _mm256_sub_epi16(_mm256_maddubs_epi16(q3l, q8), _mm256_maddubs_epi16(q3h, q8));
                    sumi[c] = _mm256_add_epi32(sumi[c], _mm256_madd_epi16(scv, p));
                }
            }
        }
        for (int c = 0; c < C; c++) {
            float dcol;
            memcpy(&dcol, acols[c] + (size_t)i * ORA_Q8K_STRIDE, 4);
            float t = dcol * d;
            t = t * (float)hsum_i32_8(sumi[c]);
            acc[c] = acc[c] + t;
        }
    }
    for (int c = 0; c < C; c++) out[c] = acc[c];
}

// ------------------------------------------------------------------------------------------------- IQ3_XXS tile

// One IQ3_XXS row against C <= 8 columns (crates/qdot/src/lib.rs:7259-7345 per column, :7412 the tile): the IQ2_XXS
// tile with eight four-magnitude grid words a sub-block, the sign/scale words behind the 64 index bytes, the
// offset 64 and d = f16 / 4.
static void dot_iq3xxs_tile(const uint8_t *wrow, const uint8_t *const *acols, int C, int nb, float *out) {
    const __m256i min_value = _mm256_set1_epi8(64);
    __m256 accd[8];
    for (int c = 0; c < C; c++) accd[c] = _mm256_setzero_ps();
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ3XXS_BLOCK;
        const uint8_t *qs = blk + 2;
        size_t at = (size_t)i * ORA_Q8K_STRIDE;
        uint16_t dh;
        memcpy(&dh, blk, 2);
        float d = 0.25f * f16c_to_f32(dh);
        float dmin = -d * 64.0f;
        __m256i words = _mm256_loadu_si256((const __m256i *)(qs + 64));
        __m256i sc32 = _mm256_or_si256(_mm256_slli_epi32(_mm256_srli_epi32(words, 28), 1), _mm256_set1_epi32(1));
        __m128i sc16 = _mm_packs_epi32(_mm256_castsi256_si128(sc32), _mm256_extracti128_si256(sc32, 1));
        __m256i mins = _mm256_set_m128i(
            _mm_shuffle_epi8(sc16, _mm_set_epi32(0x0f0e0f0e, 0x0d0c0d0c, 0x0b0a0b0a, 0x09080908)),
            _mm_shuffle_epi8(sc16, _mm_set_epi32(0x07060706, 0x05040504, 0x03020302, 0x01000100)));
        __m256i all_scales = _mm256_set_m128i(sc16, sc16);
        __m256i sumi[8];
        for (int c = 0; c < C; c++) {
            const uint8_t *col = acols[c] + at;
            float dy;
            memcpy(&dy, col, 4);
            __m256i bsums = _mm256_loadu_si256((const __m256i *)(col + 264));
            accd[c] = _mm256_fmadd_ps(_mm256_set1_ps(dmin * dy), _mm256_cvtepi32_ps(_mm256_madd_epi16(mins, bsums)),
                                      accd[c]);
        }
        for (int j = 0; j < 2; j++) {
            __m256i values[4], scales[4];
            for (int q = 0; q < 4; q++) {
                int b = 4 * j + q;
                const uint8_t *g = qs + 8 * b;
                uint32_t aux;
                memcpy(&aux, qs + 64 + 4 * b, 4);
                __m256i q3 = _mm256_set_epi32((int)ORA_IQ3XXS_GRID[g[7]], (int)ORA_IQ3XXS_GRID[g[6]], (int)ORA_IQ3XXS_GRID[g[5]],
                                              (int)ORA_IQ3XXS_GRID[g[4]], (int)ORA_IQ3XXS_GRID[g[3]], (int)ORA_IQ3XXS_GRID[g[2]],
                                              (int)ORA_IQ3XXS_GRID[g[1]], (int)ORA_IQ3XXS_GRID[g[0]]);
                __m256i sg = _mm256_set_epi64x((long long)KEVEN_SIGNS[(aux >> 21) & 127], (long long)KEVEN_SIGNS[(aux >> 14) & 127],
                                               (long long)KEVEN_SIGNS[(aux >> 7) & 127], (long long)KEVEN_SIGNS[aux & 127]);
                values[q] = _mm256_add_epi8(_mm256_sign_epi8(q3, sg), min_value);
                scales[q] = _mm256_shuffle_epi8(all_scales, _mm256_set1_epi16((short)((2 * b) | ((2 * b + 1) << 8))));
            }
            for (int c = 0; c < C; c++) {
                const uint8_t *col = acols[c] + at;
                __m256i p[4];
                for (int q = 0; q < 4; q++) {
                    __m256i q8 = _mm256_loadu_si256((const __m256i *)(col + 8 + 32 * (4 * j + q)));
                    p[q] = _mm256_madd_epi16(scales[q], _mm256_maddubs_epi16(values[q], q8));
                }
                if (j == 0) {
                    sumi[c] = _mm256_add_epi32(_mm256_add_epi32(p[0], p[2]), _mm256_add_epi32(p[1], p[3]));
                } else {
                    sumi[c] = _mm256_add_epi32(sumi[c], _mm256_add_epi32(p[0], p[2]));
                    sumi[c] = _mm256_add_epi32(sumi[c], _mm256_add_epi32(p[1], p[3]));
                }
            }
        }
        for (int c = 0; c < C; c++) {
            float dy;
            memcpy(&dy, acols[c] + at, 4);
            accd[c] = _mm256_fmadd_ps(_mm256_set1_ps(d * dy), _mm256_cvtepi32_ps(sumi[c]), accd[c]);
        }
    }
    for (int c = 0; c < C; c++) out[c] = hsum_float_8(accd[c]);
}

// -------------------------------------------------------------------------------------------------- IQ4_XS tile

// One IQ4_XS row against C <= 8 columns (crates/qdot/src/lib.rs:11062-11145): a sub-block's 32 levels come out of one
// byte shuffle of the sixteen-entry table (low nibbles in the low half, high nibbles in the high half), a level's
// magnitude goes to maddubs' unsigned side and its sign onto the activation byte, the pairs are scaled by the
// sub-block's scale in madd and added into eight i32 lanes; one fmadd a super-block.
static void dot_iq4xs_tile(const uint8_t *wrow, const uint8_t *const *acols, int C, int nb, float *out) {
    const __m256i m4 = _mm256_set1_epi8(0x0f);
    const __m128i t128 = _mm_loadu_si128((const __m128i *)ORA_KVALUES_IQ4NL);
    const __m256i table = _mm256_set_m128i(t128, t128);
    __m256 accd[8];
    for (int c = 0; c < C; c++) accd[c] = _mm256_setzero_ps();
    for (int i = 0; i < nb; i++) {
        const uint8_t *blk = wrow + (size_t)i * ORA_IQ4XS_BLOCK;
        float d = ora_half_to_f32(ora_rd16(blk));
        uint32_t scales_h = ora_rd16(blk + 2);
        __m256i values[8], scales[8];
        for (int b = 0; b < 8; b++) {
            __m128i aux = _mm_loadu_si128((const __m128i *)(blk + 8 + 16 * b));
            __m256i nib = _mm256_and_si256(_mm256_set_m128i(_mm_srli_epi16(aux, 4), aux), m4);
            values[b] = _mm256_shuffle_epi8(table, nib);
            int ls = ((blk[4 + b / 2] >> (4 * (b % 2))) & 0x0f) | (int)(((scales_h >> (2 * b)) & 3) << 4);
            scales[b] = _mm256_set1_epi16((short)(ls - 32));
        }
        for (int c = 0; c < C; c++) {
            const uint8_t *col = acols[c] + (size_t)i * ORA_Q8K_STRIDE;
            float dy;
            memcpy(&dy, col, 4);
            __m256i sumi = _mm256_setzero_si256();
            for (int b = 0; b < 8; b++) {
                __m256i q8 = _mm256_loadu_si256((const __m256i *)(col + 8 + 32 * b));
                __m256i pair = _mm256_maddubs_epi16(_mm256_sign_epi8(values[b], values[b]), _mm256_sign_epi8(q8, values[b]));
                sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(scales[b], pair));
            }
            accd[c] = _mm256_fmadd_ps(_mm256_set1_ps(d * dy), _mm256_cvtepi32_ps(sumi), accd[c]);
        }
    }
    for (int c = 0; c < C; c++) out[c] = hsum_float_8(accd[c]);
}

// ----------------------------------------------------------------------------------------------------- dispatch

// dot_row_cols (crates/qdot/src/lib.rs:905): 1..=8 columns, every value the one-column kernel's.
int ora_avx2_dot_row_cols(int wtype, const uint8_t *wrow, const uint8_t *const *acols, int cols, int k, float *out) {
    if (cols < 1 || cols > 8) return ORA_ESHAPE;
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    int nb = k / 256;
    switch (wtype) {
    case ORA_TYPE_Q3_K:
        dot_q3k_tile(wrow, acols, cols, nb, out);
        return 0;
    case ORA_TYPE_Q4_K:
        dot_q45k_tile(wrow, acols, cols, nb, 0, out);
        return 0;
    case ORA_TYPE_Q5_K:
        dot_q45k_tile(wrow, acols, cols, nb, 1, out);
        return 0;
    case ORA_TYPE_Q6_K:
        dot_q6k_tile(wrow, acols, cols, nb, out);
        return 0;
    case ORA_TYPE_IQ2_XXS:
        pthread_once(&keven_once, keven_init);
        dot_iq2xxs_tile(wrow, acols, cols, nb, out);
        return 0;
    case ORA_TYPE_IQ3_XXS:
        pthread_once(&keven_once, keven_init);
        dot_iq3xxs_tile(wrow, acols, cols, nb, out);
        return 0;
    case ORA_TYPE_IQ4_XS:
        dot_iq4xs_tile(wrow, acols, cols, nb, out);
        return 0;
    default:
        return ORA_ETYPE;
    }
}

int ora_avx2_dot_row(int wtype, const uint8_t *wrow, const uint8_t *acol, int k, float *out) {
    return ora_avx2_dot_row_cols(wtype, wrow, &acol, 1, k, out);
}

// --------------------------------------------------------------------------------- multi-threaded layer baseline

// One phase of the layer step: a list of matrix x columns products (one per expert hit and matrix) whose rows, taken
// together, are split evenly over the pool's threads - the reference's pool splits an expert matrix's rows statically
// (crates/threads/src/lib.rs:1-30); here a phase's matrices are laid end to end first, so one dispatch serves them all -
// or a list of per-slot jobs (SwiGLU and the quantizer of h).
typedef struct {
    int wtype, k, rows, cols;
    const uint8_t *w;
    const uint8_t *const *acols;
    float *const *outs;
} mt_gemv;

typedef struct {
    const mt_gemv *jobs; // kind 0
    int n_jobs;
    long total_rows;
    // kind 1: slot s: h = swiglu(g, u), then its column for the down stack
    int kind, n_slots, ff, down_type, cb_d;
    const float *g, *u;
    float *h;
    uint8_t *ad;
    volatile int *rc;
} mt_phase;

struct ora_pool;
typedef struct {
    pthread_t th;
    int tid;
    struct ora_pool *pool;
} worker;

struct ora_pool {
    int n_threads;
    worker *ws;
    volatile int quit;
    const mt_phase *volatile phase;
    // a sense-reversing barrier the threads spin on: a phase lasts tens of microseconds, a futex wake as long
    volatile int arrived, sense;
    int caller_sense; // the calling thread's side of the barrier (one caller for the pool's life)
};

static void spin_barrier(struct ora_pool *p, int *my_sense) {
    *my_sense = !*my_sense;
    if (__atomic_add_fetch(&p->arrived, 1, __ATOMIC_ACQ_REL) == p->n_threads) {
        p->arrived = 0;
        __atomic_store_n(&p->sense, *my_sense, __ATOMIC_RELEASE);
    } else {
        while (__atomic_load_n(&p->sense, __ATOMIC_ACQUIRE) != *my_sense) _mm_pause();
    }
}

static void run_rows(const mt_gemv *g, int r0, int r1) {
    int rb = ora_row_bytes(g->wtype, g->k);
    float tmp[8];
    for (int r = r0; r < r1; r++) {
        for (int c0 = 0; c0 < g->cols; c0 += 8) {
            int c = g->cols - c0 < 8 ? g->cols - c0 : 8;
            ora_avx2_dot_row_cols(g->wtype, g->w + (size_t)r * rb, g->acols + c0, c, g->k, tmp);
            for (int j = 0; j < c; j++) g->outs[c0 + j][r] = tmp[j];
        }
    }
}

static void run_share(const mt_phase *ph, int tid, int n_threads) {
    if (ph->kind == 1) {
        for (int s = tid; s < ph->n_slots; s += n_threads) {
            ora_swiglu(ph->g + (size_t)s * ph->ff, ph->u + (size_t)s * ph->ff, ph->ff, ph->h + (size_t)s * ph->ff);
            int rc = ora_avx2_quantize_col(ph->down_type, ph->h + (size_t)s * ph->ff, ph->ff, ph->ad + (size_t)s * ph->cb_d);
            if (rc) *ph->rc = rc;
        }
        return;
    }
    long per = (ph->total_rows + n_threads - 1) / n_threads;
    long lo = (long)tid * per, hi = lo + per > ph->total_rows ? ph->total_rows : lo + per;
    long at = 0;
    for (int j = 0; j < ph->n_jobs && at < hi; j++) {
        long end = at + ph->jobs[j].rows;
        long a = lo > at ? lo : at, b = hi < end ? hi : end;
        if (a < b) run_rows(&ph->jobs[j], (int)(a - at), (int)(b - at));
        at = end;
    }
}

static void *worker_main(void *arg) {
    worker *w = (worker *)arg;
    struct ora_pool *p = w->pool;
    int sense = 0;
    for (;;) {
        spin_barrier(p, &sense);
        if (p->quit) return NULL;
        run_share((const mt_phase *)p->phase, w->tid, p->n_threads);
        spin_barrier(p, &sense);
    }
}

// A resident pool (the role of crates/threads): n_threads - 1 workers plus the caller, each pinned to a CPU of the
// process's set where the system allows it.
ora_pool *ora_pool_create(int n_threads) {
    if (n_threads < 1) n_threads = 1;
    ora_pool *p = (ora_pool *)calloc(1, sizeof(ora_pool));
    p->n_threads = n_threads;
    p->ws = (worker *)calloc((size_t)n_threads, sizeof(worker));
    cpu_set_t all;
    int have = sched_getaffinity(0, sizeof all, &all) == 0 ? CPU_COUNT(&all) : 0;
    for (int t = 1; t < n_threads; t++) {
        p->ws[t].tid = t;
        p->ws[t].pool = p;
        pthread_create(&p->ws[t].th, NULL, worker_main, &p->ws[t]);
        if (have >= n_threads) { // the t-th CPU of the set
            int seen = 0;
            for (int c = 0; c < CPU_SETSIZE; c++)
                if (CPU_ISSET(c, &all) && seen++ == t) {
                    cpu_set_t one;
                    CPU_ZERO(&one);
                    CPU_SET(c, &one);
                    (void)pthread_setaffinity_np(p->ws[t].th, sizeof one, &one);
                    break;
                }
        }
    }
    return p;
}

void ora_pool_destroy(ora_pool *p) {
    if (!p) return;
    p->quit = 1;
    if (p->n_threads > 1) spin_barrier(p, &p->caller_sense);
    for (int t = 1; t < p->n_threads; t++) pthread_join(p->ws[t].th, NULL);
    free(p->ws);
    free(p);
}

static void pool_run(ora_pool *p, const mt_phase *ph) {
    if (p->n_threads == 1) {
        run_share(ph, 0, 1);
        return;
    }
    p->phase = ph;
    spin_barrier(p, &p->caller_sense);
    run_share(ph, 0, p->n_threads);
    spin_barrier(p, &p->caller_sense);
}

// The layer step of ora_moe_forward on the AVX2 kernels and the pool, slots grouped by expert so a weight row is
// read once for up to eight of its columns (crates/model/src/moe.rs:617-749 with dot_row_cols tiles). Only the experts
// the routing names are visited, and the step is three dispatches of the pool whatever their number: every hit
// expert's gate and up rows, the slots' SwiGLU and quantizer, every hit expert's down rows. The values are
// ora_moe_forward's bit for bit: every (row, column) dot is the one-column kernel's and the combine keeps its slot
// order.
int ora_avx2_moe_forward(ora_pool *p, const ora_moe_layer *L, const float *x, int m, const uint32_t *ids,
                         const float *wts, int top_k, float *y, float *h_out) {
    int hidden = L->hidden, ff = L->ff, n_slots = m * top_k;
    int cb_g = ora_col_bytes(L->gate_type, hidden), cb_u = ora_col_bytes(L->up_type, hidden);
    int cb_d = ora_col_bytes(L->down_type, ff);
    int rb_g = ora_row_bytes(L->gate_type, hidden), rb_u = ora_row_bytes(L->up_type, hidden);
    int rb_d = ora_row_bytes(L->down_type, ff);
    if (cb_g < 0 || cb_u < 0 || cb_d < 0) return ORA_ESHAPE;
    for (int s = 0; s < n_slots; s++)
        if (ids[s] >= (uint32_t)L->n_experts) return ORA_ESHAPE;
    int same_enc = ora_takes_q8k(L->gate_type) == ora_takes_q8k(L->up_type);
    uint8_t *ag = (uint8_t *)malloc((size_t)cb_g * m), *au = same_enc ? ag : (uint8_t *)malloc((size_t)cb_u * m);
    uint8_t *ad = (uint8_t *)malloc((size_t)cb_d * n_slots);
    float *g = (float *)malloc(sizeof(float) * (size_t)ff * n_slots);
    float *u = (float *)malloc(sizeof(float) * (size_t)ff * n_slots);
    float *h = h_out ? h_out : (float *)malloc(sizeof(float) * (size_t)ff * n_slots);
    float *down = (float *)malloc(sizeof(float) * (size_t)hidden * n_slots);
    int *start = (int *)calloc((size_t)L->n_experts + 1, sizeof(int));
    int *fill = (int *)malloc(sizeof(int) * (size_t)L->n_experts);
    int *order = (int *)malloc(sizeof(int) * (size_t)n_slots);
    const uint8_t **cols_g = (const uint8_t **)malloc(sizeof(void *) * (size_t)n_slots);
    const uint8_t **cols_u = (const uint8_t **)malloc(sizeof(void *) * (size_t)n_slots);
    const uint8_t **cols_d = (const uint8_t **)malloc(sizeof(void *) * (size_t)n_slots);
    float **outs_g = (float **)malloc(sizeof(void *) * (size_t)n_slots);
    float **outs_u = (float **)malloc(sizeof(void *) * (size_t)n_slots);
    float **outs_d = (float **)malloc(sizeof(void *) * (size_t)n_slots);
    mt_gemv *jobs = (mt_gemv *)malloc(sizeof(mt_gemv) * 2 * (size_t)(n_slots < L->n_experts ? n_slots : L->n_experts));
    volatile int rc = 0;
    for (int t = 0; t < m && !rc; t++) {
        rc = ora_avx2_quantize_col(L->gate_type, x + (size_t)t * hidden, hidden, ag + (size_t)t * cb_g);
        if (!rc && !same_enc)
            rc = ora_avx2_quantize_col(L->up_type, x + (size_t)t * hidden, hidden, au + (size_t)t * cb_u);
    }
    // Slots grouped by expert, ascending slot order inside an expert (the bucket table, moe.rs:281-304): a counting
    // sort over the ids.
    for (int s = 0; s < n_slots; s++) start[ids[s] + 1]++;
    for (int e = 0; e < L->n_experts; e++) start[e + 1] += start[e], fill[e] = start[e];
    for (int s = 0; s < n_slots; s++) order[fill[ids[s]]++] = s;
    for (int j = 0; j < n_slots; j++) {
        int s = order[j];
        cols_g[j] = ag + (size_t)(s / top_k) * cb_g;
        cols_u[j] = au + (size_t)(s / top_k) * cb_u;
        cols_d[j] = ad + (size_t)s * cb_d;
        outs_g[j] = g + (size_t)s * ff;
        outs_u[j] = u + (size_t)s * ff;
        outs_d[j] = down + (size_t)s * hidden;
    }
    if (!rc) {
        mt_phase ph = {0};
        for (int e = 0; e < L->n_experts; e++) {
            int first = start[e], cnt = start[e + 1] - first;
            if (!cnt) continue;
            jobs[ph.n_jobs++] = (mt_gemv){L->gate_type, hidden, ff, cnt, L->wg + (size_t)e * ff * rb_g, cols_g + first, outs_g + first};
            jobs[ph.n_jobs++] = (mt_gemv){L->up_type, hidden, ff, cnt, L->wu + (size_t)e * ff * rb_u, cols_u + first, outs_u + first};
            ph.total_rows += 2L * ff;
        }
        ph.jobs = jobs;
        pool_run(p, &ph);
        mt_phase act = {0};
        act.kind = 1, act.n_slots = n_slots, act.ff = ff, act.down_type = L->down_type, act.cb_d = cb_d;
        act.g = g, act.u = u, act.h = h, act.ad = ad, act.rc = &rc;
        pool_run(p, &act);
    }
    if (!rc) {
        mt_phase ph = {0};
        for (int e = 0; e < L->n_experts; e++) {
            int first = start[e], cnt = start[e + 1] - first;
            if (!cnt) continue;
            jobs[ph.n_jobs++] = (mt_gemv){L->down_type, ff, hidden, cnt, L->wd + (size_t)e * hidden * rb_d, cols_d + first, outs_d + first};
            ph.total_rows += hidden;
        }
        ph.jobs = jobs;
        pool_run(p, &ph);
        ora_combine_tokens(down, wts, NULL, hidden, top_k, m, y);
    }
    free(ag);
    if (!same_enc) free(au);
    free(ad);
    free(g);
    free(u);
    if (!h_out) free(h);
    free(down);
    free(start);
    free(fill);
    free(order);
    free(cols_g);
    free(cols_u);
    free(cols_d);
    free(outs_g);
    free(outs_u);
    free(outs_d);
    free(jobs);
    return rc;
}
