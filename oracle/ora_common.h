// TEST INFRASTRUCTURE ONLY. This directory is the CPU oracle of the quantized MoE expert-matmul path: a plain C
// restatement of the reference's crates/qdot + crates/gguf arithmetic. Nothing the library ships may include,
// link or call it; only the test suite, the smoke check and the benchmark's CPU-baseline leg do.
//
// Scalar helpers every oracle file shares. Build with -ffp-contract=off: a product meets a sum in one rounding
// only where the reference writes `mul_add`, and those places call fmaf() here.
#ifndef BM_ORACLE_COMMON_H
#define BM_ORACLE_COMMON_H

#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORA_Q3K_BLOCK 110    // crates/gguf/src/quant.rs:671-673: hmask[32], qs[64] @32, scales[12] @96, d @108
#define ORA_Q4K_BLOCK 144    // crates/qdot/src/lib.rs:3864
#define ORA_Q5K_BLOCK 176    // crates/qdot/src/lib.rs:4880: d, dmin, scales[12], qh[32] @16, qs[128] @48
#define ORA_Q6K_BLOCK 210    // crates/qdot/src/lib.rs:4452
#define ORA_IQ2XXS_BLOCK 66  // crates/qdot/src/lib.rs:8298
#define ORA_IQ3XXS_BLOCK 98  // crates/qdot/src/lib.rs IQ3XXS_BLOCK: d, 64 grid indices @2, eight sign/scale words @66
#define ORA_IQ4XS_BLOCK 136  // crates/qdot/src/lib.rs:11033-11037: d, scales_h u16 @2, scales_l[4] @4, qs[128] @8
#define ORA_Q8K_STRIDE 296   // crates/qdot/src/lib.rs:108
#define ORA_Q82X4_STRIDE 144 // crates/qdot/src/lib.rs:110

// Weight types, numbered as ggml numbers them (crates/gguf/src/qtype.rs:94,98,105).
#define ORA_TYPE_Q3_K 11
#define ORA_TYPE_Q4_K 12
#define ORA_TYPE_Q5_K 13
#define ORA_TYPE_Q6_K 14
#define ORA_TYPE_IQ2_XXS 16
#define ORA_TYPE_IQ3_XXS 18
#define ORA_TYPE_IQ4_XS 23

// The types whose activation column is ik's Q8_K (crates/gguf/src/qtype.rs host_act); the others here take Q8_2_X4.
static inline int ora_takes_q8k(int wtype) {
    return wtype == ORA_TYPE_Q3_K || wtype == ORA_TYPE_IQ2_XXS || wtype == ORA_TYPE_IQ3_XXS || wtype == ORA_TYPE_IQ4_XS;
}

static inline uint32_t ora_f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float ora_bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t ora_rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

static inline uint32_t ora_rd32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

static inline void ora_wr16(uint8_t *p, uint16_t v) {
    p[0] = (uint8_t)v;
    p[1] = (uint8_t)(v >> 8);
}

// f16 bits -> f32, exact, subnormals included (crates/gguf/src/quant.rs:472-494).
static inline float ora_half_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)(h >> 15)) << 31;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t mant = h & 0x3ff;
    uint32_t mag;
    if (exp == 0x1f) {
        mag = 0x7f800000u | (mant << 13);
    } else if (exp == 0) {
        if (mant == 0) {
            mag = 0;
        } else {
            uint32_t e = 127 - 14;
            uint32_t m = mant;
            while ((m & 0x400) == 0) {
                m <<= 1;
                e -= 1;
            }
            mag = (e << 23) | ((m & 0x3ff) << 13);
        }
    } else {
        mag = ((exp + 112) << 23) | (mant << 13);
    }
    return ora_bits_f32(sign | mag);
}

// f32 -> f16 bits, round to nearest even (crates/gguf/src/quant.rs:504-541).
static inline uint16_t ora_f32_to_f16_bits(float x) {
    uint32_t b = ora_f32_bits(x);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000);
    uint32_t a = b & 0x7fffffffu;
    if (a > 0x7f800000u) return sign | 0x7e00;
    int exp = (int)(a >> 23) - 127;
    uint32_t frac = a & 0x007fffffu;
    if (exp > 15) return sign | 0x7c00;
    if (exp >= -14) {
        uint32_t v = ((uint32_t)(exp + 15) << 23) | frac;
        uint32_t t = v + 0x0fff + ((v >> 13) & 1);
        uint32_t h = t >> 13;
        if ((h & 0x7c00) == 0x7c00) return sign | 0x7c00;
        return sign | (uint16_t)h;
    }
    if (exp < -25) return sign;
    uint32_t shift = (uint32_t)(-1 - exp);
    uint32_t v = 0x00800000u | frac;
    uint32_t half = 1u << (shift - 1);
    uint32_t rem = v & ((1u << shift) - 1);
    uint32_t h = v >> shift;
    if (rem > half || (rem == half && (h & 1) == 1)) h += 1;
    return sign | (uint16_t)h;
}

// f32 -> bf16 bits, round to nearest even; a NaN keeps its sign and goes quiet (crates/gguf/src/quant.rs:544-551).
static inline uint16_t ora_fp32_to_bf16_bits(float s) {
    uint32_t u = ora_f32_bits(s);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 64);
    return (uint16_t)((u + (0x7fffu + ((u >> 16) & 1))) >> 16);
}

static inline float ora_bf16_to_f32(uint16_t h) { return ora_bits_f32((uint32_t)h << 16); }

// Round to nearest even through one f32 add of 1.5 * 2^23 (crates/gguf/src/quant.rs:2222-2226).
static inline int32_t ora_nearest_int(float fval) {
    volatile float val = fval + 12582912.0f;
    uint32_t i = ora_f32_bits(val);
    return (int32_t)(i & 0x007fffffu) - 0x00400000;
}

// The q8_2 block's code multiplier from its bf16 scale bits (crates/gguf/src/quant.rs:2237-2241).
static inline float ora_q82_inverse(uint16_t t) {
    float d = ora_bf16_to_f32(t);
    float id = d > 0.0f ? 1.0f / d : 0.0f;
    return isfinite(id) ? id : 0.0f;
}

// The signed element of largest magnitude, first on ties; *bad is set when it is not finite
// (crates/gguf/src/quant.rs:2019-2034, which panics there).
static inline float ora_activation_max(const float *x, int n, int *bad) {
    float max = 0.0f;
    uint32_t amax = 0;
    for (int i = 0; i < n; i++) {
        uint32_t ax = ora_f32_bits(x[i]) & 0x7fffffffu;
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (!isfinite(max)) *bad = 1;
    return max;
}

#endif // BM_ORACLE_COMMON_H
