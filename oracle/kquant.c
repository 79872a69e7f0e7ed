// TEST INFRASTRUCTURE ONLY (see ora_common.h). Host weight quantizers for synthetic expert stacks: Q4_K and Q6_K
// by ggml's `_ref` rules as the reference restates them (crates/gguf/src/kquant.rs). Every multiply, add, divide
// and square root is its own f32 operation (build with -ffp-contract=off); MAX/MIN are `a > b ? a : b` forms and
// the searches keep the reference's candidate order and strict tie-breaks.
//
// Pinned without golden bytes (the reference checks these against ggml on its own machine only): a second spelling
// written from the reference's text in numpy, vectors over all sub-blocks at once, gives the same bytes on the reference
// tests' row generators, on N(0, 0.02) rows and on rows with zero, flat and all-positive sub-blocks, and notices one
// search step more or fewer and the other tie rule; rows built from legal blocks whose products are exact read back
// exactly; plus the reference tests' round-trip bounds (crates/gguf/src/kquant/tests.rs:5-60).
#include <pthread.h>
#include <stdlib.h>

#include "bm_oracle.h"
#include "ora_common.h"

#define GROUP_MAX_EPS 1e-15f

static inline int nint(float x) { return ora_nearest_int(x); }
static inline int imax(int a, int b) { return a > b ? a : b; }
static inline int imin(int a, int b) { return a < b ? a : b; }

// make_qx_quants at rmse_type 1 without importance: weights are x^2 (crates/gguf/src/kquant.rs:126-177).
static float make_qx_quants(int nmax, const float *x, int n, int8_t *l) {
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax < GROUP_MAX_EPS) {
        for (int i = 0; i < n; i++) l[i] = 0;
        return 0.0f;
    }
    float nmaxf = (float)nmax;
    float iscale = -nmaxf / max;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int li = imax(-nmax, imin(nmax - 1, nint(iscale * x[i])));
        l[i] = (int8_t)(li + nmax);
        float w = x[i] * x[i];
        sumlx += w * x[i] * (float)li;
        suml2 += w * (float)li * (float)li;
    }
    float scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -(nmaxf + 0.1f * (float)is) / max;
        sumlx = 0.0f;
        suml2 = 0.0f;
        for (int i = 0; i < n; i++) {
            int li = imax(-nmax, imin(nmax - 1, nint(iscale * x[i])));
            float w = x[i] * x[i];
            sumlx += w * x[i] * (float)li;
            suml2 += w * (float)li * (float)li;
        }
        if (suml2 > 0.0f && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; i++) {
                int li = nint(iscale * x[i]);
                l[i] = (int8_t)(nmax + imax(-nmax, imin(nmax - 1, li)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

// make_qkx2_quants, use_mad false (crates/gguf/src/kquant.rs:239-318). Returns the scale; *the_min = -min.
static float make_qkx2_quants(int nmax, const float *x, const float *weights, uint8_t *l, uint8_t *laux, float rmin,
                              float rdelta, int nstep, float *the_min) {
    float min = x[0], max = x[0];
    float sum_w = weights[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < 32; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0.0f) min = 0.0f;
    if (max == min) {
        for (int i = 0; i < 32; i++) l[i] = 0;
        *the_min = -min;
        return 0.0f;
    }
    float nmaxf = (float)nmax;
    float iscale = nmaxf / (max - min);
    float scale = 1.0f / iscale;
    float best_error = 0.0f;
    for (int i = 0; i < 32; i++) {
        int li = nint(iscale * (x[i] - min));
        l[i] = (uint8_t)imax(0, imin(nmax, li));
        float diff = scale * (float)l[i] + min - x[i];
        diff = diff * diff;
        best_error += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + nmaxf) / (max - min);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        for (int i = 0; i < 32; i++) {
            int li = imax(0, imin(nmax, nint(iscale * (x[i] - min))));
            laux[i] = (uint8_t)li;
            float w = weights[i];
            float lf = (float)li;
            sum_l += w * lf;
            sum_l2 += w * lf * lf;
            sum_xl += w * lf * x[i];
        }
        float d = sum_w * sum_l2 - sum_l * sum_l;
        if (d > 0.0f) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / d;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / d;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.0f;
            for (int i = 0; i < 32; i++) {
                float diff = this_scale * (float)laux[i] + this_min - x[i];
                diff = diff * diff;
                cur_error += weights[i] * diff;
            }
            if (cur_error < best_error) {
                memcpy(l, laux, 32);
                best_error = cur_error;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

static void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) { // crates/gguf/src/kquant.rs:483-492
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

// One Q4_K or Q5_K block by the `_ref` rule (crates/gguf/src/kquant.rs:528-660 kquant45_block, the branch without
// importance): `q5` takes the 5-bit levels, their search grid and the block's plane of high bits.
static void q45k_block(const float *x, uint8_t *out, int q5) {
    const int nmax = q5 ? 31 : 15;
    uint8_t l[256] = {0}, laux[32];
    float scales[8], mins[8], weights[32];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; j++) {
        const float *xs = x + 32 * j;
        float sum_x2 = 0.0f;
        for (int k = 0; k < 32; k++) sum_x2 += xs[k] * xs[k];
        float av_x = sqrtf(sum_x2 / 32.0f);
        for (int k = 0; k < 32; k++) weights[k] = av_x + fabsf(xs[k]);
        float m;
        float s = q5 ? make_qkx2_quants(nmax, xs, weights, l + 32 * j, laux, -0.5f, 0.1f, 15, &m)
                     : make_qkx2_quants(nmax, xs, weights, l + 32 * j, laux, -1.0f, 0.1f, 20, &m);
        scales[j] = s;
        mins[j] = m;
        if (s > max_scale) max_scale = s;
        if (m > max_min) max_min = m;
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint8_t ls[8], lm[8], sc[12] = {0};
    for (int j = 0; j < 8; j++) {
        uint8_t a = (uint8_t)nint(inv_scale * scales[j]), b = (uint8_t)nint(inv_min * mins[j]);
        ls[j] = a < 63 ? a : 63;
        lm[j] = b < 63 ? b : 63;
    }
    for (int j = 0; j < 8; j++) { // pack_scales, :495-508
        if (j < 4) {
            sc[j] = ls[j];
            sc[j + 4] = lm[j];
        } else {
            sc[j + 4] = (uint8_t)((ls[j] & 0xF) | ((lm[j] & 0xF) << 4));
            sc[j - 4] |= (uint8_t)((ls[j] >> 4) << 6);
            sc[j] |= (uint8_t)((lm[j] >> 4) << 6);
        }
    }
    uint16_t d_bits = ora_f32_to_f16_bits(max_scale / 63.0f);
    uint16_t dmin_bits = ora_f32_to_f16_bits(max_min / 63.0f);
    float d = ora_half_to_f32(d_bits), dmin = ora_half_to_f32(dmin_bits);
    for (int j = 0; j < 8; j++) { // requant_levels, :512-525
        uint8_t s6, m6;
        get_scale_min_k4(j, sc, &s6, &m6);
        float dd = d * (float)s6;
        if (dd == 0.0f) continue;
        float dm = dmin * (float)m6;
        for (int ii = 0; ii < 32; ii++) {
            int li = nint((x[32 * j + ii] + dm) / dd);
            l[32 * j + ii] = (uint8_t)imax(0, imin(nmax, li));
        }
    }
    ora_wr16(out, d_bits);
    ora_wr16(out + 2, dmin_bits);
    memcpy(out + 4, sc, 12);
    if (q5) { // :627-650: bit 4 of a level goes to bit n / 32 of high byte n % 32
        uint8_t *qh = out + 16, *ql = out + 48;
        memset(qh, 0, 32);
        for (int p = 0; p < 4; p++)
            for (int j = 0; j < 32; j++) {
                uint8_t l1 = l[64 * p + j], l2 = l[64 * p + j + 32];
                if (l1 > 15) {
                    l1 -= 16;
                    qh[j] |= (uint8_t)(1u << (2 * p));
                }
                if (l2 > 15) {
                    l2 -= 16;
                    qh[j] |= (uint8_t)(2u << (2 * p));
                }
                ql[32 * p + j] = (uint8_t)(l1 | (l2 << 4));
            }
        return;
    }
    uint8_t *q = out + 16;
    for (int j = 0; j < 256; j += 64)
        for (int k = 0; k < 32; k++) *q++ = (uint8_t)(l[j + k] | (l[j + k + 32] << 4));
}

// One Q6_K block by the `_ref` rule (crates/gguf/src/kquant.rs:787-842).
static void q6k_block(const float *x, uint8_t *out) {
    int8_t l[256];
    float scales[16];
    float max_scale = 0.0f, max_abs_scale = 0.0f;
    for (int ib = 0; ib < 16; ib++) {
        float scale = make_qx_quants(32, x + 16 * ib, 16, l + 16 * ib);
        scales[ib] = scale;
        float abs_scale = fabsf(scale);
        if (abs_scale > max_abs_scale) {
            max_abs_scale = abs_scale;
            max_scale = scale;
        }
    }
    if (max_abs_scale < GROUP_MAX_EPS) {
        memset(out, 0, ORA_Q6K_BLOCK);
        return;
    }
    float iscale = -128.0f / max_scale;
    uint16_t d_bits = ora_f32_to_f16_bits(1.0f / iscale);
    int8_t sc[16];
    for (int ib = 0; ib < 16; ib++) sc[ib] = (int8_t)imin(127, nint(iscale * scales[ib]));
    float d = ora_half_to_f32(d_bits);
    for (int j = 0; j < 16; j++) {
        float dd = d * (float)sc[j];
        if (dd == 0.0f) continue;
        for (int ii = 0; ii < 16; ii++) {
            int li = nint(x[16 * j + ii] / dd);
            l[16 * j + ii] = (int8_t)(imax(-32, imin(31, li)) + 32);
        }
    }
    uint8_t *ql = out, *qh = out + 128;
    for (int half = 0; half < 2; half++) {
        int j = 128 * half;
        for (int k = 0; k < 32; k++) {
            uint8_t q0 = (uint8_t)l[j + k], q1 = (uint8_t)l[j + k + 32], q2 = (uint8_t)l[j + k + 64],
                    q3 = (uint8_t)l[j + k + 96];
            ql[64 * half + k] = (uint8_t)((q0 & 0xF) | ((q2 & 0xF) << 4));
            ql[64 * half + k + 32] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
            qh[32 * half + k] = (uint8_t)((q0 >> 4) | ((q1 >> 4) << 2) | ((q2 >> 4) << 4) | ((q3 >> 4) << 6));
        }
    }
    for (int ib = 0; ib < 16; ib++) out[192 + ib] = (uint8_t)sc[ib];
    ora_wr16(out + 208, d_bits);
}

static int finite_row(const float *x, int k) {
    for (int i = 0; i < k; i++)
        if (!isfinite(x[i])) return 0;
    return 1;
}

// crates/gguf/src/kquant.rs:860-891 for Q4_K without importance.
int ora_quantize_row_q4k(const float *x, int k, uint8_t *out) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    if (!finite_row(x, k)) return ORA_ENONFINITE;
    for (int i = 0; i < k / 256; i++) q45k_block(x + 256 * i, out + (size_t)i * ORA_Q4K_BLOCK, 0);
    return 0;
}

int ora_quantize_row_q5k(const float *x, int k, uint8_t *out) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    if (!finite_row(x, k)) return ORA_ENONFINITE;
    for (int i = 0; i < k / 256; i++) q45k_block(x + 256 * i, out + (size_t)i * ORA_Q5K_BLOCK, 1);
    return 0;
}

int ora_quantize_row_q6k(const float *x, int k, uint8_t *out) {
    if (k <= 0 || k % 256 != 0) return ORA_EUNALIGNED;
    if (!finite_row(x, k)) return ORA_ENONFINITE;
    for (int i = 0; i < k / 256; i++) q6k_block(x + 256 * i, out + (size_t)i * ORA_Q6K_BLOCK);
    return 0;
}

typedef struct {
    int wtype, k, r0, r1, rc;
    const float *x;
    uint8_t *out;
} qjob;

static void *qworker(void *arg) {
    qjob *j = (qjob *)arg;
    int rb = ora_row_bytes(j->wtype, j->k);
    float *ones = NULL;
    if (j->wtype == ORA_TYPE_IQ2_XXS) {
        // An expert the importance file never counted gets all ones (crates/gguf/src/iq_quant.rs:1103-1111).
        ones = (float *)malloc(sizeof(float) * (size_t)j->k);
        for (int i = 0; i < j->k; i++) ones[i] = 1.0f;
    }
    for (int r = j->r0; r < j->r1 && !j->rc; r++) {
        const float *xr = j->x + (size_t)r * j->k;
        uint8_t *o = j->out + (size_t)r * rb;
        if (j->wtype == ORA_TYPE_Q4_K)
            j->rc = ora_quantize_row_q4k(xr, j->k, o);
        else if (j->wtype == ORA_TYPE_Q5_K)
            j->rc = ora_quantize_row_q5k(xr, j->k, o);
        else if (j->wtype == ORA_TYPE_Q6_K)
            j->rc = ora_quantize_row_q6k(xr, j->k, o);
        else if (j->wtype == ORA_TYPE_IQ2_XXS)
            j->rc = ora_quantize_row_iq2xxs(xr, ones, j->k, o);
        else
            j->rc = ORA_ETYPE; // IQ4_XS has no quantizer in the reference's gguf crate, so none here
    }
    free(ones);
    return NULL;
}

// `rows` rows of `k` values each, rows split over threads. Rows are independent, so the bytes do not depend on
// the split.
int ora_quantize_rows(int wtype, const float *x, int rows, int k, uint8_t *out, int n_threads) {
    if (ora_row_bytes(wtype, k) < 0) return ora_row_bytes(wtype, k);
    if (n_threads < 1) n_threads = 1;
    if (n_threads > 64) n_threads = 64;
    qjob jobs[64];
    pthread_t th[64];
    int per = (rows + n_threads - 1) / n_threads, n = 0;
    for (int t = 0; t < n_threads; t++) {
        int r0 = t * per, r1 = r0 + per > rows ? rows : r0 + per;
        if (r0 >= r1) break;
        jobs[n++] = (qjob){wtype, k, r0, r1, 0, x, out};
    }
    if (n == 1) {
        qworker(&jobs[0]);
    } else {
        for (int t = 0; t < n; t++) pthread_create(&th[t], NULL, qworker, &jobs[t]);
        for (int t = 0; t < n; t++) pthread_join(th[t], NULL);
    }
    for (int t = 0; t < n; t++)
        if (jobs[t].rc) return jobs[t].rc;
    return 0;
}
