// TEST INFRASTRUCTURE ONLY (see ora_common.h). The caller's side of the path: router, combine and one MoE
// layer step in the CPU engine's order (crates/model/src/moe.rs:617-749): quantize the token once per
// encoding, gate and up dots, SwiGLU, quantize with the down type's encoder, down dots, weighted sum.
#include <pthread.h>
#include <stdlib.h>

#include "bm_oracle.h"
#include "ora_common.h"

// Softmax over all experts (exp of logit - max in f32, sum in f64, one f32 divide: crates/model/src/moe.rs:246-262),
// top-k by (p descending, id ascending) (:264-279), and with `renorm` the chosen p summed in f64 in slot order,
// rounded once, each weight p / sum (crates/gpu/src/route_softmax.rs:38-51).
int ora_route_softmax_topk(const float *logits, int n_experts, int top_k, int renorm, uint32_t *ids, float *w) {
    if (n_experts <= 0 || top_k <= 0 || top_k > n_experts) return ORA_ESHAPE;
    float *p = (float *)malloc(sizeof(float) * (size_t)n_experts);
    uint8_t *taken = (uint8_t *)calloc((size_t)n_experts, 1);
    if (!p || !taken) {
        free(p);
        free(taken);
        return ORA_ESHAPE;
    }
    float max = -INFINITY;
    for (int i = 0; i < n_experts; i++) max = fmaxf(max, logits[i]);
    double sum = 0.0;
    for (int i = 0; i < n_experts; i++) {
        p[i] = expf(logits[i] - max);
        sum += (double)p[i];
    }
    for (int i = 0; i < n_experts; i++) p[i] /= (float)sum;
    for (int s = 0; s < top_k; s++) {
        int best = -1;
        for (int i = 0; i < n_experts; i++) {
            if (taken[i]) continue;
            if (best < 0 || p[i] > p[best]) best = i; // strict: ties keep the smaller id
        }
        taken[best] = 1;
        ids[s] = (uint32_t)best;
        w[s] = p[best];
    }
    if (renorm) {
        double s2 = 0.0;
        for (int s = 0; s < top_k; s++) s2 += (double)w[s];
        float denom = (float)s2;
        for (int s = 0; s < top_k; s++) w[s] = w[s] / denom;
    }
    free(p);
    free(taken);
    return 0;
}

// y[t][d] = (sum over the token's slots, ascending from 0, acc = fma(w, down, acc)) + resid[t][d]
// (crates/gpu/src/elem.rs:658-697, crates/gpu/src/arch/qwen3moe/experts.rs:293-318). `resid` may be NULL (zero).
void ora_combine_tokens(const float *down, const float *w, const float *resid, int rows, int n_slots, int m,
                        float *y) {
    for (int t = 0; t < m; t++)
        for (int d = 0; d < rows; d++) {
            float acc = 0.0f;
            for (int e = 0; e < n_slots; e++)
                acc = fmaf(w[t * n_slots + e], down[((size_t)(t * n_slots + e)) * rows + d], acc);
            y[(size_t)t * rows + d] = resid ? acc + resid[(size_t)t * rows + d] : acc;
        }
}

// y[t][d] = (the slot sum above + shexp[t][d]) + resid[t][d], the adds grouped as crates/gpu/src/moe_fused.rs:129-170
// groups them. `resid` may be NULL.
void ora_moe_combine(const float *down, const float *w, const float *shexp, const float *resid, int rows, int n_slots,
                     int m, float *y) {
    for (int t = 0; t < m; t++)
        for (int d = 0; d < rows; d++) {
            float acc = 0.0f;
            for (int e = 0; e < n_slots; e++)
                acc = fmaf(w[t * n_slots + e], down[((size_t)(t * n_slots + e)) * rows + d], acc);
            acc = acc + shexp[(size_t)t * rows + d];
            y[(size_t)t * rows + d] = resid ? acc + resid[(size_t)t * rows + d] : acc;
        }
}

typedef struct {
    int wtype, k, r0, r1, m;
    const uint8_t *w;         // expert's rows
    const uint8_t *const *acols; // m column pointers
    float *const *outs;       // m output pointers (each `rows` long)
    int rc;
} gemv_job;

static void *gemv_worker(void *arg) {
    gemv_job *j = (gemv_job *)arg;
    int rb = ora_row_bytes(j->wtype, j->k), cb = ora_col_bytes(j->wtype, j->k);
    for (int r = j->r0; r < j->r1; r++)
        for (int c = 0; c < j->m; c++) {
            int rc = ora_dot_row(j->wtype, j->w + (size_t)r * rb, rb, j->acols[c], cb, j->k, &j->outs[c][r]);
            if (rc) j->rc = rc;
        }
    return NULL;
}

// rows x m dots, rows split statically over n_threads (the pool's for_each_chunk role,
// crates/model/src/ops.rs:3123-3160).
static int gemv_mt(int wtype, const uint8_t *w, int rows, int k, const uint8_t *const *acols, float *const *outs,
                   int m, int n_threads) {
    if (n_threads < 1) n_threads = 1;
    if (n_threads > 256) n_threads = 256;
    gemv_job jobs[256];
    pthread_t th[256];
    int per = (rows + n_threads - 1) / n_threads, n = 0;
    for (int t = 0; t < n_threads; t++) {
        int r0 = t * per, r1 = r0 + per > rows ? rows : r0 + per;
        if (r0 >= r1) break;
        jobs[n] = (gemv_job){wtype, k, r0, r1, m, w, acols, outs, 0};
        n++;
    }
    if (n == 1) {
        gemv_worker(&jobs[0]);
    } else {
        for (int t = 0; t < n; t++) pthread_create(&th[t], NULL, gemv_worker, &jobs[t]);
        for (int t = 0; t < n; t++) pthread_join(th[t], NULL);
    }
    for (int t = 0; t < n; t++)
        if (jobs[t].rc) return jobs[t].rc;
    return 0;
}

int ora_moe_forward(const ora_moe_layer *L, const float *x, int m, const uint32_t *ids, const float *wts, int top_k,
                    float *y, float *h_out, int n_threads) {
    int hidden = L->hidden, ff = L->ff;
    int cb_g = ora_col_bytes(L->gate_type, hidden), cb_u = ora_col_bytes(L->up_type, hidden);
    int cb_d = ora_col_bytes(L->down_type, ff);
    int rb_g = ora_row_bytes(L->gate_type, hidden), rb_u = ora_row_bytes(L->up_type, hidden);
    int rb_d = ora_row_bytes(L->down_type, ff);
    if (cb_g < 0 || cb_u < 0 || cb_d < 0) return cb_g < 0 ? cb_g : (cb_u < 0 ? cb_u : cb_d);
    int n_slots = m * top_k, rc = 0;
    for (int s = 0; s < n_slots; s++)
        if (ids[s] >= (uint32_t)L->n_experts) return ORA_ESHAPE;
    // x quantized once per (token, encoding) (crates/model/src/ops.rs:554).
    int same_enc = ora_takes_q8k(L->gate_type) == ora_takes_q8k(L->up_type);
    uint8_t *ag = (uint8_t *)malloc((size_t)cb_g * m), *au = same_enc ? ag : (uint8_t *)malloc((size_t)cb_u * m);
    uint8_t *ad = (uint8_t *)malloc((size_t)cb_d);
    float *g = (float *)malloc(sizeof(float) * ff), *u = (float *)malloc(sizeof(float) * ff);
    float *h = (float *)malloc(sizeof(float) * ff);
    float *down = (float *)malloc(sizeof(float) * (size_t)n_slots * hidden);
    for (int t = 0; t < m && !rc; t++) {
        rc = ora_quantize_col(L->gate_type, x + (size_t)t * hidden, hidden, ag + (size_t)t * cb_g);
        if (!rc && !same_enc) rc = ora_quantize_col(L->up_type, x + (size_t)t * hidden, hidden, au + (size_t)t * cb_u);
    }
    for (int s = 0; s < n_slots && !rc; s++) {
        int t = s / top_k;
        uint32_t e = ids[s];
        const uint8_t *cg = ag + (size_t)t * cb_g, *cu = au + (size_t)t * cb_u;
        float *og = g, *ou = u;
        rc = gemv_mt(L->gate_type, L->wg + (size_t)e * ff * rb_g, ff, hidden, &cg, &og, 1, n_threads);
        if (!rc) rc = gemv_mt(L->up_type, L->wu + (size_t)e * ff * rb_u, ff, hidden, &cu, &ou, 1, n_threads);
        if (rc) break;
        ora_swiglu(g, u, ff, h);
        if (h_out) memcpy(h_out + (size_t)s * ff, h, sizeof(float) * ff);
        // The down type's encoder (crates/model/src/moe.rs:675-691).
        rc = ora_quantize_col(L->down_type, h, ff, ad);
        if (rc) break;
        const uint8_t *cd = ad;
        float *od = down + (size_t)s * hidden;
        rc = gemv_mt(L->down_type, L->wd + (size_t)e * hidden * rb_d, hidden, ff, &cd, &od, 1, n_threads);
    }
    if (!rc) ora_combine_tokens(down, wts, NULL, hidden, top_k, m, y);
    free(ag);
    if (!same_enc) free(au);
    free(ad);
    free(g);
    free(u);
    free(h);
    free(down);
    return rc;
}

// ------------------------------------------------------------------------------- the norm and the router's logits

// sum of (x[i] * x[i]) as f64, f32 squares, in the vector kernel's lane order (crates/qdot/src/lib.rs:11418-11456): two
// registers of four f64 lanes take values 8i .. 8i + 3 and 8i + 4 .. 8i + 7, are added lane by lane, the upper pair
// onto the lower, then the two; a tail past the last eight is added left to right.
double ora_sum_sq_f64(const float *x, int n) {
    double a0[4] = {0, 0, 0, 0}, a1[4] = {0, 0, 0, 0};
    int full = n / 8 * 8;
    for (int i = 0; i < full; i += 8)
        for (int l = 0; l < 4; l++) {
            float s0 = x[i + l] * x[i + l], s1 = x[i + 4 + l] * x[i + 4 + l];
            a0[l] += (double)s0;
            a1[l] += (double)s1;
        }
    double a[4], lo[2];
    for (int l = 0; l < 4; l++) a[l] = a0[l] + a1[l];
    lo[0] = a[0] + a[2];
    lo[1] = a[1] + a[3];
    double total = lo[0] + lo[1];
    for (int i = full; i < n; i++) {
        float s = x[i] * x[i];
        total += (double)s;
    }
    return total;
}

// RMS norm with a gain (crates/model/src/ops.rs:350-368): the mean of the squares narrowed to f32, eps inside the
// square root, then (scale * gain) * x in that order.
void ora_rms_norm(const float *x, const float *gain, float eps, int n, float *out) {
    float mean = (float)(ora_sum_sq_f64(x, n) / (double)n);
    float scale = 1.0f / sqrtf(mean + eps);
    for (int i = 0; i < n; i++) {
        float sg = scale * gain[i];
        out[i] = sg * x[i];
    }
}

// One f32 weight row . an f32 column in the reference's float-kernel order (crates/qdot/src/lib.rs:11349-11386): eight
// lane accumulators, the first block a product, every later one a fused multiply-add, then (l0 + l4 + l2 + l6) +
// (l1 + l5 + l3 + l7). n a positive multiple of eight (the reference hands other widths back to its caller).
int ora_dot_f32(const float *w, const float *x, int n, float *out) {
    if (n <= 0 || n % 8 != 0) return ORA_EUNALIGNED;
    float acc[8];
    for (int l = 0; l < 8; l++) acc[l] = x[l] * w[l];
    for (int i = 1; i < n / 8; i++)
        for (int l = 0; l < 8; l++) acc[l] = fmaf(x[8 * i + l], w[8 * i + l], acc[l]);
    float s[4] = {acc[0] + acc[4], acc[1] + acc[5], acc[2] + acc[6], acc[3] + acc[7]};
    *out = (s[0] + s[2]) + (s[1] + s[3]);
    return 0;
}

// The router's logits of m tokens (crates/model/src/moe.rs:246: matmul_q over the f32 gate_inp rows): logits[t *
// n_experts + e] = row e . token t's row, after the norm when a gain is given.
int ora_router_logits(const float *router, int n_experts, int hidden, const float *x, const float *gain, float eps, int m,
                      float *normed_out, float *logits) {
    float *row = (float *)malloc(sizeof(float) * (size_t)hidden);
    int rc = 0;
    for (int t = 0; t < m && !rc; t++) {
        const float *xt = x + (size_t)t * hidden;
        if (gain)
            ora_rms_norm(xt, gain, eps, hidden, row);
        else
            memcpy(row, xt, sizeof(float) * (size_t)hidden);
        if (normed_out) memcpy(normed_out + (size_t)t * hidden, row, sizeof(float) * (size_t)hidden);
        for (int e = 0; e < n_experts && !rc; e++)
            rc = ora_dot_f32(router + (size_t)e * hidden, row, hidden, &logits[(size_t)t * n_experts + e]);
    }
    free(row);
    return rc;
}
