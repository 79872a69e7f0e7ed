// TEST INFRASTRUCTURE ONLY (see bm_oracle.h). The AVX2+FMA+F16C twin of the scalar oracle, and the resident
// thread pool the CPU baseline runs it on.
#ifndef BM_ORACLE_AVX2_H
#define BM_ORACLE_AVX2_H

#include "bm_oracle.h"

#ifdef __cplusplus
extern "C" {
#endif

int ora_avx2_supported(void);
int ora_avx2_quantize_q82x4(const float *x, int k, uint8_t *out);
int ora_avx2_quantize_q8k(const float *x, int k, uint8_t *out);
int ora_avx2_quantize_col(int wtype, const float *x, int k, uint8_t *out);
int ora_avx2_dot_row(int wtype, const uint8_t *wrow, const uint8_t *acol, int k, float *out);
int ora_avx2_dot_row_cols(int wtype, const uint8_t *wrow, const uint8_t *const *acols, int cols, int k, float *out);

typedef struct ora_pool ora_pool;
ora_pool *ora_pool_create(int n_threads);
void ora_pool_destroy(ora_pool *p);
int ora_avx2_moe_forward(ora_pool *p, const ora_moe_layer *L, const float *x, int m, const uint32_t *ids,
                         const float *wts, int top_k, float *y, float *h_out);

#ifdef __cplusplus
}
#endif

#endif // BM_ORACLE_AVX2_H
