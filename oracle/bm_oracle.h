// TEST INFRASTRUCTURE ONLY. CPU oracle of the quantized MoE expert-matmul path: a plain C restatement of the
// reference's crates/qdot (activation encoders, Q3_K / Q4_K / Q5_K / Q6_K / IQ2_XXS / IQ3_XXS / IQ4_XS row dots, SwiGLU), crates/gguf (block
// layouts, dequantizers, K-quant and IQ2_XXS weight quantizers) and the caller-side router/combine order of
// crates/model/src/moe.rs. Each function cites the reference lines it follows. The shipped library never links
// or calls this; the test suite, the smoke check and the benchmark's CPU-baseline leg do.
//
// What pins each function (the reference itself cannot be built here: it is Rust and the image has no rustc):
//   encoders        the reference tests' known answers (bf16 scale bits 0x3F80/0x4000/0x3F80/0x3F82, saturation
//                   ends, 1e-40 / 1e-38 flushes, first-max ties, round-half-even codes), an independent
//                   closed-form restatement in the test suite, and the isum / bsums invariants;
//   integer sums    brute-force sums over independently decoded codes in the test suite;
//   fp32 dots       bit-equality with an AVX2-intrinsics restatement of the reference's vector kernels (its own
//                   first gate) and an f64 band around the dequantized dot;
//   dequantizers    the reference's ggml-made IQ2_XXS block (66 bytes -> 256 f32 bit patterns), table digests,
//                   independent decoders written from the layout text in the test suite (all five types);
//   expf / SwiGLU   libm band and special-case paths;
//   card rule       (card.c) the quantizer by the worked cases of the reference's own test (ties, near ties, the clamp,
//                   zero / subnormal / underflowed scales, refused blocks, the sums) and a numpy restatement; the
//                   32-lane walks by a second spelling from the device's loops over independently decoded blocks,
//                   one-lane rows that separate the split order from the fused one, and the reference test's f64 band;
//   weight quantizers   no golden bytes exist (the reference checks them against ggml on its own machine): a second
//                   spelling in numpy written from the reference's text gives the same bytes (K-quants and IQ2_XXS) and
//                   notices a wrong step count or tie rule; exactly representable rows read back exactly; an IQ2_XXS
//                   group's signs are the input's but for the flip its parity bit forces; the reference tests' bounds.
#ifndef BM_ORACLE_H
#define BM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Refusals (the reference panics or returns QdotError, crates/qdot/src/lib.rs:127-160).
#define ORA_EUNALIGNED (-1) // k is not a whole number of 256-value super-blocks
#define ORA_ETYPE (-2)      // weight type outside {Q3_K = 11, Q4_K = 12, Q5_K = 13, Q6_K = 14, IQ2_XXS = 16, IQ3_XXS = 18, IQ4_XS = 23}
#define ORA_ESHORTROW (-3)
#define ORA_ESHORTCOL (-4)
#define ORA_ENONFINITE (-5) // an activation value that is not finite
#define ORA_ESHAPE (-6)
#define ORA_ESTATUS (-7) // the IQ2_XXS search left the grid (crates/gguf/src/iq_quant.rs:52-61)

int ora_col_bytes(int wtype, int k);
int ora_row_bytes(int wtype, int k);

int ora_quantize_q82x4(const float *x, int k, uint8_t *out);
int ora_quantize_q8k(const float *x, int k, uint8_t *out);
int ora_quantize_col(int wtype, const float *x, int k, uint8_t *out);

float ora_dot_q4k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb);
float ora_dot_q5k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb);
float ora_dot_q6k_q82x4(const uint8_t *wrow, const uint8_t *acol, int nb);
float ora_dot_q3k_q8k(const uint8_t *wrow, const uint8_t *acol, int nb);
float ora_dot_iq2xxs_q8k(const uint8_t *wrow, const uint8_t *acol, int nb);
float ora_dot_iq3xxs_q8k(const uint8_t *wrow, const uint8_t *acol, int nb);
float ora_dot_iq4xs_q8k(const uint8_t *wrow, const uint8_t *acol, int nb);
int ora_dot_row(int wtype, const uint8_t *wrow, size_t wrow_len, const uint8_t *acol, size_t acol_len, int k,
                float *out);
int ora_gemv(int wtype, const uint8_t *w, int rows, int k, const uint8_t *act, int m, float *y);

void ora_q3k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *s_out);
void ora_q4k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *a_out, int32_t *isum_out);
void ora_q5k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *a_out, int32_t *isum_out);
void ora_q6k_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int fold, int32_t *s_out);
void ora_iq2xxs_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *i_out, int32_t *sc_out,
                           int32_t *codes_out, int32_t *fold_out);
void ora_iq3xxs_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int32_t *i_out, int32_t *sc_out,
                           int32_t *codes_out, int32_t *fold_out);
void ora_iq4xs_block_sums(const uint8_t *wrow, const uint8_t *acol, int nb, int fold, int32_t *i_out,
                          int32_t *lanes_out);

int ora_dequant_row(int wtype, const uint8_t *src, int k, float *dst);
int ora_dequant_col(int wtype, const uint8_t *acol, int k, float *dst);

float ora_expf_ik(float x);
void ora_swiglu(const float *gate, const float *up, int n, float *out);
int ora_gate_rule(int rule, float limit, const float *gate, const float *up, int n, float *out);

// Router and combine, in the caller's order (harness side of the path).
int ora_route_softmax_topk(const float *logits, int n_experts, int top_k, int renorm, uint32_t *ids, float *w);
void ora_combine_tokens(const float *down, const float *w, const float *resid, int rows, int n_slots, int m,
                        float *y);
void ora_moe_combine(const float *down, const float *w, const float *shexp, const float *resid, int rows, int n_slots,
                     int m, float *y);

// Weight quantizers (offline, host).
int ora_quantize_row_q4k(const float *x, int k, uint8_t *out);
int ora_quantize_row_q5k(const float *x, int k, uint8_t *out);
int ora_quantize_row_q6k(const float *x, int k, uint8_t *out);
int ora_quantize_row_iq2xxs(const float *x, const float *qw, int k, uint8_t *out);
int ora_quantize_rows(int wtype, const float *x, int rows, int k, uint8_t *out, int n_threads);
int ora_iq2xxs_grid_codes(uint32_t *codes256, int *kmap_neg_count, int *neighbour_words);

// Whole layers, for parity tests and the CPU baseline. Weights are GGUF block bytes, expert-major, rows back to
// back. `n_threads` splits rows statically; each (row, column) value is ora_dot_row's whatever the split.
typedef struct {
    int hidden, ff, n_experts;
    int gate_type, up_type, down_type;
    const uint8_t *wg, *wu, *wd;
} ora_moe_layer;

// One decode step of `m` tokens: x[m][hidden], ids/wts[m][top_k] -> y[m][hidden] (no residual),
// optionally h[m*top_k][ff] (the SwiGLU outputs). Returns 0 or a refusal.
int ora_moe_forward(const ora_moe_layer *L, const float *x, int m, const uint32_t *ids, const float *wts, int top_k,
                    float *y, float *h_out, int n_threads);

// The step before the path: the FFN norm and the router's f32 logits (crates/model/src/ops.rs:350-368,
// crates/qdot/src/lib.rs:11349-11456).
double ora_sum_sq_f64(const float *x, int n);
void ora_rms_norm(const float *x, const float *gain, float eps, int n, float *out);
int ora_dot_f32(const float *w, const float *x, int n, float *out);
int ora_router_logits(const float *router, int n_experts, int hidden, const float *x, const float *gain, float eps, int m,
                      float *normed_out, float *logits);

// The card rule (card.c): the reference's CPU mirrors of its GPU tier's q8_1 activations and 32-lane row walks
// (crates/qdot/src/lib.rs:2885-3620). ora_card_q8_1 returns the number of refused (non-finite) blocks.
int ora_card_q8_1(const float *x, int k, int8_t *codes, float *d8, int32_t *s8, uint8_t *refused);
int ora_card_dot_row(int wtype, const uint8_t *wrow, int k, const int8_t *codes, const float *d8, const int32_t *s8, float *out);
int ora_card_gemv(int wtype, const uint8_t *w, int rows, int k, const int8_t *codes, const float *d8, const int32_t *s8, int m, float *y);
int ora_card_gemv_sel(int wtype, const uint8_t *w, int n_experts, int rows_per_expert, int k, const int8_t *codes, const float *d8,
                      const int32_t *s8, const uint32_t *sel, int n_slots, float *y);

#ifdef __cplusplus
}
#endif

#endif // BM_ORACLE_H
