/* bm_moe.h - C ABI of libbm_moe_hip.so: quantized MoE expert matmul on MI355X (gfx950).
 *
 * Q3_K / Q4_K / Q5_K / Q6_K / IQ2_XXS / IQ3_XXS / IQ4_XS GGUF weight blocks dotted with Q8-quantized activations (Q8_2_X4 for Q4_K, Q5_K and
 * Q6_K, Q8_K for Q3_K and the IQ types), in the arithmetic of the reference's CPU path crates/qdot: activation bytes and per-block
 * integer sums are bit-exact with it, and the decode kernels keep its fp32 operation order.
 *
 * The entry points stand where the reference's crates/gpu launchers stand (each declaration cites the one it
 * replaces). Conventions shared by all of them, as in the reference (crates/gpu/src/q4k_sel.rs:926-936,973):
 *   - every launcher is asynchronous on the context's stream, allocates nothing, never synchronises, and reads
 *     expert ids from device memory, so it can be captured into a HIP graph and replayed over new ids;
 *   - the caller owns every buffer; handles are created at load time and are not thread-safe;
 *   - geometry the host can check is refused before launch with a negative code and a message naming the entry
 *     point and the lengths (bm_last_error); conditions only the device can see raise the fault word.
 * Pointers named *_dev are device pointers; weights are the file's block bytes verbatim, rows back to back
 * (crates/gpu/src/weights.rs:69-86).
 */
#ifndef BM_MOE_H
#define BM_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Weight types, numbered as ggml numbers them (crates/gguf/src/qtype.rs:94,98,105). */
#define BM_TYPE_Q3_K 11    /* 110 B / 256 values; activations Q8_K */
#define BM_TYPE_Q4_K 12    /* 144 B / 256 values; activations Q8_2_X4 */
#define BM_TYPE_Q5_K 13    /* 176 B / 256 values; activations Q8_2_X4 */
#define BM_TYPE_Q6_K 14    /* 210 B / 256 values; activations Q8_2_X4 */
#define BM_TYPE_IQ2_XXS 16 /* 66 B / 256 values; activations Q8_K */
#define BM_TYPE_IQ3_XXS 18 /* 98 B / 256 values; activations Q8_K */
#define BM_TYPE_IQ4_XS 23  /* 136 B / 256 values; activations Q8_K */

/* Return codes: 0 is success (crates/gpu/src/lib.rs:175-313 GpuError). */
#define BM_OK 0
#define BM_ESHAPE (-1)   /* GpuError::Shape: lengths that do not fit the launch */
#define BM_EDRIVER (-2)  /* GpuError::Driver: a HIP call failed */
#define BM_ETYPE (-3)    /* a weight type or type combination with no kernel */
#define BM_EARG (-4)     /* a null handle or pointer */
#define BM_EFAULT (-5)   /* bm_fault_check: the fault word is raised */

/* Fault word (crates/device/src/fault.rs:9-60): u32[BM_FAULT_WORDS] on the device. Word 0 holds
 * (layer << 8) | site of the earliest layer and smallest site raised there (atomic minimum; BM_FAULT_NONE while
 * clean); word 1 + layer is that layer's site mask. Sticky until bm_fault_clear. */
#define BM_FAULT_NONE 0xFFFFFFFFu
#define BM_LAYER_NONE 0xFFFFu
#define BM_FAULT_WORDS (1 + 0xFFFF + 1)
#define BM_SITE_QUANT_COLUMN 1 /* a quantizer met a value that is not finite: NaN scale, zero codes */
#define BM_SITE_ROUTER 5       /* a token's logits hold a value that is not finite */
#define BM_SITE_EXPERT_ID 7    /* an expert id at or past the stack */
#define BM_SITE_F32_PRODUCT 21 /* a gate or up sum that is not finite met a clamped gate rule: the value is NaN */

/* The id of a slot served elsewhere (crates/gpu/src/host/slots.rs:10): every routed entry skips it silently - the
 * gate . up entries write nothing for it (no h rows, no activation block) and the down entries leave its rows as they
 * were; nothing is raised (crates/gpu/src/kquant/sel.rs:22-28,153-161). */
#define BM_HOST_SLOT 0xFFFFFFFFu

typedef struct bm_ctx bm_ctx;         /* crates/gpu/src/lib.rs:2529 Gpu: device, stream, fault word */
typedef struct bm_weights bm_weights; /* crates/gpu/src/tensor.rs:588-616 DeviceTensor<u32>: rows of block bytes */
typedef struct bm_act bm_act;         /* crates/gpu/src/tensor.rs:811-948 Q8Act: m quantized columns of k values */

/* The rule a gate . up entry (bm_gate_up, bm_gate_up_x, bm_moe_decode, bm_moe_decode_noalloc, bm_gate_up_tiles,
 * bm_swiglu_quant) applies to a row's gate sum g and up sum u: the Act argument of the reference's launchers
 * (crates/gpu/src/kquant/act.rs:21-57 Act, device codes :46-56; GateUpAct.rule of crates/gpu/src/kquant/sel.rs), passed
 * with each launch. An entry whose rule argument is NULL takes the context's rule, which bm_set_gate_rule sets
 * (BM_ACT_SILU_MUL until then). The numbers are the CPU path's (crates/qdot/src/lib.rs:11467 swiglu, :11492
 * swiglu_clamp, swiglu_oai, :11617 swiglu_gclamp; crates/model/src/ops.rs:2345 situ_into), every exponential ik's.
 *   BM_ACT_SILU_MUL       silu(g) * u (the default; limit ignored)
 *   BM_ACT_SWIGLU_CLAMP   min(silu(g), limit) * clamp(u, -limit, limit); limit <= 1e-6 clamps nothing; limit finite
 *   BM_ACT_SWIGLU_OAI     x = min(g, limit), y = clamp(u, -limit, limit): x / (1 + e^(-1.702 x)) * (y + 1); limit finite, >= 0
 *   BM_ACT_SITU           (beta tanh(g / beta) * sigmoid(g)) * (25 tanh(u / 25)), beta = limit, finite and positive; each
 *                         scale by the f32 reciprocal, the products in that order (act.rs:152-163 situ). The tanh is the
 *                         device library's f32 one where the CPU path calls the host's: a value can differ from the CPU
 *                         path's in its last bits (the reference says the same of its own card and host), so under this rule
 *                         the contract is 1e-5 relative on h (crates/model/src/ops.rs:7124-7131), not bits
 *   BM_ACT_SWIGLU_GCLAMP  silu(min(g, limit)) * clamp(u, -limit, limit); limit finite and positive
 * Under every rule but the first a sum that is not finite raises BM_SITE_F32_PRODUCT and its value is NaN (act.rs:166-175
 * apply_checked; the CPU path's rules refuse such a block). A rule or limit outside the above is refused by the entry
 * (BM_ETYPE / BM_ESHAPE) before anything is enqueued, as Act::code refuses it (act.rs:71-125). */
#define BM_ACT_SILU_MUL 0
#define BM_ACT_SWIGLU_CLAMP 1
#define BM_ACT_SWIGLU_OAI 2
#define BM_ACT_SITU 3
#define BM_ACT_SWIGLU_GCLAMP 4
typedef struct bm_gate_act {
    int rule;    /* one of BM_ACT_* */
    float limit; /* the clamp limit, or SiTU's beta */
} bm_gate_act;
int bm_set_gate_rule(bm_ctx *ctx, int rule, float limit);

/* ------------------------------------------------------------------------------------------------ context */

/* A context on `device` with a stream of its own (default priority) and a clean fault word. */
int bm_ctx_create(int device, bm_ctx **out);
/* As bm_ctx_create, on a stream the caller owns (a hipStream_t); the context never destroys it. */
int bm_ctx_create_on_stream(int device, void *hip_stream, bm_ctx **out);
void bm_ctx_destroy(bm_ctx *ctx);
/* The context's hipStream_t. */
void *bm_ctx_stream(bm_ctx *ctx);
/* hipStreamSynchronize on the context's stream. */
int bm_ctx_sync(bm_ctx *ctx);
/* The message of the last refusal on this context (or on the creating thread when ctx is NULL). */
const char *bm_last_error(const bm_ctx *ctx);
/* The layer later launches raise faults with (default BM_LAYER_NONE). */
int bm_set_layer(bm_ctx *ctx, uint32_t layer);
/* Synchronise and read word 0 and the site mask of `layer` (either pointer may be NULL). */
int bm_fault_read(bm_ctx *ctx, uint32_t layer, uint32_t *word0, uint32_t *mask);
/* Reset the fault word to clean (asynchronous, a fill kernel on the stream). */
int bm_fault_clear(bm_ctx *ctx);
/* Device pointer of the fault word. */
uint32_t *bm_fault_word_dev(bm_ctx *ctx);

/* Bytes of one weight row / one activation column of k values (crates/qdot/src/lib.rs:381-422,1727-1762);
 * negative for a type with no kernel or a k that is not a multiple of 256. */
int64_t bm_row_bytes(int wtype, int k);
int64_t bm_col_bytes(int wtype, int k);

/* ------------------------------------------------------------------------------------------------ buffers */

/* Device memory helpers for callers without a HIP binding of their own (the test suite). */
int bm_dev_alloc(bm_ctx *ctx, size_t bytes, void **out_dev);
int bm_dev_free(bm_ctx *ctx, void *dev);
int bm_dev_upload(bm_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);   /* synchronous */
int bm_dev_download(bm_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes); /* synchronous */
int bm_dev_memset(bm_ctx *ctx, void *dst_dev, int byte, size_t bytes);               /* synchronous */

/* An expert stack (or one matrix): `rows` rows of `k` values in `wtype` blocks, uploaded from `host_bytes`
 * (rows * bm_row_bytes bytes). Load time only. */
int bm_weights_create(bm_ctx *ctx, int wtype, int64_t rows, int k, const void *host_bytes, bm_weights **out);
/* As bm_weights_create over device memory the caller already holds (no copy; the caller keeps ownership). */
int bm_weights_wrap(bm_ctx *ctx, int wtype, int64_t rows, int k, const void *dev_bytes, bm_weights **out);
void bm_weights_destroy(bm_weights *w);
const void *bm_weights_dev(const bm_weights *w);

/* Activation scratch for up to `m_cap` columns of `k` values in the form `wtype` dots against
 * (Q8Act::with_k / with_slots). Load time only. On the device a column is the reference CPU path's column bytes
 * followed, for the Q8_2_X4 form, by two small tables the dot kernels read (per-block f32 scale and scale * sum,
 * per-16 code sums); bm_act_download / bm_act_upload move the reference bytes only, so a column can be handed to
 * or taken from a host tier unchanged. */
int bm_act_create(bm_ctx *ctx, int wtype, int k, int m_cap, bm_act **out);
void bm_act_destroy(bm_act *act);
/* Synchronise and copy column `col`'s bytes (bm_col_bytes of them) to the host. */
int bm_act_download(bm_ctx *ctx, const bm_act *act, int col, void *host_bytes);
/* Upload column `col` from host bytes in the same layout (the tables are rebuilt on the device). */
int bm_act_upload(bm_ctx *ctx, bm_act *act, int col, const void *host_bytes);

/* ------------------------------------------------------------------------------- decode: quantize and gemv */

/* Gpu::enqueue_quantize_q8_1 (crates/gpu/src/lib.rs:3275), in the CPU path's rule (crates/qdot/src/lib.rs:434
 * quantize_col): x_dev holds m columns of act's k values, column c at x_dev + c * k; columns 0..m of act are
 * written. A block holding a value that is not finite raises BM_SITE_QUANT_COLUMN, gets a NaN scale and zero
 * codes (crates/gpu/src/lib.rs:925-933). */
int bm_quantize(bm_ctx *ctx, const float *x_dev, int m, bm_act *act);

/* Gpu::enqueue_gemv_q4k / enqueue_gemv_q6k (crates/gpu/src/lib.rs:3495,3839) and the IQ2_XXS row kernel
 * (crates/gpu/src/iq.rs:1405): y_dev[row * m + c] = row `row` of w . column c of act, m = `m` columns, 1..=8. */
int bm_gemv(bm_ctx *ctx, const bm_weights *w, const bm_act *act, int m, float *y_dev);
/* bm_quantize + bm_gemv in one launch (the reference issues the two, crates/gpu/src/lib.rs:3275 then :3495): column c is
 * the f32 row x_dev + c * k, quantized by every workgroup for itself, so y_dev[r * m + c] holds bm_gemv's bits of
 * bm_quantize's columns without a column passing through memory. act_out (optional, made for w's type, m_cap >= m)
 * receives the columns as bm_quantize would leave them. A value that is not finite raises QuantColumn as bm_quantize
 * does. x_dev 16-byte aligned. */
int bm_gemv_x(bm_ctx *ctx, const bm_weights *w, const float *x_dev, int m, bm_act *act_out, float *y_dev);

/* -------------------------------------------------------------------------- decode: the routed expert chain */

/* ExpertKernels::enqueue_gate_up(GateUpArgs) (crates/gpu/src/arch/qwen3moe/experts.rs:326-335,462), for Q4_K,
 * Q5_K (crates/gpu/src/kquant/tiles.rs:120-190), Q6_K (crates/gpu/src/q6k_sel.rs:633), IQ2_XXS (crates/gpu/src/iq_sel.rs:1357) and IQ4_XS (iq_sel.rs, iq4_xs_gate_up_sel) stacks of one type:
 * slot s < n_slots reads expert sel_dev[s]'s rows of both stacks against activation column s / slots_per_col and
 * writes h_dev[s * rows_per_expert + r] = the rule's value of (gate_r, up_r) - rule is GateUpArgs' act, NULL for the
 * context's; silu(gate_r) * up_r in the CPU path's SwiGLU (crates/qdot/src/lib.rs:11467) by default. An id at or past the stack raises BM_SITE_EXPERT_ID and writes NaN into the
 * slot's rows (and a NaN-scaled block into act_h); BM_HOST_SLOT is skipped: nothing written, nothing raised.
 * h_dev may be NULL when act_h is given.
 * act_h (optional, NULL to skip): the down projection's activation, quantized in the same launch from the rows
 * just written, column s of act_h for slot s, in the form of act_h's type (Q8_2_X4 only; rows_per_expert must
 * then be act_h's k). The reference runs this as a separate quantizer launch (dispatch.rs:1343). */
int bm_gate_up(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_act *act, const uint32_t *sel_dev,
               int n_slots, int rows_per_expert, int slots_per_col, const bm_gate_act *rule, float *h_dev, bm_act *act_h);

/* Q4kSelKernels::enqueue_gemv_q4k_sel (crates/gpu/src/q4k_sel.rs:978), Q6kSelKernels::enqueue_gemv_q6k_sel
 * (crates/gpu/src/q6k_sel.rs:513), QuantSelKernels::enqueue_down (crates/gpu/src/iq_sel.rs:1557): slot s writes
 * y_dev[s * rows_per_expert + r] = row r of expert sel_dev[s] . column s of act. An id at or past the stack
 * leaves the slot's rows untouched and, unless it is BM_HOST_SLOT, raises BM_SITE_EXPERT_ID. */
int bm_gemv_sel(bm_ctx *ctx, const bm_weights *w, const bm_act *act, const uint32_t *sel_dev, int n_slots,
                int rows_per_expert, float *y_dev);

/* ExpertKernels::enqueue_combine_tokens(CombineArgs) (crates/gpu/src/arch/qwen3moe/experts.rs:341-349,529):
 * y[t * rows + d] = (acc = 0; for slot e ascending: acc = fma(w[t * n_slots + e], down[(t * n_slots + e) * rows
 * + d], acc)) + resid[t * rows + d] for t < m. resid_dev may be NULL (no residual add). */
int bm_combine_tokens(bm_ctx *ctx, const float *down_dev, const float *w_dev, const float *resid_dev, int rows,
                      int n_slots, int m, float *y_dev);
/* The combine of a layer with a shared expert, MoeFusedKernels' moe_combine (crates/gpu/src/moe_fused.rs:129-170), for m
 * tokens: y[t * rows + d] = (the slot sum above + shexp[t * rows + d]) + resid[t * rows + d], the two adds grouped as
 * the reference groups them (f32 addition is not associative). resid_dev may be NULL. */
int bm_moe_combine(bm_ctx *ctx, const float *down_dev, const float *w_dev, const float *shexp_dev, const float *resid_dev,
                   int rows, int n_slots, int m, float *y_dev);

/* bm_gemv_sel and bm_combine_tokens in one launch (no counterpart launch in the reference, which keeps the two
 * apart: dispatch.rs:1346-1424): the slot values never reach memory. Same values as the two calls: every slot
 * dot is bm_gemv_sel's and the sum keeps the slot order. A refused id contributes nothing to the sum. */
int bm_down_combine(bm_ctx *ctx, const bm_weights *w, const bm_act *act, const uint32_t *sel_dev,
                    const float *w_dev, const float *resid_dev, int n_slots_per_token, int m, int rows_per_expert,
                    float *y_dev);

/* bm_quantize of the slots' f32 rows of h and bm_down_combine in one launch, in the column form w's type dots against.
 * It is how a down stack on Q8_K columns (Q3_K and the IQ types) joins the fused step; for the K-quants on Q8_2_X4
 * columns it serves a caller that holds f32 rows only (where bm_gate_up / bm_gate_up_x can write the columns, that is
 * the faster way: every workgroup here quantizes its token's rows again). Slot s reads h_dev[s * k .. (s + 1) * k),
 * k = w's k, 16-byte aligned. act_h (optional) receives the quantized columns. Same bits as the two calls. No
 * counterpart launch in the reference. */
int bm_down_combine_h(bm_ctx *ctx, const bm_weights *w, const float *h_dev, bm_act *act_h, const uint32_t *sel_dev,
                      const float *w_dev, const float *resid_dev, int n_slots_per_token, int m, int rows_per_expert,
                      float *y_dev);

/* The whole decode step of one MoE layer for m tokens with every quantizer folded in (no counterpart in the
 * reference, whose step is the chain quantize, gate_up, quantize, down, combine: dispatch.rs:1245-1436): x_dev
 * holds m rows of hidden = wg's k f32 values (16-byte aligned); token t's slots are sel_dev / w_dev[t *
 * n_slots_per_token ..]; y_dev[t * hidden + d] gets bm_combine_tokens' value. Same bits as bm_quantize, bm_gate_up
 * (with act_h) and bm_down_combine run one after the other. Gate and up are of one type; every type of this library
 * goes on either side. A slot whose id is BM_HOST_SLOT
 * is skipped by both halves (its h rows and activation column keep what they held, it adds nothing to the sum, nothing is
 * raised); any other id at or past the stack raises BM_SITE_EXPERT_ID and adds nothing. act_h is caller-held scratch
 * (m * n_slots_per_token columns of ff = wd's k, in the form wd dots against) and holds the quantized h afterwards;
 * act_x (optional, in the form wg dots against) receives the quantized x columns; h_dev receives the f32 h rows:
 * optional, except that a down stack on Q8_K columns needs it (16-byte aligned): a Q8_K block spans eight gate . up
 * workgroups, so that launch leaves f32 rows and the down launch quantizes them (bm_down_combine_h). m <= 1024.
 * Two launches: gate . up with both quantizers folded in (bm_gate_up_x), then down + combine (bm_down_combine). */
int bm_moe_decode(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_weights *wd, const float *x_dev,
                  const uint32_t *sel_dev, const float *w_dev, const float *resid_dev, int n_slots_per_token, int m,
                  const bm_gate_act *rule, bm_act *act_h, bm_act *act_x, float *h_dev, float *y_dev);
/* The first launch of bm_moe_decode on its own: bm_quantize, bm_gate_up and the quantizer of h in one
 * launch, from the f32 token rows (gate and up of one type; rows_per_expert = ff a multiple of 256). act_h: Q8_2_X4
 * columns for the down stack, or NULL; h_dev: the f32 h rows, or NULL; one of the two at least. Ids as bm_gate_up
 * takes them (BM_HOST_SLOT skipped silently). Follow it with
 * bm_down_combine or bm_gemv_sel over act_h, or bm_down_combine_h over h_dev. */
int bm_gate_up_x(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const float *x_dev, const uint32_t *sel_dev,
                 int n_slots_per_token, int m, int rows_per_expert, const bm_gate_act *rule, bm_act *act_h, bm_act *act_x,
                 float *h_dev);
/* bm_moe_decode for callers that cannot allocate device memory or hold a scratch handle: code
 * under HIP graph capture, serving loops and harnesses that forbid hipMalloc. It has no counterpart in the reference,
 * whose callers make their Q8Act scratch at load time. The quantized h between the two launches (bm_moe_decode's act_h,
 * and its h_dev rows for a down stack on Q8_K columns) lives in an array the library holds on each device for the life
 * of the process (about 360 KiB), so the call allocates nothing, on the device or through any library. Same arguments
 * and same bits in y_dev as bm_moe_decode. Limit: m * n_slots_per_token * ff <= 65536 values of h (8 slots of ff 8192,
 * 32 of ff 2048, 85 of ff 768); more is refused with BM_ESHAPE. Every call on a device shares that device's array, which
 * keeps the last call's contents: calls that overlap on one device (two streams, two contexts) race; calls in stream
 * order do not, and nothing in the array has to start at zero. */
int bm_moe_decode_noalloc(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_weights *wd, const float *x_dev,
                          const uint32_t *sel_dev, const float *w_dev, const float *resid_dev, int n_slots_per_token, int m,
                          const bm_gate_act *rule, float *y_dev);

/* ------------------------------------------------------------- decode of several tokens: grouped by expert */

/* The grouped slot table (crates/gpu/src/q4k_sel.rs:20-41). Buffers the caller holds on the device:
 *   order[n_slots]      the card's slots listed by expert, ascending inside a run;
 *   start[n_experts+1]  expert e's run is order[start[e] .. start[e + 1]]; start[n_experts] = slots listed;
 *   tiles[cap + 1]      cap = bm_tile_cap(n_slots, n_experts): tiles[0] = count, tiles[1 + g] = (e << 22) | j,
 *                       tile g = up to 8 consecutive entries of expert e's run from entry j.
 * The layouts are the reference's, so a caller's tables interchange. At most 1024 experts, 2^22 slots. */

/* tile_cap (crates/gpu/src/q4k_sel.rs:96): min(n_slots, (n_slots + 7 * n_experts) / 8). */
int bm_tile_cap(int n_slots, int n_experts);
/* Q4kSelKernels::enqueue_buckets (crates/gpu/src/q4k_sel.rs:1103): order and start from sel_dev[n_slots]. An id
 * at or past n_experts joins no run and, unless it is BM_HOST_SLOT, raises BM_SITE_EXPERT_ID. */
int bm_buckets(bm_ctx *ctx, const uint32_t *sel_dev, int n_slots, int n_experts, uint32_t *order_dev, uint32_t *start_dev);
/* Q4kSelKernels::enqueue_grouped_tiles (crates/gpu/src/q4k_sel.rs:1152): the tile table of start_dev. A run
 * outside the table raises BM_SITE_EXPERT_ID and leaves a count of 0. */
int bm_tiles(bm_ctx *ctx, const uint32_t *start_dev, int n_experts, int n_slots, uint32_t *tiles_dev);
/* bm_buckets then bm_tiles as one launch: order_dev, start_dev and tiles_dev hold what the two calls would leave. */
int bm_tables(bm_ctx *ctx, const uint32_t *sel_dev, int n_slots, int n_experts, uint32_t *order_dev, uint32_t *start_dev,
              uint32_t *tiles_dev);
/* bm_tables and bm_quantize(ctx, x_dev, m, act) as one launch: the two depend on nothing of each other and are each a few
 * microseconds of latency, so the grouped step starts one launch sooner. The same tables and the same column bytes. No
 * counterpart in the reference, which enqueues the two separately (crates/gpu/src/q4k_sel.rs:1103,1152 and the card's
 * quantizer). Rows that are not 16-byte aligned or not whole super-blocks go through the two launches. */
int bm_tables_quantize(bm_ctx *ctx, const uint32_t *sel_dev, int n_slots, int n_experts, uint32_t *order_dev, uint32_t *start_dev,
                       uint32_t *tiles_dev, const float *x_dev, int m, bm_act *act);
/* Q4kSelKernels::enqueue_quantize_ord (crates/gpu/src/q4k_sel.rs:1255): the first start_dev[n_experts] columns
 * of x_dev (at most m_cols, the columns launched) into the same columns of act, bm_quantize's bytes; every other
 * column keeps what it held. */
int bm_quantize_ord(bm_ctx *ctx, const float *x_dev, const uint32_t *start_dev, int n_experts, int m_cols, bm_act *act);
/* The grouped gate . up (crates/gpu/src/kquant/tiles.rs:62-118,1055; kq_card_gather :10-14 folded in): table
 * entry j is slot order[j]; it reads the activation column of its token (column order[j] / slots_per_col of act)
 * and writes h_dev[j * rows_per_expert + r] - by entry, not by slot - bm_gate_up's value for that slot. An expert's
 * rows are read once for up to eight of its slots. act_h (optional, Q8_2_X4, k = rows_per_expert): column j gets
 * the quantized rows of entry j in the same launch (the reference's bm_quantize_ord step). An entry that names no
 * slot raises BM_SITE_EXPERT_ID and writes NaN. */
int bm_gate_up_tiles(bm_ctx *ctx, const bm_weights *wg, const bm_weights *wu, const bm_act *act, const uint32_t *order_dev,
                     const uint32_t *start_dev, const uint32_t *tiles_dev, int n_slots, int rows_per_expert,
                     int slots_per_col, const bm_gate_act *rule, float *h_dev, bm_act *act_h);
/* Q4kSelKernels::enqueue_gemv_q4k_tiles (crates/gpu/src/q4k_sel.rs:1208; Q5K/Q6K/IQ forms kquant/tiles.rs:120-190):
 * the grouped down. Entry j reads column j of act and writes y_dev[order[j] * rows_per_expert + r], bm_gemv_sel's
 * value for that slot. An entry that names no slot raises BM_SITE_EXPERT_ID and writes nothing. */
int bm_gemv_tiles(bm_ctx *ctx, const bm_weights *w, const bm_act *act, const uint32_t *order_dev, const uint32_t *start_dev,
                  const uint32_t *tiles_dev, int n_slots, int rows_per_expert, float *y_dev);

/* -------------------------------------------------------------------- prefill: route table and grouped GEMM */

typedef struct bm_route bm_route; /* crates/gpu/src/gemm/route.rs:109-125 GemmRoute */

/* GemmRoute::new (crates/gpu/src/gemm/route.rs:127-155): a table for up to max_slots (1..=40960) slots over a
 * stack of n_experts (1..=1024) experts. Load time only. */
int bm_route_create(bm_ctx *ctx, int max_slots, int n_experts, bm_route **out);
void bm_route_destroy(bm_route *route);
/* GemmKernels::enqueue_route (crates/gpu/src/gemm/route.rs:351): the table of ids_dev[0 .. n_slots) (slot =
 * token * top_k + k), built on the device: the slots grouped by expert, ascending inside an expert, cut into
 * tiles of at most 64. An id at or past the stack raises BM_SITE_EXPERT_ID; its slot is left out of the tiles
 * and listed as refused, and every bm_gemm over the table writes NaN into its rows. A slot whose id is BM_HOST_SLOT is
 * not listed at all and raises nothing (crates/gpu/src/kquant/sel.rs:22-28): no bm_gemm over the table touches its rows. */
int bm_route_fill(bm_ctx *ctx, const uint32_t *ids_dev, int n_slots, bm_route *route);
/* bm_route_fill and bm_quantize(ctx, x_dev, m, act) as one launch (the prefill step's two first launches depend on nothing of
 * each other): the same table and the same column bytes. No counterpart in the reference, which enqueues the two separately
 * (crates/gpu/src/gemm/route.rs:351 and the card's quantizer). Rows that are not 16-byte aligned or not whole super-blocks go
 * through the two launches. */
int bm_route_fill_quantize(bm_ctx *ctx, const uint32_t *ids_dev, int n_slots, bm_route *route, const float *x_dev, int m, bm_act *act);
/* GemmRoute::read_back / refused_back (route.rs:188-245): synchronise and copy the table out. cols_host (optional)
 * takes the n_slots slot list (refused slots last; behind them BM_HOST_SLOT once for every slot that is not listed);
 * tiles_host (optional) two words a tile: expert, then first index | length << 16. */
int bm_route_read(bm_ctx *ctx, const bm_route *route, uint32_t *cols_host, uint32_t *tiles_host, int *n_tiles, int *n_refused);
/* GemmKernels::enqueue_gemm(GemmArgs) (crates/gpu/src/gemm/grouped.rs:2125-2133,2300), Q4_K, Q5_K and Q6_K stacks against
 * Q8_2_X4 columns and IQ2_XXS, IQ3_XXS, IQ4_XS and Q3_K stacks (crates/gpu/src/gemm/kernels.rs:867 gemm_iq2xxs, :1139
 * gemm_iq3xxs, :1248 gemm_iq4xs, :759 gemm_q3k) against Q8_K columns:
 * y_dev[s * rows_per_expert + r] = row r of expert e(s) . column c(s) of act for every slot s of the table's last
 * fill; c(s) = s / top_k (GemmInput::Shared) or s when top_k is 0 (GemmInput::PerSlot). rows_per_expert a
 * multiple of 16. Every value is bm_gemv_sel's for that slot, bit for bit; the integer sums are formed on the int8
 * matrix cores. A refused slot gets NaN in every row. */
int bm_gemm(bm_ctx *ctx, const bm_weights *w, int rows_per_expert, const bm_act *act, const bm_route *route, int top_k,
            float *y_dev);
/* How bm_gemm sums in f32 (the integer block sums are exact either way):
 *   BM_GEMM_EXACT (default): the CPU path's eight accumulators and closing order; bit-identical to bm_gemv_sel;
 *   BM_GEMM_FAST: one accumulator a value, blocks in increasing k; differs from the exact value by f32 rounding
 *     only (observed below 1e-6 of the row's largest magnitude; the contract's tolerance is 1e-4), about 1.9x the
 *     speed of a Q4_K / Q6_K layer step. No counterpart in the reference, whose grouped GEMM has one order (gemm/grouped.rs:33-58).
 *     IQ3_XXS, IQ4_XS and Q3_K stacks have the exact order only and run in it under every mode.
 *   BM_GEMM_FAST_F16: the tolerance mode with both scales folded into f16 matrix operands (the sub-scale times the 4-bit
 *     code on the weight side, the block scale times the int8 code as an f16 value and its remainder on the column side), so
 *     the matrix cores deliver scaled sums and the vector ALU is left with two multiply-adds a super-block. The same
 *     tolerance (observed 3e-7). Q4_K stacks only; other types run as under BM_GEMM_FAST. Measured slower than BM_GEMM_FAST on
 *     MI355X (167 against 125 us for the 2048-token gate GEMM) and kept as the measured alternative form. */
#define BM_GEMM_EXACT 0
#define BM_GEMM_FAST 1
#define BM_GEMM_FAST_F16 2
int bm_set_gemm_mode(bm_ctx *ctx, int mode);
/* How the down + combine launch (bm_down_combine, the second launch of bm_moe_decode and of the per-slot path of bm_moe_forward)
 * walks a weight row; the bits of y are the same either way. No counterpart in the reference (its down launch has one form,
 * crates/gpu/src/arch/qwen3moe/experts.rs:227-318): a measurement switch.
 *   BM_DOWN_RING (default): four lanes a (row, slot), the row's super-blocks one after the other through a ring of registers;
 *   BM_DOWN_SPLIT: the row's super-blocks dealt to the waves of a larger workgroup (every super-block asked for at once, three
 *     waves a SIMD), the f32 chain run by the last super-block's wave in the CPU path's order. Built for Q6_K stacks of 768-value
 *     rows with 1, 2, 4 or 8 slots a token; every other launch runs as under BM_DOWN_RING. Measured slower on MI355X (5.6 against
 *     5.2 us at 2048 rows x 8 slots) and kept as the measured alternative form. */
#define BM_DOWN_RING 0
#define BM_DOWN_SPLIT 1
int bm_set_down_form(bm_ctx *ctx, int form);
/* GemmKernels::enqueue_swiglu_quant (crates/gpu/src/gemm/swiglu.rs:46): column c of act = the quantized
 * silu(g) * u of g_dev / u_dev[c * k .. (c + 1) * k), k = act's k, slot-major as the gate and up GEMMs write them;
 * bm_quantize's bytes of the CPU path's SwiGLU, in the column form of act's type (Q8_2_X4 or Q8_K). */
int bm_swiglu_quant(bm_ctx *ctx, const float *g_dev, const float *u_dev, int n_cols, const bm_gate_act *rule, bm_act *act);
/* GemmKernels::enqueue_swiglu_act_quant_sel (crates/gpu/src/gemm/swiglu.rs:96-140): bm_swiglu_quant over the columns of
 * slots 0 .. n_cols whose expert sel_dev[c] is on the stack. The column of a slot served elsewhere (BM_HOST_SLOT) is left
 * exactly as it stands, whatever its g / u rows hold, and raises nothing (a bm_gemm over the route reads listed columns
 * only); any other id at or past n_experts raises BM_SITE_EXPERT_ID with nothing stored. The written columns' bytes are
 * bm_swiglu_quant's. */
int bm_swiglu_quant_sel(bm_ctx *ctx, const float *g_dev, const float *u_dev, const uint32_t *sel_dev, int n_experts, int n_cols,
                        const bm_gate_act *rule, bm_act *act);


/* ------------------------------------------------------------------ one entry for every number of tokens */

/* The expert step of a layer for any number of tokens through one call, which picks among the three ways above by the
 * number of tokens - the reference's cut between its gemv arm and its wide arm (crates/gpu/src/arch/qwen3moe/wide.rs:75-77
 * GEMV_COLS, prefill.rs:602-604 WIDE_FROM, :147 wide_steps), here with a grouped arm between the two:
 *   BM_PATH_PER_SLOT  bm_moe_decode: two launches, every slot streams its expert's rows (repeats come from the caches);
 *   BM_PATH_GROUPED   bm_tables_quantize, bm_gate_up_tiles (bm_quantize_ord for a down stack on Q8_K columns),
 *                     bm_gemv_tiles, the slots' sum: an expert's rows are read once for all of its slots;
 *   BM_PATH_GEMM      bm_route_fill_quantize, bm_gemm twice, bm_swiglu_quant_sel, bm_gemm, the slots' sum: the int8 matrix
 *                     cores (in the f32 order bm_set_gemm_mode sets; every stack type bm_gemm takes).
 * In the exact mode all three give the same bits in y_dev. bm_scratch holds what the paths need between their launches for
 * up to max_tokens tokens (made at load time and shared by every layer of the same shape, as the reference's Q8Act scratch
 * is): max_tokens * n_slots_per_token <= 40960. BM_PATH_AUTO (the default) takes the per-slot path below grouped_from
 * tokens, the grouped path below gemm_from and the GEMM from there; the defaults are the crossovers measured on MI355X at
 * the Qwen3-30B-A3B layer shape: 22 tokens, and 448 tokens in the exact mode of bm_gemm or 96 in its tolerance mode (96 in
 * either mode where the gate/up stack dots against Q8_K columns: Q3_K, IQ2_XXS, IQ3_XXS, IQ4_XS; where the down stack does so
 * too and hidden x ff is 2^23 or more, the grouped path from the first token). On the grouped path a batch with no more slots
 * than experts whose h crosses in f32 rows takes the per-slot gate . up launch (over columns made in the tables' launch) and
 * the tile launch for down.
 * bm_scratch_set_path sets others (0 keeps a value; gemm_from then holds for both modes) or forces one path.
 * bm_scratch_path_for: the path a call with m tokens takes. A slot whose id names no expert of the stack adds nothing to
 * the sum and raises BM_SITE_EXPERT_ID unless it is BM_HOST_SLOT, which every path skips silently (the GEMM path's route
 * table does not list it, and its SwiGLU quantizer is bm_swiglu_quant_sel). Calls that share a scratch must not overlap. */
typedef struct bm_scratch bm_scratch;
#define BM_PATH_AUTO 0
#define BM_PATH_PER_SLOT 1
#define BM_PATH_GROUPED 2
#define BM_PATH_GEMM 3
int bm_scratch_create(bm_ctx *ctx, int gate_type, int down_type, int hidden, int ff, int n_experts, int n_slots_per_token,
                      int max_tokens, bm_scratch **out);
void bm_scratch_destroy(bm_scratch *scratch);
int bm_scratch_set_path(bm_scratch *scratch, int path, int grouped_from, int gemm_from);
int bm_scratch_path_for(const bm_scratch *scratch, int m);
int bm_moe_forward(bm_ctx *ctx, bm_scratch *scratch, const bm_weights *wg, const bm_weights *wu, const bm_weights *wd,
                   const float *x_dev, const uint32_t *sel_dev, const float *w_dev, const float *resid_dev, int m,
                   const bm_gate_act *rule, float *y_dev);

/* ------------------------------------------------------------------------------------------------- router */

/* The step before the experts: RouterKernels::enqueue_route, kernel softmax_router_route
 * (crates/gpu/src/route_softmax.rs:1643, :1203), in the CPU path's numbers (crates/model/src/moe.rs:246-279).
 * logits_dev: n_tokens rows of n_experts f32 (1 .. 1024 experts). Per token: the softmax probabilities (exp of
 * logit - max in f32, their sum in f64, one f32 divide) into probs_dev[t * n_experts ..] (probs_dev may be NULL),
 * the top_k (1 .. 32) experts by descending probability, ties toward the smaller id, into ids_dev[t * top_k ..],
 * and their weights into weights_dev[t * top_k ..]: with renorm != 0 each probability over the f32 rounding of the
 * chosen probabilities' f64 sum in slot order (norm_topk_prob), else the probability itself. The outputs are the
 * sel / weights arguments of the entries above. A token with a logit that is not finite raises BM_SITE_ROUTER, gets
 * NaN probabilities and weights, and keeps its ids as they stand. */
int bm_route_softmax(bm_ctx *ctx, const float *logits_dev, int n_tokens, int n_experts, int top_k, int renorm,
                     float *probs_dev, uint32_t *ids_dev, float *weights_dev);
/* The FFN norm and the router's logits, the step before bm_route_softmax (RouterKernels::enqueue_norm_fused,
 * crates/gpu/src/route_softmax.rs:1667-1674, does norm, quantizer and routing in one launch; here: this launch, then
 * bm_route_softmax, and the quantizer rides in bm_moe_decode / bm_gate_up_x over normed_dev). In the CPU path's numbers:
 * normed[t] = (scale * gain) * x[t] with scale = 1 / sqrt(mean of squares + eps), the squares summed in f64 and the mean
 * narrowed to f32 (crates/model/src/ops.rs:350-368); logits[t * n_experts + e] = router row e . normed[t] in
 * qdot::dot_f32's eight-lane order (crates/qdot/src/lib.rs:11349-11386). gain_dev NULL: no norm, the rows are dotted as
 * they are. router_dev: n_experts rows of hidden f32, x_dev: n_tokens rows; hidden a multiple of 8; normed_dev
 * (optional) receives the normed rows; every pointer 16-byte aligned. */
int bm_router_logits(bm_ctx *ctx, const float *router_dev, const float *x_dev, const float *gain_dev, float eps, int n_tokens,
                     int n_experts, int hidden, float *normed_dev, float *logits_dev);
/* bm_router_logits and bm_route_softmax as one launch (RouterKernels::enqueue_norm_fused / enqueue_norm_fused_m,
 * crates/gpu/src/route_softmax.rs:1667-1679: norm, logits, routing and the activation quantizer of the tokens in one
 * launch). Same arguments and the same bits in every output as the two calls one after the other. act_x (optional; hidden a
 * multiple of 256): the tokens' normed rows as quantized columns in the form the bm_act was made for, the bytes bm_quantize
 * makes of normed_dev (the launch's act_ffn), written by one more workgroup a token that the routing does not wait for:
 * bm_gate_up over act_x then takes the place of bm_gate_up_x / bm_moe_decode's first launch over normed_dev. One workgroup
 * a token, behind the logits' workgroups in the grid, takes the token's logits as they land (words of the context that
 * hold an armed pattern between launches; its wait is bounded: BM_SITE_ROUTER and NaN weights if a logit never came) and
 * routes the token (after a wait that ran out: bm_fault_clear, which arms the words again, before the next call).
 * logits_dev is required; 1 .. 4096 tokens a launch. Launches of this entry that share a context must not
 * overlap (they share those words). */
int bm_norm_route(bm_ctx *ctx, const float *router_dev, const float *x_dev, const float *gain_dev, float eps, int n_tokens,
                  int n_experts, int hidden, int top_k, int renorm, float *normed_dev, float *logits_dev, float *probs_dev,
                  uint32_t *ids_dev, float *weights_dev, bm_act *act_x);


/* ------------------------------------------------------------------------------------------- the card rule */

/* The reference's GPU tier has an activation form and row walks of its own, and its CPU crate restates them so the
 * tiers can be compared bit for bit (crates/qdot/src/lib.rs:2885 card_q8_1, :3558 card_q4k_dot_row, :3346
 * card_q3k_dot_row; the device side: q3k_quantize_q8_1 crates/gpu/src/lib.rs:1448, q4k_gemv :1617, q4k_gemv_sel
 * crates/gpu/src/q4k_sel.rs:358). These entries give those values on this GPU, so a caller holding outputs of the
 * reference's CUDA tier can compare them with this library's bit for bit. They are a second arithmetic beside the
 * CPU path's that every other entry follows, not a faster one.
 *
 * A card q8_1 column of k values (a multiple of 256) is three planes in value order: codes i8[k]; d8 f32[k / 128],
 * a 128-value block's amax / 127 (1 for a zero block); s8 i32[k / 32], the code sum of 32 values. Codes are
 * v / d rounded half away from zero and held to +-127. A block holding a value that is not finite is refused: NaN
 * scale, zero codes and sums, and the fault word takes QuantColumn. m columns lie back to back in each plane. */
int bm_card_quantize(bm_ctx *ctx, const float *x_dev, int m, int k, int8_t *codes_dev, float *d8_dev, int32_t *s8_dev);
/* y_dev[r * m + c] = row r of w (Q4_K or Q3_K) against column c, by the 32-lane walk and its butterfly. */
int bm_card_gemv(bm_ctx *ctx, const bm_weights *w, const int8_t *codes_dev, const float *d8_dev, const int32_t *s8_dev, int m,
                 float *y_dev);
/* The MoE down step of the card tier: y_dev[s * rows_per_expert + r] = row r of expert sel_dev[s] against column s.
 * Ids as bm_gemv_sel takes them (past the stack: ExpertId raised, the slot's rows untouched; 0xffffffff skipped). */
int bm_card_gemv_sel(bm_ctx *ctx, const bm_weights *w, const int8_t *codes_dev, const float *d8_dev, const int32_t *s8_dev,
                     const uint32_t *sel_dev, int n_slots, int rows_per_expert, float *y_dev);

/* ------------------------------------------------------------------------------------------- model files */

/* A GGUF file's header and a read-only mapping of it: the part of the reference's reader (crates/gguf/src/lib.rs:
 * Gguf::open :319, find :540, data :557, value :439; TensorInfo :103) that hands a model file's expert stacks to
 * bm_weights_create. Host code; no context is needed. Versions 2 and 3, little-endian. Every length, count and
 * offset of the file is checked against its size at open (LoadError::OutOfBounds and friends are refusals here);
 * bm_gguf_last_error() holds the message of the calling thread's last refusal. */
typedef struct bm_gguf bm_gguf;
typedef struct bm_gguf_tensor {
    const char *name;  /* owned by the bm_gguf */
    int type;          /* the ggml type id as the file states it (BM_TYPE_Q3_K = 11, BM_TYPE_Q4_K = 12, BM_TYPE_Q5_K = 13, BM_TYPE_Q6_K = 14, BM_TYPE_IQ2_XXS = 16, BM_TYPE_IQ3_XXS = 18, BM_TYPE_IQ4_XS = 23, 0 = F32 ...) */
    int n_dims;        /* 1 .. 4 */
    uint64_t dims[4];  /* ggml ne[] order: dims[0] is the contiguous axis; unused dims are 1 */
    uint64_t offset;   /* from the file's data section */
    uint64_t nbytes;   /* type_size * (dims[0] / block) * dims[1] * ...; 0 for a type this build cannot size */
    const void *data;  /* the tensor's bytes in the mapping (valid until bm_gguf_close); NULL when nbytes is 0 */
} bm_gguf_tensor;
int bm_gguf_open(const char *path, bm_gguf **out);
/* A model as one file or as llama.cpp's split set, opened by its first shard (crates/gguf/src/lib.rs:617-630 Split,
 * :835-875 Split::open_model): a file without "split.count" is a set of one. The siblings of
 * <prefix>-00001-of-%05d.gguf are <prefix>-%05d-of-%05d.gguf; every shard's "split.no" is its place (from 0), every
 * "split.count" agrees, the shards' tensor counts sum to the first shard's "split.tensors.count" and no tensor name
 * appears twice, or the set is refused with the file and key named. The handle then answers for the whole set: tensors
 * in shard order, each one's offset and data within its own shard, key-values from the first shard (the splitter
 * writes the model's keys there alone). bm_gguf_open on a shard reads that one file (Gguf::open_split_shard, :359). */
int bm_gguf_open_split(const char *first_shard_path, bm_gguf **out);
void bm_gguf_close(bm_gguf *g);
const char *bm_gguf_last_error(void);
int bm_gguf_version(const bm_gguf *g);
int64_t bm_gguf_tensor_count(const bm_gguf *g);
int bm_gguf_tensor_at(const bm_gguf *g, int64_t i, bm_gguf_tensor *out);
int bm_gguf_find(const bm_gguf *g, const char *name, bm_gguf_tensor *out);
/* Key-values: an integer of any width that is not negative (Value::as_u64, crates/gguf/src/lib.rs:1510), an f32, a
 * string (NULL when the key is absent or not a string). "<arch>.expert_count", "<arch>.expert_used_count" and
 * "general.architecture" are what the MoE caller reads (crates/gguf/src/lib.rs:512-516,453). */
int bm_gguf_get_u64(const bm_gguf *g, const char *key, uint64_t *out);
int bm_gguf_get_f32(const bm_gguf *g, const char *key, float *out);
const char *bm_gguf_get_str(const bm_gguf *g, const char *key);
/* The tensor `name` of the file as a weight stack on the device: a matrix {k, rows} or an expert stack
 * {k, rows_per_expert, n_experts} (crates/model/src/moe.rs:330 expert_view: expert e's matrix is the e-th equal part),
 * rows back to back as bm_weights_create takes them. The tensor's type must be one this library computes in
 * (BM_TYPE_Q3_K, BM_TYPE_Q4_K, BM_TYPE_Q5_K, BM_TYPE_Q6_K, BM_TYPE_IQ2_XXS, BM_TYPE_IQ3_XXS, BM_TYPE_IQ4_XS); rows_per_expert and n_experts (either may be NULL) receive dims[1] and dims[2]. */
int bm_weights_from_gguf(bm_ctx *ctx, const bm_gguf *g, const char *name, bm_weights **out, int *rows_per_expert, int *n_experts);

/* ------------------------------------------------------------------------------------------- verification */

/* The exact per-block integers the kernels above form for row `row` of w against column `col` of act, written
 * to out_dev as i32, through the same device code the launchers run:
 *   Q4_K, Q5_K: per super-block 8 sums A[s] = sum q * a over sub-block s (q the 4- or 5-bit code), then the 8
 *            activation isums (16 words);
 *   Q6_K:    per super-block 16 sums S[g] = sum (q6 - 32) * a over 16-value group g (16 words);
 *   Q3_K:    per super-block 16 sums S[g] = sum (q3 - 4) * a over 16-value group g (16 words);
 *   IQ2_XXS, IQ3_XXS: per super-block 8 sums I[b] = sum (+-grid) * a over sub-block b, then the 8 scales 2s + 1
 *            (16 words);
 *   IQ4_XS:  per super-block 8 sums I[b] = sum level * a over sub-block b, then the CPU path's 8 i32 lanes
 *            L[l] = sum_b scale_b * (sum over values 4l .. 4l + 3 of sub-block b of level * a) (16 words).
 * out_dev holds 16 * (k / 256) words. These are the integers crates/qdot's lanes hold (its gates pin them by
 * bit identity, crates/qdot/tests/qdot.rs:738,818,2664). */
int bm_block_sums(bm_ctx *ctx, const bm_weights *w, int64_t row, const bm_act *act, int col, int32_t *out_dev);

/* ------------------------------------------------------------------------------------ graphs and events */

typedef struct bm_graph bm_graph; /* an instantiated HIP graph of launches captured on the context's stream */
typedef struct bm_event bm_event; /* a HIP event on the context's stream */

/* The reference replays each decode step as one captured graph (crates/gpu/src/arch/qwen3moe/dispatch.rs, the
 * launchers' "capturable" contract, crates/gpu/src/q4k_sel.rs:973). bm_capture_begin starts capturing the
 * context's stream (thread-local mode); the launchers called until bm_capture_end become the graph's nodes.
 * Ids, activations and outputs are read and written through their device pointers at replay time. */
int bm_capture_begin(bm_ctx *ctx);
int bm_capture_end(bm_ctx *ctx, bm_graph **out);
int bm_graph_launch(bm_ctx *ctx, bm_graph *graph);
void bm_graph_destroy(bm_graph *graph);

int bm_event_create(bm_ctx *ctx, bm_event **out);
int bm_event_record(bm_ctx *ctx, bm_event *event);
/* The work enqueued on the context's stream after this call waits for `event`, which another context may have recorded on
 * its own stream (`Stream::wait`, crates/device/src/lib.rs:821, crates/gpu/src/device.rs:244): the fork and join of two
 * streams. Under capture a wait for an event recorded on the capturing stream draws the waiting context's stream into the same
 * graph, where the two streams' launches become branches that may run side by side (the capturing context must wait for an
 * event recorded at the end of the other stream's work before bm_capture_end). */
int bm_event_wait(bm_ctx *ctx, bm_event *event);
/* Waits for `stop`, then the milliseconds from `start` to `stop`. */
int bm_event_elapsed_ms(bm_ctx *ctx, bm_event *start, bm_event *stop, float *ms);
void bm_event_destroy(bm_event *event);

/* Library version: major * 10000 + minor * 100 + patch. */
int bm_version(void);

#ifdef __cplusplus
}
#endif

#endif /* BM_MOE_H */
