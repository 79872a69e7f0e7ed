// Host-callable launch functions of the HIP kernels (bm_kernels.hip). Geometry is checked by the C ABI layer
// (bm_capi.cpp) before any of these is called; they enqueue on `stream`, allocate nothing and never synchronise.
#ifndef BM_KERNELS_H
#define BM_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bmk {

// The rule a gate . up launch applies to a row's two sums (crates/gpu/src/kquant/act.rs:21-57 Act and its device
// codes): silu(g) * u, ik's clamped SwiGLU, the gpt-oss / MiniMax SwiGLU at alpha 1.702, SiTU-GLU at linear beta 25
// (limit carries the gate's beta), ggml's gate-first clamp.
struct GateRule {
    uint32_t act;
    float limit;
};
constexpr uint32_t kActSiluMul = 0, kActSwigluClamp = 1, kActSwigluOai = 2, kActSitu = 3, kActSwigluGclamp = 4;

struct Launch {
    hipStream_t stream;
    uint32_t *fault; // device fault word, u32[BM_FAULT_WORDS]
    uint32_t layer;  // layer the launch raises with
    GateRule rule;   // what the gate . up launches apply
    int down_form = 0; // BM_DOWN_RING or BM_DOWN_SPLIT: how down_combine walks a row (bm_set_down_form)
};

// Largest dynamic LDS a launch may ask for (gfx950 has 160 KiB a workgroup).
constexpr int kMaxLds = 160 * 1024;

hipError_t fill_u32(const Launch &L, uint32_t *dst, uint32_t value, size_t n);

// Bytes of one activation column of k values on the device, in the form weight type `wtype` dots against: the CPU
// path's bytes, and for the Q8_2_X4 form two tables after them (bm_device.hpp).
int act_col_bytes(int wtype, int k);

// `live` (optional): a device word holding how many of the m columns to quantize; the rest keep what they held.
hipError_t quantize(const Launch &L, int wtype, const float *x, int m, int k, uint8_t *act,
                    const uint32_t *live = nullptr, const uint32_t *sel = nullptr, uint32_t n_experts = 0);

// Rebuilds the tables of m Q8_2_X4 device columns whose reference bytes were just written by a copy.
hipError_t q82_tables(const Launch &L, uint8_t *act, int m, int k);

// Columns that fit one gemv launch's LDS for this type and k (at most 8).
int gemv_max_cols(int wtype, int k);
hipError_t gemv(const Launch &L, int wtype, const uint8_t *w, int64_t rows, int k, const uint8_t *act, int m_total,
                int col0, int m, float *y);

hipError_t gate_up(const Launch &L, int wtype, const uint8_t *wg, const uint8_t *wu, int n_experts, int k,
                   const uint8_t *act, const uint32_t *sel, int n_slots, int rows_per_expert, int slots_per_col,
                   float *h, uint8_t *act_h);

hipError_t gemv_sel(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                    const uint32_t *sel, int n_slots, int rows_per_expert, float *y);

// sel (optional): a slot whose id is at or past n_experts adds nothing
hipError_t combine_tokens(const Launch &L, const float *down, const float *w, const float *shexp, const float *resid,
                          int rows, int n_slots, int m, float *y, const uint32_t *sel = nullptr, uint32_t n_experts = 0);

// Slots a token may have in the fused down + combine launch.
constexpr int kMaxCombineSlots = 64;
hipError_t down_combine(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                        const uint32_t *sel, const float *wts, const float *resid, int slots_per_token, int m,
                        int rows_per_expert, float *y);

// The whole decode step: quantize x, gate . up . SwiGLU, quantize h, down, weighted slot sum, in two launches: gate . up
// with the quantizers folded in, then down + combine.
constexpr int kMaxDecodeTokens = 1024;
bool moe_decode_supported(int gate_type, int down_type);
// gate . up . SwiGLU from f32 token rows, the token quantizer folded in: the first launch of moe_decode. act_h
// (Q8_2_X4 columns, or NULL when the down stack takes Q8_K ones) is quantized in the same launch; h (f32 rows) is
// optional beside act_h and the output without it.
hipError_t gate_up_x(const Launch &L, int gate_type, const float *x, const uint8_t *wg, const uint8_t *wu,
                     int n_experts, int hidden, int ff, const uint32_t *sel, int slots_per_token, int m,
                     uint8_t *act_x, uint8_t *act_h, float *h);
hipError_t down_combine_hq(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const float *h,
                           uint8_t *act_h, const uint32_t *sel, const float *wts, const float *resid,
                           int slots_per_token, int m, int rows_per_expert, float *y);
hipError_t moe_decode(const Launch &L, int gate_type, int down_type, const float *x, const uint8_t *wg, const uint8_t *wu,
                      const uint8_t *wd, int n_experts, int hidden, int ff, const uint32_t *sel, const float *wts,
                      const float *resid, int slots_per_token, int m, uint8_t *act_x, uint8_t *act_h, float *h, float *y);

// moe_decode's two launches with act_h and h in a file-scope device array instead of caller memory: no allocation
// anywhere on the way. static_scratch_init(device), called with that device current (the context's creation does),
// looks the array's address up once a device; kStaticValues = the most values of h (tokens x slots x ff) a call may ask
// for. Calls on one device share the array: two that overlap race.
constexpr size_t kStaticValues = 65536;
hipError_t static_scratch_init(int device);
hipError_t moe_decode_static(const Launch &L, int device, int gate_type, int down_type, const float *x, const uint8_t *wg,
                             const uint8_t *wu, const uint8_t *wd, int n_experts, int hidden, int ff, const uint32_t *sel,
                             const float *wts, const float *resid, int slots_per_token, int m, float *y);

// ------------------------------------------------------------------------------ grouped decode (bm_grouped.hip)

// crates/gpu/src/q4k_sel.rs:68-97: a tile is up to 8 consecutive entries of one expert's run; word (e << 22) | j.
constexpr int kTileCols = 8;
constexpr int kTileExpertShift = 22;
constexpr int kBucketExperts = 1024;
constexpr int kTileMaxSlots = 1 << kTileExpertShift;
int tile_cap(int n_slots, int n_experts);

hipError_t buckets(const Launch &L, const uint32_t *sel, int n_slots, int n_experts, uint32_t *order, uint32_t *start);
hipError_t tiles(const Launch &L, const uint32_t *start, int n_experts, int n_slots, uint32_t *tiles);
// buckets, then tiles, in one launch
hipError_t tables(const Launch &L, const uint32_t *sel, int n_slots, int n_experts, uint32_t *order, uint32_t *start,
                  uint32_t *tiles);
// LDS bytes a tile launch of this type and k asks for (0 if eight columns do not fit a workgroup's LDS).
size_t tiles_lds(int wtype, int k);
// tables() and quantize() of m rows of k f32 values (k a multiple of 256, x 16-byte aligned) into the column form wtype
// dots against, as one launch.
hipError_t tables_quant(const Launch &L, const uint32_t *sel, int n_slots, int n_experts, uint32_t *order, uint32_t *start,
                        uint32_t *tiles_out, int wtype, const float *x, int m, int k, uint8_t *act);
hipError_t gate_up_tiles(const Launch &L, int wtype, const uint8_t *wg, const uint8_t *wu, int n_experts, int k,
                         const uint8_t *act, int act_cols, const uint32_t *order, const uint32_t *start,
                         const uint32_t *tiles, int n_slots, int rows_per_expert, int slots_per_col, float *h,
                         uint8_t *act_h);
hipError_t gemv_tiles(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                      const uint32_t *order, const uint32_t *start, const uint32_t *tiles, int n_slots,
                      int rows_per_expert, float *y, bool by_slot = false);

// ------------------------------------------------------------------------------------- prefill (bm_prefill.hip)

// crates/gpu/src/gemm/mod.rs:97-101, route.rs:11-13.
constexpr int kGemmBN = 64, kGemmBM = 64;
constexpr int kGemmMaxSlots = 40960, kGemmMaxExperts = 1024;
int gemm_max_tiles(int n_slots, int n_experts);
// cols[n_slots], tiles[2 * gemm_max_tiles], n_tiles[3]: tiles, refused slots, slots served elsewhere (not listed)
// x (optional; 16-byte aligned, k a multiple of 256): in the same launch, quantize() of m rows of k f32 values into act, the
// column form wtype dots against.
hipError_t route(const Launch &L, const uint32_t *ids, int n_slots, int n_experts, uint32_t *cols, uint32_t *tiles,
                 uint32_t *n_tiles, int wtype = 0, const float *x = nullptr, int m = 0, int k = 0, uint8_t *act = nullptr);
// q8k: the columns are Q8_K ones (else Q8_2_X4)
// sel (optional): column c is slot c's; a slot served elsewhere is left as it stands, another id at or past n_experts raises
hipError_t swiglu_quant(const Launch &L, const float *g, const float *u, int m, int k, uint8_t *act, bool q8k,
                        const uint32_t *sel = nullptr, uint32_t n_experts = 0);
bool gemm_supported(int wtype);
// slot_div: slots a token when every slot of a token reads the token's column, 1 when each slot reads its own.
// mode 0: the CPU path's eight-accumulator f32 order (bit-identical to the row dots); 1: one accumulator a value, int8
// matrix instructions; 2: one accumulator, f16 matrix instructions with the scales in the operands (Q4_K; else as 1).
hipError_t gemm(const Launch &L, int wtype, const uint8_t *w, int n_experts, int rows_per_expert, int k,
                const uint8_t *act, const uint32_t *cols, const uint32_t *tiles, const uint32_t *n_tiles, int n_slots,
                int slot_div, float *y, int mode);

// The tolerance mode on f16 matrix instructions with both scales folded into the operands (bm_gemm_half.hip): gemm()'s
// mode 2 where a type has that form; mode 1 is the int8 form.
bool gemm_half_supported(int wtype);
hipError_t gemm_half(const Launch &L, int wtype, const uint8_t *w, int n_experts, int rows_per_expert, int k, const uint8_t *act,
                     const uint32_t *cols, const uint32_t *tiles, const uint32_t *n_tiles, int n_slots, int slot_div, float *y);

// ---------------------------------------------------------------------------------------- router (bm_router.hip)

constexpr int kRouteMaxExperts = 1024, kRouteMaxPicks = 32;
// probs may be NULL. logits[n_tok * n_exp], ids / weights[n_tok * used].
hipError_t route_softmax(const Launch &L, const float *logits, int n_tok, int n_exp, int used, int renorm, float *probs,
                         uint32_t *ids, float *weights);

// The FFN norm (gain NULL: none) and the router's f32 logits: router[n_exp * hidden], x[m * hidden], logits[m * n_exp],
// normed_out (optional) [m * hidden]. hidden a multiple of 8.
bool router_logits_fits(int hidden);
// router_logits and route_softmax as one launch: a token's logits reach its routing wave through `hand`, a word a (token,
// expert) of the launch (m * n_exp of them) that holds kRouteArmed between launches (left so); launches that share it must
// not overlap. kRouteArmed is a signalling NaN's pattern: no logit has it, arithmetic only ever leaves the quiet form.
constexpr int kNormRouteMaxTokens = 4096;
constexpr uint32_t kRouteArmed = 0x7fa00001u;
// polls after which a routing wave gives a token up (BM_SITE_ROUTER, NaN weights): some ten seconds; only a launch that
// lost its other workgroups gets there
constexpr uint32_t kRoutePolls = 1u << 24;
// act_x (optional; hidden a multiple of 256): the tokens' normed rows as quantized columns (q8k: Q8_K, else Q8_2_X4 with tables)
hipError_t norm_route(const Launch &L, const float *router, const float *x, const float *gain, float eps, int m, int n_exp,
                      int hidden, float *normed_out, float *logits, int used, int renorm, float *probs, uint32_t *ids,
                      float *weights, uint32_t *hand, uint8_t *act_x = nullptr, bool q8k = false, uint32_t max_polls = kRoutePolls);
hipError_t router_logits(const Launch &L, const float *router, const float *x, const float *gain, float eps, int m, int n_exp,
                         int hidden, float *normed_out, float *logits);

// gemv from f32 columns x[m * k], the quantizer folded in: y[row * m + c]; act_out (optional) receives the columns' bytes
// in the device form of an activation column.
size_t gemv_x_lds(int wtype, int k);
hipError_t gemv_x(const Launch &L, int wtype, const uint8_t *w, int64_t rows, int k, const float *x, int m, uint8_t *act_out,
                  float *y);

hipError_t block_sums(const Launch &L, int wtype, const uint8_t *wrow, int k, const uint8_t *col, int32_t *out);

// The card rule (bm_card.hip): the reference GPU tier's q8_1 columns (codes[m * k], d8[m * k / 128], s8[m * k / 32]) and
// its 32-lane Q4_K / Q3_K row walks. codes must be 16-byte aligned.
bool card_type(int wtype);
hipError_t card_quantize(const Launch &L, const float *x, int m, int k, int8_t *codes, float *d8, int32_t *s8);
hipError_t card_gemv(const Launch &L, int wtype, const uint8_t *w, long rows, int k, const int8_t *codes, const float *d8,
                     const int32_t *s8, int m, float *y);
hipError_t card_gemv_sel(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const int8_t *codes, const float *d8,
                         const int32_t *s8, const uint32_t *sel, int n_slots, int rows_per_expert, float *y);

} // namespace bmk

#endif // BM_KERNELS_H
