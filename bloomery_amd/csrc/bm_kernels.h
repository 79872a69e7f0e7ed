// Host-callable launch functions of the HIP kernels (bm_kernels.hip). Geometry is checked by the C ABI layer
// (bm_capi.cpp) before any of these is called; they enqueue on `stream`, allocate nothing and never synchronise.
#ifndef BM_KERNELS_H
#define BM_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bmk {

struct Launch {
    hipStream_t stream;
    uint32_t *fault; // device fault word, u32[BM_FAULT_WORDS]
    uint32_t layer;  // layer the launch raises with
};

// Largest dynamic LDS a launch may ask for (gfx950 has 160 KiB a workgroup).
constexpr int kMaxLds = 160 * 1024;

hipError_t fill_u32(const Launch &L, uint32_t *dst, uint32_t value, size_t n);

hipError_t quantize(const Launch &L, int wtype, const float *x, int m, int k, uint8_t *act);

// Columns that fit one gemv launch's LDS for this type and k (at most 8).
int gemv_max_cols(int wtype, int k);
hipError_t gemv(const Launch &L, int wtype, const uint8_t *w, int64_t rows, int k, const uint8_t *act, int m_total,
                int col0, int m, float *y);

hipError_t gate_up(const Launch &L, int wtype, const uint8_t *wg, const uint8_t *wu, int n_experts, int k,
                   const uint8_t *act, const uint32_t *sel, int n_slots, int rows_per_expert, int slots_per_col,
                   float *h, uint8_t *act_h);

hipError_t gemv_sel(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                    const uint32_t *sel, int n_slots, int rows_per_expert, float *y);

hipError_t combine_tokens(const Launch &L, const float *down, const float *w, const float *resid, int rows,
                          int n_slots, int m, float *y);

// Slots a token may have in the fused down + combine launch.
constexpr int kMaxCombineSlots = 64;
hipError_t down_combine(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                        const uint32_t *sel, const float *wts, const float *resid, int slots_per_token, int m,
                        int rows_per_expert, float *y);

hipError_t block_sums(const Launch &L, int wtype, const uint8_t *wrow, int k, const uint8_t *col, int32_t *out);

} // namespace bmk

#endif // BM_KERNELS_H
