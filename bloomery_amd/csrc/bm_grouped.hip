// Grouped decode: the routed expert chain of several tokens with each expert's rows read once for up to eight of
// its slots. The tables are the reference's (crates/gpu/src/q4k_sel.rs:20-41): `order` lists the card's slots by
// expert, expert e's run is order[start[e] .. start[e + 1]], and the tile table cuts every run into tiles of up to
// eight consecutive entries, tile g the word (e << 22) | j at tiles[1 + g], their count at tiles[0]. Every slot's
// value is its slot-by-slot launch's, bit for bit: a column of the multi-column dot is the one-column dot.
#include "bm_stream.hpp"

namespace bmk {

constexpr u32 kHostSlot = 0xffffffffu; // crates/gpu/src/host/slots.rs:10

int tile_cap(int n_slots, int n_experts) { // crates/gpu/src/q4k_sel.rs:96-98
    const long a = ((long)n_slots + (long)(kTileCols - 1) * n_experts) / kTileCols;
    return (int)(a < n_slots ? a : n_slots);
}

// ---------------------------------------------------------------------------------------------- tables

// crates/gpu/src/q4k_sel.rs:480-560 grouped_buckets: one workgroup of 1024 threads. Slots keep their order inside
// a run. An id at or past the stack that is not the host's raises ExpertId and joins no run.
__global__ __launch_bounds__(1024) void k_buckets(const u32 *sel, u32 n_slots, u32 n_experts, u32 *order, u32 *start,
                                                  u32 *fault, u32 layer) {
    __shared__ GroupLds g;
    group_slots(g, n_slots, n_experts, order, [&](u32 s) {
        const u32 p = sel[s];
        if (p < n_experts) return p;
        if (p != kHostSlot) bm_raise(fault, layer, kSiteExpertId);
        return kNoBucket;
    });
    for (u32 e = threadIdx.x; e <= n_experts; e += kGroupThreads) start[e] = g.base[e];
}

// crates/gpu/src/q4k_sel.rs:562-680 grouped_tiles. A run outside 0 .. start[n_experts] <= n_slots, or more tiles
// than `cap`, raise ExpertId and leave a count of 0.
__device__ __forceinline__ void tiles_body(const u32 *start, u32 n_experts, u32 n_slots, u32 cap, u32 *tiles, u32 *fault,
                                           u32 layer) {
    __shared__ u32 scan[17];
    __shared__ u32 bad;
    const u32 tid = threadIdx.x;
    const u32 end = start[n_experts];
    if (tid == 0) bad = 0;
    __syncthreads();
    u32 j0 = 0, j1 = 0, c = 0;
    if (tid < n_experts) {
        j0 = start[tid];
        j1 = start[tid + 1];
        if (j0 <= j1 && j1 <= end && end <= n_slots)
            c = (j1 - j0 + kTileCols - 1) / kTileCols; // at most 2^19: the sum of 1024 of them fits a word
        else
            bad = 1;
    }
    u32 total;
    u32 g = block_scan_1024(c, scan, &total); // its barriers publish `bad`
    const bool refuse = bad != 0 || total > cap;
    if (tid == 0) {
        if (refuse) bm_raise(fault, layer, kSiteExpertId);
        tiles[0] = refuse ? 0 : total;
    }
    if (tid < n_experts && !refuse)
        for (u32 j = j0; j < j1; j += kTileCols) tiles[1 + g++] = (tid << kTileExpertShift) | j;
}

__global__ __launch_bounds__(1024) void k_tiles(const u32 *start, u32 n_experts, u32 n_slots, u32 cap, u32 *tiles,
                                                u32 *fault, u32 layer) {
    tiles_body(start, n_experts, n_slots, cap, tiles, fault, layer);
}

// k_buckets, then k_tiles over the runs it has just written: the grouped step's two table launches as one.
__global__ __launch_bounds__(1024) void k_tables(const u32 *sel, u32 n_slots, u32 n_experts, u32 cap, u32 *order, u32 *start,
                                                 u32 *tiles, u32 *fault, u32 layer) {
    __shared__ GroupLds g;
    group_slots(g, n_slots, n_experts, order, [&](u32 s) {
        const u32 p = sel[s];
        if (p < n_experts) return p;
        if (p != kHostSlot) bm_raise(fault, layer, kSiteExpertId);
        return kNoBucket;
    });
    for (u32 e = threadIdx.x; e <= n_experts; e += kGroupThreads) start[e] = g.base[e];
    __threadfence_block();
    __syncthreads(); // the runs are the workgroup's own writes: visible to it past the barrier
    tiles_body(start, n_experts, n_slots, cap, tiles, fault, layer);
}

// k_tables with a quantizer beside it: workgroup 0 makes the tables, the others the quantized columns of m rows of k f32
// values - Q8_K: a wave a 256-value block, the bytes of k_quantize_q8k; Q8_2_X4: eight values a thread, a block a quad of
// lanes, the bytes of k_quantize_q82x4 - two short launches that do not depend on each other as one.
template <bool Q8K>
__global__ __launch_bounds__(1024) void k_tables_quant(const u32 *sel, u32 n_slots, u32 n_experts, u32 cap, u32 *order, u32 *start,
                                                       u32 *tiles, const float *x, int m, int k, uint8_t *act, u32 *fault, u32 layer) {
    if (blockIdx.x != 0) {
        if constexpr (Q8K) {
            const int b = (int)(blockIdx.x - 1) * 16 + (int)(threadIdx.x >> 6), lane = (int)(threadIdx.x & 63);
            if (b >= m * (k / 256)) return; // whole waves leave
            q8k_wave_block(*reinterpret_cast<const float4 *>(x + (size_t)b * 256 + 4 * lane), act + (size_t)b * BM_Q8K_STRIDE, lane, fault, layer);
        } else {
            const long at = ((long)(blockIdx.x - 1) * 1024 + threadIdx.x) * 8;
            if (at >= (long)m * k) return; // whole quads leave: a block is 32 values, k a multiple of 256
            const int col = (int)(at / k), o = (int)(at % k);
            const float4 a = *reinterpret_cast<const float4 *>(x + at), b = *reinterpret_cast<const float4 *>(x + at + 4);
            const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            q82_quad8(v, act + (size_t)col * (k / 256) * BM_Q82_SB_EXT, k / 256, o >> 5, threadIdx.x & 3, fault, layer);
        }
        return;
    }
    __shared__ GroupLds g;
    group_slots(g, n_slots, n_experts, order, [&](u32 s) {
        const u32 p = sel[s];
        if (p < n_experts) return p;
        if (p != kHostSlot) bm_raise(fault, layer, kSiteExpertId);
        return kNoBucket;
    });
    for (u32 e = threadIdx.x; e <= n_experts; e += kGroupThreads) start[e] = g.base[e];
    __threadfence_block();
    __syncthreads();
    tiles_body(start, n_experts, n_slots, cap, tiles, fault, layer);
}

hipError_t tables_quant(const Launch &L, const uint32_t *sel, int n_slots, int n_experts, uint32_t *order, uint32_t *start,
                        uint32_t *tiles_out, int wtype, const float *x, int m, int k, uint8_t *act) {
    if (k % 256 != 0 || (reinterpret_cast<uintptr_t>(x) & 15) != 0) return hipErrorInvalidValue;
    const u32 cap = (u32)tile_cap(n_slots, n_experts);
    if (bm_takes_q8k(wtype)) {
        const unsigned grid = 1 + (unsigned)((m * (k / 256) + 15) / 16);
        hipLaunchKernelGGL(k_tables_quant<true>, dim3(grid), dim3(1024), 0, L.stream, sel, (u32)n_slots, (u32)n_experts, cap, order, start,
                           tiles_out, x, m, k, act, L.fault, L.layer);
    } else {
        const unsigned grid = 1 + (unsigned)(((long)m * k + 8191) / 8192);
        hipLaunchKernelGGL(k_tables_quant<false>, dim3(grid), dim3(1024), 0, L.stream, sel, (u32)n_slots, (u32)n_experts, cap, order, start,
                           tiles_out, x, m, k, act, L.fault, L.layer);
    }
    return hipGetLastError();
}

hipError_t tables(const Launch &L, const uint32_t *sel, int n_slots, int n_experts, uint32_t *order, uint32_t *start,
                  uint32_t *tiles_out) {
    hipLaunchKernelGGL(k_tables, dim3(1), dim3(1024), 0, L.stream, sel, (u32)n_slots, (u32)n_experts,
                       (u32)tile_cap(n_slots, n_experts), order, start, tiles_out, L.fault, L.layer);
    return hipGetLastError();
}

hipError_t buckets(const Launch &L, const uint32_t *sel, int n_slots, int n_experts, uint32_t *order, uint32_t *start) {
    hipLaunchKernelGGL(k_buckets, dim3(1), dim3(1024), 0, L.stream, sel, (u32)n_slots, (u32)n_experts, order, start,
                       L.fault, L.layer);
    return hipGetLastError();
}

hipError_t tiles(const Launch &L, const uint32_t *start, int n_experts, int n_slots, uint32_t *tiles_out) {
    hipLaunchKernelGGL(k_tiles, dim3(1), dim3(1024), 0, L.stream, start, (u32)n_experts, (u32)n_slots,
                       (u32)tile_cap(n_slots, n_experts), tiles_out, L.fault, L.layer);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------- tile kernels

// A launch's workgroup as every tile kernel reads it (crates/gpu/src/q4k_sel.rs:101-151 tile_at, :186-234
// tile_block): workgroup b is tile g = b mod cap of row block b / cap. False: no tile (past the count, or a word
// that names no run of the table, which raises ExpertId).
struct Tile {
    int e, j, m, row_block;
    u32 entry; // threads 0 .. 7: order[j + thread] (0 past the table), requested together with the run's end
};
// The lookups are a chain of memory round trips in front of everything a workgroup does, so each step asks for all it
// can: the count and the word together (the table holds cap + 1 words, so word g is there whatever the count), then
// the run's end together with the tile's entries of `order`.
__device__ __forceinline__ bool tile_of_block(const u32 *tiles, const u32 *start, const u32 *order, u32 n_experts, u32 n_slots,
                                              u32 cap, Tile *t, u32 *fault, u32 layer) {
    const u32 g = blockIdx.x % cap;
    t->row_block = (int)(blockIdx.x / cap);
    const u32 count = tiles[0], word = tiles[1 + g];
    if (g >= count) return false;
    const u32 e = word >> kTileExpertShift, j = word & ((1u << kTileExpertShift) - 1);
    const u32 at = j + threadIdx.x;
    t->entry = threadIdx.x < (u32)kTileCols && at < n_slots ? order[at] : 0;
    const u32 j1 = e < n_experts ? start[e + 1] : 0;
    if (!(j < j1 && j1 <= n_slots)) {
        if (threadIdx.x == 0) bm_raise(fault, layer, kSiteExpertId);
        return false;
    }
    t->e = (int)e;
    t->j = (int)j;
    t->m = (int)(j1 - j < (u32)kTileCols ? j1 - j : (u32)kTileCols);
    return true;
}

// The tile's m activation columns into LDS, column c from `src_col(c)` of act (a column index, or -1: none).
template <class ColOf>
__device__ __forceinline__ void stage_tile_cols(uint8_t *cols, const uint8_t *act, int col_bytes, int m,
                                                const ColOf &src_col) {
    for (int c = 0; c < m; c++) {
        const int sc = src_col(c);
        if (sc >= 0) stage_bytes(cols + (size_t)c * col_bytes, act + (size_t)sc * col_bytes, col_bytes);
    }
}

// crates/gpu/src/kquant/tiles.rs:62-118 GateUpTiles: workgroup = tile x 32 rows of the tile's expert, eight lanes a
// row (a quad on the gate row, a quad on the up row), all m columns in one pass over the two rows. Entry j + c reads
// the activation column of the token of slot order[j + c] and writes h[(j + c) * rpe + r]: by entry, not by slot.
// With act_h the 32 values of each column become block rb of column j + c of act_h in the same launch.
// MC: the columns this launch has LDS for; it takes the tiles of m_lo < m <= MC columns and leaves the others to the
// launch of the other width (see tile_widths below). PASSES: it takes every tile, MC columns at a pass over the rows
// (a wider tile's rows are then read and unpacked again for every pass: the form for batches whose tiles are nearly all
// narrow, where it saves the second launch; a variant of its own, so that the one-pass kernels stay straight-line code).
template <int WT, int U, int NB, int MC, bool PASSES>
__global__ __launch_bounds__(256) void k_gate_up_tiles(const uint8_t *wg, const uint8_t *wu, u32 n_experts, int nb,
                                                       const uint8_t *act, int act_cols, const u32 *order,
                                                       const u32 *start, const u32 *tiles, u32 n_slots, u32 cap,
                                                       int rpe, int slots_per_col, float *h, uint8_t *act_h, int m_lo,
                                                       GateRule rule, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3, which = (tid >> 2) & 1;
    Tile t;
    if (!tile_of_block(tiles, start, order, n_experts, n_slots, cap, &t, fault, layer)) return; // raising twice is raising once
    if (!PASSES && (t.m <= m_lo || t.m > MC)) return;
    __shared__ u32 s_entry[kTileCols];
    if (PASSES && tid < kTileCols) s_entry[tid] = t.entry;
    const int rb = t.row_block;
    const int r = rb * 32 + (tid >> 3);
    const bool active = r < rpe;
    const int n = NB > 0 ? NB : nb;
    const int nb_h = rpe / 256;
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const uint8_t *wrow = (which ? wu : wg) + ((size_t)t.e * rpe + (active ? r : 0)) * row_bytes;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *cols = lds + tab_bytes<WT>();
    float *hbuf = reinterpret_cast<float *>(cols + (size_t)MC * col_bytes); // [MC][32]
    u32 *bad = reinterpret_cast<u32 *>(hbuf + MC * 32);                      // [MC]: entry names no slot
    for (int c0 = 0; c0 < (PASSES ? t.m : 1); c0 += MC) { // one pass, but for a tile wider than MC under PASSES
        const int mc = !PASSES ? t.m : t.m - c0 < MC ? t.m - c0 : MC;
        if (PASSES) __syncthreads(); // s_entry is written; the pass before is done with cols, hbuf and bad
        if (PASSES && c0) preload<WT, U>(b, wrow, q);
        if (tid < MC) {
            const u32 s = tid < mc ? (PASSES ? s_entry[c0 + tid] : t.entry) : 0;
            const bool none = tid < mc && (s >= n_slots || (int)(s / slots_per_col) >= act_cols);
            if (none) bm_raise(fault, layer, kSiteExpertId);
            bad[tid] = none ? 0xffffffffu : s / slots_per_col;
        }
        __syncthreads();
        stage_tile_cols(cols, act, col_bytes, mc, [&](int c) { return bad[c] == 0xffffffffu ? 0 : (int)bad[c]; });
        __syncthreads();
        float v[MC];
        row_dot<WT, U, NB, MC>(b, wrow, cols, col_bytes, mc, n, q, tb, v, NoTap{});
#pragma unroll
        for (int c = 0; c < MC; c++) {
            float hv = swiglu_of_pair(c < mc ? v[c] : 0.0f, which, rule, fault, layer);
            if (c < mc) {
                if (bad[c] == 0xffffffffu) hv = bm_bits_f32(0x7fc00000u);
                if (h && active && (tid & 7) == 0) h[(size_t)(t.j + c0 + c) * rpe + r] = hv;
                if (act_h && (tid & 7) == 0) hbuf[c * 32 + (tid >> 3)] = hv;
            }
        }
        if (act_h) { // rpe is a multiple of 256 here, so every row of the block is live
            __syncthreads();
            const int c = tid >> 5; // half wave c: column c
            if (c < mc)
                quantize_h_block(hbuf + c * 32, act_h + (size_t)(t.j + c0 + c) * nb_h * BM_Q82_SB_EXT, nb_h, rb, tid & 31, fault,
                                 layer);
        }
    }
}

// crates/gpu/src/kquant/tiles.rs:120-190 GemvTiles: workgroup = tile x 64 rows (a quad a row); entry j + c reads
// column j + c of act and writes row r of its slot order[j + c]. An entry that names no slot raises ExpertId.
// by_slot: the columns of act lie in slot order instead (entry j + c reads column order[j + c]): what a per-slot gate . up launch
// leaves, so a step can take that launch for gate . up and this one for down.
template <int WT, int U, int NB, int MC, bool PASSES>
__global__ __launch_bounds__(256) void k_gemv_tiles(const uint8_t *w, u32 n_experts, int nb, const uint8_t *act,
                                                    const u32 *order, const u32 *start, const u32 *tiles, u32 n_slots,
                                                    u32 cap, int rpe, float *y, int m_lo, int by_slot, u32 *fault, u32 layer) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, q = tid & 3;
    Tile t;
    if (!tile_of_block(tiles, start, order, n_experts, n_slots, cap, &t, fault, layer)) return;
    if (!PASSES && (t.m <= m_lo || t.m > MC)) return;
    __shared__ u32 s_entry[kTileCols];
    if (PASSES && tid < kTileCols) s_entry[tid] = t.entry;
    const int r = t.row_block * 64 + (tid >> 2);
    const bool active = r < rpe;
    const int n = NB > 0 ? NB : nb;
    const int col_bytes = bm_act_col_bytes<WT>(n);
    const size_t row_bytes = (size_t)n * bm_block_bytes<WT>();
    const uint8_t *wrow = w + ((size_t)t.e * rpe + (active ? r : 0)) * row_bytes;
    Blk<WT> b[U];
    preload<WT, U>(b, wrow, q);
    const Iq2Tables tb = stage_tables<WT>(lds);
    uint8_t *cols = lds + tab_bytes<WT>();
    u32 *slot_of = reinterpret_cast<u32 *>(cols + (size_t)MC * col_bytes); // [MC]
    for (int c0 = 0; c0 < (PASSES ? t.m : 1); c0 += MC) { // one pass, but for a tile wider than MC under PASSES
        const int mc = !PASSES ? t.m : t.m - c0 < MC ? t.m - c0 : MC;
        if (PASSES) __syncthreads(); // s_entry is written; the pass before is done with cols and slot_of
        if (PASSES && c0) preload<WT, U>(b, wrow, q);
        if (tid < MC) {
            const u32 s = tid < mc ? (PASSES ? s_entry[c0 + tid] : t.entry) : 0;
            if (tid < mc && s >= n_slots && t.row_block == 0) bm_raise(fault, layer, kSiteExpertId);
            slot_of[tid] = s;
        }
        if (by_slot) {
            __syncthreads(); // slot_of is written
            for (int c = 0; c < mc; c++)
                stage_bytes(cols + (size_t)c * col_bytes, act + (size_t)(slot_of[c] < n_slots ? slot_of[c] : 0) * col_bytes, col_bytes);
        } else {
            stage_bytes(cols, act + (size_t)(t.j + c0) * col_bytes, mc * col_bytes); // the tile's columns lie side by side
        }
        __syncthreads();
        float v[MC];
        row_dot<WT, U, NB, MC>(b, wrow, cols, col_bytes, mc, n, q, tb, v, NoTap{});
        if (q == 0 && active) {
#pragma unroll
            for (int c = 0; c < MC; c++)
                if (c < mc && slot_of[c] < n_slots) y[(size_t)slot_of[c] * rpe + r] = v[c];
        }
    }
}

// ------------------------------------------------------------------------------------------------ launchers

static size_t tiles_lds_of(int wtype, int k, int cols) {
    return tab_bytes_rt(wtype) + (size_t)cols * act_col_bytes(wtype, k) + (size_t)cols * 32 * sizeof(float) + cols * sizeof(u32);
}
size_t tiles_lds(int wtype, int k) {
    const size_t lds = tiles_lds_of(wtype, k, kTileCols);
    return lds <= (size_t)kMaxLds ? lds : 0;
}

// Eight columns of a long row take most of a CU's LDS (IQ2_XXS at 7168 values: 66 KB, two workgroups a CU), and with
// few tokens over many experts most tiles hold one or two slots. Past kTileSplitLds a tile launch therefore goes as two:
// one with LDS for two columns takes the tiles of up to two slots at several times the occupancy, one with LDS for
// eight takes the rest; a workgroup whose tile is the other launch's returns at once. With no more than two slots an
// expert of the stack on average nearly every tile is narrow, and the narrow launch alone takes them all, a wider tile
// in passes of two columns: one launch instead of two. Values do not depend on the width: every column is its own row dot.
constexpr size_t kTileSplitLds = 40 * 1024;
constexpr int kTileNarrow = 2;
static bool tile_widths_split(int wtype, int k) { return tiles_lds_of(wtype, k, kTileCols) > kTileSplitLds; }
static bool tiles_mostly_narrow(int n_slots, int n_experts) { return n_slots <= kTileNarrow * n_experts; }

hipError_t gate_up_tiles(const Launch &L, int wtype, const uint8_t *wg, const uint8_t *wu, int n_experts, int k,
                         const uint8_t *act, int act_cols, const uint32_t *order, const uint32_t *start,
                         const uint32_t *tiles_dev, int n_slots, int rows_per_expert, int slots_per_col, float *h,
                         uint8_t *act_h) {
    const int nb = k / 256, rpe = rows_per_expert;
    const bool split = tile_widths_split(wtype, k), narrow = tiles_mostly_narrow(n_slots, n_experts);
    const u32 cap = (u32)tile_cap(n_slots, n_experts);
    const unsigned grid = cap * (unsigned)((rpe + 31) / 32);
#define BM_TILE_LAUNCH(MC, M_LO, PASSES)                                                                               \
    {                                                                                                                  \
        const size_t lds = tiles_lds_of(wtype, k, MC);                                                                 \
        auto kern = k_gate_up_tiles<WT, U, NB, MC, PASSES>;                                                                    \
        hipError_t e = allow_lds(kern, lds);                                                                           \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, wg, wu, (u32)n_experts, nb, act, act_cols,      \
                           order, start, tiles_dev, (u32)n_slots, cap, rpe, slots_per_col, h, act_h, M_LO, L.rule,     \
                           L.fault, L.layer);                                                                          \
    }
#define CALL_BODY                                                                                                      \
    if (split && narrow) BM_TILE_LAUNCH(kTileNarrow, 0, true)                                                          \
    else {                                                                                                             \
        if (split) BM_TILE_LAUNCH(kTileNarrow, 0, false)                                                               \
        BM_TILE_LAUNCH(kTileCols, split ? kTileNarrow : 0, false)                                                      \
    }
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
#undef BM_TILE_LAUNCH
    return hipGetLastError();
}

hipError_t gemv_tiles(const Launch &L, int wtype, const uint8_t *w, int n_experts, int k, const uint8_t *act,
                      const uint32_t *order, const uint32_t *start, const uint32_t *tiles_dev, int n_slots,
                      int rows_per_expert, float *y, bool by_slot) {
    const int nb = k / 256, rpe = rows_per_expert;
    const bool split = tile_widths_split(wtype, k), narrow = tiles_mostly_narrow(n_slots, n_experts);
    const u32 cap = (u32)tile_cap(n_slots, n_experts);
    const unsigned grid = cap * (unsigned)((rpe + 63) / 64);
#define BM_TILE_LAUNCH(MC, M_LO, PASSES)                                                                               \
    {                                                                                                                  \
        const size_t lds = tiles_lds_of(wtype, k, MC);                                                                 \
        auto kern = k_gemv_tiles<WT, U, NB, MC, PASSES>;                                                                       \
        hipError_t e = allow_lds(kern, lds);                                                                           \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, w, (u32)n_experts, nb, act, order, start,       \
                           tiles_dev, (u32)n_slots, cap, rpe, y, M_LO, by_slot ? 1 : 0, L.fault, L.layer);             \
    }
#define CALL_BODY                                                                                                      \
    if (split && narrow) BM_TILE_LAUNCH(kTileNarrow, 0, true)                                                          \
    else {                                                                                                             \
        if (split) BM_TILE_LAUNCH(kTileNarrow, 0, false)                                                               \
        BM_TILE_LAUNCH(kTileCols, split ? kTileNarrow : 0, false)                                                      \
    }
    BM_DISPATCH(wtype, nb)
#undef CALL_BODY
#undef BM_TILE_LAUNCH
    return hipGetLastError();
}

} // namespace bmk
