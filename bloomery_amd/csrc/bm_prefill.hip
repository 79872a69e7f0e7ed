// Prefill: the grouped expert GEMM over a route table, on the int8 matrix cores, and the SwiGLU quantizer between
// a gate/up pair and its down (crates/gpu/src/gemm/mod.rs:1-50).
//
// The route table is the reference's (crates/gpu/src/gemm/route.rs:1-60,109-125): `cols` lists the slots grouped by
// expert, ascending slot order inside an expert, the refused slots (an id past the stack) at its end; `tiles` holds
// a pair of words a tile, (expert, first index | length << 16), tiles of at most 64 slots; `n_tiles` = {tile count,
// refused count}.
//
// The GEMM's numbers are the decode path's, bit for bit: every (row, slot) value is the one-column row dot of
// bm_device.hpp. The integer sums of each 16-value group come out of v_mfma_i32_16x16x32_i8 (16 rows x 16 slots,
// exact; the other half of the 32 values zeroed on the weight side), and each enters the f32 accumulator of the CPU path's lane that
// owns it, in the CPU path's order (crates/qdot/src/lib.rs:4363-4447 Q4_K, :4776-4874 Q6_K): eight accumulators a
// value, the min term first, then the groups in increasing k, and the closing sum (t0 + t2) + (t1 + t3).
// Activation scales come per 32 values in this form, so every group's sum is scaled on the vector ALU before it is
// added: three operations a (row, slot, group) against one matrix instruction per 1024 of them. The kernel is bound
// by that arithmetic, not by the matrix cores.
#include <type_traits>

#include "bm_gemm.hpp"

namespace bmk {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kRouteThreads = 1024;

int gemm_max_tiles(int n_slots, int n_experts) { // crates/gpu/src/gemm/route.rs:55-57
    return n_slots / kGemmBN + (n_experts < n_slots ? n_experts : n_slots);
}

// ------------------------------------------------------------------------------------------------ route

// The slots listed by expert in ascending slot order, bucket n_experts collecting the refused ones at the list's end
// (group_slots_part: as many workgroups as the list has parts, each placing its part; one workgroup on a single compute
// unit took 23 us over 16384 slots, bound by that unit's instruction rate and by lanes queueing on a popular expert's
// counter); one workgroup more places nothing and writes the tiles, an expert's run cut into runs of at most 64. A slot served elsewhere (id 0xffffffff, crates/gpu/src/kquant/sel.rs:22-28) is not
// listed and raises nothing: the list is that many entries shorter, the entries past it hold 0xffffffff, and n_tiles[2]
// counts them.
struct RouteLds {
    GroupLds g;
    u32 off[kGroupBuckets];
};
// With `x`: behind the table's workgroups (route_blocks of them) further ones quantize m rows of k f32 values into `act`,
// the column form picked by q8k (Q8_K: a wave a 256-value block; Q8_2_X4: eight values a thread): the prefill step's two
// first launches, which depend on nothing of each other, as one.
__global__ __launch_bounds__(kRouteThreads) void k_route(const u32 *ids, u32 n_slots, u32 n_experts, u32 *cols,
                                                         u32 *tiles, u32 *n_tiles, u32 route_blocks, const float *x, int m, int k,
                                                         int q8k, uint8_t *act, u32 *fault, u32 layer) {
    if (blockIdx.x >= route_blocks) {
        const u32 qb = blockIdx.x - route_blocks;
        if (q8k) {
            const int b = (int)qb * 16 + (int)(threadIdx.x >> 6), lane = (int)(threadIdx.x & 63);
            if (b >= m * (k / 256)) return; // whole waves leave
            q8k_wave_block(*reinterpret_cast<const float4 *>(x + (size_t)b * 256 + 4 * lane), act + (size_t)b * BM_Q8K_STRIDE, lane, fault, layer);
        } else {
            const long at = ((long)qb * kRouteThreads + threadIdx.x) * 8;
            if (at >= (long)m * k) return; // whole quads leave: a block is 32 values, k a multiple of 256
            const int col = (int)(at / k), o = (int)(at % k);
            const float4 a = *reinterpret_cast<const float4 *>(x + at), b = *reinterpret_cast<const float4 *>(x + at + 4);
            const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            q82_quad8(v, act + (size_t)col * (k / 256) * BM_Q82_SB_EXT, k / 256, o >> 5, threadIdx.x & 3, fault, layer);
        }
        return;
    }
    __shared__ RouteLds lds;
    GroupLds &g = lds.g;
    const u32 tid = threadIdx.x;
    group_slots_part(g, lds.off, n_slots, n_experts + 1, blockIdx.x, cols, [&](u32 s) {
        const u32 id = ids[s];
        return id < n_experts ? id : id == 0xffffffffu ? kNoBucket : n_experts;
    });
    if (blockIdx.x + 1 != route_blocks) return;
    const u32 listed = g.base[n_experts + 1];
    for (u32 i = listed + tid; i < n_slots; i += kRouteThreads) cols[i] = 0xffffffffu;
    u32 j0 = 0, j1 = 0;
    if (tid < n_experts) {
        j0 = g.base[tid];
        j1 = g.base[tid + 1];
    }
    u32 total;
    u32 t = block_scan_1024((j1 - j0 + kGemmBN - 1) / kGemmBN, g.scan, &total);
    for (u32 j = j0; j < j1; j += kGemmBN, t++) {
        const u32 len = j1 - j < (u32)kGemmBN ? j1 - j : (u32)kGemmBN;
        tiles[2 * t] = tid;
        tiles[2 * t + 1] = j | (len << 16);
    }
    if (tid == 0) {
        const u32 refused = g.base[n_experts + 1] - g.base[n_experts];
        if (refused) bm_raise(fault, layer, kSiteExpertId);
        n_tiles[0] = total;
        n_tiles[1] = refused;
        n_tiles[2] = n_slots - listed;
    }
}

hipError_t route(const Launch &L, const uint32_t *ids, int n_slots, int n_experts, uint32_t *cols, uint32_t *tiles_out,
                 uint32_t *n_tiles, int wtype, const float *x, int m, int k, uint8_t *act) {
    const u32 route_blocks = group_parts((u32)n_slots, (u32)n_experts + 1) + 1;
    u32 quant_blocks = 0;
    const bool q8k = x && bm_takes_q8k(wtype);
    if (x) {
        if (k % 256 != 0 || (reinterpret_cast<uintptr_t>(x) & 15) != 0) return hipErrorInvalidValue;
        quant_blocks = q8k ? (u32)((m * (k / 256) + 15) / 16) : (u32)(((long)m * k + 8 * kRouteThreads - 1) / (8 * kRouteThreads));
    }
    hipLaunchKernelGGL(k_route, dim3(route_blocks + quant_blocks), dim3(kRouteThreads), 0, L.stream, ids, (u32)n_slots, (u32)n_experts,
                       cols, tiles_out, n_tiles, route_blocks, x, m, k, q8k ? 1 : 0, act, L.fault, L.layer);
    return hipGetLastError();
}

// --------------------------------------------------------------------------------------- SwiGLU + quantize

// crates/gpu/src/gemm/swiglu.rs:46-58 in the CPU path's rules: column c of act = Q8_2_X4(swiglu(g, u)) over the k
// values g[c * k ..], u[c * k ..]. One half wave a 32-value block.
// `sel` (optional; crates/gpu/src/gemm/swiglu.rs:96-140 enqueue_swiglu_act_quant_sel): column c belongs to slot c; a slot
// served elsewhere (id 0xffffffff) keeps its column as it stands and raises nothing, any other id at or past n_experts
// raises ExpertId with nothing stored.
__device__ __forceinline__ bool swiglu_column_skipped(const u32 *sel, u32 n_experts, int col, bool first, u32 *fault, u32 layer) {
    if (!sel) return false;
    const u32 id = sel[col];
    if (id < n_experts) return false;
    if (id != 0xffffffffu && first) bm_raise(fault, layer, kSiteExpertId);
    return true;
}

__global__ __launch_bounds__(256) void k_swiglu_quant(const float *g, const float *u, int m, int k, uint8_t *act,
                                                      GateRule rule, const u32 *sel, u32 n_experts, u32 *fault, u32 layer) {
    const int bpc = k / 32;
    const long gblk = (long)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (gblk >= (long)m * bpc) return;
    const int col = (int)(gblk / bpc), blk = (int)(gblk % bpc), lane32 = threadIdx.x & 31;
    if (swiglu_column_skipped(sel, n_experts, col, blk == 0 && lane32 == 0, fault, layer)) return; // uniform over the half wave
    const size_t at = (size_t)col * k + 32 * blk + lane32;
    bool odd;
    const float v = bm_gate_rule(rule.act, rule.limit, g[at], u[at], odd);
    if (odd) bm_raise(fault, layer, kSiteF32Product);
    Q82Head hd;
    int s16;
    const int code = q82_block(v, &hd, &s16);
    if (hd.bad && lane32 == 0) bm_raise(fault, layer, kSiteQuantColumn);
    q82_store(act + (size_t)col * (k / 256) * BM_Q82_SB_EXT, k / 256, blk, lane32, code, hd, s16);
}

// The same into Q8_K columns, for a down stack that dots against those (IQ2_XXS, ...): one workgroup a 256-value block.
__global__ __launch_bounds__(256) void k_swiglu_quant_q8k(const float *g, const float *u, int m, int k, uint8_t *act,
                                                          GateRule rule, const u32 *sel, u32 n_experts, u32 *fault, u32 layer) {
    const int bpc = k / 256;
    const int col = blockIdx.x / bpc, blk = blockIdx.x % bpc;
    if (swiglu_column_skipped(sel, n_experts, col, blk == 0 && threadIdx.x == 0, fault, layer)) return; // uniform over the workgroup
    const size_t at = (size_t)col * k + 256 * blk + threadIdx.x;
    bool odd;
    const float v = bm_gate_rule(rule.act, rule.limit, g[at], u[at], odd);
    if (odd) bm_raise(fault, layer, kSiteF32Product);
    q8k_block_by_workgroup(v, act + ((size_t)col * bpc + blk) * BM_Q8K_STRIDE, fault, layer);
}

// The Q8_2_X4 form with eight values a thread, a block a quad of lanes: two 16-byte loads of each input a thread.
__global__ __launch_bounds__(256) void k_swiglu_quant_wide(const float *g, const float *u, int m, int k, uint8_t *act,
                                                           GateRule rule, const u32 *sel, u32 n_experts, u32 *fault, u32 layer) {
    const long at = ((long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (at >= (long)m * k) return;
    const int col = (int)(at / k), o = (int)(at % k);
    if (swiglu_column_skipped(sel, n_experts, col, o == 0, fault, layer)) return; // uniform over a block's quad of lanes
    const float4 g0 = *reinterpret_cast<const float4 *>(g + at), g1 = *reinterpret_cast<const float4 *>(g + at + 4);
    const float4 u0 = *reinterpret_cast<const float4 *>(u + at), u1 = *reinterpret_cast<const float4 *>(u + at + 4);
    const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
    const float uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
    float v[8];
    bool any_odd = false;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        bool odd;
        v[i] = bm_gate_rule(rule.act, rule.limit, gv[i], uv[i], odd);
        any_odd |= odd;
    }
    if (any_odd) bm_raise(fault, layer, kSiteF32Product);
    q82_quad8(v, act + (size_t)col * (k / 256) * BM_Q82_SB_EXT, k / 256, o >> 5, threadIdx.x & 3, fault, layer);
}

hipError_t swiglu_quant(const Launch &L, const float *g, const float *u, int m, int k, uint8_t *act, bool q8k, const uint32_t *sel,
                        uint32_t n_experts) {
    if (!q8k && (((uintptr_t)g | (uintptr_t)u) & 15) == 0) {
        const long threads = (long)m * k / 8;
        hipLaunchKernelGGL(k_swiglu_quant_wide, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, L.stream, g, u, m, k, act,
                           L.rule, sel, n_experts, L.fault, L.layer);
        return hipGetLastError();
    }
    if (q8k) {
        hipLaunchKernelGGL(k_swiglu_quant_q8k, dim3((unsigned)(m * (k / 256))), dim3(256), 0, L.stream, g, u, m, k, act, L.rule,
                           sel, n_experts, L.fault, L.layer);
        return hipGetLastError();
    }
    const long blocks = (long)m * (k / 32);
    hipLaunchKernelGGL(k_swiglu_quant, dim3((unsigned)((blocks + 7) / 8)), dim3(256), 0, L.stream, g, u, m, k, act,
                       L.rule, sel, n_experts, L.fault, L.layer);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------- GEMM

// LDS of one workgroup: a super-block of the tile's 64 activation columns and of the slab's 64 weight rows, and the
// rows' scale products. Strides are padded off the 128-byte bank period.
constexpr int kActSb = BM_Q82_SB_REF + 64;   // a column's super-block: its two groups and its (d8, d8 * isum) pairs
constexpr int kActStride = kActSb + 8;       // 360

// (q6 - 32) of four codes a word, as signed bytes: q6 in 0..63.
__device__ __forceinline__ u32 q6_minus_32(u32 q) {
    const u32 t = q ^ 0x20202020u;        // q >= 32: q - 32; q < 32: q + 32
    const u32 m = ~q & 0x20202020u;       // the bytes that went up: they want -64, the two top bits
    return t | (m << 1) | (m << 2);
}

// LDS of the exact kernel, two buffers of: the part's activation columns (a super-block each), the slab's 64 weight
// rows unpacked to a signed byte a code (Q4_K 0..15, Q6_K q6 - 32), so the arithmetic reads matrix operands as they
// are, and the rows' 16 x 64 scale products. A page of zeros stands in for the half of an operand that must not count.
// Strides: an operand read is 8 bytes a lane, served sixteen lanes at a time, the sixteen a wave's rows (or slots) at
// one piece of a block: a stride of 8 x an odd number puts them on sixteen different bank pairs (rows 8 x 33, columns
// 8 x 45). Strides of 16-byte multiples, which would let the staging store 16 bytes a lane, measured slower: the reads
// then collide in pairs.
constexpr int kRowStride = 256 + 8;
constexpr int kColStride = kActStride; // 360
constexpr int kRsStride = 68; // floats a row of the 16 x 64 scale products
constexpr int kZeroPage = 256;
__host__ __device__ constexpr size_t gemm_exact_buf_bytes(int slots) {
    return (size_t)slots * kColStride + (size_t)kGemmBM * kRowStride + 16 * kRsStride * sizeof(float);
}
__host__ __device__ constexpr size_t gemm_exact_lds_bytes(int slots) {
    return sizeof(GemmLds) + kZeroPage + 2 * gemm_exact_buf_bytes(slots);
}

// Byte j (0..11) of the twelve scale bytes a Q4_K block holds after d and dmin, the bytes given as three words.
__device__ __forceinline__ u32 q4k_scale_byte(u32 y, u32 z, u32 w, int j) {
    const unsigned long long yz = ((unsigned long long)z << 32) | y;
    const u32 a = (u32)(yz >> ((8 * j) & 63)), b = w >> ((8 * j) & 31);
    return (j < 8 ? a : b) & 0xffu;
}

// A workgroup of 4 CH waves takes 16 T CH slots of a tile (all 64, or a part of it: a tile's parts are workgroups of
// their own) and a slab of 64 rows. Wave w works on rows 16 * (w & 3) .. and slots 16 T * (w >> 2) ..: T 16 x 16
// products a 16-value group. v_mfma_i32_16x16x32_i8 sums over 32 values, lane / 16 = k / 8; a 16-value half comes out
// of it when the lanes of the other half hand in zeros: those lanes read their weight operand from the zero page (an
// address picked once, no instruction a product). 4 T results a lane, 32 T accumulators.
// The next super-block is loaded to registers before the arithmetic on the present one and stored to the other
// buffer after it: one barrier a super-block. Parts of 32 slots put two workgroups on a CU, and one's loads, LDS
// stores and barrier then run under the other's arithmetic.
template <int WT, int T, int CH>
__global__ __launch_bounds__(256 * CH) void k_gemm(const uint8_t *w, int rpe, int nb, const uint8_t *act, const u32 *cols,
                                                 const u32 *tiles, const u32 *n_tiles, u32 n_units, u32 slot_div,
                                                 u32 n_slots, float *y) {
    constexpr int kSlots = 16 * T * CH, kParts = kGemmBN / kSlots, kThreads = 256 * CH;
    static_assert(kThreads == 8 * kGemmBM, "a thread a (row, eighth of the row's codes)");
    constexpr size_t kBuf = gemm_exact_buf_bytes(kSlots);
    constexpr int kWtsAt = kSlots * kColStride, kRsAt = kWtsAt + kGemmBM * kRowStride;
    extern __shared__ __align__(16) uint8_t lds[];
    GemmLds *tab = reinterpret_cast<GemmLds *>(lds);
    uint8_t *zeros = lds + sizeof(GemmLds);
    uint8_t *buf0 = zeros + kZeroPage;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const u32 g = tile_of_block(blockIdx.x, n_units); // a unit: a row slab and a part of the tile
    const u32 unit = slab_of_block(blockIdx.x, n_units);
    const int row0 = (int)(unit / kParts) * kGemmBM, part0 = (int)(unit % kParts) * kSlots;
    const u32 count = n_tiles[0];
    if (g > count) return;
    if (g == count) { // the refused slots' rows: NaN (crates/gpu/src/gemm/grouped.rs:2283-2287)
        const u32 refused = part0 == 0 ? n_tiles[1] : 0u;
        for (u32 i = tid; i < refused * kGemmBM; i += blockDim.x) {
            const u32 s = cols[n_slots - n_tiles[2] - refused + i / kGemmBM];
            const int r = row0 + (int)(i % kGemmBM);
            if (r < rpe) y[(size_t)s * rpe + r] = bm_bits_f32(0x7fc00000u);
        }
        return;
    }
    const u32 e = tiles[2 * g], word = tiles[2 * g + 1];
    const int start = (int)(word & 0xffffu) + part0, len = (int)(word >> 16) - part0;
    if (len <= 0) return; // the tile ends before this part
    if (tid < kSlots) {
        const u32 s = cols[start + (tid < len ? tid : 0)];
        tab->slot[tid] = s;
        tab->col[tid] = s / slot_div;
    }
    if (tid < kZeroPage / 4) reinterpret_cast<u32 *>(zeros)[tid] = 0u;
    __syncthreads();
    constexpr int kBlock = bm_block_bytes<WT>();
    constexpr bool kQ45 = WT == BM_Q4K || WT == BM_Q5K; // one walk: Q5_K is Q4_K with a fifth bit a code
    constexpr int kCodesAt = WT == BM_Q5K ? 48 : 16;    // where a Q4_K / Q5_K block's nibbles start
    const u32 row_bytes = (u32)nb * kBlock, col_bytes = (u32)nb * BM_Q82_SB_EXT;

    // What a thread stages of every super-block: kActLoads 16-byte chunks of the activations (a column's super-block
    // is 18 chunks of codes and 4 of (d8, d8 * isum) pairs), 16 code bytes of row tid / 8 (Q6_K: with the 16 bytes of
    // high bits that go with them), and two of that row's sixteen scale products. The sources are fixed but for the
    // super-block's offset: 32-bit offsets from the activations and from the expert's rows.
    constexpr int kAc = kActSb / 16; // 22
    constexpr int kActLoads = (kSlots * kAc + kThreads - 1) / kThreads;
    u32 src_a[kActLoads], step_a[kActLoads]; // a chunk's offset in super-block 0 and its step a super-block
    int dst_a[kActLoads];
#pragma unroll
    for (int t = 0; t < kActLoads; t++) {
        int c = t * kThreads + tid;
        c = c < kSlots * kAc ? c : kSlots * kAc - 1;
        const int n = c / kAc, k = c % kAc;
        const u32 colp = tab->col[n] * col_bytes;
        // chunk k < 18: the codes, a step of 288 a super-block; else the pairs behind all the codes, a step of 64
        src_a[t] = k < 18 ? colp + 16 * k : colp + (u32)nb * BM_Q82_SB_REF + 16 * (k - 18);
        step_a[t] = k < 18 ? BM_Q82_SB_REF : 64;
        dst_a[t] = n * kColStride + 16 * k;
    }
    const uint8_t *we = w + (size_t)e * rpe * row_bytes;
    const int wr = tid >> 3, pc = tid & 7; // the row and the eighth of its codes
    const u32 src_w = (u32)(row0 + wr < rpe ? row0 + wr : rpe - 1) * row_bytes;
    uint4 ra[kActLoads], rw, rqh, rhd = make_uint4(0, 0, 0, 0);
    auto fetch = [&](int i) {
#pragma unroll
        for (int t = 0; t < kActLoads; t++) ra[t] = *reinterpret_cast<const uint4 *>(act + (src_a[t] + (u32)i * step_a[t]));
        const uint8_t *blk = we + (src_w + (u32)i * kBlock);
        if constexpr (kQ45) {
            rw = *reinterpret_cast<const uint4 *>(blk + kCodesAt + 16 * pc);
            if (pc == 0) rhd = *reinterpret_cast<const uint4 *>(blk); // d, dmin, the twelve scale bytes
            // Q5_K: value n's fifth bit is bit n / 32 of high byte n % 32 (crates/gguf/src/quant.rs:769-816); these
            // code bytes hold values 64 (pc / 2) + 16 (pc % 2) .. and the values 32 on
            if constexpr (WT == BM_Q5K) rqh = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * (pc & 1));
        } else { // half pc / 4: its ql bytes 16 (pc % 4) .. and the qh bytes that go with them
            rw = bm_ld16u(blk + 64 * (pc >> 2) + 16 * (pc & 3));
            rqh = bm_ld16u(blk + 128 + 32 * (pc >> 2) + 16 * (pc & 1));
            rhd.x = bm_ld2u(blk + 208);          // d
            rhd.y = bm_ld2u(blk + 192 + 2 * pc); // scales 2 pc, 2 pc + 1
        }
    };
    auto put16 = [](uint8_t *dst, u32 a, u32 b, u32 c, u32 d) {
        *reinterpret_cast<uint2 *>(dst) = make_uint2(a, b);
        *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(c, d);
    };
    auto stash = [&](uint8_t *buf) {
#pragma unroll
        for (int t = 0; t < kActLoads; t++)
            if (t * kThreads + tid < kSlots * kAc) put16(buf + dst_a[t], ra[t].x, ra[t].y, ra[t].z, ra[t].w);
        const u32 ml = 0x0f0f0f0fu;
        uint8_t *codes = buf + kWtsAt + wr * kRowStride;
        float *rs = reinterpret_cast<float *>(buf + kRsAt); // [16][kRsStride]
        if constexpr (kQ45) {
            // code bytes 16 pc ..: values 64 (pc / 2) + 16 (pc % 2) .. (low nibbles) and 32 on (high nibbles)
            uint8_t *dst = codes + 64 * (pc >> 1) + 16 * (pc & 1);
            if constexpr (WT == BM_Q5K) {
                const u32 one = 0x01010101u;
                const int s0 = 2 * (pc >> 1), s1 = s0 + 1; // the sub-blocks of the low and of the high nibbles
                put16(dst, (rw.x & ml) | (((rqh.x >> s0) & one) << 4), (rw.y & ml) | (((rqh.y >> s0) & one) << 4),
                      (rw.z & ml) | (((rqh.z >> s0) & one) << 4), (rw.w & ml) | (((rqh.w >> s0) & one) << 4));
                put16(dst + 32, ((rw.x >> 4) & ml) | (((rqh.x >> s1) & one) << 4), ((rw.y >> 4) & ml) | (((rqh.y >> s1) & one) << 4),
                      ((rw.z >> 4) & ml) | (((rqh.z >> s1) & one) << 4), ((rw.w >> 4) & ml) | (((rqh.w >> s1) & one) << 4));
            } else {
                put16(dst, rw.x & ml, rw.y & ml, rw.z & ml, rw.w & ml);
                put16(dst + 32, (rw.x >> 4) & ml, (rw.y >> 4) & ml, (rw.z >> 4) & ml, (rw.w >> 4) & ml);
            }
            // the row's header from the lane that read it; scale and min of sub-block pc
            // (crates/gguf/src/quant.rs:620-628 get_scale_min_k4)
            const int from = 4 * (lane & ~7);
            const u32 h0 = (u32)__builtin_amdgcn_ds_bpermute(from, (int)rhd.x), h1 = (u32)__builtin_amdgcn_ds_bpermute(from, (int)rhd.y),
                      h2 = (u32)__builtin_amdgcn_ds_bpermute(from, (int)rhd.z), h3 = (u32)__builtin_amdgcn_ds_bpermute(from, (int)rhd.w);
            const float d = bm_half_to_f32((unsigned short)(h0 & 0xffffu));
            const float dmin = bm_half_to_f32((unsigned short)(h0 >> 16));
            const u32 lo = q4k_scale_byte(h1, h2, h3, pc < 4 ? pc : pc + 4);     // pc < 4: sc[pc]; else sc[pc + 4]
            const u32 b4 = q4k_scale_byte(h1, h2, h3, pc < 4 ? pc + 4 : pc - 4); // pc < 4: sc[pc + 4]; else sc[pc - 4]
            const u32 b0 = q4k_scale_byte(h1, h2, h3, pc);                       // sc[pc]
            const u32 scv = pc < 4 ? (lo & 63u) : ((lo & 15u) | ((b4 >> 6) << 4));
            const u32 mv = pc < 4 ? (b4 & 63u) : ((lo >> 4) | ((b0 >> 6) << 4));
            rs[pc * kRsStride + wr] = d * (float)scv;
            rs[(8 + pc) * kRsStride + wr] = -(dmin * (float)mv);
        } else {
            // low nibbles are quarter (pc % 4) / 2 of the half, high nibbles that quarter + 2; values 16 (pc % 2) ..
#pragma unroll
            for (int hn = 0; hn < 2; hn++) {
                const int a4 = ((pc & 3) >> 1) + 2 * hn, ns = 4 * hn, hs = 2 * a4;
                uint8_t *dst = codes + 128 * (pc >> 2) + 32 * a4 + 16 * (pc & 1);
                const u32 mh = 0x03030303u;
                put16(dst, q6_minus_32(((rw.x >> ns) & ml) | (((rqh.x >> hs) & mh) << 4)),
                      q6_minus_32(((rw.y >> ns) & ml) | (((rqh.y >> hs) & mh) << 4)),
                      q6_minus_32(((rw.z >> ns) & ml) | (((rqh.z >> hs) & mh) << 4)),
                      q6_minus_32(((rw.w >> ns) & ml) | (((rqh.w >> hs) & mh) << 4)));
            }
            const float d = bm_half_to_f32((unsigned short)rhd.x);
            rs[(2 * pc) * kRsStride + wr] = d * (float)(int)(signed char)(rhd.y & 0xffu);
            rs[(2 * pc + 1) * kRsStride + wr] = d * (float)(int)(signed char)(rhd.y >> 8);
        }
    };
    // this lane in its wave's 16 x 16 products: operand row / slot lane % 16, values 8 * (lane / 16) .. + 8 of a
    // 32-value block; its four results of each product are rows 4 * (lane / 16) + v of slot lane % 16
    const int rg = wv & 3, ch = wv >> 2, l16 = lane & 15, kg = lane >> 4;
    int my_act[T];
#pragma unroll
    for (int t = 0; t < T; t++) my_act[t] = (16 * T * ch + 16 * t + l16) * kColStride;
    // the weight operand of half h of a block: this lane's eight codes when they are of that half, else zeros
    // (offsets from the buffer; the zero page lies below both buffers)
    const int my_row = kWtsAt + (16 * rg + l16) * kRowStride + 8 * kg;
    const int rbase = 16 * rg + 4 * kg; // result v sits in row rbase + v of the slab
    const bool live = 16 * T * ch < len; // else none of this wave's slots is real
    float acc[T][4][8];
#pragma unroll
    for (int t = 0; t < T; t++)
#pragma unroll
        for (int v = 0; v < 4; v++)
#pragma unroll
            for (int l = 0; l < 8; l++) acc[t][v][l] = 0.0f;

    auto arithmetic = [&](const uint8_t *buf) __attribute__((always_inline)) {
        const float *rs = reinterpret_cast<const float *>(buf + kRsAt);
        const uint8_t *my_a[2] = {kg < 2 ? buf + my_row : zeros, kg < 2 ? zeros : buf + my_row};
        const float2 *pair[T]; // (d8, d8 * isum) a 32-block
#pragma unroll
        for (int t = 0; t < T; t++) pair[t] = reinterpret_cast<const float2 *>(buf + my_act[t] + BM_Q82_SB_REF);
        if constexpr (kQ45) {
            // the min terms first: accumulator l takes sub-block l's (crates/qdot/src/lib.rs:4389-4394)
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const float4 mn = *reinterpret_cast<const float4 *>(&rs[(8 + s) * kRsStride + rbase]);
#pragma unroll
                for (int t = 0; t < T; t++) {
                    const float my = pair[t][s].y;
                    acc[t][0][s] = fmaf(my, mn.x, acc[t][0][s]);
                    acc[t][1][s] = fmaf(my, mn.y, acc[t][1][s]);
                    acc[t][2][s] = fmaf(my, mn.z, acc[t][2][s]);
                    acc[t][3][s] = fmaf(my, mn.w, acc[t][3][s]);
                }
            }
        }
        if constexpr (T == 1) {
            // one product a 16-value group, sixteen a super-block: a group's matrix instruction is issued one group ahead
            // of the vector work on its sums, and a block's LDS operands are read two blocks ahead
            long a[2][2], b[2];
            float d8[2];
            float4 sv[2][2];
            v4i sum[2];
            auto rd = [&](int bk) {
#pragma unroll
                for (int h = 0; h < 2; h++) a[bk & 1][h] = *reinterpret_cast<const long *>(my_a[h] + 32 * bk);
                b[bk & 1] = *reinterpret_cast<const long *>(buf + my_act[0] + (bk >> 2) * BM_Q82X4_STRIDE + 16 + 32 * (bk & 3) + 8 * kg);
                d8[bk & 1] = pair[0][bk].x;
                sv[bk & 1][0] = *reinterpret_cast<const float4 *>(&rs[(kQ45 ? bk : 2 * bk) * kRsStride + rbase]);
                if constexpr (!kQ45) sv[bk & 1][1] = *reinterpret_cast<const float4 *>(&rs[(2 * bk + 1) * kRsStride + rbase]);
            };
            auto product = [&](int g) {
                const v4i z = {0, 0, 0, 0};
                sum[g & 1] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[(g >> 1) & 1][g & 1], b[(g >> 1) & 1], z, 0, 0, 0);
            };
            rd(0);
            rd(1);
            product(0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 16; g++) {
                const int bk = g >> 1, h = g & 1, l = 4 * h + (bk & 3);
                if (g + 1 < 16) product(g + 1);
                __builtin_amdgcn_sched_barrier(0);
                // Q4_K, Q5_K: one scale a block; Q6_K: one a group (crates/qdot/src/lib.rs:4403-4440, :4794-4809)
                const float4 r = sv[bk & 1][kQ45 ? 0 : h];
                const float dc = d8[bk & 1];
                acc[0][0][l] = fmaf(r.x * dc, (float)sum[g & 1][0], acc[0][0][l]);
                acc[0][1][l] = fmaf(r.y * dc, (float)sum[g & 1][1], acc[0][1][l]);
                acc[0][2][l] = fmaf(r.z * dc, (float)sum[g & 1][2], acc[0][2][l]);
                acc[0][3][l] = fmaf(r.w * dc, (float)sum[g & 1][3], acc[0][3][l]);
                __builtin_amdgcn_sched_barrier(0);
                if (h == 1 && bk + 2 < 8) rd(bk + 2);
            }
            return;
        }
#pragma unroll
        for (int bk = 0; bk < 8; bk++) { // 32-value block bk of the super-block: groups 2 bk (half 0) and 2 bk + 1
            long a[2], b[T];
#pragma unroll
            for (int h = 0; h < 2; h++) a[h] = *reinterpret_cast<const long *>(my_a[h] + 32 * bk);
            float d8[T];
#pragma unroll
            for (int t = 0; t < T; t++) {
                b[t] = *reinterpret_cast<const long *>(buf + my_act[t] + (bk >> 2) * BM_Q82X4_STRIDE + 16 + 32 * (bk & 3) + 8 * kg);
                d8[t] = pair[t][bk].x;
            }
#pragma unroll
            for (int h = 0; h < 2; h++) {
                // Q4_K, Q5_K: one scale a block; Q6_K: one a group (crates/qdot/src/lib.rs:4403-4440, :4794-4809)
                const float4 sv = *reinterpret_cast<const float4 *>(&rs[(kQ45 ? bk : 2 * bk + h) * kRsStride + rbase]);
                const int l = 4 * h + (bk & 3);
#pragma unroll
                for (int t = 0; t < T; t++) {
                    const v4i z = {0, 0, 0, 0};
                    const v4i sum = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[h], b[t], z, 0, 0, 0);
                    acc[t][0][l] = fmaf(sv.x * d8[t], (float)sum[0], acc[t][0][l]);
                    acc[t][1][l] = fmaf(sv.y * d8[t], (float)sum[1], acc[t][1][l]);
                    acc[t][2][l] = fmaf(sv.z * d8[t], (float)sum[2], acc[t][2][l]);
                    acc[t][3][l] = fmaf(sv.w * d8[t], (float)sum[3], acc[t][3][l]);
                }
            }
        }
    };

    fetch(0);
    stash(buf0);
    __syncthreads();
    for (int i = 0; i < nb; i++) {
        const bool more = i + 1 < nb;
        if (more) fetch(i + 1);
        if (live) arithmetic(buf0 + (size_t)(i & 1) * kBuf);
        // the other buffer's last readers passed the barrier that ended the super-block before this one
        if (more) stash(buf0 + (size_t)((i + 1) & 1) * kBuf);
        __syncthreads();
    }
    // the closing sum of the eight lanes (crates/qdot/src/lib.rs:4128 hsum_float_8's order) and the store
#pragma unroll
    for (int t = 0; t < T; t++) {
        const int n = 16 * T * ch + 16 * t + l16;
        if (n < len) {
            const size_t out = (size_t)tab->slot[n] * rpe + row0;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int r = rbase + v;
                const float t0 = acc[t][v][0] + acc[t][v][4], t1 = acc[t][v][1] + acc[t][v][5];
                const float t2 = acc[t][v][2] + acc[t][v][6], t3 = acc[t][v][3] + acc[t][v][7];
                if (row0 + r < rpe) y[out + r] = (t0 + t2) + (t1 + t3);
            }
        }
    }
}

// ------------------------------------------------------ one accumulator a value: whole-block matrix instructions

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// The tolerance mode (BM_GEMM_FAST). The integer sums are the exact ones, formed by matrix instructions whose K is
// exactly the span one scale covers, so no issued multiply is wasted:
//   Q4_K, Q5_K: a 32-value sub-block of a row against a 32-value block of a column is one v_mfma_i32_32x32x32_i8 over 32
//         rows and 32 slots; the min terms, sum over a super-block's eight sub-blocks of -(dmin m)[row] x (d8 isum)[slot],
//         are a product of two thin matrices and go to v_mfma_f32_32x32x2_f32 (four a super-block), into the same
//         accumulators;
//   Q6_K: a 16-value group, whose scale is its own, is one v_mfma_i32_32x32x16_i8.
// The product of a row's scale and a column's d8 for a whole 32 x 32 tile is an outer product, so it goes to the matrix
// cores too: v_mfma_f32_32x32x8_bf16_1k over K slots that hold the row scale as three bf16 pieces (8 + 8 + 8 bits: the
// f32 exactly) against the column's d8 (a bf16 value as it stands) in the same three slots. Each of the three products
// is exact in f32; their sum is the f32 product to within a rounding. Lanes 32 .. 63 carry K slots 4 .. 7: the row side
// reads a zero there.
// What is left for the vector ALU is two operations a (row, slot, unit): the integer to a float and the multiply-add into
// the one accumulator a value (the CPU path keeps eight and a fixed order: that is the exact mode; this one differs from
// it by f32 rounding only).
// A workgroup of eight waves takes 128 rows and a tile's 64 slots, a wave 32 x 32 of them. LDS holds one super-block: the
// columns' codes, the slab's codes unpacked to a signed byte each, and the scale operands; 72 KB and at most 128 registers,
// so two workgroups, four waves a SIMD, share a CU and fill each other's staging gaps and waits (a wave alone issues a
// vector instruction every five to six cycles, the SIMD takes one every four). The next super-block's global loads are in flight during the
// arithmetic on the present one. Inside a wave a unit's matrix instructions are issued one unit ahead of the vector work
// on their results, and its LDS operands are read two units ahead.
constexpr int kFastRows = 128;
constexpr int kFastThreads = 512;
constexpr int kFastRowLine = kFastRows + 4; // entries a line of the row tables ([unit][row]); entry kFastRows of a line holds zero
constexpr int kFastColLine = kGemmBN + 4;   // entries a line of the column tables ([block][slot])
// a row's or a column's 256 codes, padded so that the operand reads of consecutive rows fall on different banks: the
// reads are 16 bytes a lane for K = 32 and 8 bytes a lane for K = 16
template <int WT>
__host__ __device__ constexpr int fast_code_stride() {
    return WT == BM_Q6K ? 256 + 8 : 256 + 16;
}
template <int WT>
__host__ __device__ constexpr int fast_units() { // scaled units a super-block
    return WT == BM_Q6K ? 16 : 8;
}
template <int WT>
__host__ __device__ constexpr size_t fast_lds_bytes() {
    // codes of both sides; the columns' scale operands ([block][slot], 8 bytes) and d8 * isum; the rows' scale operands
    // ([unit][row], 8 bytes) and mins
    constexpr bool mins = WT != BM_Q6K;
    return sizeof(GemmLds) + (size_t)(kGemmBN + kFastRows) * fast_code_stride<WT>() + 8 * kFastColLine * (8 + (mins ? sizeof(float) : 0)) +
           (size_t)fast_units<WT>() * kFastRowLine * (8 + (mins ? sizeof(float) : 0));
}

__device__ __forceinline__ uint2 scale_operand_row(float v) {
    const u32 hi = bm_f32_bits(v) & 0xffff0000u;
    const float r1 = v - bm_bits_f32(hi);
    const u32 mid = bm_f32_bits(r1) & 0xffff0000u;
    const float r2 = r1 - bm_bits_f32(mid);
    return make_uint2((hi >> 16) | mid, bm_f32_bits(r2) >> 16);
}
__device__ __forceinline__ uint2 scale_operand_col(u32 d8_bits) {
    const u32 h = d8_bits >> 16;
    return make_uint2(h | (h << 16), h);
}
typedef short v4s __attribute__((ext_vector_type(4)));

template <int WT>
__global__ __launch_bounds__(kFastThreads, 2) void k_gemm_fast(const uint8_t *w, int rpe, int nb, const uint8_t *act, const u32 *cols,
                                                      const u32 *tiles, const u32 *n_tiles, u32 n_slabs, u32 slot_div,
                                                      u32 n_slots, float *y) {
    constexpr bool kQ45 = WT == BM_Q4K || WT == BM_Q5K;
    constexpr int kStride = fast_code_stride<WT>(), kUnitsSb = fast_units<WT>(), kBlock = bm_block_bytes<WT>();
    constexpr int kOp = kQ45 ? 16 : 8; // operand bytes a lane
    extern __shared__ __align__(16) uint8_t lds[];
    GemmLds *tab = reinterpret_cast<GemmLds *>(lds);
    uint8_t *a_codes = lds + sizeof(GemmLds);
    uint8_t *w_codes = a_codes + (size_t)kGemmBN * kStride;
    uint2 *d8_t = reinterpret_cast<uint2 *>(w_codes + (size_t)kFastRows * kStride); // [block][slot]
    uint2 *sv_t = d8_t + 8 * kFastColLine;                                           // [unit][row]
    float *my_t = reinterpret_cast<float *>(sv_t + kUnitsSb * kFastRowLine);         // Q4_K, Q5_K only, as is mn_t
    float *mn_t = my_t + 8 * kFastColLine;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const u32 g = tile_of_block(blockIdx.x, n_slabs);
    const int row0 = (int)slab_of_block(blockIdx.x, n_slabs) * kFastRows;
    const u32 count = n_tiles[0];
    if (g > count) return;
    if (g == count) { // the refused slots' rows: NaN (crates/gpu/src/gemm/grouped.rs:2283-2287)
        const u32 refused = n_tiles[1];
        for (u32 i = tid; i < refused * kFastRows; i += kFastThreads) {
            const u32 s = cols[n_slots - n_tiles[2] - refused + i / kFastRows];
            const int r = row0 + (int)(i % kFastRows);
            if (r < rpe) y[(size_t)s * rpe + r] = bm_bits_f32(0x7fc00000u);
        }
        return;
    }
    const u32 e = tiles[2 * g], word = tiles[2 * g + 1];
    const int start = (int)(word & 0xffffu), len = (int)(word >> 16);
    if (tid < kGemmBN) {
        const u32 s = cols[start + (tid < len ? tid : 0)];
        tab->slot[tid] = s;
        tab->col[tid] = s / slot_div;
    }
    if (tid < kUnitsSb) sv_t[tid * kFastRowLine + kFastRows] = make_uint2(0u, 0u);
    __syncthreads();
    const u32 row_bytes = (u32)nb * kBlock, col_bytes = (u32)nb * BM_Q82_SB_EXT;
    // what this thread stages of every super-block:
    //   two 16-byte pieces of column codes (column tid / 16 + 32 j, piece tid % 16 of the sixteen: a column's
    //   super-block is two groups of 144 bytes whose first 16 are scales and sums, skipped here),
    //   one (d8, d8 * isum) pair (column tid / 8, block tid % 8),
    //   two 16-byte pieces of weight codes (row tid / 8 + 64 j, piece tid % 8 of the row's eight: eight consecutive lanes
    //   read 128 consecutive bytes),
    //   a quarter of a weight row's scales (row tid / 4)
    const int ac = tid >> 4, ap = tid & 15;
    u32 src_a[2];
#pragma unroll
    for (int j = 0; j < 2; j++) src_a[j] = tab->col[ac + 32 * j] * col_bytes + 16u * (u32)(1 + ap + (ap >> 3));
    const int pcol = tid >> 3, pb = tid & 7;
    const u32 src_p = tab->col[pcol] * col_bytes + (u32)nb * BM_Q82_SB_REF + 8u * (u32)pb;
    const int wr = tid >> 2, wq = tid & 3;
    const uint8_t *we = w + (size_t)e * rpe * row_bytes;
    const u32 src_w = (u32)(row0 + wr < rpe ? row0 + wr : rpe - 1) * row_bytes;
    const int crow = tid >> 3, cc = tid & 7;
    constexpr int kCodesAt = WT == BM_Q5K ? 48 : WT == BM_Q4K ? 16 : 0;
    u32 src_c[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
        src_c[j] = (u32)(row0 + crow + 64 * j < rpe ? row0 + crow + 64 * j : rpe - 1) * row_bytes + kCodesAt + 16u * (u32)cc;
    // the bytes that carry the high bits of piece cc, from the piece's own address: Q5_K's 32 high-bit bytes (value n's
    // fifth bit is bit n / 32 of byte n % 32), Q6_K's qh (piece cc of ql goes with qh piece cc % 2 of its half)
    const int high_at = WT == BM_Q5K ? 16 * (cc & 1) - 32 - 16 * cc : 128 + 32 * (cc >> 2) + 16 * (cc & 1) - 16 * cc;
    uint4 ra0, ra1, rq[2], rh, rx[WT == BM_Q4K ? 1 : 2];
    uint2 rp;
    auto fetch = [&](int i) {
        ra0 = *reinterpret_cast<const uint4 *>(act + (src_a[0] + (u32)i * BM_Q82_SB_REF));
        ra1 = *reinterpret_cast<const uint4 *>(act + (src_a[1] + (u32)i * BM_Q82_SB_REF));
        rp = *reinterpret_cast<const uint2 *>(act + (src_p + (u32)i * 64u));
        const uint8_t *blk = we + (src_w + (u32)i * kBlock);
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint8_t *piece = we + (src_c[j] + (u32)i * kBlock);
            if constexpr (kQ45) {
                rq[j] = *reinterpret_cast<const uint4 *>(piece);
                if constexpr (WT == BM_Q5K) rx[j] = *reinterpret_cast<const uint4 *>(piece + high_at);
            } else {
                rq[j] = bm_ld16u(piece);
                rx[j] = bm_ld16u(piece + high_at);
            }
        }
        if constexpr (kQ45) {
            rh = *reinterpret_cast<const uint4 *>(blk); // d, dmin, the twelve scale bytes
        } else { // scales 4 wq .. 4 wq + 3 of the sixteen, and d
            rh.x = bm_ld2u(blk + 192 + 4 * wq) | (bm_ld2u(blk + 194 + 4 * wq) << 16);
            rh.y = bm_ld2u(blk + 208);
        }
    };
    auto put16 = [](uint8_t *dst, u32 a, u32 b, u32 c, u32 d) {
        if constexpr (kOp == 16) {
            *reinterpret_cast<uint4 *>(dst) = make_uint4(a, b, c, d);
        } else { // rows 8 bytes apart modulo 16
            *reinterpret_cast<uint2 *>(dst) = make_uint2(a, b);
            *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(c, d);
        }
    };
    auto stash = [&]() {
        uint8_t *acol = a_codes + ac * kStride + 16 * ap;
        put16(acol, ra0.x, ra0.y, ra0.z, ra0.w);
        put16(acol + 32 * kStride, ra1.x, ra1.y, ra1.z, ra1.w);
        d8_t[pb * kFastColLine + pcol] = scale_operand_col(rp.x);
        if constexpr (kQ45) my_t[pb * kFastColLine + pcol] = bm_bits_f32(rp.y);
        const u32 ml = 0x0f0f0f0fu;
        if constexpr (kQ45) {
            // nibble piece cc of a row: code bytes 16 cc ..: the low nibbles are sub-block 2 p, values 16 (cc % 2) .., the
            // high nibbles sub-block 2 p + 1, the same values, with p = cc / 2
            const int p = cc >> 1, at = 16 * (cc & 1);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint8_t *row = w_codes + (crow + 64 * j) * kStride;
                u32 lo[4] = {rq[j].x & ml, rq[j].y & ml, rq[j].z & ml, rq[j].w & ml};
                u32 hi[4] = {(rq[j].x >> 4) & ml, (rq[j].y >> 4) & ml, (rq[j].z >> 4) & ml, (rq[j].w >> 4) & ml};
                if constexpr (WT == BM_Q5K) { // high-bit bytes 16 (cc % 2) ..: bit 2 p for the low nibbles, 2 p + 1 for the high
                    const u32 hw[4] = {rx[j].x, rx[j].y, rx[j].z, rx[j].w};
                    const u32 one = 0x01010101u;
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        lo[k] |= ((hw[k] >> (2 * p)) & one) << 4;
                        hi[k] |= ((hw[k] >> (2 * p + 1)) & one) << 4;
                    }
                }
                put16(row + 64 * p + at, lo[0], lo[1], lo[2], lo[3]);
                put16(row + 64 * p + 32 + at, hi[0], hi[1], hi[2], hi[3]);
            }
            // scale and min of sub-blocks 2 wq and 2 wq + 1 (crates/gguf/src/quant.rs:620-628 get_scale_min_k4): with the
            // twelve bytes as q[0 .. 11], sub-block j < 4 has q[j] & 63 and q[j + 4] & 63; j >= 4 has
            // (q[j + 4] & 15) | (q[j - 4] >> 6) << 4 and (q[j + 4] >> 4) | (q[j] >> 6) << 4
            const float d = bm_half_to_f32(rh.x & 0xffffu), dmin = bm_half_to_f32(rh.x >> 16);
            const bool upper = wq >= 2;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const u32 sh = 8u * (u32)(2 * (wq & 1) + i);
                const u32 qa = (rh.y >> sh) & 0xffu, qb = (rh.z >> sh) & 0xffu, qc = (rh.w >> sh) & 0xffu;
                const u32 scv = upper ? ((qc & 15u) | ((qa >> 6) << 4)) : (qa & 63u);
                const u32 mv = upper ? ((qc >> 4) | ((qb >> 6) << 4)) : (qb & 63u);
                sv_t[(2 * wq + i) * kFastRowLine + wr] = scale_operand_row(d * (float)scv);
                mn_t[(2 * wq + i) * kFastRowLine + wr] = -(dmin * (float)mv);
            }
        } else {
            // ql piece cc of a row (bytes 16 cc ..: half cc / 4, piece c = cc % 4 of it) with qh piece c % 2 of that half: the
            // low nibbles are quarter c / 2 of the half, values 16 (c % 2) .., the high nibbles quarter 2 + c / 2; a quarter's
            // high bits are bits 2 a .. of qh (crates/gguf/src/quant.rs:826-859). Each is one 16-value group: group
            // 8 (cc / 4) + 2 a + c % 2.
            const u32 mh = 0x03030303u;
            const int half = cc >> 2, c = cc & 3;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint8_t *row = w_codes + (crow + 64 * j) * kStride;
                const uint4 hq = rx[j];
#pragma unroll
                for (int hn = 0; hn < 2; hn++) {
                    const int a4 = (c >> 1) + 2 * hn, ns = 4 * hn, hs = 2 * a4;
                    put16(row + 128 * half + 32 * a4 + 16 * (c & 1),
                          q6_minus_32(((rq[j].x >> ns) & ml) | (((hq.x >> hs) & mh) << 4)),
                          q6_minus_32(((rq[j].y >> ns) & ml) | (((hq.y >> hs) & mh) << 4)),
                          q6_minus_32(((rq[j].z >> ns) & ml) | (((hq.z >> hs) & mh) << 4)),
                          q6_minus_32(((rq[j].w >> ns) & ml) | (((hq.w >> hs) & mh) << 4)));
                }
            }
            const float d = bm_half_to_f32(rh.y & 0xffffu);
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
                sv_t[(4 * wq + jj) * kFastRowLine + wr] = scale_operand_row(d * (float)(int)(signed char)((rh.x >> (8 * jj)) & 0xffu));
        }
    };
    // this wave's 32 rows (32 rg ..) and 32 slots (32 t ..); this lane in the 32 x 32 product: operand row / slot lane % 32,
    // its share of the unit's values (lane / 32); result v is row 8 (v / 4) + 4 (lane / 32) + v % 4 of slot lane % 32
    const int rg = wv & 3, t = wv >> 2;
    const int l32 = lane & 31, kh = lane >> 5;
    const uint8_t *my_w = w_codes + (32 * rg + l32) * kStride + kOp * kh;
    const uint8_t *my_a = a_codes + (32 * t + l32) * kStride + kOp * kh;
    const uint2 *my_sv = sv_t + (kh ? kFastRows : 32 * rg + l32); // lanes 32 .. 63: the line's zero
    const uint2 *my_d8 = d8_t + 32 * t + l32;
    const bool live = t == 0 || len > 32; // else this wave's slots are all padding
    v16f acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;

    // One super-block's products. A step is a unit: its integer sums (one matrix instruction, issued a step ahead), its
    // scale products (another, issued at the end of the step before, behind that step's last use of the one buffer), and on
    // the vector ALU the sums to floats and the multiply-adds.
    auto blocks = [&]() __attribute__((always_inline)) {
        typedef typename std::conditional<kQ45, v4i, long>::type Operand;
        Operand a[2], b[2];
        uint2 sa[2], sb[2];
        v16i sum[2];
        v16f pr;
        auto rd = [&](int u) {
            a[u & 1] = *reinterpret_cast<const Operand *>(my_w + 2 * kOp * u);
            b[u & 1] = *reinterpret_cast<const Operand *>(my_a + 2 * kOp * u);
            sa[u & 1] = my_sv[u * kFastRowLine];
            sb[u & 1] = my_d8[(kQ45 ? u : u >> 1) * kFastColLine];
        };
        auto product = [&](int u) {
            const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            if constexpr (kQ45) sum[u & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u & 1], b[u & 1], z, 0, 0, 0);
            else sum[u & 1] = __builtin_amdgcn_mfma_i32_32x32x16_i8(a[u & 1], b[u & 1], z, 0, 0, 0);
        };
        auto scales = [&](int u) {
            const v16f z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            pr = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(v4s, sa[u & 1]), __builtin_bit_cast(v4s, sb[u & 1]), z, 0, 0,
                                                         0);
        };
        rd(0);
        rd(1);
        product(0);
        scales(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < kUnitsSb; u++) {
            if (u + 1 < kUnitsSb) product(u + 1);
            __builtin_amdgcn_sched_barrier(0);
            float f[16];
#pragma unroll
            for (int v = 0; v < 16; v++) f[v] = (float)sum[u & 1][v];
#pragma unroll
            for (int v = 0; v < 16; v++) acc[v] = fmaf(pr[v], f[v], acc[v]);
            __builtin_amdgcn_sched_barrier(0);
            if (u + 1 < kUnitsSb) scales(u + 1);
            // the operands two units on, into the buffers of this unit, whose last instructions have been issued
            if (u + 2 < kUnitsSb) rd(u + 2);
        }
        if constexpr (kQ45) {
            // the min terms last, into the same accumulators: a 32 x 8 by 8 x 32 product in f32, two of the eight
            // sub-blocks an instruction; they run on the matrix cores while the workgroup goes through its barrier and the
            // next staging
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(mn_t[(2 * j + kh) * kFastRowLine + 32 * rg + l32],
                                                           my_t[(2 * j + kh) * kFastColLine + 32 * t + l32], acc, 0, 0, 0);
        }
    };

    fetch(0);
    for (int i = 0; i < nb; i++) {
        if (i) __syncthreads(); // the readers of the super-block before are done
        stash();
        __syncthreads();
        if (i + 1 < nb) fetch(i + 1);
        if (live) blocks();
    }
    const int n = 32 * t + l32;
    if (n < len) {
        float *out = y + (size_t)tab->slot[n] * rpe + row0 + 32 * rg + 4 * kh;
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            // rows_per_expert is a multiple of 16 and these four rows start at a multiple of 4: all inside or all outside
            if (row0 + 32 * rg + 4 * kh + 8 * q4 < rpe)
                *reinterpret_cast<float4 *>(out + 8 * q4) = make_float4(acc[4 * q4 + 0], acc[4 * q4 + 1], acc[4 * q4 + 2], acc[4 * q4 + 3]);
        }
    }
}

// ------------------------------------------------------------------------------------- IQ2_XXS on Q8_K columns

// The grouped GEMM for IQ2_XXS stacks (crates/gpu/src/gemm/kernels.rs:867 gemm_iq2xxs; the arithmetic is
// crates/gpu/src/gemm/grouped.rs:33-58 with the CPU path's lanes, crates/qdot/src/lib.rs:8677-8724). A super-block of a
// row against a super-block of a Q8_K column is, in the CPU path, eight accumulators: accumulator l first takes
// (dmin dy) (2 s_l + 1) (bsum[2l] + bsum[2l + 1]), then (d dy) sumi[l] with
//     sumi[l] = sum over the eight sub-blocks b of (2 s_b + 1) * sum over i < 4 of u[b][4l + i] a[b][4l + i],
// u = +-grid + 43 the unsigned code byte. sumi[l] is a 32-term integer dot whose weight-side terms (2 s_b + 1) u are at most
// 31 * 86 = 2666: too wide for an int8 operand, so each is split into two signed bytes, 256 h + lo with lo = the low byte
// read as signed and h = (term + 128) >> 8 (0 .. 10), and the dot is two v_mfma_i32_32x32x32_i8 whose sums meet as
// (H << 8) + L, exactly. The LDS copy of a row's (and a column's) super-block is laid out lane-major, [l][b][i], so a matrix
// operand is 16 consecutive bytes. With EXACT the eight accumulators and their order are the CPU path's, bit for bit
// (the value bm_gemv_sel gives); without it one accumulator takes d dy times the super-block's whole sum
// sum_b (2 s_b + 1) sum_n (u - 43) a, the 43s taken out in integers through two more matrix instructions over the
// column's 32-value sums (split into two bytes the same way): f32 rounding is the only difference.
// A workgroup of four waves takes 64 rows and a tile's 64 slots, a wave 32 x 32 of them.
constexpr int kIqRows = 64;
constexpr int kIqStride = 256 + 16; // bytes a row's or a column's 256 codes take in LDS
constexpr int kIqLine = 64 + 4;     // floats a line of the per-lane tables
template <int WT, bool EXACT>
__host__ __device__ constexpr size_t gemm_iq_lds_bytes() {
    return sizeof(GemmLds) + (size_t)tab_bytes<WT>() + 3 * (size_t)64 * kIqStride + 2 * 64 * sizeof(float) +
           (EXACT ? 2 * 8 * kIqLine * sizeof(float) : 3 * 64 * 16);
}

// (2 s + 1) u for the four code bytes of `u`, each product split into the signed low byte (lo) and what is left over 256
// (hi): 256 hi + lo is the product.
__device__ __forceinline__ void iq2_planes(u32 u, u32 sc, u32 &hi, u32 &lo) {
    const u32 even = __builtin_amdgcn_perm(0u, u, 0x0c020c00u), odd = __builtin_amdgcn_perm(0u, u, 0x0c030c01u);
    const u32 pe = even * sc, po = odd * sc; // two 16-bit fields each, at most 2666
    lo = __builtin_amdgcn_perm(po, pe, 0x06020400u);
    hi = __builtin_amdgcn_perm(po + 0x00800080u, pe + 0x00800080u, 0x07030501u);
}

// The same split for a product of four signed bytes with a signed scale (|product| <= 4064): lo the low byte read as signed,
// hi what is left over 256.
__device__ __forceinline__ void iq_planes_signed(u32 v, int sc, u32 &hi, u32 &lo) {
    const int p0 = bm_mul24(__builtin_amdgcn_sbfe((int)v, 0, 8), sc), p1 = bm_mul24(__builtin_amdgcn_sbfe((int)v, 8, 8), sc);
    const int p2 = bm_mul24(__builtin_amdgcn_sbfe((int)v, 16, 8), sc), p3 = bm_mul24(__builtin_amdgcn_sbfe((int)v, 24, 8), sc);
    lo = ((u32)p0 & 0xffu) | (((u32)p1 & 0xffu) << 8) | (((u32)p2 & 0xffu) << 16) | ((u32)p3 << 24);
    hi = ((u32)((p0 + 128) >> 8) & 0xffu) | (((u32)((p1 + 128) >> 8) & 0xffu) << 8) | (((u32)((p2 + 128) >> 8) & 0xffu) << 16) |
         ((u32)((p3 + 128) >> 8) << 24);
}

// The types that dot against Q8_K columns (crates/gpu/src/gemm/kernels.rs:867 gemm_iq2xxs, :759 gemm_q3k, :1139 gemm_iq3xxs,
// :1248 gemm_iq4xs). What differs between them is how a row's super-block becomes signed code x scale terms (the staging) and
// the f32 step a super-block; the columns, the lane-major operands, the two byte planes and the products are the same.
//   IQ2_XXS, IQ3_XXS: terms (2 s + 1) (offset + u), offset 43 / 64, the offsets folded out through the column's sums first,
//     eight accumulators, d = f16 / 8 and f16 / 4;
//   IQ4_XS: terms scale x level (scale -32 .. 31, the sixteen levels), eight accumulators, one multiply-add a super-block each
//     (crates/qdot/src/lib.rs:11171-11173);
//   Q3_K: terms scale x (u - 4) over the sixteen 16-value groups, one integer a super-block and one accumulator, the float step
//     acc + (dcol d) sum with every operation rounded on its own (crates/qdot/src/lib.rs:2223-2245).
// EXACT only for the three added types: the tolerance mode runs them in this order too.
template <int WT>
struct IqGemm {
    static constexpr bool kFold = WT == BM_IQ2XXS || WT == BM_IQ3XXS;
    static constexpr int kOff = WT == BM_IQ2XXS ? 43 : 64;
    static constexpr int kLanes = WT == BM_Q3K ? 1 : 8;
    static constexpr int kBlock = WT == BM_IQ2XXS ? BM_IQ2XXS_BLOCK : WT == BM_IQ3XXS ? BM_IQ3XXS_BLOCK : WT == BM_IQ4XS ? BM_IQ4XS_BLOCK : BM_Q3K_BLOCK;
};

template <int WT, bool EXACT>
__global__ __launch_bounds__(256, 2) void k_gemm_iq(const uint8_t *w, int rpe, int nb, const uint8_t *act, const u32 *cols,
                                                    const u32 *tiles, const u32 *n_tiles, u32 n_slabs, u32 slot_div,
                                                    u32 n_slots, float *y) {
    static_assert(EXACT || WT == BM_IQ2XXS, "the one-accumulator form is IQ2_XXS's");
    using G = IqGemm<WT>;
    extern __shared__ __align__(16) uint8_t lds[];
    GemmLds *tab = reinterpret_cast<GemmLds *>(lds);
    [[maybe_unused]] const Iq2Tables tb = stage_tables<WT>(lds + sizeof(GemmLds));
    uint8_t *a_codes = lds + sizeof(GemmLds) + tab_bytes<WT>();
    uint8_t *w_hi = a_codes + 64 * kIqStride;
    uint8_t *w_lo = w_hi + 64 * kIqStride;
    float *dy_t = reinterpret_cast<float *>(w_lo + 64 * kIqStride); // [slot]
    float *d_t = dy_t + 64;                                          // [row]
    float *bs_t = d_t + 64;                                          // EXACT: [l][slot] the 32-value sums, as floats
    float *sc_t = bs_t + 8 * kIqLine;                                // EXACT: [l][row] the scales 2 s + 1, as floats
    uint8_t *x_sc = reinterpret_cast<uint8_t *>(d_t + 64);           // else: [row][16] the scales as bytes, zeros behind
    uint8_t *x_bl = x_sc + 64 * 16;                                  // [slot][16] the sums' low bytes, zeros behind
    uint8_t *x_bh = x_bl + 64 * 16;                                  // [slot][16] what is left of the sums over 256
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const u32 g = tile_of_block(blockIdx.x, n_slabs);
    const int row0 = (int)slab_of_block(blockIdx.x, n_slabs) * kIqRows;
    const u32 count = n_tiles[0];
    if (g > count) return;
    if (g == count) { // the refused slots' rows: NaN (crates/gpu/src/gemm/grouped.rs:2283-2287)
        const u32 refused = n_tiles[1];
        for (u32 i = tid; i < refused * kIqRows; i += 256) {
            const u32 s = cols[n_slots - n_tiles[2] - refused + i / kIqRows];
            const int r = row0 + (int)(i % kIqRows);
            if (r < rpe) y[(size_t)s * rpe + r] = bm_bits_f32(0x7fc00000u);
        }
        return;
    }
    const u32 e = tiles[2 * g], word = tiles[2 * g + 1];
    const int start = (int)(word & 0xffffu), len = (int)(word >> 16);
    if (tid < kGemmBN) {
        const u32 s = cols[start + (tid < len ? tid : 0)];
        tab->slot[tid] = s;
        tab->col[tid] = s / slot_div;
    }
    __syncthreads();
    const u32 row_bytes = (u32)nb * G::kBlock, col_bytes = (u32)nb * BM_Q8K_STRIDE;
    // what this thread stages of every super-block:
    //   four 16-byte pieces of column codes (column tid / 16 + 16 j, piece tid % 16 of the sixteen): values 16 (piece % 2) ..
    //   of sub-block piece / 2, i.e. the four-value groups of lanes 4 (piece % 2) .. + 3, one word each;
    //   threads below 64: column tid's scale and its sixteen 16-value sums;
    //   two sub-blocks of a weight row (row tid / 4, sub-blocks 2 (tid % 4) and the one after), the first of the four
    //   also the row's d
    const int ac = tid >> 4, ap = tid & 15;
    u32 src_a[4];
#pragma unroll
    for (int j = 0; j < 4; j++) src_a[j] = tab->col[ac + 16 * j] * col_bytes + 8u + 16u * (u32)ap;
    const u32 src_c = tab->col[tid & 63] * col_bytes;
    const int wr = tid >> 2, wq = tid & 3;
    const uint8_t *we = w + (size_t)e * rpe * row_bytes;
    const u32 src_w = (u32)(row0 + wr < rpe ? row0 + wr : rpe - 1) * row_bytes;
    const int a_dst = ac * kIqStride + 32 * (4 * (ap & 1)) + 4 * (ap >> 1); // word k of a piece: + 32 k

    // A super-block's bytes are asked for one super-block ahead (fetch_rows, fetch_cols: into registers, behind the staging of
    // the present one and before its products) and unpacked into LDS when their turn comes (stage): the loads' way through memory runs
    // under the matrix work instead of in front of it.
    uint4 ra[4];
    uint4 rq = make_uint4(0, 0, 0, 0), rq2 = rq, rq3 = rq, rq4 = rq;
    uint2 rx = make_uint2(0, 0);
    u32 rd = 0, ra2 = 0;
    float cdy = 0.0f;
    uint4 cb0 = make_uint4(0, 0, 0, 0), cb1 = cb0;
    auto fetch_cols = [&](int i) {
#pragma unroll
        for (int j = 0; j < 4; j++) __builtin_memcpy(&ra[j], act + (src_a[j] + (u32)i * BM_Q8K_STRIDE), 16);
        if (tid < 64) {
            const uint8_t *cs = act + (src_c + (u32)i * BM_Q8K_STRIDE);
            cdy = *reinterpret_cast<const float *>(cs);
            __builtin_memcpy(&cb0, cs + 264, 16);
            __builtin_memcpy(&cb1, cs + 280, 16);
        }
    };
    auto fetch_rows = [&](int i) {
        const uint8_t *blk = we + (src_w + (u32)i * G::kBlock);
        // the row's two sub-blocks 2 wq and 2 wq + 1, as the type lays them out
        if constexpr (WT == BM_IQ2XXS) {
            rq = bm_ld16u(blk + 2 + 16 * wq);
            rd = bm_ld2u(blk);
        } else if constexpr (WT == BM_IQ3XXS) {
            rq = bm_ld16u(blk + 2 + 16 * wq); // the index bytes of the two sub-blocks
            __builtin_memcpy(&rx, blk + 66 + 8 * wq, 8); // their sign/scale words
            rd = bm_ld2u(blk);
        } else if constexpr (WT == BM_IQ4XS) {
            __builtin_memcpy(&rx, blk, 8); // d | scales_h << 16, scales_l
            rq = bm_ld16u(blk + 8 + 32 * wq);
            rq2 = bm_ld16u(blk + 24 + 32 * wq);
            rd = rx.x & 0xffffu;
        } else { // Q3_K: the 32 field bytes of half wq / 2, the 32 high-bit bytes, the scales and d
            rq = bm_ld16u(blk + 32 + 32 * (wq >> 1));
            rq2 = bm_ld16u(blk + 48 + 32 * (wq >> 1));
            rq3 = bm_ld16u(blk);
            rq4 = bm_ld16u(blk + 16);
            const uint4 tail = bm_ld16u(blk + 94); // the twelve scale bytes at 2 .., d at 14
            rx = make_uint2((tail.x >> 16) | (tail.y << 16), (tail.y >> 16) | (tail.z << 16)); // scale words a0, a1
            ra2 = (tail.z >> 16) | (tail.w << 16);                                             // a2: their high bits
            rd = tail.w >> 16;
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint8_t *dst = a_codes + a_dst + 16 * j * kIqStride;
            *reinterpret_cast<u32 *>(dst) = ra[j].x;
            *reinterpret_cast<u32 *>(dst + 32) = ra[j].y;
            *reinterpret_cast<u32 *>(dst + 64) = ra[j].z;
            *reinterpret_cast<u32 *>(dst + 96) = ra[j].w;
        }
        if (tid < 64) {
            dy_t[tid] = cdy;
            const u32 bw[8] = {cb0.x, cb0.y, cb0.z, cb0.w, cb1.x, cb1.y, cb1.z, cb1.w};
            u32 bl[2] = {0, 0}, bh[2] = {0, 0};
#pragma unroll
            for (int l = 0; l < 8; l++) { // the two 16-value sums of sub-block l
                const int bs = (int)(short)(bw[l] & 0xffffu) + (int)(short)(bw[l] >> 16);
                if constexpr (EXACT) {
                    if constexpr (G::kFold) bs_t[l * kIqLine + tid] = (float)bs;
                } else { // 256 hi + lo with lo the low byte read as signed
                    bl[l >> 2] |= ((u32)bs & 0xffu) << (8 * (l & 3));
                    bh[l >> 2] |= ((u32)((bs + 128) >> 8) & 0xffu) << (8 * (l & 3));
                }
            }
            if constexpr (!EXACT) {
                *reinterpret_cast<uint4 *>(x_bl + 16 * tid) = make_uint4(bl[0], bl[1], 0u, 0u);
                *reinterpret_cast<uint4 *>(x_bh + 16 * tid) = make_uint4(bh[0], bh[1], 0u, 0u);
            }
        }
        if (wq == 0) {
            const float dh = bm_half_to_f32((unsigned short)rd);
            d_t[wr] = WT == BM_IQ2XXS ? 0.125f * dh : WT == BM_IQ3XXS ? 0.25f * dh : dh;
        }
        [[maybe_unused]] u32 scs[2] = {0, 0};
#pragma unroll
        for (int e2 = 0; e2 < 2; e2++) {
            const int b = 2 * wq + e2;
            // the four values 4 l .. 4 l + 3 of sub-block b, times the scale, as the two byte planes at lane l's place
            auto put = [&](int l, u32 h, u32 lo) {
                const int at = wr * kIqStride + 32 * l + 4 * b;
                *reinterpret_cast<u32 *>(w_hi + at) = h;
                *reinterpret_cast<u32 *>(w_lo + at) = lo;
            };
            if constexpr (WT == BM_IQ2XXS || WT == BM_IQ3XXS) {
                const u32 aux = WT == BM_IQ2XXS ? (e2 ? rq.w : rq.y) : (e2 ? rx.y : rx.x);
                const u32 sc = 2u * (aux >> 28) + 1u;
                scs[e2] = sc;
                if constexpr (EXACT) sc_t[b * kIqLine + wr] = (float)sc;
#pragma unroll
                for (int q = 0; q < 4; q++) { // values 8 q .. 8 q + 7: lanes 2 q and 2 q + 1
                    u32 c_lo, c_hi;
                    if constexpr (WT == BM_IQ2XXS) {
                        const u32 idx = e2 ? rq.z : rq.x;
                        bm_iq2_codes(tb, (idx >> (8 * q)) & 0xffu, (aux >> (7 * q)) & 127u, c_lo, c_hi);
                    } else { // index bytes 2 q and 2 q + 1 of the sub-block's eight, sign group q
                        const u32 word = e2 ? ((q & 2) ? rq.w : rq.z) : ((q & 2) ? rq.y : rq.x);
                        const u32 pair = word >> (16 * (q & 1));
                        const uint2 g0 = tb.grid3[pair & 0xffu], g1 = tb.grid3[(pair >> 8) & 0xffu];
                        const uint2 sg = tb.signs[(aux >> (7 * q)) & 127u];
                        c_lo = bm_iq_pick(g0.x, g0.y, sg.x);
                        c_hi = bm_iq_pick(g1.x, g1.y, sg.y);
                    }
                    u32 h0, l0, h1, l1;
                    iq2_planes(c_lo, sc, h0, l0);
                    iq2_planes(c_hi, sc, h1, l1);
                    put(2 * q, h0, l0);
                    put(2 * q + 1, h1, l1);
                }
            } else if constexpr (WT == BM_IQ4XS) {
                // crates/gguf/src/quant.rs:1989-1991: nibble b % 2 of scales_l[b / 2] under bits 2b .. of scales_h, less 32
                const u32 sl = (rx.y >> (8 * wq + 4 * e2)) & 15u, sh = (rx.x >> (16 + 4 * wq + 2 * e2)) & 3u;
                const int sc = (int)(sl | (sh << 4)) - 32;
                const uint4 cw = e2 ? rq2 : rq;
                const u32 qw[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
                for (int l = 0; l < 4; l++) { // low nibbles: values 4 l ..; high nibbles: values 16 + 4 l ..
                    u32 h, lo;
                    iq_planes_signed(bm_iq4_levels<0>(qw[l]), sc, h, lo);
                    put(l, h, lo);
                    iq_planes_signed(bm_iq4_levels<4>(qw[l]), sc, h, lo);
                    put(4 + l, h, lo);
                }
            } else { // Q3_K: sub-block b = 4 j + f is field f of the half's 32 cells; cell p is value p of the sub-block
                const int j = wq >> 1, f = 2 * (wq & 1) + e2;
                // the sixteen six-bit scales (crates/qdot/src/lib.rs:2162-2174): group 8 j + 2 f + odd
                const u32 lo4 = j ? (rx.x >> 4) : rx.x, lo41 = j ? (rx.y >> 4) : rx.y, hi2 = ra2 >> (4 * j);
                const u32 w0 = (lo4 & 0x0f0f0f0fu) | ((hi2 & 0x03030303u) << 4);
                const u32 w1 = (lo41 & 0x0f0f0f0fu) | (((hi2 >> 2) & 0x03030303u) << 4);
                const u32 sword = (f >> 1) ? w1 : w0;
                const u32 qs[8] = {rq.x, rq.y, rq.z, rq.w, rq2.x, rq2.y, rq2.z, rq2.w};
                const u32 hm[8] = {rq3.x, rq3.y, rq3.z, rq3.w, rq4.x, rq4.y, rq4.z, rq4.w};
#pragma unroll
                for (int t = 0; t < 8; t++) { // cells 4 t .. 4 t + 3: lane t
                    const int sc = (int)((sword >> (8 * (2 * (f & 1) + (t >> 2)))) & 0xffu) - 32;
                    const u32 low = (qs[t] >> (2 * f)) & 0x03030303u, high = (hm[t] >> (4 * j + f)) & 0x01010101u;
                    const u32 v = __builtin_amdgcn_perm(0x03020100u, 0xfffefdfcu, (high << 2) | low); // u - 4
                    u32 h, lo;
                    iq_planes_signed(v, sc, h, lo);
                    put(t, h, lo);
                }
            }
        }
        if constexpr (!EXACT) { // the row's eight scales as bytes: the thread of sub-blocks 2 wq, 2 wq + 1 writes its two
            *reinterpret_cast<unsigned short *>(x_sc + 16 * wr + 2 * wq) = (unsigned short)(scs[0] | (scs[1] << 8));
            if (wq == 0) *reinterpret_cast<uint2 *>(x_sc + 16 * wr + 8) = make_uint2(0u, 0u);
        }
    };

    // this lane in its wave's 32 x 32 product: operand row / slot lane % 32, terms 16 (lane / 32) .. of the 32; result v
    // is row 8 (v / 4) + 4 (lane / 32) + v % 4 of slot lane % 32
    const int l32 = lane & 31, kh = lane >> 5;
    const int wrow = 32 * (wv & 1), wslot = 32 * (wv >> 1);
    const uint8_t *my_h = w_hi + (wrow + l32) * kIqStride + 16 * kh;
    const uint8_t *my_l = w_lo + (wrow + l32) * kIqStride + 16 * kh;
    const uint8_t *my_a = a_codes + (wslot + l32) * kIqStride + 16 * kh;
    const bool live = wslot < len; // else none of this wave's slots is real
    const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    constexpr int kAcc = EXACT ? G::kLanes : 1;
    v16f acc[kAcc];
#pragma unroll
    for (int l = 0; l < kAcc; l++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[l][v] = 0.0f;

    // (the columns' bytes too where the registers allow: the exact forms of the types with eight accumulators a value have few
    // to spare - with everything held over they spilled and ran 6 % slower - so there only the rows' bytes, which come from
    // HBM, are asked for ahead, and the columns', which the cache holds, when their turn comes)
    constexpr bool kColsAhead = !EXACT || G::kLanes == 1;
    fetch_rows(0);
    if constexpr (kColsAhead) fetch_cols(0);
    for (int i = 0; i < nb; i++) {
        if (i) __syncthreads(); // the readers of the super-block before are done
        if constexpr (!kColsAhead) fetch_cols(i);
        stage();
        if (i + 1 < nb) {
            fetch_rows(i + 1);
            if constexpr (kColsAhead) fetch_cols(i + 1);
        }
        __syncthreads();
        if (!live) continue;
        const float dy = dy_t[wslot + l32];
        float dd[16];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const float4 d4 = *reinterpret_cast<const float4 *>(d_t + wrow + 8 * q4 + 4 * kh);
            dd[4 * q4 + 0] = d4.x;
            dd[4 * q4 + 1] = d4.y;
            dd[4 * q4 + 2] = d4.z;
            dd[4 * q4 + 3] = d4.w;
        }
        if constexpr (EXACT && G::kLanes == 1) {
            // Q3_K: one integer a super-block, then acc + (dcol d) sum, each operation rounded on its own
            v16i hs = z, ls = z;
#pragma unroll
            for (int l = 0; l < 8; l++) {
                const v4i b = *reinterpret_cast<const v4i *>(my_a + 32 * l);
                hs = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i *>(my_h + 32 * l), b, hs, 0, 0, 0);
                ls = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i *>(my_l + 32 * l), b, ls, 0, 0, 0);
            }
#pragma unroll
            for (int v = 0; v < 16; v++)
                acc[0][v] = __fadd_rn(acc[0][v], __fmul_rn(__fmul_rn(dy, dd[v]), (float)(hs[v] * 256 + ls[v])));
        } else if constexpr (EXACT) {
            if constexpr (G::kFold) {
                // the fold of the offsets first: accumulator l takes sub-block l's scale on its two sums
                // (crates/qdot/src/lib.rs:8691-8694); the product of the two small integers is exact in f32
#pragma unroll
                for (int l = 0; l < 8; l++) {
                    const float bs = bs_t[l * kIqLine + wslot + l32];
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) {
                        const float4 s4 = *reinterpret_cast<const float4 *>(sc_t + l * kIqLine + wrow + 8 * q4 + 4 * kh);
                        const float sv[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            const float dmin = -dd[4 * q4 + k] * (float)G::kOff;
                            acc[l][4 * q4 + k] = fmaf(dmin * dy, sv[k] * bs, acc[l][4 * q4 + k]);
                        }
                    }
                }
            }
#pragma unroll
            for (int l = 0; l < 8; l++) {
                const v4i b = *reinterpret_cast<const v4i *>(my_a + 32 * l);
                const v16i hs = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i *>(my_h + 32 * l), b, z, 0, 0, 0);
                const v16i ls = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i *>(my_l + 32 * l), b, z, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[l][v] = fmaf(dd[v] * dy, (float)(hs[v] * 256 + ls[v]), acc[l][v]);
            }
        } else {
            v16i hs = z, ls = z;
#pragma unroll
            for (int l = 0; l < 8; l++) {
                const v4i b = *reinterpret_cast<const v4i *>(my_a + 32 * l);
                hs = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i *>(my_h + 32 * l), b, hs, 0, 0, 0);
                ls = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i *>(my_l + 32 * l), b, ls, 0, 0, 0);
            }
            // sum_b (2 s_b + 1) (the sub-block's sum of a): the scales against the sums' two bytes, terms 8 .. 31 zero
            const v4i zero4 = {0, 0, 0, 0};
            const v4i xs = kh ? zero4 : *reinterpret_cast<const v4i *>(x_sc + 16 * (wrow + l32));
            const v4i xl = kh ? zero4 : *reinterpret_cast<const v4i *>(x_bl + 16 * (wslot + l32));
            const v4i xh = kh ? zero4 : *reinterpret_cast<const v4i *>(x_bh + 16 * (wslot + l32));
            const v16i ml = __builtin_amdgcn_mfma_i32_32x32x32_i8(xs, xl, z, 0, 0, 0);
            const v16i mh = __builtin_amdgcn_mfma_i32_32x32x32_i8(xs, xh, z, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int total = ((hs[v] << 8) + ls[v]) - 43 * ((mh[v] << 8) + ml[v]);
                acc[0][v] = fmaf(dd[v] * dy, (float)total, acc[0][v]);
            }
        }
    }
    const int n = wslot + l32;
    if (live && n < len) {
        float *out = y + (size_t)tab->slot[n] * rpe + row0 + wrow + 4 * kh;
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            // rows_per_expert is a multiple of 16 and these four rows start at a multiple of 4: all inside or all outside
            if (row0 + wrow + 4 * kh + 8 * q4 < rpe) {
                float r[4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int v = 4 * q4 + k;
                    if constexpr (EXACT && G::kLanes == 8) { // the closing sum of the eight lanes (crates/qdot/src/lib.rs:4128 hsum_float_8's order)
                        const float t0 = acc[0][v] + acc[4][v], t1 = acc[1][v] + acc[5][v];
                        const float t2 = acc[2][v] + acc[6][v], t3 = acc[3][v] + acc[7][v];
                        r[k] = (t0 + t2) + (t1 + t3);
                    } else {
                        r[k] = acc[0][v];
                    }
                }
                *reinterpret_cast<float4 *>(out + 8 * q4) = make_float4(r[0], r[1], r[2], r[3]);
            }
        }
    }
}

bool gemm_supported(int wtype) {
    return wtype == BM_Q4K || wtype == BM_Q5K || wtype == BM_Q6K || wtype == BM_IQ2XXS || wtype == BM_IQ3XXS || wtype == BM_IQ4XS ||
           wtype == BM_Q3K;
}

hipError_t gemm(const Launch &L, int wtype, const uint8_t *w, int n_experts, int rows_per_expert, int k,
                const uint8_t *act, const uint32_t *cols, const uint32_t *tiles_dev, const uint32_t *n_tiles, int n_slots,
                int slot_div, float *y, int mode) {
    const int nb = k / 256;
    const u32 max_tiles = (u32)gemm_max_tiles(n_slots, n_experts) + 1; // one more: the block that fills refused slots
    const u32 n_slabs = (u32)((rows_per_expert + kGemmBM - 1) / kGemmBM);
    // parts: workgroups a tile's 64 slots are shared among (each takes every row slab)
    auto launch = [&](auto kern, unsigned threads, size_t lds, unsigned parts) {
        hipError_t e = allow_lds(kern, lds);
        if (e != hipSuccess) return e;
        const u32 n_units = n_slabs * parts;
        const unsigned grid = ((max_tiles + 7) / 8) * 8 * n_units;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, L.stream, w, rows_per_expert, nb, act, cols, tiles_dev, n_tiles,
                           n_units, (u32)slot_div, (u32)n_slots, y);
        return hipGetLastError();
    };
    if (bm_takes_q8k(wtype)) {
        auto launch_iq = [&](auto kern, size_t lds) {
            hipError_t e = allow_lds(kern, lds);
            if (e != hipSuccess) return e;
            const u32 n_slabs_q = (u32)((rows_per_expert + kIqRows - 1) / kIqRows);
            const unsigned grid = ((max_tiles + 7) / 8) * 8 * n_slabs_q;
            hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, w, rows_per_expert, nb, act, cols, tiles_dev, n_tiles,
                               n_slabs_q, (u32)slot_div, (u32)n_slots, y);
            return hipGetLastError();
        };
        if (wtype == BM_IQ3XXS) return launch_iq(k_gemm_iq<BM_IQ3XXS, true>, gemm_iq_lds_bytes<BM_IQ3XXS, true>());
        if (wtype == BM_IQ4XS) return launch_iq(k_gemm_iq<BM_IQ4XS, true>, gemm_iq_lds_bytes<BM_IQ4XS, true>());
        if (wtype == BM_Q3K) return launch_iq(k_gemm_iq<BM_Q3K, true>, gemm_iq_lds_bytes<BM_Q3K, true>());
        if (wtype != BM_IQ2XXS) return hipErrorInvalidValue;
        if (mode != 0) return launch_iq(k_gemm_iq<BM_IQ2XXS, false>, gemm_iq_lds_bytes<BM_IQ2XXS, false>());
        return launch_iq(k_gemm_iq<BM_IQ2XXS, true>, gemm_iq_lds_bytes<BM_IQ2XXS, true>());
    }
    if (mode == 2 && gemm_half_supported(wtype)) // the f16 form of the tolerance mode, where the type has one
        return gemm_half(L, wtype, w, n_experts, rows_per_expert, k, act, cols, tiles_dev, n_tiles, n_slots, slot_div, y);
    if (mode == 1 || mode == 2) {
        auto launch_fast = [&](auto kern, size_t lds) {
            hipError_t e = allow_lds(kern, lds);
            if (e != hipSuccess) return e;
            const u32 n_slabs_f = (u32)((rows_per_expert + kFastRows - 1) / kFastRows);
            const unsigned grid = ((max_tiles + 7) / 8) * 8 * n_slabs_f;
            hipLaunchKernelGGL(kern, dim3(grid), dim3(kFastThreads), lds, L.stream, w, rows_per_expert, nb, act, cols, tiles_dev, n_tiles,
                               n_slabs_f, (u32)slot_div, (u32)n_slots, y);
            return hipGetLastError();
        };
        if (wtype == BM_Q4K) return launch_fast(k_gemm_fast<BM_Q4K>, fast_lds_bytes<BM_Q4K>());
        if (wtype == BM_Q5K) return launch_fast(k_gemm_fast<BM_Q5K>, fast_lds_bytes<BM_Q5K>());
        if (wtype == BM_Q6K) return launch_fast(k_gemm_fast<BM_Q6K>, fast_lds_bytes<BM_Q6K>());
    }
    // 512 threads on 32 slots of a tile for both types (Q4_K 114 registers, Q6_K 121): two workgroups a CU. Measured
    // against 1024 threads on all 64 slots (Q4_K gate 362 -> 342 us), 512 threads with two slot groups a wave on 64
    // (Q6_K down 489 -> 407 us), and 256 threads on 16 or 32 slots (slower: the rows are staged once a workgroup).
    if (wtype == BM_Q4K) return launch(k_gemm<BM_Q4K, 1, 2>, 512, gemm_exact_lds_bytes(32), 2);
    if (wtype == BM_Q5K) return launch(k_gemm<BM_Q5K, 1, 2>, 512, gemm_exact_lds_bytes(32), 2);
    if (wtype == BM_Q6K) return launch(k_gemm<BM_Q6K, 1, 2>, 512, gemm_exact_lds_bytes(32), 2);
    return hipErrorInvalidValue;
}

} // namespace bmk
