// Prefill: the grouped expert GEMM over a route table, on the int8 matrix cores, and the SwiGLU quantizer between
// a gate/up pair and its down (crates/gpu/src/gemm/mod.rs:1-50).
//
// The route table is the reference's (crates/gpu/src/gemm/route.rs:1-60,109-125): `cols` lists the slots grouped by
// expert, ascending slot order inside an expert, the refused slots (an id past the stack) at its end; `tiles` holds
// a pair of words a tile, (expert, first index | length << 16), tiles of at most 64 slots; `n_tiles` = {tile count,
// refused count}.
//
// The GEMM's numbers are the decode path's, bit for bit: every (row, slot) value is the one-column row dot of
// bm_device.cuh. The integer sums of each 16-value group come out of v_mfma_i32_16x16x32_i8 (16 rows x 16 slots,
// exact; the other half of the 32 values zeroed on the weight side), and each enters the f32 accumulator of the CPU path's lane that
// owns it, in the CPU path's order (crates/qdot/src/lib.rs:4363-4447 Q4_K, :4776-4874 Q6_K): eight accumulators a
// value, the min term first, then the groups in increasing k, and the closing sum (t0 + t2) + (t1 + t3).
// Activation scales come per 32 values in this form, so every group's sum is scaled on the vector ALU before it is
// added: three operations a (row, slot, group) against one matrix instruction per 1024 of them. The kernel is bound
// by that arithmetic, not by the matrix cores.
#include "bm_stream.cuh"

namespace bmk {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kRouteThreads = 1024;

int gemm_max_tiles(int n_slots, int n_experts) { // crates/gpu/src/gemm/route.rs:55-57
    return n_slots / kGemmBN + (n_experts < n_slots ? n_experts : n_slots);
}

// ------------------------------------------------------------------------------------------------ route

// One workgroup: the slots listed by expert in ascending slot order (group_slots), bucket n_experts collecting the
// refused ones at the list's end; then the tiles, an expert's run cut into runs of at most 64.
__global__ __launch_bounds__(kRouteThreads) void k_route(const u32 *ids, u32 n_slots, u32 n_experts, u32 *cols,
                                                         u32 *tiles, u32 *n_tiles, u32 *fault, u32 layer) {
    __shared__ GroupLds g;
    const u32 tid = threadIdx.x;
    group_slots(g, n_slots, n_experts + 1, cols, [&](u32 s) {
        const u32 id = ids[s];
        return id < n_experts ? id : n_experts;
    });
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
    }
}

hipError_t route(const Launch &L, const uint32_t *ids, int n_slots, int n_experts, uint32_t *cols, uint32_t *tiles_out,
                 uint32_t *n_tiles) {
    hipLaunchKernelGGL(k_route, dim3(1), dim3(kRouteThreads), 0, L.stream, ids, (u32)n_slots, (u32)n_experts, cols,
                       tiles_out, n_tiles, L.fault, L.layer);
    return hipGetLastError();
}

// --------------------------------------------------------------------------------------- SwiGLU + quantize

// crates/gpu/src/gemm/swiglu.rs:46-58 in the CPU path's rules: column c of act = Q8_2_X4(swiglu(g, u)) over the k
// values g[c * k ..], u[c * k ..]. One half wave a 32-value block.
__global__ __launch_bounds__(256) void k_swiglu_quant(const float *g, const float *u, int m, int k, uint8_t *act,
                                                      GateRule rule, u32 *fault, u32 layer) {
    const int bpc = k / 32;
    const long gblk = (long)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (gblk >= (long)m * bpc) return;
    const int col = (int)(gblk / bpc), blk = (int)(gblk % bpc), lane32 = threadIdx.x & 31;
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

hipError_t swiglu_quant(const Launch &L, const float *g, const float *u, int m, int k, uint8_t *act) {
    const long blocks = (long)m * (k / 32);
    hipLaunchKernelGGL(k_swiglu_quant, dim3((unsigned)((blocks + 7) / 8)), dim3(256), 0, L.stream, g, u, m, k, act,
                       L.rule, L.fault, L.layer);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------- GEMM

// LDS of one workgroup: a super-block of the tile's 64 activation columns and of the slab's 64 weight rows, and the
// rows' scale products. Strides are padded off the 128-byte bank period.
constexpr int kActSb = BM_Q82_SB_REF + 64;   // a column's super-block: its two groups and its (d8, d8 * isum) pairs
constexpr int kActStride = kActSb + 8;       // 360
template <int WT>
__host__ __device__ constexpr int wt_stride() {
    return WT == BM_Q4K ? 152 : 232; // 144 and 224 (14 chunks of 16) padded
}
template <int WT>
__host__ __device__ constexpr int wt_chunks() {
    return WT == BM_Q4K ? 9 : 14;
}

struct GemmLds {
    u32 col[kGemmBN];  // the tile's activation columns
    u32 slot[kGemmBN]; // and slots
};

template <int WT>
__host__ __device__ constexpr size_t gemm_lds_bytes() {
    return sizeof(GemmLds) + (size_t)kGemmBN * kActStride + (size_t)kGemmBM * wt_stride<WT>() + 16 * kGemmBM * sizeof(float);
}

// Workgroup b of a GEMM grid: tile and row slab. Workgroups go to the chip's eight dies in turn (b to die b % 8,
// each with its own L2), so a tile's row slabs are consecutive workgroups of one die: the tile's activation columns
// come from memory once and serve all the slabs from that L2. The grid is 8 * ceil(tiles / 8) * n_slabs workgroups.
__device__ __forceinline__ u32 tile_of_block(u32 b, u32 n_slabs) { return ((b >> 3) / n_slabs) * 8 + (b & 7); }
__device__ __forceinline__ u32 slab_of_block(u32 b, u32 n_slabs) { return (b >> 3) % n_slabs; }

// (q6 - 32) of four codes a word, as signed bytes: q6 in 0..63.
__device__ __forceinline__ u32 q6_minus_32(u32 q) {
    const u32 t = q ^ 0x20202020u;        // q >= 32: q - 32; q < 32: q + 32
    const u32 m = ~q & 0x20202020u;       // the bytes that went up: they want -64, the two top bits
    return t | (m << 1) | (m << 2);
}

// A workgroup of 1024 / T threads takes a tile of <= 64 slots and a slab of 64 rows. Wave w works on rows
// 16 * (w & 3) .. and slots 16 T * (w >> 2) ..: T 16 x 16 products a 32-value block and half. v_mfma_i32_16x16x32_i8 sums over 32
// values; a 16-value half comes out of it by zeroing the other half's weight codes, the lanes of one half of the
// k range holding them (lane / 16 = k / 8). 4 T results a lane, 32 T accumulators: two to four waves a SIMD
// stay resident and hide each other's LDS and matrix latencies.
template <int WT, int T>
__global__ __launch_bounds__(1024 / T) void k_gemm(const uint8_t *w, int rpe, int nb, const uint8_t *act, const u32 *cols,
                                                 const u32 *tiles, const u32 *n_tiles, u32 n_slabs, u32 slot_div,
                                                 u32 n_slots, float *y) {
    extern __shared__ __align__(16) uint8_t lds[];
    GemmLds *tab = reinterpret_cast<GemmLds *>(lds);
    uint8_t *acts = lds + sizeof(GemmLds);
    uint8_t *wts = acts + (size_t)kGemmBN * kActStride;
    float *rs = reinterpret_cast<float *>(wts + (size_t)kGemmBM * wt_stride<WT>()); // [16][64]
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const u32 g = tile_of_block(blockIdx.x, n_slabs);
    const int row0 = (int)slab_of_block(blockIdx.x, n_slabs) * kGemmBM;
    const u32 count = n_tiles[0];
    if (g > count) return;
    if (g == count) { // the refused slots' rows: NaN (crates/gpu/src/gemm/grouped.rs:2283-2287)
        const u32 refused = n_tiles[1];
        for (u32 i = tid; i < refused * kGemmBM; i += blockDim.x) {
            const u32 s = cols[n_slots - refused + i / kGemmBM];
            const int r = row0 + (int)(i % kGemmBM);
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
    constexpr int kBlock = WT == BM_Q4K ? BM_Q4K_BLOCK : BM_Q6K_BLOCK;
    constexpr int kWc = wt_chunks<WT>();
    const size_t row_bytes = (size_t)nb * kBlock;
    const int col_bytes = nb * BM_Q82_SB_EXT;
    // staging: kGemmBN * 22 chunks of 16 bytes of activations, kGemmBM * kWc of weights, a super-block
    constexpr int kAc = kActSb / 16; // 22
    constexpr int kThreads = 1024 / T; // 16 / T waves: four row groups x (4 / T) slot groups of 16 T slots
    constexpr int kActLoads = (kGemmBN * kAc + kThreads - 1) / kThreads, kWtLoads = (kGemmBM * kWc + kThreads - 1) / kThreads;
    uint4 ra[kActLoads], rw[kWtLoads];
    auto fetch = [&](int i) {
#pragma unroll
        for (int t = 0; t < kActLoads; t++) {
            int c = t * kThreads + tid;
            c = c < kGemmBN * kAc ? c : kGemmBN * kAc - 1;
            const int n = c / kAc, k = c % kAc;
            const uint8_t *colp = act + (size_t)tab->col[n] * col_bytes;
            const uint8_t *src = k < 18 ? colp + (size_t)i * BM_Q82_SB_REF + 16 * k
                                        : colp + (size_t)nb * BM_Q82_SB_REF + (size_t)i * 64 + 16 * (k - 18);
            ra[t] = *reinterpret_cast<const uint4 *>(src);
        }
#pragma unroll
        for (int t = 0; t < kWtLoads; t++) {
            int c = t * kThreads + tid;
            c = c < kGemmBM * kWc ? c : kGemmBM * kWc - 1;
            int r = row0 + c / kWc;
            const int k = c % kWc;
            r = r < rpe ? r : rpe - 1;
            const uint8_t *blk = w + ((size_t)e * rpe + r) * row_bytes + (size_t)i * kBlock;
            // Q6_K: 210 bytes are 13 chunks and a last one that ends with the block (bytes 194 .. 210)
            rw[t] = bm_ld16u(blk + ((WT == BM_Q6K && k == 13) ? 194 : 16 * k));
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int t = 0; t < kActLoads; t++) {
            const int c = t * kThreads + tid;
            if (c < kGemmBN * kAc) {
                uint8_t *dst = acts + (c / kAc) * kActStride + 16 * (c % kAc);
                *reinterpret_cast<uint2 *>(dst) = make_uint2(ra[t].x, ra[t].y);
                *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(ra[t].z, ra[t].w);
            }
        }
#pragma unroll
        for (int t = 0; t < kWtLoads; t++) {
            const int c = t * kThreads + tid;
            if (c < kGemmBM * kWc) {
                uint8_t *dst = wts + (c / kWc) * wt_stride<WT>() + 16 * (c % kWc);
                *reinterpret_cast<uint2 *>(dst) = make_uint2(rw[t].x, rw[t].y);
                *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(rw[t].z, rw[t].w);
            }
        }
    };
    // this lane in its wave's two 16 x 16 products: operand row / slot lane % 16, values 8 * (lane / 16) .. + 8 of
    // a 32-value block; its four results of each product are rows 4 * (lane / 16) + v of slot lane % 16
    const int rg = wv & 3, ch = wv >> 2, l16 = lane & 15, kg = lane >> 4;
    const uint8_t *my_act[T];
#pragma unroll
    for (int t = 0; t < T; t++) my_act[t] = acts + (16 * T * ch + 16 * t + l16) * kActStride;
    const uint8_t *my_wt = wts + (16 * rg + l16) * wt_stride<WT>();
    const int rbase = 16 * rg + 4 * kg; // result v sits in row rbase + v of the slab
    const u32 keep[2] = {kg < 2 ? 0xffffffffu : 0u, kg < 2 ? 0u : 0xffffffffu}; // this lane's codes are of half kg / 2
    float acc[T][4][8];
#pragma unroll
    for (int t = 0; t < T; t++)
#pragma unroll
        for (int v = 0; v < 4; v++)
#pragma unroll
            for (int l = 0; l < 8; l++) acc[t][v][l] = 0.0f;

    fetch(0);
    for (int i = 0; i < nb; i++) {
        __syncthreads(); // the previous super-block's readers are done
        stash();
        __syncthreads();
        if (i + 1 < nb) fetch(i + 1);
        // the rows' scale products: rs[s][row]
        {
            const int r = (tid >> 3) & 63, part = tid & 7;
            const uint8_t *blk = wts + r * wt_stride<WT>();
            if (tid < 512) {
                if constexpr (WT == BM_Q4K) {
                    const float d = bm_half_to_f32(*reinterpret_cast<const unsigned short *>(blk));
                    const float dmin = bm_half_to_f32(*reinterpret_cast<const unsigned short *>(blk + 2));
                    const uint8_t *sc = blk + 4;
                    const int s = part; // crates/gguf/src/quant.rs:620-628 get_scale_min_k4
                    int scv, mv;
                    if (s < 4) {
                        scv = sc[s] & 63;
                        mv = sc[s + 4] & 63;
                    } else {
                        scv = (sc[s + 4] & 15) | ((sc[s - 4] >> 6) << 4);
                        mv = (sc[s + 4] >> 4) | ((sc[s] >> 6) << 4);
                    }
                    rs[s * kGemmBM + r] = d * (float)scv;
                    rs[(8 + s) * kGemmBM + r] = -(dmin * (float)mv);
                } else {
                    const float d = bm_half_to_f32(*reinterpret_cast<const unsigned short *>(blk + 222));
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        const int gq = 2 * part + t;
                        rs[gq * kGemmBM + r] = d * (float)(int)(signed char)blk[192 + gq];
                    }
                }
            }
        }
        __syncthreads();
        if (16 * T * ch >= len) continue; // none of this wave's slots is real (the barriers above are the loop's only ones)
        const float2 *pair[T]; // (d8, d8 * isum) a 32-block
#pragma unroll
        for (int t = 0; t < T; t++) pair[t] = reinterpret_cast<const float2 *>(my_act[t] + BM_Q82_SB_REF);
        if constexpr (WT == BM_Q4K) {
            // the min terms first: accumulator l takes sub-block l's (crates/qdot/src/lib.rs:4389-4394)
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const float4 mn = *reinterpret_cast<const float4 *>(&rs[(8 + s) * kGemmBM + rbase]);
#pragma unroll
                for (int t = 0; t < T; t++) {
                    const float my = pair[t][s].y;
                    acc[t][0][s] = fmaf(my, mn.x, acc[t][0][s]);
                    acc[t][1][s] = fmaf(my, mn.y, acc[t][1][s]);
                    acc[t][2][s] = fmaf(my, mn.z, acc[t][2][s]);
                    acc[t][3][s] = fmaf(my, mn.w, acc[t][3][s]);
                }
            }
#pragma unroll
            for (int p = 0; p < 4; p++) { // code bytes 32p ..: low nibbles sub-block 2p, high nibbles 2p + 1
                const uint2 wq = *reinterpret_cast<const uint2 *>(my_wt + 16 + 32 * p + 8 * kg);
#pragma unroll
                for (int en = 0; en < 2; en++) {
                    const int s = 2 * p + en;
                    const u32 ax = (wq.x >> (4 * en)) & 0x0f0f0f0fu, ay = (wq.y >> (4 * en)) & 0x0f0f0f0fu;
                    const float4 sv = *reinterpret_cast<const float4 *>(&rs[s * kGemmBM + rbase]);
                    float f[T][4];
                    long b[T];
#pragma unroll
                    for (int t = 0; t < T; t++) {
                        const float d8 = pair[t][s].x;
                        f[t][0] = sv.x * d8;
                        f[t][1] = sv.y * d8;
                        f[t][2] = sv.z * d8;
                        f[t][3] = sv.w * d8;
                        const uint2 bq = *reinterpret_cast<const uint2 *>(my_act[t] + (s >> 2) * BM_Q82X4_STRIDE + 16 +
                                                                          32 * (s & 3) + 8 * kg);
                        b[t] = (long)(((unsigned long long)bq.y << 32) | bq.x);
                    }
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const long a = (long)(((unsigned long long)(ay & keep[h]) << 32) | (ax & keep[h]));
                        const int l = 4 * h + (s & 3);
#pragma unroll
                        for (int t = 0; t < T; t++) {
                            const v4i z = {0, 0, 0, 0};
                            const v4i sum = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b[t], z, 0, 0, 0);
#pragma unroll
                            for (int v = 0; v < 4; v++) acc[t][v][l] = fmaf(f[t][v], (float)sum[v], acc[t][v][l]);
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int bk = 0; bk < 8; bk++) { // 32-block bk of the super-block: quarter bk % 4 of half bk / 4
                const int c2 = bk >> 2, a4 = bk & 3;
                const uint2 ql = *reinterpret_cast<const uint2 *>(my_wt + 64 * c2 + 32 * (a4 & 1) + 8 * kg);
                const uint2 qh = *reinterpret_cast<const uint2 *>(my_wt + 128 + 32 * c2 + 8 * kg);
                const int ns = 4 * (a4 >> 1), hs = 2 * a4;
                const u32 ax = q6_minus_32(((ql.x >> ns) & 0x0f0f0f0fu) | (((qh.x >> hs) & 0x03030303u) << 4));
                const u32 ay = q6_minus_32(((ql.y >> ns) & 0x0f0f0f0fu) | (((qh.y >> hs) & 0x03030303u) << 4));
                long b[T];
                float d8[T];
#pragma unroll
                for (int t = 0; t < T; t++) {
                    const uint2 bq = *reinterpret_cast<const uint2 *>(my_act[t] + (bk >> 2) * BM_Q82X4_STRIDE + 16 + 32 * (bk & 3) +
                                                                      8 * kg);
                    b[t] = (long)(((unsigned long long)bq.y << 32) | bq.x);
                    d8[t] = pair[t][bk].x;
                }
#pragma unroll
                for (int hh = 0; hh < 2; hh++) { // 16-value group 2 bk + hh
                    const long a = (long)(((unsigned long long)(ay & keep[hh]) << 32) | (ax & keep[hh]));
                    const float4 sv = *reinterpret_cast<const float4 *>(&rs[(2 * bk + hh) * kGemmBM + rbase]);
                    const int l = 4 * hh + (bk & 3); // crates/qdot/src/lib.rs:4794-4809
#pragma unroll
                    for (int t = 0; t < T; t++) {
                        const v4i z = {0, 0, 0, 0};
                        const v4i sum = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b[t], z, 0, 0, 0);
                        acc[t][0][l] = fmaf(sv.x * d8[t], (float)sum[0], acc[t][0][l]);
                        acc[t][1][l] = fmaf(sv.y * d8[t], (float)sum[1], acc[t][1][l]);
                        acc[t][2][l] = fmaf(sv.z * d8[t], (float)sum[2], acc[t][2][l]);
                        acc[t][3][l] = fmaf(sv.w * d8[t], (float)sum[3], acc[t][3][l]);
                    }
                }
            }
        }
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

// The same product with one accumulator a value: each 32-value block's integer sum (Q4_K: two chained matrix
// instructions) or 16-value group's (Q6_K) is scaled and added in increasing k, a block's min term just before it.
// The integers are the exact ones; the f32 sum is not in the CPU path's eight-lane order, so a value differs from
// the exact kernel's by rounding only (a few 1e-7 of the row's magnitude; the contract's tolerance is 1e-4). A third
// fewer vector operations and an eighth of the accumulator registers: 32 x 32 tiles, four waves, several
// workgroups a CU.
typedef int v16i __attribute__((ext_vector_type(16)));

template <int WT>
__global__ __launch_bounds__(256) void k_gemm_fast(const uint8_t *w, int rpe, int nb, const uint8_t *act, const u32 *cols,
                                                   const u32 *tiles, const u32 *n_tiles, u32 n_slabs, u32 slot_div,
                                                   u32 n_slots, float *y) {
    extern __shared__ __align__(16) uint8_t lds[];
    GemmLds *tab = reinterpret_cast<GemmLds *>(lds);
    uint8_t *acts = lds + sizeof(GemmLds);
    uint8_t *wts = acts + (size_t)kGemmBN * kActStride;
    float *rs = reinterpret_cast<float *>(wts + (size_t)kGemmBM * wt_stride<WT>()); // [16][64]
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const u32 g = tile_of_block(blockIdx.x, n_slabs);
    const int row0 = (int)slab_of_block(blockIdx.x, n_slabs) * kGemmBM;
    const u32 count = n_tiles[0];
    if (g > count) return;
    if (g == count) {
        const u32 refused = n_tiles[1];
        for (u32 i = tid; i < refused * kGemmBM; i += blockDim.x) {
            const u32 s = cols[n_slots - refused + i / kGemmBM];
            const int r = row0 + (int)(i % kGemmBM);
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
    constexpr int kBlock = WT == BM_Q4K ? BM_Q4K_BLOCK : BM_Q6K_BLOCK;
    constexpr int kWc = wt_chunks<WT>();
    const size_t row_bytes = (size_t)nb * kBlock;
    const int col_bytes = nb * BM_Q82_SB_EXT;
    constexpr int kAc = kActSb / 16; // 22
    constexpr int kActLoads = (kGemmBN * kAc + 255) / 256, kWtLoads = (kGemmBM * kWc + 255) / 256;
    uint4 ra[kActLoads], rw[kWtLoads];
    auto fetch = [&](int i) {
#pragma unroll
        for (int t = 0; t < kActLoads; t++) {
            int c = t * 256 + tid;
            c = c < kGemmBN * kAc ? c : kGemmBN * kAc - 1;
            const int n = c / kAc, k = c % kAc;
            const uint8_t *colp = act + (size_t)tab->col[n] * col_bytes;
            const uint8_t *src = k < 18 ? colp + (size_t)i * BM_Q82_SB_REF + 16 * k
                                        : colp + (size_t)nb * BM_Q82_SB_REF + (size_t)i * 64 + 16 * (k - 18);
            ra[t] = *reinterpret_cast<const uint4 *>(src);
        }
#pragma unroll
        for (int t = 0; t < kWtLoads; t++) {
            int c = t * 256 + tid;
            c = c < kGemmBM * kWc ? c : kGemmBM * kWc - 1;
            int r = row0 + c / kWc;
            const int k = c % kWc;
            r = r < rpe ? r : rpe - 1;
            const uint8_t *blk = w + ((size_t)e * rpe + r) * row_bytes + (size_t)i * kBlock;
            rw[t] = bm_ld16u(blk + ((WT == BM_Q6K && k == 13) ? 194 : 16 * k));
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int t = 0; t < kActLoads; t++) {
            const int c = t * 256 + tid;
            if (c < kGemmBN * kAc) {
                uint8_t *dst = acts + (c / kAc) * kActStride + 16 * (c % kAc);
                *reinterpret_cast<uint2 *>(dst) = make_uint2(ra[t].x, ra[t].y);
                *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(ra[t].z, ra[t].w);
            }
        }
#pragma unroll
        for (int t = 0; t < kWtLoads; t++) {
            const int c = t * 256 + tid;
            if (c < kGemmBM * kWc) {
                uint8_t *dst = wts + (c / kWc) * wt_stride<WT>() + 16 * (c % kWc);
                *reinterpret_cast<uint2 *>(dst) = make_uint2(rw[t].x, rw[t].y);
                *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(rw[t].z, rw[t].w);
            }
        }
    };
    // v_mfma_i32_32x32x16_i8: operand row / slot lane % 32, values 8 * (lane / 32) .. + 8 of a 16-value group; result v
    // is row 8 * (v / 4) + 4 * (lane / 32) + v % 4 of slot lane % 32
    const int wr = wv & 1, wc = wv >> 1, l32 = lane & 31, kh = lane >> 5;
    const uint8_t *my_act = acts + (32 * wc + l32) * kActStride;
    const uint8_t *my_wt = wts + (32 * wr + l32) * wt_stride<WT>();
    const int rbase = 32 * wr + 4 * kh;
    float acc[16];
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;

    fetch(0);
    for (int i = 0; i < nb; i++) {
        __syncthreads();
        stash();
        __syncthreads();
        if (i + 1 < nb) fetch(i + 1);
        {
            const int r = tid >> 2, part = tid & 3;
            const uint8_t *blk = wts + r * wt_stride<WT>();
            if constexpr (WT == BM_Q4K) {
                const float d = bm_half_to_f32(*reinterpret_cast<const unsigned short *>(blk));
                const float dmin = bm_half_to_f32(*reinterpret_cast<const unsigned short *>(blk + 2));
                const uint8_t *sc = blk + 4;
#pragma unroll
                for (int t = 0; t < 2; t++) { // crates/gguf/src/quant.rs:620-628 get_scale_min_k4
                    const int s = 2 * part + t;
                    int scv, mv;
                    if (s < 4) {
                        scv = sc[s] & 63;
                        mv = sc[s + 4] & 63;
                    } else {
                        scv = (sc[s + 4] & 15) | ((sc[s - 4] >> 6) << 4);
                        mv = (sc[s + 4] >> 4) | ((sc[s] >> 6) << 4);
                    }
                    rs[s * kGemmBM + r] = d * (float)scv;
                    rs[(8 + s) * kGemmBM + r] = -(dmin * (float)mv);
                }
            } else {
                const float d = bm_half_to_f32(*reinterpret_cast<const unsigned short *>(blk + 222));
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const int gq = 4 * part + t;
                    rs[gq * kGemmBM + r] = d * (float)(int)(signed char)blk[192 + gq];
                }
            }
        }
        __syncthreads();
        if (32 * wc >= len) continue; // none of this wave's slots is real (the barriers above are the loop's only ones)
        const float2 *pair = reinterpret_cast<const float2 *>(my_act + BM_Q82_SB_REF);
        if constexpr (WT == BM_Q4K) {
#pragma unroll
            for (int p = 0; p < 4; p++) {
                uint2 wq[2];
#pragma unroll
                for (int h = 0; h < 2; h++) wq[h] = *reinterpret_cast<const uint2 *>(my_wt + 16 + 32 * p + 16 * h + 8 * kh);
#pragma unroll
                for (int en = 0; en < 2; en++) {
                    const int s = 2 * p + en;
                    v16i sum = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const u32 ax = (wq[h].x >> (4 * en)) & 0x0f0f0f0fu, ay = (wq[h].y >> (4 * en)) & 0x0f0f0f0fu;
                        const uint2 bq = *reinterpret_cast<const uint2 *>(my_act + (s >> 2) * BM_Q82X4_STRIDE + 16 +
                                                                          32 * (s & 3) + 16 * h + 8 * kh);
                        sum = __builtin_amdgcn_mfma_i32_32x32x16_i8((long)(((unsigned long long)ay << 32) | ax),
                                                                    (long)(((unsigned long long)bq.y << 32) | bq.x), sum, 0, 0, 0);
                    }
                    const float d8 = pair[s].x, my = pair[s].y;
#pragma unroll
                    for (int qd = 0; qd < 4; qd++) {
                        const float4 mn = *reinterpret_cast<const float4 *>(&rs[(8 + s) * kGemmBM + rbase + 8 * qd]);
                        const float4 sv = *reinterpret_cast<const float4 *>(&rs[s * kGemmBM + rbase + 8 * qd]);
                        acc[4 * qd + 0] = fmaf(sv.x * d8, (float)sum[4 * qd + 0], fmaf(my, mn.x, acc[4 * qd + 0]));
                        acc[4 * qd + 1] = fmaf(sv.y * d8, (float)sum[4 * qd + 1], fmaf(my, mn.y, acc[4 * qd + 1]));
                        acc[4 * qd + 2] = fmaf(sv.z * d8, (float)sum[4 * qd + 2], fmaf(my, mn.z, acc[4 * qd + 2]));
                        acc[4 * qd + 3] = fmaf(sv.w * d8, (float)sum[4 * qd + 3], fmaf(my, mn.w, acc[4 * qd + 3]));
                    }
                }
            }
        } else {
#pragma unroll
            for (int gq = 0; gq < 16; gq++) {
                const int c2 = gq >> 3, a4 = (gq & 7) >> 1, hh = gq & 1, bk = gq >> 1;
                const int l0 = 16 * hh + 8 * kh;
                const uint2 ql = *reinterpret_cast<const uint2 *>(my_wt + 64 * c2 + 32 * (a4 & 1) + l0);
                const uint2 qh = *reinterpret_cast<const uint2 *>(my_wt + 128 + 32 * c2 + l0);
                const int ns = 4 * (a4 >> 1), hs = 2 * a4;
                const u32 ax = q6_minus_32(((ql.x >> ns) & 0x0f0f0f0fu) | (((qh.x >> hs) & 0x03030303u) << 4));
                const u32 ay = q6_minus_32(((ql.y >> ns) & 0x0f0f0f0fu) | (((qh.y >> hs) & 0x03030303u) << 4));
                const uint2 bq = *reinterpret_cast<const uint2 *>(my_act + (bk >> 2) * BM_Q82X4_STRIDE + 16 + 32 * (bk & 3) +
                                                                  16 * hh + 8 * kh);
                const float d8 = pair[bk].x;
                const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const v16i sum = __builtin_amdgcn_mfma_i32_32x32x16_i8((long)(((unsigned long long)ay << 32) | ax),
                                                                       (long)(((unsigned long long)bq.y << 32) | bq.x), z, 0, 0, 0);
#pragma unroll
                for (int qd = 0; qd < 4; qd++) {
                    const float4 sv = *reinterpret_cast<const float4 *>(&rs[gq * kGemmBM + rbase + 8 * qd]);
                    acc[4 * qd + 0] = fmaf(sv.x * d8, (float)sum[4 * qd + 0], acc[4 * qd + 0]);
                    acc[4 * qd + 1] = fmaf(sv.y * d8, (float)sum[4 * qd + 1], acc[4 * qd + 1]);
                    acc[4 * qd + 2] = fmaf(sv.z * d8, (float)sum[4 * qd + 2], acc[4 * qd + 2]);
                    acc[4 * qd + 3] = fmaf(sv.w * d8, (float)sum[4 * qd + 3], acc[4 * qd + 3]);
                }
            }
        }
    }
    const int n = 32 * wc + l32;
    if (n < len) {
        const size_t out = (size_t)tab->slot[n] * rpe + row0;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int r = rbase + 8 * (v >> 2) + (v & 3);
            if (row0 + r < rpe) y[out + r] = acc[v];
        }
    }
}

bool gemm_supported(int wtype) { return wtype == BM_Q4K || wtype == BM_Q6K; }

hipError_t gemm(const Launch &L, int wtype, const uint8_t *w, int n_experts, int rows_per_expert, int k,
                const uint8_t *act, const uint32_t *cols, const uint32_t *tiles_dev, const uint32_t *n_tiles, int n_slots,
                int slot_div, float *y, int mode) {
    const int nb = k / 256;
    const u32 max_tiles = (u32)gemm_max_tiles(n_slots, n_experts) + 1; // one more: the block that fills refused slots
    const u32 n_slabs = (u32)((rows_per_expert + kGemmBM - 1) / kGemmBM);
    const unsigned grid = ((max_tiles + 7) / 8) * 8 * n_slabs;
    auto launch = [&](auto kern, unsigned threads, size_t lds) {
        hipError_t e = allow_lds(kern, lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, L.stream, w, rows_per_expert, nb, act, cols, tiles_dev, n_tiles,
                           n_slabs, (u32)slot_div, (u32)n_slots, y);
        return hipGetLastError();
    };
    if (mode == 1) {
        if (wtype == BM_Q4K) return launch(k_gemm_fast<BM_Q4K>, 256, gemm_lds_bytes<BM_Q4K>());
        if (wtype == BM_Q6K) return launch(k_gemm_fast<BM_Q6K>, 256, gemm_lds_bytes<BM_Q6K>());
        return hipErrorInvalidValue;
    }
    // slot groups of 16 a wave (T): 1 -> 1024 threads a workgroup, 2 -> 512; the faster of the two for each type
    if (wtype == BM_Q4K) return launch(k_gemm<BM_Q4K, 1>, 1024, gemm_lds_bytes<BM_Q4K>());
    if (wtype == BM_Q6K) return launch(k_gemm<BM_Q6K, 2>, 512, gemm_lds_bytes<BM_Q6K>());
    return hipErrorInvalidValue;
}

} // namespace bmk
