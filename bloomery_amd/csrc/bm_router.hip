// The softmax router over given logits (crates/gpu/src/route_softmax.rs:1203 softmax_router_route, the routing body
// :177 route_warp): a token's probabilities, its top `used` experts by probability and their weights, renormalised
// to sum to one when the model's rule says so.
//
// Numbers, op for op (crates/model/src/moe.rs:246-279, crates/gpu/src/route_softmax.rs:38-51): the max of the logits
// (exact, any order); exp(logit - max) in f32; the sum of the exps in f64; each probability the f32 divide by the sum
// rounded to f32; the top `used` by descending probability, ties toward the smaller id; the chosen probabilities
// summed in f64 in slot order, rounded once, each weight the f32 divide of its probability by it.
// exp: the CPU path's is the host library's expf, correctly rounded in all but rare cases; here exp in f64 rounded to
// f32, which is the correctly rounded value in all but rare cases too. The f64 sums are taken lane by lane and then
// over the lanes (the order the reference's launch takes them in); they differ from a serial sum below 2^-50 of the
// sum, which its rounding to f32 hides except on an exact tie of that rounding.
//
// A token with a logit that is not finite has no defined routing: it raises Router on the fault word, gets NaN
// probabilities and weights, and keeps its ids as they stand (crates/gpu/src/route_softmax.rs:53-62).
#include "bm_stream.hpp"

namespace bmk {

// Timeline of the router launch, in measurement builds only (-DBM_TIMELINE, the library bench.py --timeline loads): thread 0 of
// workgroup b keeps the device's constant-rate counter (100 MHz) in registers at six points of router_logits_body and stores
// them at its end in row b: start, the token's row arrived, normed, rows and token in LDS (behind the barrier), dots done,
// the routing done (the workgroup that routes).
#ifdef BM_TIMELINE
constexpr int kRouterTimelineRows = 1024;
__device__ unsigned long long g_router_timeline[kRouterTimelineRows * 8];
#define BM_RTICK(var, dep)                                                                                             \
    do {                                                                                                               \
        __asm__ volatile("" ::"v"(dep) : "memory");                                                                    \
        var = wall_clock64();                                                                                          \
    } while (0)
#define BM_RTOCK(mark, var)                                                                                            \
    do {                                                                                                               \
        if (threadIdx.x == 0 && blockIdx.x < (unsigned)kRouterTimelineRows) g_router_timeline[blockIdx.x * 8 + (mark)] = var; \
    } while (0)
#else
#define BM_RTICK(var, dep)                                                                                             \
    do {                                                                                                               \
    } while (0)
#define BM_RTOCK(mark, var)                                                                                            \
    do {                                                                                                               \
    } while (0)
#endif


constexpr u32 kSiteRouter = 5; // crates/device/src/fault.rs:84-86

// Sum / maximum over the wave, every lane ending with it: pairs, quads, eights and sixteens by data-parallel-primitive moves
// (a few cycles each, where a shuffle through the LDS crossbar is a hundred), the two sixteens of a half by one swizzle, the
// halves by two lane reads. The sum's association: ((pairs) quads) ... halves, lower half first.
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v) {
    return __hiloint2double((int)bm_dpp<CTRL>((u32)__double2hiint(v)), (int)bm_dpp<CTRL>((u32)__double2loint(v)));
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    v += dpp_f64<kDppXor1>(v);
    v += dpp_f64<kDppXor2>(v);
    v += dpp_f64<kDppHalfMirror>(v);
    v += dpp_f64<kDppMirror>(v);
    v += __hiloint2double((int)bm_swap16((u32)__double2hiint(v)), (int)bm_swap16((u32)__double2loint(v)));
    const int lo = __double2loint(v), hi = __double2hiint(v);
    const double a = __hiloint2double(__builtin_amdgcn_readlane(hi, 0), __builtin_amdgcn_readlane(lo, 0));
    const double b = __hiloint2double(__builtin_amdgcn_readlane(hi, 32), __builtin_amdgcn_readlane(lo, 32));
    return a + b;
}
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, bm_dppf<kDppXor1>(v));
    v = fmaxf(v, bm_dppf<kDppXor2>(v));
    v = fmaxf(v, bm_dppf<kDppHalfMirror>(v));
    v = fmaxf(v, bm_dppf<kDppMirror>(v));
    v = fmaxf(v, bm_bits_f32(bm_swap16(bm_f32_bits(v))));
    const int bits = (int)bm_f32_bits(v);
    return fmaxf(bm_bits_f32((u32)__builtin_amdgcn_readlane(bits, 0)), bm_bits_f32((u32)__builtin_amdgcn_readlane(bits, 32)));
}

// Token t's routing by one wave; lane L owns experts L + 64 j, j < PER. `v`: this lane's logits, expert lane + 64 j in v[j]
// (-inf past n_exp). First the probabilities (p[j]; stored if asked for): false, with NaN probabilities and weights and
// BM_SITE_ROUTER raised, when a logit is not finite.
template <int PER>
__device__ __forceinline__ bool route_probs_wave(const float (&v)[PER], u32 t, u32 n_exp, u32 used, float *probs, float *weights,
                                                 u32 *fault, u32 layer, float (&p)[PER]) {
    const u32 lane = threadIdx.x & 63;
    bool odd = false;
#pragma unroll
    for (int j = 0; j < PER; j++) odd |= lane + 64 * j < n_exp && !(fabsf(v[j]) <= 3.402823466e38f);
    if (__ballot(odd) != 0) {
        const float nan = bm_bits_f32(0x7fc00000u);
        if (probs) {
#pragma unroll
            for (int j = 0; j < PER; j++)
                if (lane + 64 * j < n_exp) probs[(size_t)t * n_exp + lane + 64 * j] = nan;
        }
        if (lane < used) weights[(size_t)t * used + lane] = nan;
        if (lane == 0) bm_raise(fault, layer, kSiteRouter);
        return false;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; j++) mx = fmaxf(mx, v[j]);
    mx = wave_max_f32(mx);
    [[maybe_unused]] unsigned long long tl_a = 0, tl_b = 0, tl_c = 0;
    BM_RTICK(tl_a, mx);
    double sum = 0.0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        p[j] = lane + 64 * j < n_exp ? (float)exp((double)(v[j] - mx)) : 0.0f;
        sum += (double)p[j];
    }
    sum = wave_sum_f64(sum);
    BM_RTICK(tl_b, sum);
    const float inv = (float)sum;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        p[j] = p[j] / inv;
        if (probs && lane + 64 * j < n_exp) probs[(size_t)t * n_exp + lane + 64 * j] = p[j];
    }
    BM_RTICK(tl_c, p[0]);
    BM_RTOCK(1, tl_a);
    BM_RTOCK(2, tl_b);
    BM_RTOCK(3, tl_c);
    return true;
}

// Then the picks, by the wave alone: `used` rounds of a wave argmax under (probability descending, id ascending): the
// largest probability left (its bits order as its value: not negative) as one unsigned maximum over the wave, then the
// smallest id that holds it: expert lane + 64 j, so the first j with a holder and that ballot's lowest lane. The winning
// lane marks its entry.
template <int PER>
__device__ __forceinline__ void route_pick_rounds(const float (&p)[PER], u32 t, u32 n_exp, u32 used, u32 renorm, u32 *ids,
                                                  float *weights) {
    const u32 lane = threadIdx.x & 63;
    u32 taken = 0;
    double chosen = 0.0;
    float mine = 0.0f;
    for (u32 s = 0; s < used; s++) {
        u32 best = 0;
        bool any = false;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const bool open = lane + 64 * j < n_exp && !((taken >> j) & 1u);
            const u32 bits = bm_f32_bits(p[j]);
            best = open && bits > best ? bits : best;
            any |= open;
        }
        const u32 half = bm_max32(best);
        const u32 m0 = (u32)__builtin_amdgcn_readlane((int)half, 0), m1 = (u32)__builtin_amdgcn_readlane((int)half, 32);
        const u32 top = m0 > m1 ? m0 : m1;
        u32 bi = 0xffffffffu; // none left
        if (__ballot(any) != 0) {
#pragma unroll
            for (int j = PER - 1; j >= 0; j--) {
                const bool open = lane + 64 * j < n_exp && !((taken >> j) & 1u);
                const unsigned long long holders = __ballot(open && bm_f32_bits(p[j]) == top);
                if (holders) bi = (u32)(64 * j + __builtin_ctzll(holders)); // uniform; the smallest j wins: it comes last
            }
        }
        const float bv = bi != 0xffffffffu ? bm_bits_f32(top) : 0.0f;
        if ((bi & 63u) == lane && bi != 0xffffffffu) taken |= 1u << (bi >> 6);
        if (lane == 0) ids[(size_t)t * used + s] = bi;
        chosen += (double)bv;
        if (lane == s) mine = bv;
    }
    if (lane < used) weights[(size_t)t * used + lane] = renorm ? mine / (float)chosen : mine;
}

template <int PER>
__device__ __forceinline__ void route_softmax_wave(const float (&v)[PER], u32 t, u32 n_exp, u32 used, u32 renorm, float *probs,
                                                   u32 *ids, float *weights, u32 *fault, u32 layer) {
    float p[PER];
    if (route_probs_wave<PER>(v, t, n_exp, used, probs, weights, fault, layer, p)) route_pick_rounds<PER>(p, t, n_exp, used, renorm, ids, weights);
}

// The same picks by a workgroup of 256 threads for up to 256 experts (n_exp >= used), the probabilities in LDS: an entry's
// place in the order (probability descending, id ascending) is the number of entries ahead of it, counted by comparing it
// with every other - independent instructions spread over four waves, where the wave's rounds are a chain of some eighty
// dependent ones each (2.0 us of a 2.6 us routing at 128 experts, 8 picks). What is counted is the entries not smaller
// (one compare and one add with carry an entry; probabilities are not negative, so their bits order as signed integers,
// and the places past n_exp hold -1): without the entry itself that is its place unless another entry has its bits, and then
// some place below `used` is taken twice or not at all - seen by counting the takers of every place - and the first wave
// picks by its rounds instead. The entry with `s` ahead of it is pick s: the rounds' ids, and the same weights from the
// same sums (the chosen probabilities added in pick order).
// A barrier that waits for the wave's LDS traffic only: the routing workgroup's waves meet over LDS while the first wave's
// stores to memory (the words armed again, the probabilities) are still on their way, and a barrier that waited for those to
// be acknowledged cost the routing 1 us.
__device__ __forceinline__ void lds_barrier() { __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

struct PickLds {
    __align__(16) float p[256];      // entry e's probability, -1 past n_exp
    u32 ahead[256];    // zero on entry
    u32 takers[32];    // zero on entry
    u32 pick_id[32];
    __align__(16) float pick_p[32];
    u32 ok;
};
// Every thread of the workgroup calls it; true: the picks are written; false (first wave: pick by rounds): two entries tie.
__device__ __forceinline__ bool route_pick_ranks(PickLds &L, u32 t, u32 n_exp, u32 used, u32 renorm, u32 *ids, float *weights) {
    const u32 tid = threadIdx.x;
    // the entries padded to 64 << k; a thread an (entry, part of the others): 4 >> k parts of 16 << 2 k entries, a wave's
    // threads all of one part, so its reads of the others are broadcasts
    const u32 k = n_exp <= 64 ? 0u : n_exp <= 128 ? 1u : 2u;
    const u32 n_pad = 64u << k, chunk = 16u << (2 * k);
    const u32 i = tid & (n_pad - 1), j0 = (tid >> (6 + k)) * chunk;
    if (i < n_exp) {
        const int ki = (int)bm_f32_bits(L.p[i]);
        u32 cnt = 0;
        for (u32 j = j0; j < j0 + chunk; j += 16) { // sixteen entries' reads in flight, then their compares (chunk: 16, 64 or 256)
            float4 o[4];
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = *reinterpret_cast<const float4 *>(&L.p[j + 4 * k]);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                cnt += (int)bm_f32_bits(o[k].x) >= ki;
                cnt += (int)bm_f32_bits(o[k].y) >= ki;
                cnt += (int)bm_f32_bits(o[k].z) >= ki;
                cnt += (int)bm_f32_bits(o[k].w) >= ki;
            }
        }
        if (cnt) atomicAdd(&L.ahead[i], cnt);
    }
    [[maybe_unused]] unsigned long long tl_cnt = 0, tl_place = 0;
    BM_RTICK(tl_cnt, tid);
    lds_barrier();
    BM_RTICK(tl_place, tid);
    BM_RTOCK(6, tl_cnt);
    BM_RTOCK(7, tl_place);
    if (tid < n_exp) {
        const u32 r = L.ahead[tid] - 1; // (itself among the counted)
        if (r < used) {
            L.pick_id[r] = tid, L.pick_p[r] = L.p[tid];
            atomicAdd(&L.takers[r], 1u);
        }
    }
    lds_barrier();
    if (tid >= 64) return true;
    if (__ballot(tid < used && L.takers[tid] != 1u) != 0) return false;
    if (tid < used) {
        double chosen = 0.0;
        for (u32 s0 = 0; s0 < used; s0 += 8) { // eight reads at a time, then their adds in pick order
            const float4 a = *reinterpret_cast<const float4 *>(&L.pick_p[s0]), b = *reinterpret_cast<const float4 *>(&L.pick_p[s0 + 4]);
            const float q[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (s0 + k < used) chosen += (double)q[k];
        }
        ids[(size_t)t * used + tid] = L.pick_id[tid];
        weights[(size_t)t * used + tid] = renorm ? L.pick_p[tid] / (float)chosen : L.pick_p[tid];
    }
    return true;
}

// One wave a token.
template <int PER>
__global__ __launch_bounds__(256) void k_route_softmax(const float *logits, u32 n_tok, u32 n_exp, u32 used, u32 renorm,
                                                       float *probs, u32 *ids, float *weights, u32 *fault, u32 layer) {
    const u32 t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tok) return; // whole waves leave
    float v[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const u32 e = (threadIdx.x & 63) + 64 * j;
        v[j] = e < n_exp ? logits[(size_t)t * n_exp + e] : -INFINITY;
    }
    route_softmax_wave<PER>(v, t, n_exp, used, renorm, probs, ids, weights, fault, layer);
}

hipError_t route_softmax(const Launch &L, const float *logits, int n_tok, int n_exp, int used, int renorm, float *probs,
                         uint32_t *ids, float *weights) {
    const dim3 grid((unsigned)((n_tok + 3) / 4)), block(256);
    if (n_exp <= 128)
        hipLaunchKernelGGL(k_route_softmax<2>, grid, block, 0, L.stream, logits, (u32)n_tok, (u32)n_exp, (u32)used, (u32)renorm,
                           probs, ids, weights, L.fault, L.layer);
    else if (n_exp <= 256)
        hipLaunchKernelGGL(k_route_softmax<4>, grid, block, 0, L.stream, logits, (u32)n_tok, (u32)n_exp, (u32)used, (u32)renorm,
                           probs, ids, weights, L.fault, L.layer);
    else
        hipLaunchKernelGGL(k_route_softmax<16>, grid, block, 0, L.stream, logits, (u32)n_tok, (u32)n_exp, (u32)used,
                           (u32)renorm, probs, ids, weights, L.fault, L.layer);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------- the norm and the router's logits

// The FFN norm and the router's f32 logits of m tokens (crates/gpu/src/route_softmax.rs:1667-1674 enqueue_norm_fused does
// norm, quantizer and routing in one launch; here the norm and the logits are this launch, the routing
// k_route_softmax's, and the quantizer is folded into the expert launches). Numbers, op for op: the norm
// (crates/model/src/ops.rs:350-368) sums the f32 squares in f64 - lane by lane and then over the lanes; any order gives
// the same f32 mean except on an exact tie of that rounding, as the reference notes of its own two orders - narrows the
// mean to f32, takes scale = 1 / sqrt(mean + eps) and writes (scale * gain) * x; a logit is the f32 row dot of
// crates/qdot/src/lib.rs:11349-11386: eight lane accumulators (a product, then fused multiply-adds in increasing k) and
// (l0 + l4 + l2 + l6) + (l1 + l5 + l3 + l7).
//
// A workgroup takes one token and R router rows: the token's row is normed into LDS by all 256 threads while the rows'
// bytes arrive (both requested at once), then eight lanes a row walk it, lane l the accumulator l.
// Floats a line of the accumulator-major LDS rows.
__host__ __device__ inline int router_line(int hidden) { return ((hidden / 8 + 3) & ~3) + 8; }

// (k_norm_route's arguments: what the head of a logits workgroup needs stands in the first fourteen words, which are in registers when a
// wave starts - m_word is the token count, bit 31 set where the quantized column is asked for - and the rest travels as one
// struct behind them that a workgroup reads when it gets there: see bm_kernarg_at.)
struct NormRouteLate {
    u32 used, renorm;
    float *probs;
    u32 *ids;
    float *weights;
    u32 *hand;
    uint8_t *act_x;
    int q8k;
    u32 layer;
    u32 *fault;
    u32 max_polls, unused;
};
struct NormRouteArgs { // k_norm_route's argument block
    const float *router, *x, *gain;
    float eps;
    int n_exp, hidden;
    u32 m_word;
    float *normed_out, *logits;
    NormRouteLate late;
};
static_assert(offsetof(NormRouteArgs, late) == 56, "fourteen words in front of the late arguments");

// t: the token; e0: the first of the workgroup's R router rows, or -1 for a workgroup that only norms the token's row into LDS
// (k_norm_route's quantizer workgroups): no router rows, no logits.
template <int R, bool COH = false>
__device__ __forceinline__ void router_logits_body(uint8_t *lds, const float *router, const float *x, const float *gain, float eps,
                                                   int n_exp, int hidden, float *normed_out, float *logits, int t, int e0) {
    // The token's row and the R router rows lie accumulator-major in LDS: value k at line k % 8, place k / 8, so that the
    // lane that owns accumulator l reads four consecutive steps' operands as 16 bytes. A line is hidden / 8 floats, rounded up
    // to whole 16 bytes, + 8 (the eight lines of a row 8 banks apart), a router row four floats past the one before (rows r
    // and r + 1 on different banks).
    const int line = router_line(hidden), wrow_floats = 8 * line + 4;
    float *xs = reinterpret_cast<float *>(lds);  // [8][line]
    float *ws = xs + 8 * line;                   // [R][8][line] (+ 4 a row)
    auto put4 = [&](float *base, int c, const float4 v) { // the four values 4 c .. 4 c + 3 of a row
        float *at = base + (4 * (c & 1)) * line + (c >> 1);
        at[0] = v.x, at[line] = v.y, at[2 * line] = v.z, at[3 * line] = v.w;
    };
    __shared__ double s_part[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    [[maybe_unused]] unsigned long long tl_start = 0, tl_row = 0, tl_norm = 0, tl_lds = 0, tl_dots = 0;
    BM_RTICK(tl_start, tid);
    const float *xt = x + (size_t)t * hidden;
    // the rows' bytes on their way first: they do not depend on the norm. Eight 16-byte loads a thread are asked for together
    // and go to LDS once the token's row has been asked for too and normed
    const int n4 = hidden / 4;
    // A thread's pieces of the R rows: row 0's pieces tid, tid + 256, ..., then row 1's, ...: piece n of the thread is (row, place)
    // by counting on, no division by a length only known at run time in front of the first request.
    constexpr int kBatch = 8;
    float4 rv[kBatch];
    struct Piece {
        int r, c;
    };
    const int rows_here = e0 >= 0 ? R : 0;
    auto step = [&](Piece &p) {
        p.c += 256;
        if (p.c >= n4) p.r++, p.c = tid;
    };
    const Piece first = {tid < n4 ? 0 : rows_here, tid};
    auto ask = [&](Piece p) { // asks for the next kBatch pieces from p on; returns the piece behind them
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            if (p.r < rows_here) {
                const int e = e0 + p.r < n_exp ? e0 + p.r : n_exp - 1;
                rv[u] = reinterpret_cast<const float4 *>(router + (size_t)e * hidden)[p.c];
                step(p);
            }
        }
        return p;
    };
    auto park = [&](Piece p) {
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            if (p.r < rows_here) {
                put4(ws + (size_t)p.r * wrow_floats, p.c, rv[u]);
                step(p);
            }
        }
        return p;
    };
    ask(first);
    double sum = 0.0;
    constexpr int kInRegs = 8; // float4s of the row a thread can hold: rows of up to 8192 values stay in registers
    if (gain && n4 <= 256 * kInRegs) {
        // the row and the gain requested together and kept in registers: one pass, no second wait on memory
        float4 xv[kInRegs], gv[kInRegs];
#pragma unroll
        for (int j = 0; j < kInRegs; j++) {
            const int i = tid + 256 * j;
            if (i < n4) {
                xv[j] = reinterpret_cast<const float4 *>(xt)[i];
                gv[j] = reinterpret_cast<const float4 *>(gain)[i];
            }
        }
#pragma unroll
        for (int j = 0; j < kInRegs; j++)
            if (tid + 256 * j < n4) {
                sum += (double)__fmul_rn(xv[j].x, xv[j].x);
                sum += (double)__fmul_rn(xv[j].y, xv[j].y);
                sum += (double)__fmul_rn(xv[j].z, xv[j].z);
                sum += (double)__fmul_rn(xv[j].w, xv[j].w);
            }
        BM_RTICK(tl_row, sum);
        sum = wave_sum_f64(sum);
        if (lane == 0) s_part[wave] = sum;
        __syncthreads();
        const double total = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
        const float mean = (float)(total / (double)hidden);
        const float scale = __fdiv_rn(1.0f, bm_sqrt_rn(__fadd_rn(mean, eps)));
        BM_RTICK(tl_norm, scale);
#pragma unroll
        for (int j = 0; j < kInRegs; j++) {
            const int i = tid + 256 * j;
            if (i < n4) {
                const float4 v = make_float4(__fmul_rn(__fmul_rn(scale, gv[j].x), xv[j].x), __fmul_rn(__fmul_rn(scale, gv[j].y), xv[j].y),
                                             __fmul_rn(__fmul_rn(scale, gv[j].z), xv[j].z), __fmul_rn(__fmul_rn(scale, gv[j].w), xv[j].w));
                put4(xs, i, v);
                if (normed_out && e0 == 0) reinterpret_cast<float4 *>(normed_out + (size_t)t * hidden)[i] = v;
            }
        }
    } else {
        for (int i = tid; i < n4; i += 256) {
            const float4 v = reinterpret_cast<const float4 *>(xt)[i];
            put4(xs, i, v);
            if (gain) {
                sum += (double)__fmul_rn(v.x, v.x);
                sum += (double)__fmul_rn(v.y, v.y);
                sum += (double)__fmul_rn(v.z, v.z);
                sum += (double)__fmul_rn(v.w, v.w);
            }
        }
        if (gain) {
            sum = wave_sum_f64(sum);
            if (lane == 0) s_part[wave] = sum;
            __syncthreads();
            const double total = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
            const float mean = (float)(total / (double)hidden);
            const float scale = __fdiv_rn(1.0f, bm_sqrt_rn(__fadd_rn(mean, eps)));
            for (int i = tid; i < hidden; i += 256) {
                float *at = xs + (i & 7) * line + (i >> 3);
                const float v = __fmul_rn(__fmul_rn(scale, gain[i]), *at); // written before the barrier above
                *at = v;
                if (normed_out && e0 == 0) normed_out[(size_t)t * hidden + i] = v;
            }
        }
    }
    Piece parked = park(first);
    while (parked.r < rows_here) { // (no barrier inside: a thread with fewer pieces leaves earlier)
        ask(parked);
        parked = park(parked);
    }
    __syncthreads();
    BM_RTICK(tl_lds, tid);
    // (k_norm_route's hand-over words: an argument behind the preloaded ones, read here, where its way through memory runs under
    // the dots)
    [[maybe_unused]] u32 *hand = nullptr;
    if constexpr (COH) hand = bm_global(bm_kernarg_at<u32 *>(offsetof(NormRouteArgs, late) + offsetof(NormRouteLate, hand)));
    if (!gain && normed_out && e0 == 0) // the rows as they are (read after the barrier: other threads staged them)
        for (int i = tid; i < hidden; i += 256) normed_out[(size_t)t * hidden + i] = xs[(i & 7) * line + (i >> 3)];
    // every thread that stores a logit below is of the first wave: k_norm_route's hand-over (a device-scope count updated by
    // thread 0 behind the workgroup's barrier) publishes that wave's stores and relies on it
    static_assert(8 * R <= 64, "the logits of a workgroup are stored by its first wave");
    if (e0 >= 0 && tid < 8 * R) {
        const int r = tid >> 3, l = tid & 7;
        const float4 *xl = reinterpret_cast<const float4 *>(xs + l * line);
        const float4 *wl = reinterpret_cast<const float4 *>(ws + (size_t)r * wrow_floats + l * line);
        // the chain is serial by the order's definition (a product, then fused multiply-adds in increasing k); the reads
        // are not: sixteen steps' operands, four 16-byte reads a side, a batch
        const float *xf = xs + l * line, *wf = ws + (size_t)r * wrow_floats + l * line;
        const int steps = hidden / 8;
        float acc = __fmul_rn(xf[0], wf[0]);
        int i = 1;
        for (; i < 4 && i < steps; i++) acc = fmaf(xf[i], wf[i], acc);
        auto rd = [&](float4(&a)[4], float4(&b)[4], int at) {
#pragma unroll
            for (int u = 0; u < 4; u++) a[u] = xl[at / 4 + u], b[u] = wl[at / 4 + u];
        };
        auto chain = [&](const float4(&a)[4], const float4(&b)[4]) {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                acc = fmaf(a[u].x, b[u].x, acc), acc = fmaf(a[u].y, b[u].y, acc);
                acc = fmaf(a[u].z, b[u].z, acc), acc = fmaf(a[u].w, b[u].w, acc);
            }
        };
        if (i + 16 <= steps) {
            // two batches a turn in two sets of registers: a batch's operands are read while the batch before runs its chain
            float4 a0[4], b0[4], a1[4], b1[4];
            rd(a0, b0, i);
            for (; i + 48 <= steps; i += 32) {
                rd(a1, b1, i + 16);
                __builtin_amdgcn_sched_barrier(0);
                chain(a0, b0);
                __builtin_amdgcn_sched_barrier(0);
                rd(a0, b0, i + 32);
                __builtin_amdgcn_sched_barrier(0);
                chain(a1, b1);
                __builtin_amdgcn_sched_barrier(0);
            }
            chain(a0, b0);
            i += 16;
            for (; i + 16 <= steps; i += 16) {
                rd(a0, b0, i);
                chain(a0, b0);
            }
        }
        for (; i < steps; i++) acc = fmaf(xf[i], wf[i], acc);
        // s_l = acc_l + acc_{l+4} on lanes 0..3 of the row's eight, then (s0 + s2) + (s1 + s3)
        // (lane i reads lane i + n of its sixteen: right for the lanes of the eight whose value is used)
        const float s = __fadd_rn(acc, bm_dppf<kDppShl4>(acc));
        const float pair = __fadd_rn(s, bm_dppf<kDppShl2>(s)); // lane 0: s0 + s2, lane 1: s1 + s3
        const float out = __fadd_rn(pair, bm_dppf<kDppShl1>(pair));
        BM_RTICK(tl_dots, out);
        if (l == 0 && e0 + r < n_exp) {
            logits[(size_t)t * n_exp + e0 + r] = out;
            // k_norm_route's hand-over: the logit as a device-scope store of its own, into a word that held the armed pattern
            if constexpr (COH) __hip_atomic_store(hand + (size_t)t * n_exp + e0 + r, bm_f32_bits(out), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    BM_RTOCK(0, tl_start);
    BM_RTOCK(1, tl_row);
    BM_RTOCK(2, tl_norm);
    BM_RTOCK(3, tl_lds);
    BM_RTOCK(4, tl_dots);
}

template <int R>
__global__ __launch_bounds__(256) void k_router_logits(const float *router, const float *x, const float *gain, float eps,
                                                       int n_exp, int hidden, float *normed_out, float *logits) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int blocks_per_token = (n_exp + R - 1) / R;
    router_logits_body<R>(lds, router, x, gain, eps, n_exp, hidden, normed_out, logits, blockIdx.x / blocks_per_token,
                          (blockIdx.x % blocks_per_token) * R);
}

// Norm, logits and routing in one launch (crates/gpu/src/route_softmax.rs:1667-1674 enqueue_norm_fused; the quantizer of
// that launch is an option here, see below). The workgroups are k_router_logits's, and behind them in the grid one more a
// token, whose first wave routes it with k_route_softmax's numbers. The hand-over is one trip through memory: `hand` holds a
// word a (token, expert) that is armed between launches - kRouteArmed, a signalling NaN pattern, which no arithmetic
// leaves behind (an operation on it gives the quiet form) - each logit is stored over its word with a device-scope store as
// soon as it is formed, and the routing wave reads its words with device-scope loads until none is armed, so it has the
// logits the moment the last one lands: no acknowledgement is waited for, no count is kept, nothing is read back (the form
// before, a count raised behind acknowledged stores by the last workgroup to finish, which then read the logits back: 10.3
// us a token against this one's figure in the bench line). The wave arms its words again before it ends, so a graph replay
// needs no memset. A routing workgroup comes after every workgroup it waits for in the grid, so those are dispatched
// whatever else the card runs; the wait is bounded all the same (max_polls polls, kRoutePolls = 2^24 or some ten seconds unless the caller says otherwise - an XCD busy with another stream's work may hold some of them back for
// a while - then BM_SITE_ROUTER and NaN weights), and
// every wave ends. Launches over the same `hand` must not overlap.
// With act_x (the reference launch's quantizer, route_softmax.rs:1679): one more workgroup a token, between the two kinds in
// the grid, norms the token's row the same way and leaves it as the token's quantized column (q8k: a Q8_K column, else a
// Q8_2_X4 one with its tables), the bytes bm_quantize makes of normed_out. The routing waits for none of it.
template <int R, int PER>
__global__ __launch_bounds__(256) void k_norm_route(const float *router, const float *x, const float *gain, float eps, int n_exp,
                                                    int hidden, u32 m_word, float *normed_out, float *logits, NormRouteLate) {
    extern __shared__ __align__(16) uint8_t lds[];
    const u32 blocks_per_token = (u32)((n_exp + R - 1) / R);
    const u32 m = m_word & 0x7fffffffu;
    const u32 n_logit_blocks = m * blocks_per_token, n_quant_blocks = (m_word >> 31) ? m : 0u;
    if (blockIdx.x >= n_logit_blocks + n_quant_blocks) { // a routing workgroup: its first wave takes the logits
        __shared__ PickLds pick;
        const u32 t = blockIdx.x - n_logit_blocks - n_quant_blocks, lane = threadIdx.x;
        const NormRouteLate late = bm_kernarg_at<NormRouteLate>(offsetof(NormRouteArgs, late));
        const u32 used = late.used, renorm = late.renorm, layer = late.layer, max_polls = late.max_polls;
        float *const probs = bm_global(late.probs), *const weights = bm_global(late.weights);
        u32 *const ids = bm_global(late.ids), *const hand = bm_global(late.hand), *const fault = bm_global(late.fault);
        constexpr bool kRanks = PER <= 4; // up to 256 experts: the picks by the whole workgroup
        if constexpr (kRanks) {
            pick.p[threadIdx.x] = -1.0f, pick.ahead[threadIdx.x] = 0;
            if (threadIdx.x < 32) pick.takers[threadIdx.x] = 0;
            lds_barrier();
        } else {
            if (threadIdx.x >= 64) return;
        }
        [[maybe_unused]] float p[PER];
        if (threadIdx.x < 64) {
            u32 *mine = hand + (size_t)t * n_exp;
            [[maybe_unused]] unsigned long long tl_start = 0, tl_seen = 0;
            BM_RTICK(tl_start, lane);
            u32 w[PER];
            bool late = true;
            for (u32 spin = 0; spin < max_polls && late; spin++) {
                bool armed = false;
#pragma unroll
                for (int j = 0; j < PER; j++) {
                    const u32 e = lane + 64 * j;
                    w[j] = e < (u32)n_exp ? __hip_atomic_load(mine + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
                    armed |= w[j] == kRouteArmed;
                }
                late = __ballot(armed) != 0;
            }
            BM_RTICK(tl_seen, w[0]);
            BM_RTOCK(0, tl_start);
            BM_RTOCK(4, tl_seen);
            float v[PER];
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const u32 e = lane + 64 * j;
                // (a word still armed after the last poll: the NaN it is, which the routing refuses as it refuses any)
                v[j] = e < (u32)n_exp ? bm_bits_f32(w[j]) : -INFINITY;
                if (e < (u32)n_exp) __hip_atomic_store(mine + e, kRouteArmed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if constexpr (!kRanks) route_softmax_wave<PER>(v, t, (u32)n_exp, used, renorm, probs, ids, weights, fault, layer);
            if constexpr (kRanks) {
                const bool ok = route_probs_wave<PER>(v, t, (u32)n_exp, used, probs, weights, fault, layer, p);
                if (lane == 0) pick.ok = ok;
#pragma unroll
                for (int j = 0; j < PER; j++)
                    if (ok && lane + 64 * j < (u32)n_exp) pick.p[lane + 64 * j] = p[j];
            }
        }
        if constexpr (kRanks) {
            lds_barrier();
            if (pick.ok && !route_pick_ranks(pick, t, (u32)n_exp, used, renorm, ids, weights))
                route_pick_rounds<PER>(p, t, (u32)n_exp, used, renorm, ids, weights); // (the first wave, which holds p)
        }
        [[maybe_unused]] unsigned long long tl_routed = 0;
        BM_RTICK(tl_routed, threadIdx.x);
        BM_RTOCK(5, tl_routed);
        return;
    }
    if (blockIdx.x >= n_logit_blocks) { // a quantizer workgroup
        const int tq = (int)(blockIdx.x - n_logit_blocks);
        router_logits_body<R>(lds, router, x, gain, eps, n_exp, hidden, nullptr, nullptr, tq, -1);
        const NormRouteLate late = bm_kernarg_at<NormRouteLate>(offsetof(NormRouteArgs, late));
        uint8_t *const act_x = bm_global(late.act_x);
        u32 *const fault = bm_global(late.fault);
        const u32 layer = late.layer;
        const int q8k = late.q8k;
        const int line = router_line(hidden), nb = hidden / 256, tid = threadIdx.x;
        const float *xs = reinterpret_cast<const float *>(lds); // value k at line k % 8, place k / 8
        if (q8k) {
            uint8_t *col = act_x + (size_t)tq * nb * BM_Q8K_STRIDE;
            for (int b = tid >> 6; b < nb; b += 4) { // a wave a 256-value block, four consecutive values a lane
                const int k = 256 * b + 4 * (tid & 63);
                const float *at = xs + (k & 7) * line + (k >> 3);
                q8k_wave_block(make_float4(at[0], at[line], at[2 * line], at[3 * line]), col + (size_t)b * BM_Q8K_STRIDE, tid & 63, fault, layer);
            }
        } else {
            uint8_t *col = act_x + (size_t)tq * nb * BM_Q82_SB_EXT;
            for (int k = 8 * tid; k < hidden; k += 2048) { // a quad of lanes a 32-value block, eight consecutive values a lane
                float v8[8];
#pragma unroll
                for (int j = 0; j < 8; j++) v8[j] = xs[j * line + (k >> 3)];
                q82_quad8(v8, col, nb, k >> 5, tid & 3, fault, layer);
            }
        }
        return;
    }
    const u32 t = blockIdx.x / blocks_per_token;
    router_logits_body<R, true>(lds, router, x, gain, eps, n_exp, hidden, normed_out, logits, (int)t, (int)(blockIdx.x % blocks_per_token) * R);
}

// LDS of a workgroup of R rows: the token's row and the router rows, each as eight lines.
static size_t router_lds_bytes(int rows, int hidden) {
    return ((size_t)(rows + 1) * 8 * router_line(hidden) + 4 * (size_t)rows) * sizeof(float);
}

// Rows a workgroup takes: four where they fit the LDS beside the token's row, else two, else one - and no more than leaves
// a workgroup for every compute unit: a workgroup's time goes to bringing its rows in and laying them out in LDS (the dots of
// its rows run side by side on one wave), so with few tokens fewer rows a workgroup is the shorter launch.
static int router_rows(int hidden, int m = 1 << 20, int n_exp = 1 << 20) {
    int fit = 0;
    for (int r = 4; r >= 1; r >>= 1)
        if (router_lds_bytes(r, hidden) <= (size_t)kMaxLds - 1024) {
            fit = r;
            break;
        }
    while (fit > 1 && (long)m * ((n_exp + fit - 1) / fit) < 256) fit >>= 1;
    return fit;
}

bool router_logits_fits(int hidden) { return router_rows(hidden) > 0; }

hipError_t router_logits(const Launch &L, const float *router, const float *x, const float *gain, float eps, int m, int n_exp,
                         int hidden, float *normed_out, float *logits) {
    const int rows = router_rows(hidden, m, n_exp);
    if (rows == 0) return hipErrorInvalidValue;
    const size_t lds = router_lds_bytes(rows, hidden);
    const unsigned grid = (unsigned)m * (unsigned)((n_exp + rows - 1) / rows);
#define BM_RL(R)                                                                                                       \
    {                                                                                                                  \
        auto kern = k_router_logits<R>;                                                                                \
        hipError_t e = allow_lds(kern, lds);                                                                           \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, router, x, gain, eps, n_exp, hidden, normed_out, \
                           logits);                                                                                    \
    }
    if (rows == 4) BM_RL(4)
    else if (rows == 2) BM_RL(2)
    else BM_RL(1)
#undef BM_RL
    return hipGetLastError();
}

hipError_t norm_route(const Launch &L, const float *router, const float *x, const float *gain, float eps, int m, int n_exp,
                      int hidden, float *normed_out, float *logits, int used, int renorm, float *probs, uint32_t *ids,
                      float *weights, uint32_t *hand, uint8_t *act_x, bool q8k, uint32_t max_polls) {
    const int rows = router_rows(hidden, m, n_exp);
    if (rows == 0) return hipErrorInvalidValue;
    if (act_x && hidden % 256 != 0) return hipErrorInvalidValue;
    const size_t lds = router_lds_bytes(rows, hidden);
    const unsigned grid = (unsigned)m * (unsigned)((n_exp + rows - 1) / rows) + (act_x ? (unsigned)m : 0u) + (unsigned)m;
#define BM_NR(R, PER)                                                                                                  \
    {                                                                                                                  \
        auto kern = k_norm_route<R, PER>;                                                                              \
        hipError_t e = allow_lds(kern, lds);                                                                           \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, L.stream, router, x, gain, eps, n_exp, hidden,           \
                           (u32)m | (act_x ? 0x80000000u : 0u), normed_out, logits,                                    \
                           NormRouteLate{(u32)used, (u32)renorm, probs, ids, weights, hand, act_x, q8k ? 1 : 0, L.layer, L.fault, max_polls, 0u}); \
    }
#define BM_NR_ROWS(PER)                                                                                                \
    {                                                                                                                  \
        if (rows == 4) BM_NR(4, PER)                                                                                   \
        else if (rows == 2) BM_NR(2, PER)                                                                              \
        else BM_NR(1, PER)                                                                                             \
    }
    if (n_exp <= 128) BM_NR_ROWS(2)
    else if (n_exp <= 256) BM_NR_ROWS(4)
    else BM_NR_ROWS(16)
#undef BM_NR_ROWS
#undef BM_NR
    return hipGetLastError();
}

} // namespace bmk

#ifdef BM_TIMELINE
// The router's table, copied to the host: dst holds 1024 * 8 words. Measurement builds only; not part of the C ABI.
extern "C" int bm_router_timeline_read(unsigned long long *dst) {
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(bmk::g_router_timeline), sizeof(unsigned long long) * bmk::kRouterTimelineRows * 8);
}
#endif
