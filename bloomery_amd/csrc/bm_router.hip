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
#include "bm_stream.cuh"

namespace bmk {

constexpr u32 kSiteRouter = 5; // crates/device/src/fault.rs:84-86

__device__ __forceinline__ double shfl_xor_f64(double v, int mask) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __shfl_xor(lo, mask);
    hi = __shfl_xor(hi, mask);
    return __hiloint2double(hi, lo);
}

// One wave a token; lane L owns experts L + 64 j, j < PER.
template <int PER>
__global__ __launch_bounds__(256) void k_route_softmax(const float *logits, u32 n_tok, u32 n_exp, u32 used, u32 renorm,
                                                       float *probs, u32 *ids, float *weights, u32 *fault, u32 layer) {
    const u32 lane = threadIdx.x & 63, t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tok) return; // whole waves leave
    const float *row = logits + (size_t)t * n_exp;
    float v[PER];
    bool odd = false;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const u32 e = lane + 64 * j;
        v[j] = e < n_exp ? row[e] : -INFINITY;
        odd |= e < n_exp && !(fabsf(v[j]) <= 3.402823466e38f);
    }
    if (__ballot(odd) != 0) {
        const float nan = bm_bits_f32(0x7fc00000u);
        if (probs) {
#pragma unroll
            for (int j = 0; j < PER; j++)
                if (lane + 64 * j < n_exp) probs[(size_t)t * n_exp + lane + 64 * j] = nan;
        }
        if (lane < used) weights[(size_t)t * used + lane] = nan;
        if (lane == 0) bm_raise(fault, layer, kSiteRouter);
        return;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; j++) mx = fmaxf(mx, v[j]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float p[PER];
    double sum = 0.0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        p[j] = lane + 64 * j < n_exp ? (float)exp((double)(v[j] - mx)) : 0.0f;
        sum += (double)p[j];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += shfl_xor_f64(sum, off);
    const float inv = (float)sum;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        p[j] = p[j] / inv;
        if (probs && lane + 64 * j < n_exp) probs[(size_t)t * n_exp + lane + 64 * j] = p[j];
    }
    // `used` rounds of a wave argmax under (probability descending, id ascending); the winning lane marks its entry
    u32 taken = 0;
    double chosen = 0.0;
    float mine = 0.0f;
    for (u32 s = 0; s < used; s++) {
        float bv = -INFINITY;
        u32 bi = 0xffffffffu;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const u32 e = lane + 64 * j;
            if (e < n_exp && !((taken >> j) & 1u) && p[j] > bv) { // strict: a lane's ids ascend with j
                bv = p[j];
                bi = e;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off);
            const u32 oi = (u32)__shfl_xor((int)bi, off);
            if (ov > bv || (ov == bv && oi < bi)) {
                bv = ov;
                bi = oi;
            }
        }
        if ((bi & 63u) == lane && bi != 0xffffffffu) taken |= 1u << (bi >> 6);
        if (lane == 0) ids[(size_t)t * used + s] = bi;
        chosen += (double)bv;
        if (lane == s) mine = bv;
    }
    if (lane < used) weights[(size_t)t * used + lane] = renorm ? mine / (float)chosen : mine;
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

} // namespace bmk
