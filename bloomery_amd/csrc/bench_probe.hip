// Measurement only, not part of the library's C ABI: the launches bench.py reads the decode kernels' times against.
// Built into a library of its own (libbm_bench_probe.so) that only the benchmark and its test load.
#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

namespace {

// n_wg workgroups read `bytes` (a multiple of 16) as plain 16-byte loads, workgroup b the b-th equal share, four loads a
// thread in flight, and leave one word a workgroup in `sink`. With bytes = 0 it is an empty launch. What a decode
// launch's time is to be read against: its bytes fetched by a kernel that does nothing else.
__global__ __launch_bounds__(256) void k_probe_read(const uint4 *src, size_t n16, uint32_t *sink) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t lo = per * blockIdx.x, hi = lo + per < n16 ? lo + per : n16;
    uint32_t acc = 0;
    size_t i = lo + threadIdx.x;
    for (; i + 768 < hi; i += 1024) {
        const uint4 a = src[i], b = src[i + 256], c = src[i + 512], d = src[i + 768];
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < hi; i += 256) {
        const uint4 a = src[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u && threadIdx.x == 0) sink[blockIdx.x] = acc; // the loads must happen; the store almost never does
}

// What a hand-over between workgroups inside one launch costs, to be read against a launch boundary. 256 workgroups, one a
// compute unit. Workgroup 0, `delay_ticks` (of 10 ns) after its start, stores 64 words with device-scope stores, waits for
// their acknowledgement, takes the time and stores a flag the same way; workgroups 8, 16, 248 (dispatched to workgroup 0's
// XCD: the dispatcher deals workgroups round over the eight XCDs, and out[8 b] holds the XCD each one ran on) and 1, 4, 255
// (other XCDs) poll the flag with device-scope loads (a bounded number of times), then read the 64 words and take the time.
// load 0: the other workgroups end at once; 1: each of their waves reads 1 MiB of `src` meanwhile; 2: waves 1 to 3 of the
// seven workgroups above do so too. out[8 b + 0..5] of workgroup b: XCD, start time, (0: words acknowledged | poller: flag
// seen), (0: flag acknowledged | poller: words read), words right, polls.
__global__ __launch_bounds__(256) void k_probe_handoff(uint32_t gen, int load, const uint4 *src, size_t n16, uint32_t *flag,
                                                        uint32_t *words, unsigned long long *out, uint32_t *sink,
                                                        int delay_ticks) {
    const int wg = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    uint32_t xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    const unsigned long long t0 = wall_clock64();
    if (tid == 0) out[wg * 8 + 0] = xcc & 15u, out[wg * 8 + 1] = t0;
    const bool poller = wg == 8 || wg == 16 || wg == 248 || wg == 1 || wg == 4 || wg == 255;
    if ((wg != 0 && !poller) ? load >= 1 : (wave > 0 && load == 2)) {
        const size_t per_wave = 16384; // 16-byte words: 256 KiB a pass, four passes, another place each launch
        size_t base = ((size_t)(gen * 1024u + wg * 4 + wave) * per_wave) % (n16 - per_wave);
        uint4 acc = make_uint4(0, 0, 0, 0);
        for (int pass = 0; pass < 4; pass++) {
            for (size_t i = lane; i < per_wave; i += 64 * 8) {
                uint4 v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = src[base + ((i + 64 * u) % per_wave)];
#pragma unroll
                for (int u = 0; u < 8; u++) acc.x ^= v[u].x, acc.y ^= v[u].y, acc.z ^= v[u].z, acc.w ^= v[u].w;
            }
            base = (base + per_wave * 7168) % (n16 - per_wave);
        }
        if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[tid] = acc.x;
        return;
    }
    if (wave > 0) return;
    if (wg == 0) {
        while (wall_clock64() - t0 < (unsigned long long)delay_ticks) {}
        __hip_atomic_store(words + lane, gen * 64u + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const unsigned long long t1 = wall_clock64();
        if (lane == 0) __hip_atomic_store(flag, gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const unsigned long long t2 = wall_clock64();
        if (lane == 0) out[2] = t1, out[3] = t2;
        return;
    }
    uint32_t polls = 0;
    bool seen = false;
    while (polls < 400000u && !seen) { // bounded: the launch ends whatever happens
        seen = __builtin_amdgcn_readfirstlane(__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) == gen;
        polls++;
    }
    const unsigned long long t1 = wall_clock64();
    const uint32_t v = __hip_atomic_load(words + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool right = __ballot(seen && v == gen * 64u + lane) == ~0ull;
    const unsigned long long t2 = wall_clock64();
    if (lane == 0) out[wg * 8 + 2] = t1, out[wg * 8 + 3] = t2, out[wg * 8 + 4] = right ? 1 : 0, out[wg * 8 + 5] = polls;
}

// The read patterns of the two decode launches with nothing computed, to be read against their times: what the requests
// alone cost, and what other ways of asking for the same bytes would.
// Gate . up (rows of 8 super-blocks of 144 bytes, a workgroup of T threads takes T / 8 row pairs (gate row, up row) of one slot):
//   pattern 0: a quad a row as k_gate_up_x asks: lane q of the quad the 16 bytes at 16 + 32 q and at 32 + 32 q and the 4 at 4 q of
//              a super-block, `ahead` super-blocks asked for up front and one more behind every one consumed;
//   pattern 1: eight lanes a row pair: lane k the 16 code bytes at 16 + 16 k of the gate row's and of the up row's super-block
//              and the two 16-byte headers (four requests a super-block, every one of a row 16-byte contiguous over the octet);
//   pattern 2: the workgroup's rows of each matrix are contiguous in memory: plain 16-byte loads over them, thread by thread.
//   pattern 3: loads that land in LDS (global_load_lds_dwordx4: no register holds them, any lane may ask for any piece): a wave
//              takes its own 8 row pairs, super-block by super-block, nine lanes a (row, super-block)'s 144 contiguous bytes,
//              all asked for up front; the bytes are then read back from LDS;
//   pattern 4: the same loads over the wave's rows as they lie (8 gate rows, then 8 up rows: 9 KB contiguous each).
typedef __attribute__((address_space(1))) const void probe_gptr;
typedef __attribute__((address_space(3))) void probe_lptr;
template <int T, int PATTERN, int AHEAD>
__global__ __launch_bounds__(T) void k_probe_gate_up_rows(const uint8_t *wg, const uint8_t *wu, const uint32_t *sel, int ff,
                                                          uint32_t *sink) {
    constexpr int RP = T / 8;
    const int tid = threadIdx.x, q = tid & 3, which = (tid >> 2) & 1;
    const int per_slot = ff / RP;
    const int slot = blockIdx.x / per_slot, rb = blockIdx.x % per_slot;
    const uint32_t id = sel[slot];
    uint4 acc = make_uint4(0, 0, 0, 0);
    if constexpr (PATTERN == 0) {
        const uint8_t *wrow = (which ? wu : wg) + ((size_t)id * ff + rb * RP + (tid >> 3)) * 1152;
        uint4 a[8], b[8];
        uint32_t c[8];
        auto ask = [&](int i) {
            const uint8_t *p = wrow + i * 144;
            a[i] = *reinterpret_cast<const uint4 *>(p + 16 + 32 * q);
            b[i] = *reinterpret_cast<const uint4 *>(p + 32 + 32 * q);
            c[i] = *reinterpret_cast<const uint32_t *>(p + 4 * q);
        };
#pragma unroll
        for (int i = 0; i < AHEAD; i++) ask(i);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            acc.x ^= a[i].x ^ b[i].x ^ c[i], acc.y ^= a[i].y ^ b[i].y, acc.z ^= a[i].z ^ b[i].z, acc.w ^= a[i].w ^ b[i].w;
            if (i + AHEAD < 8) ask(i + AHEAD);
        }
    } else if constexpr (PATTERN == 1) {
        const int k = tid & 7;
        const size_t row = ((size_t)id * ff + rb * RP + (tid >> 3)) * 1152;
        uint4 qg[8], qu[8], hg[8], hu[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            qg[i] = *reinterpret_cast<const uint4 *>(wg + row + i * 144 + 16 + 16 * k);
            hg[i] = *reinterpret_cast<const uint4 *>(wg + row + i * 144);
            qu[i] = *reinterpret_cast<const uint4 *>(wu + row + i * 144 + 16 + 16 * k);
            hu[i] = *reinterpret_cast<const uint4 *>(wu + row + i * 144);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            acc.x ^= qg[i].x ^ qu[i].x ^ hg[i].x ^ hu[i].x, acc.y ^= qg[i].y ^ qu[i].y ^ hg[i].y ^ hu[i].y;
            acc.z ^= qg[i].z ^ qu[i].z ^ hg[i].z ^ hu[i].z, acc.w ^= qg[i].w ^ qu[i].w ^ hg[i].w ^ hu[i].w;
        }
    } else if constexpr (PATTERN == 3 || PATTERN == 4) {
        static_assert(T == 256, "four waves of 8 row pairs");
        extern __shared__ __align__(16) uint8_t lds[];
        const int lane = tid & 63, wave = tid >> 6;
        uint8_t *mine = lds + wave * 24576; // 16 rows of 1152 bytes (pattern 3: 24 requests of 1 KB)
        const size_t row0 = ((size_t)id * ff + rb * RP + 8 * wave) * 1152;
        if constexpr (PATTERN == 3) {
            // piece P = 64 j + lane of a super-block's 144: row P / 9 of the wave's 16 (8 gate, 8 up), part P % 9
            const uint8_t *src[3];
#pragma unroll
            for (int j = 0; j < 3; j++) {
                int pc = 64 * j + lane;
                pc = pc < 144 ? pc : 143;
                const int r16 = pc / 9, part = pc % 9;
                src[j] = (r16 < 8 ? wg : wu) + row0 + (size_t)(r16 & 7) * 1152 + 16 * part;
            }
#pragma unroll
            for (int i = 0; i < 8; i++)
#pragma unroll
                for (int j = 0; j < 3; j++)
                    __builtin_amdgcn_global_load_lds((probe_gptr *)(src[j] + 144 * i), (probe_lptr *)(mine + (3 * i + j) * 1024), 16, 0, 0);
            __builtin_amdgcn_s_waitcnt(0);
#pragma unroll
            for (int k = 0; k < 24; k++) {
                const uint4 v = *reinterpret_cast<const uint4 *>(mine + k * 1024 + 16 * lane);
                acc.x ^= v.x, acc.y ^= v.y, acc.z ^= v.z, acc.w ^= v.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 18; k++)
                __builtin_amdgcn_global_load_lds((probe_gptr *)((k < 9 ? wg : wu) + row0 + (size_t)(k % 9) * 1024 + 16 * lane),
                                                 (probe_lptr *)(mine + k * 1024), 16, 0, 0);
            __builtin_amdgcn_s_waitcnt(0);
#pragma unroll
            for (int k = 0; k < 18; k++) {
                const uint4 v = *reinterpret_cast<const uint4 *>(mine + k * 1024 + 16 * lane);
                acc.x ^= v.x, acc.y ^= v.y, acc.z ^= v.z, acc.w ^= v.w;
            }
        }
    } else {
        constexpr int N16 = RP * 1152 / 16, PER = (2 * N16 + T - 1) / T;
        const uint8_t *g0 = wg + ((size_t)id * ff + rb * RP) * 1152, *u0 = wu + ((size_t)id * ff + rb * RP) * 1152;
        uint4 v[PER];
#pragma unroll
        for (int k = 0; k < PER; k++) {
            int ch = k * T + tid;
            ch = ch < 2 * N16 ? ch : 2 * N16 - 1;
            v[k] = *reinterpret_cast<const uint4 *>((ch < N16 ? g0 : u0) + (size_t)(ch % N16) * 16);
        }
#pragma unroll
        for (int k = 0; k < PER; k++) acc.x ^= v[k].x, acc.y ^= v[k].y, acc.z ^= v[k].z, acc.w ^= v[k].w;
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[tid] = acc.x;
}

// Down (rows of 3 Q6_K super-blocks; a workgroup of 256 threads takes 8 rows of each of the token's 8 experts, a quad a
// (row, expert)): layout 0: the rows as they are, super-blocks of 210 bytes back to back, the six requests a lane and
// super-block of the six-load form (ql, qh, ql, qh, scales, d); layout 1: the same requests over rows laid out as planes (ql of
// the three super-blocks, then qh, scales, d) in 640 bytes, every piece 16-byte aligned; `w` must hold n_experts * rpe rows
// of 630 or 640 bytes.
template <int LAYOUT>
__global__ __launch_bounds__(256) void k_probe_down_rows(const uint8_t *w, const uint32_t *sel, int rpe, uint32_t *sink) {
    const int tid = threadIdx.x, q = tid & 3, quad = tid >> 2, c = q & 1, h = q >> 1;
    const int e = quad % 8, r = blockIdx.x * 8 + quad / 8;
    const uint32_t id = sel[e];
    const uint8_t *wrow = w + ((size_t)id * rpe + r) * (LAYOUT == 0 ? 630 : 640);
    auto ld16 = [](const uint8_t *p) {
        uint4 v;
        __builtin_memcpy(&v, p, 16);
        return v;
    };
    uint4 v[3][5];
    uint32_t d[3];
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const uint8_t *ql = LAYOUT == 0 ? wrow + i * 210 : wrow + i * 128;
        const uint8_t *qh = LAYOUT == 0 ? wrow + i * 210 + 128 : wrow + 384 + i * 64;
        const uint8_t *sc = LAYOUT == 0 ? wrow + i * 210 + 192 : wrow + 576 + i * 16;
        const uint8_t *dd = LAYOUT == 0 ? wrow + i * 210 + 208 : wrow + 624 + i * 2;
        v[i][0] = ld16(ql + 32 * c + 16 * h), v[i][1] = ld16(qh + 16 * h), v[i][2] = ld16(ql + 64 + 32 * c + 16 * h);
        v[i][3] = ld16(qh + 32 + 16 * h), v[i][4] = ld16(sc);
        unsigned short d16;
        __builtin_memcpy(&d16, dd, 2);
        d[i] = d16;
    }
    uint4 acc = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 3; i++) {
#pragma unroll
        for (int j = 0; j < 5; j++) acc.x ^= v[i][j].x, acc.y ^= v[i][j].y, acc.z ^= v[i][j].z, acc.w ^= v[i][j].w;
        acc.x ^= d[i];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[tid] = acc.x;
}

} // namespace

// Enqueues a gate . up read pattern over 8 slots of sel_dev: pattern 0 .. 4 as above, threads 256 or 192 a workgroup (ff a
// multiple of threads / 8; patterns 3 and 4: 256), ahead 4 or 8 (pattern 0 only). Returns 0, -1 for a refused argument, or the HIP error.
extern "C" int bm_bench_probe_gate_up_rows(void *hip_stream, const void *wg_dev, const void *wu_dev, const uint32_t *sel_dev, int ff,
                                           int pattern, int threads, int ahead, uint32_t *sink_dev) {
    if (!wg_dev || !wu_dev || !sel_dev || !sink_dev || ff < 1) return -1;
    if ((threads != 256 && threads != 192) || ff % (threads / 8) != 0) return -1;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const uint8_t *g = static_cast<const uint8_t *>(wg_dev), *u = static_cast<const uint8_t *>(wu_dev);
    const dim3 grid((unsigned)(8 * ff / (threads / 8)));
#define BM_PROBE_ROWS(T, P, A) hipLaunchKernelGGL((k_probe_gate_up_rows<T, P, A>), grid, dim3(T), 0, s, g, u, sel_dev, ff, sink_dev)
    if (pattern == 0 && threads == 256 && ahead == 4) BM_PROBE_ROWS(256, 0, 4);
    else if (pattern == 0 && threads == 256 && ahead == 8) BM_PROBE_ROWS(256, 0, 8);
    else if (pattern == 0 && threads == 192 && ahead == 4) BM_PROBE_ROWS(192, 0, 4);
    else if (pattern == 0 && threads == 192 && ahead == 8) BM_PROBE_ROWS(192, 0, 8);
    else if (pattern == 1 && threads == 256) BM_PROBE_ROWS(256, 1, 8);
    else if (pattern == 1 && threads == 192) BM_PROBE_ROWS(192, 1, 8);
    else if (pattern == 2 && threads == 256) BM_PROBE_ROWS(256, 2, 8);
    else if (pattern == 2 && threads == 192) BM_PROBE_ROWS(192, 2, 8);
    else if ((pattern == 3 || pattern == 4) && threads == 256) {
        constexpr int kLds = 4 * 24 * 1024; // a wave: 24 KB (pattern 3 leaves the third request of a super-block a quarter full)
        auto k3 = k_probe_gate_up_rows<256, 3, 8>;
        auto k4 = k_probe_gate_up_rows<256, 4, 8>;
        auto kern = pattern == 3 ? k3 : k4;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, grid, dim3(256), kLds, s, g, u, sel_dev, ff, sink_dev);
    } else return -1;
#undef BM_PROBE_ROWS
    return (int)hipGetLastError();
}

// Enqueues the down read pattern over the 8 experts of sel_dev: rows_per_expert a multiple of 8, layout 0 or 1 as above.
extern "C" int bm_bench_probe_down_rows(void *hip_stream, const void *w_dev, const uint32_t *sel_dev, int rows_per_expert, int layout,
                                        uint32_t *sink_dev) {
    if (!w_dev || !sel_dev || !sink_dev || rows_per_expert < 8 || rows_per_expert % 8 != 0) return -1;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const dim3 grid((unsigned)(rows_per_expert / 8));
    if (layout == 0) hipLaunchKernelGGL(k_probe_down_rows<0>, grid, dim3(256), 0, s, static_cast<const uint8_t *>(w_dev), sel_dev, rows_per_expert, sink_dev);
    else if (layout == 1) hipLaunchKernelGGL(k_probe_down_rows<1>, grid, dim3(256), 0, s, static_cast<const uint8_t *>(w_dev), sel_dev, rows_per_expert, sink_dev);
    else return -1;
    return (int)hipGetLastError();
}

// Enqueues the hand-over probe: src_dev of src_bytes (at least 64 MiB, a multiple of 16), flag_dev of 65 words (the flag,
// then the words; `gen` must differ from what the flag holds: count launches from 1 over a zeroed flag), out_dev of 2048
// 64-bit words, sink_dev of 256 words. Returns 0, -1 for a refused argument, or the HIP error of the launch.
extern "C" int bm_bench_probe_handoff(void *hip_stream, const void *src_dev, size_t src_bytes, uint32_t *flag_dev,
                                      unsigned long long *out_dev, uint32_t *sink_dev, uint32_t gen, int load, int delay_ticks) {
    if (!src_dev || !flag_dev || !out_dev || !sink_dev) return -1;
    if (src_bytes < ((size_t)64 << 20) || src_bytes % 16 != 0 || ((uintptr_t)src_dev & 15) != 0) return -1;
    if (load < 0 || load > 2 || delay_ticks < 0 || delay_ticks > 100000) return -1;
    hipLaunchKernelGGL(k_probe_handoff, dim3(256), dim3(256), 0, static_cast<hipStream_t>(hip_stream), gen, load,
                       static_cast<const uint4 *>(src_dev), src_bytes / 16, flag_dev, flag_dev + 1, out_dev, sink_dev, delay_ticks);
    return (int)hipGetLastError();
}

// Enqueues the probe on `hip_stream` (a hipStream_t). Returns 0, -1 for a refused argument (bytes and src_dev multiples of
// 16, 1 .. 65536 workgroups, sink_dev of n_workgroups words), or the HIP error of the launch.
extern "C" int bm_bench_probe_read(void *hip_stream, const void *src_dev, size_t bytes, int n_workgroups, uint32_t *sink_dev) {
    if (!sink_dev || (!src_dev && bytes)) return -1;
    if (bytes % 16 != 0 || ((uintptr_t)src_dev & 15) != 0) return -1;
    if (n_workgroups < 1 || n_workgroups > 65536) return -1;
    hipLaunchKernelGGL(k_probe_read, dim3((unsigned)n_workgroups), dim3(256), 0, static_cast<hipStream_t>(hip_stream),
                       static_cast<const uint4 *>(src_dev), bytes / 16, sink_dev);
    return (int)hipGetLastError();
}
