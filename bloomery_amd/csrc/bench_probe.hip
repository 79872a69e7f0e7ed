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

} // namespace

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
