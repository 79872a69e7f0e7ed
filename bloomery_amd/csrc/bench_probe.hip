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

} // namespace

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
