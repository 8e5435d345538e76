// Measurement aid, built into a library of its own (libcq_bench.so) that only the benchmark loads: a plain streaming read of
// a device buffer, the yardstick the decode matvec is held against (what this GPU delivers to a kernel that only reads,
// at the same launch size and from the same memory).  Not part of the quantized-matmul C ABI.
#include "cq_device.h"

namespace {

// 256 workgroups of 1024 threads like the matvec; each workgroup walks its own contiguous share with four 16-byte
// loads per lane in flight.  The result is never stored for real data (the xor of the words would have to hit one
// value), it only keeps the loads alive.
__global__ __launch_bounds__(1024) void read_kernel(const u32x4 *__restrict__ p, int64_t n16, uint32_t *__restrict__ sink) {
    const int64_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const int64_t lo = (int64_t)blockIdx.x * per, hi = min(lo + per, n16);
    uint32_t acc = 0;
    int64_t i = lo + threadIdx.x;
    for (; i + 3 * 1024 < hi; i += 4 * 1024) {
        const u32x4 a = p[i], b = p[i + 1024], c = p[i + 2048], d = p[i + 3072];
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < hi; i += 1024) {
        const u32x4 a = p[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;
}

// The same read in the launch shape that a sweep over grid x block x loads in flight found fastest for tens of megabytes
// per launch: 768 workgroups of 512 threads walking the buffer interleaved, eight 16-byte loads per lane in flight.
__global__ __launch_bounds__(512) void read_interleaved_kernel(const u32x4 *__restrict__ p, int64_t n16, uint32_t *__restrict__ sink) {
    const int64_t stride = (int64_t)gridDim.x * 512;
    uint32_t acc = 0;
    int64_t i = (int64_t)blockIdx.x * 512 + threadIdx.x;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = p[i + u * stride];
#pragma unroll
        for (int u = 0; u < 8; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const u32x4 a = p[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;
}

}  // namespace

// Reads `bytes` (a multiple of 16) of `src_dev` (16-byte aligned) on `stream`; `sink_dev` holds at least 4 bytes.
// Returns 0, -2 for a bad size, -4 for a null pointer, -3 for a misaligned one, or the hipError_t of the launch.
extern "C" int cq_bench_read(const void *src_dev, int64_t bytes, void *sink_dev, void *stream) {
    if (bytes < 0 || bytes % 16) return -2;
    if (bytes == 0) return 0;
    if (!src_dev || !sink_dev) return -4;
    if (((uintptr_t)src_dev & 15) || ((uintptr_t)sink_dev & 3)) return -3;
    hipLaunchKernelGGL(read_kernel, dim3(256), dim3(1024), 0, (hipStream_t)stream, (const u32x4 *)src_dev, bytes / 16, (uint32_t *)sink_dev);
    return (int)hipGetLastError();
}

// cq_bench_read in the fastest launch shape found (see read_interleaved_kernel); same arguments and return values.
extern "C" int cq_bench_read_best(const void *src_dev, int64_t bytes, void *sink_dev, void *stream) {
    if (bytes < 0 || bytes % 16) return -2;
    if (bytes == 0) return 0;
    if (!src_dev || !sink_dev) return -4;
    if (((uintptr_t)src_dev & 15) || ((uintptr_t)sink_dev & 3)) return -3;
    hipLaunchKernelGGL(read_interleaved_kernel, dim3(768), dim3(512), 0, (hipStream_t)stream, (const u32x4 *)src_dev, bytes / 16, (uint32_t *)sink_dev);
    return (int)hipGetLastError();
}
