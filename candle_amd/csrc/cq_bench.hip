// Measurement aid: a plain streaming read of a device buffer, the yardstick the decode matvec is held against
// (what this GPU delivers to a kernel that only reads, at the same launch size and from the same memory).
#include "cq_device.h"
#include "cq_launch.h"

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

}  // namespace

int cq_bench_read_launch(const void *src, int64_t bytes, void *sink, hipStream_t s) {
    hipLaunchKernelGGL(read_kernel, dim3(256), dim3(1024), 0, s, (const u32x4 *)src, bytes / 16, (uint32_t *)sink);
    return (int)hipGetLastError();
}
