// Prefill matmul over pre-quantized activations, and the f32 -> f16/bf16 output conversion.
#include "cq_device.h"
#include "cq_launch.h"

namespace {

__global__ __launch_bounds__(256) void convert_f32_kernel(const float *__restrict__ src, void *__restrict__ dst, int dst_dtype, int64_t count) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    float v = src[i];
    if (dst_dtype == CQ_F16) {
        ((uint16_t *)dst)[i] = f2h_bits(v);
    } else {
        uint32_t b = __float_as_uint(v);
        uint32_t r = (b & 0x7fffffffu) > 0x7f800000u ? (b | 0x00400000u) : b + 0x7fffu + ((b >> 16) & 1u);
        ((uint16_t *)dst)[i] = (uint16_t)(r >> 16);
    }
}

}  // namespace

int cq_convert_f32_launch(const float *src, void *dst, int dst_dtype, int64_t count, hipStream_t s) {
    if (count == 0) return CQ_OK;
    if (dst_dtype != CQ_F16 && dst_dtype != CQ_BF16) return CQ_ERR_DTYPE;
    int64_t grid = (count + 255) / 256;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    hipLaunchKernelGGL(convert_f32_kernel, dim3((unsigned)grid), dim3(256), 0, s, src, dst, dst_dtype, count);
    return (int)hipGetLastError();
}

// Row-chunked matvec: every chunk of 8 activation rows streams W once.
int cq_matmul_launch(int w_dtype, const void *w, const void *scratch, float *dst, int64_t k, int64_t n, int64_t rows,
                     int64_t stride_dst, hipStream_t s) {
    ActView av = cq_act_view(scratch, w_dtype, k, rows);
    for (int64_t r0 = 0; r0 < rows; r0 += CQ_MATVEC_MAX_ROWS) {
        int64_t nb = rows - r0 < CQ_MATVEC_MAX_ROWS ? rows - r0 : CQ_MATVEC_MAX_ROWS;
        ActView c = cq_act_view_rows(av, w_dtype, k, r0);
        int rc = cq_matvec_launch_av(w_dtype, w, c, dst + r0 * stride_dst, CQ_F32, k, n, nb, stride_dst, s);
        if (rc) return rc;
    }
    return CQ_OK;
}
