// Stand-alone activation quantization kernels: one wave64 per 256-element span, writing the
// device-private scratch layout of cq_device.h.  The arithmetic lives in cq_actquant.h.
#include "cq_actquant.h"
#include "cq_launch.h"

namespace {

template <int XDT>
__global__ __launch_bounds__(256) void quantize_q8k_kernel(const void *__restrict__ x, int8_t *__restrict__ qs,
                                                           float *__restrict__ dout, int16_t *__restrict__ bsums, int64_t n_blocks) {
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;
    cq_quantize_q8k_span<XDT>(x, blk, threadIdx.x & 63, qs, dout, bsums);
}

template <int XDT>
__global__ __launch_bounds__(256) void quantize_q80_kernel(const void *__restrict__ x, int8_t *__restrict__ qs,
                                                           float *__restrict__ ds, int64_t total) {
    const int64_t span = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    cq_quantize_q80_span<XDT>(x, span, threadIdx.x & 63, total, qs, ds);
}

template <int XDT>
int launch_quantize_act(int w_dtype, const void *x, void *scratch, int64_t k, int64_t rows, hipStream_t s) {
    ActLayout L = cq_act_layout(w_dtype, k, rows);
    uint8_t *b = (uint8_t *)scratch;
    int64_t total = rows * k;
    int64_t spans = (total + 255) / 256;
    if (spans == 0) return CQ_OK;
    int64_t grid = (spans + 3) / 4;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (cq_is_kquant(w_dtype))
        hipLaunchKernelGGL((quantize_q8k_kernel<XDT>), dim3((unsigned)grid), dim3(256), 0, s, x, (int8_t *)(b + L.qs_off),
                           (float *)(b + L.d_off), (int16_t *)(b + L.bs_off), total / 256);
    else
        hipLaunchKernelGGL((quantize_q80_kernel<XDT>), dim3((unsigned)grid), dim3(256), 0, s, x, (int8_t *)(b + L.qs_off),
                           (float *)(b + L.d_off), total);
    return (int)hipGetLastError();
}

}  // namespace

// k is a multiple of the weight type's block size (256 for K-quants, 32 for Q4_0 / Q8_0); the API
// layer checks it.
int cq_quantize_act_launch(int w_dtype, const void *x, int x_dtype, void *scratch, int64_t k, int64_t rows, hipStream_t s) {
    switch (x_dtype) {
        case CQ_F32: return launch_quantize_act<CQ_F32>(w_dtype, x, scratch, k, rows, s);
        case CQ_F16: return launch_quantize_act<CQ_F16>(w_dtype, x, scratch, k, rows, s);
        case CQ_BF16: return launch_quantize_act<CQ_BF16>(w_dtype, x, scratch, k, rows, s);
    }
    return CQ_ERR_DTYPE;
}
