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

// Gathering variants (f32 rows): destination row i of the scratch is row row_map[i] of x.  k is a multiple of 256.
__global__ __launch_bounds__(256) void quantize_q8k_gather_kernel(const float *__restrict__ x, const int *__restrict__ row_map, int kb,
                                                                  int8_t *__restrict__ qs, float *__restrict__ dout, int16_t *__restrict__ bsums,
                                                                  int64_t n_blocks) {
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;
    const int lane = threadIdx.x & 63;
    const int64_t row = blk / kb, b = blk - row * kb;
    float v[4];
    cq_load4<CQ_F32>(x, ((int64_t)row_map[row] * kb + b) * 256 + lane * 4, v);
    cq_quantize_q8k_vals(v, blk, lane, qs, dout, bsums);
}
__global__ __launch_bounds__(256) void quantize_q80_gather_kernel(const float *__restrict__ x, const int *__restrict__ row_map, int kb,
                                                                  int8_t *__restrict__ qs, float *__restrict__ ds, int64_t n_spans) {
    const int64_t span = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (span >= n_spans) return;
    const int lane = threadIdx.x & 63;
    const int64_t row = span / kb, b = span - row * kb;
    float v[4];
    cq_load4<CQ_F32>(x, ((int64_t)row_map[row] * kb + b) * 256 + lane * 4, v);
    cq_quantize_q80_vals(v, true, span * 256 + lane * 4, lane, qs, ds);
}

__global__ __launch_bounds__(256) void quantize_q8k_swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up, int64_t gate_stride,
                                                                  int64_t up_stride, int kb, int8_t *__restrict__ qs, float *__restrict__ dout,
                                                                  int16_t *__restrict__ bsums, int64_t n_blocks) {
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;
    const int lane = threadIdx.x & 63;
    const int64_t row = blk / kb, off = (blk - row * kb) * 256 + lane * 4;
    float v[4];
    cq_load_swiglu4(gate, up, row * gate_stride + off, row * up_stride + off, v);
    cq_quantize_q8k_vals(v, blk, lane, qs, dout, bsums);
}
__global__ __launch_bounds__(256) void quantize_q80_swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up, int64_t gate_stride,
                                                                  int64_t up_stride, int kb, int8_t *__restrict__ qs, float *__restrict__ ds,
                                                                  int64_t n_spans) {
    const int64_t span = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (span >= n_spans) return;
    const int lane = threadIdx.x & 63;
    const int64_t row = span / kb, off = (span - row * kb) * 256 + lane * 4;
    float v[4];
    cq_load_swiglu4(gate, up, row * gate_stride + off, row * up_stride + off, v);
    cq_quantize_q80_vals(v, true, span * 256 + lane * 4, lane, qs, ds);
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

// Scratch row i = quantized silu(gate[row_map[i]]) * up[row_map[i]] (rows of k contiguous floats), and scale_out[i] =
// scale_in[row_map[i]], for i < *n_valid: the down projection of an expert MLP over pairs that an earlier call has bucketed by expert.
__global__ __launch_bounds__(256) void quantize_q8k_swiglu_gather_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                                                         const int *__restrict__ row_map, const int *__restrict__ n_valid,
                                                                         const float *__restrict__ scale_in, float *__restrict__ scale_out, int kb,
                                                                         int8_t *__restrict__ qs, float *__restrict__ dout,
                                                                         int16_t *__restrict__ bsums, int64_t n_blocks) {
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;
    const int lane = threadIdx.x & 63;
    const int64_t row = blk / kb, b = blk - row * kb;
    const int src = row < *n_valid ? row_map[row] : 0;          // (rows behind the last valid pair are in no tile: any valid source)
    const int64_t off = ((int64_t)src * kb + b) * 256 + lane * 4;
    float v[4];
    cq_load_swiglu4(gate, up, off, off, v);
    cq_quantize_q8k_vals(v, blk, lane, qs, dout, bsums);
    if (b == 0 && lane == 0) scale_out[row] = scale_in[src];
}
__global__ __launch_bounds__(256) void quantize_q80_swiglu_gather_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                                                         const int *__restrict__ row_map, const int *__restrict__ n_valid,
                                                                         const float *__restrict__ scale_in, float *__restrict__ scale_out, int kb,
                                                                         int8_t *__restrict__ qs, float *__restrict__ ds, int64_t n_spans) {
    const int64_t span = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (span >= n_spans) return;
    const int lane = threadIdx.x & 63;
    const int64_t row = span / kb, b = span - row * kb;
    const int src = row < *n_valid ? row_map[row] : 0;          // (rows behind the last valid pair are in no tile: any valid source)
    const int64_t off = ((int64_t)src * kb + b) * 256 + lane * 4;
    float v[4];
    cq_load_swiglu4(gate, up, off, off, v);
    cq_quantize_q80_vals(v, true, span * 256 + lane * 4, lane, qs, ds);
    if (b == 0 && lane == 0) scale_out[row] = scale_in[src];
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

// Scratch rows [0, rows) = quantized x[row_map[i]]; the layout is that of `rows_alloc` rows (rows_alloc >= rows).
int cq_quantize_act_gather_launch(int w_dtype, const float *x, const int *row_map, void *scratch, int64_t k, int64_t rows, int64_t rows_alloc,
                                  hipStream_t s) {
    if (k % 256) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    ActLayout L = cq_act_layout(w_dtype, k, rows_alloc);
    uint8_t *b = (uint8_t *)scratch;
    const int64_t spans = rows * (k / 256);
    const int64_t grid = (spans + 3) / 4;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (cq_is_kquant(w_dtype))
        hipLaunchKernelGGL(quantize_q8k_gather_kernel, dim3((unsigned)grid), dim3(256), 0, s, x, row_map, (int)(k / 256), (int8_t *)(b + L.qs_off),
                           (float *)(b + L.d_off), (int16_t *)(b + L.bs_off), spans);
    else
        hipLaunchKernelGGL(quantize_q80_gather_kernel, dim3((unsigned)grid), dim3(256), 0, s, x, row_map, (int)(k / 256), (int8_t *)(b + L.qs_off),
                           (float *)(b + L.d_off), spans);
    return (int)hipGetLastError();
}

// Scratch rows [0, rows) = quantized silu(gate[row_map[i]]) * up[row_map[i]], scale_out[i] = scale_in[row_map[i]].
int cq_quantize_act_swiglu_gather_launch(int w_dtype, const float *gate, const float *up, const int *row_map, const int *n_valid, const float *scale_in,
                                         float *scale_out, void *scratch, int64_t k, int64_t rows, int64_t rows_alloc, hipStream_t s) {
    if (k % 256) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    ActLayout L = cq_act_layout(w_dtype, k, rows_alloc);
    uint8_t *b = (uint8_t *)scratch;
    const int64_t spans = rows * (k / 256);
    const int64_t grid = (spans + 3) / 4;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (cq_is_kquant(w_dtype))
        hipLaunchKernelGGL(quantize_q8k_swiglu_gather_kernel, dim3((unsigned)grid), dim3(256), 0, s, gate, up, row_map, n_valid, scale_in, scale_out, (int)(k / 256),
                           (int8_t *)(b + L.qs_off), (float *)(b + L.d_off), (int16_t *)(b + L.bs_off), spans);
    else
        hipLaunchKernelGGL(quantize_q80_swiglu_gather_kernel, dim3((unsigned)grid), dim3(256), 0, s, gate, up, row_map, n_valid, scale_in, scale_out, (int)(k / 256),
                           (int8_t *)(b + L.qs_off), (float *)(b + L.d_off), spans);
    return (int)hipGetLastError();
}

// Scratch rows [0, rows) = quantized silu(gate[r]) * up[r].  k is a multiple of 256; strides in floats, multiples of 4.
int cq_quantize_act_swiglu_launch(int w_dtype, const float *gate, const float *up, int64_t gate_stride, int64_t up_stride, void *scratch, int64_t k,
                                  int64_t rows, hipStream_t s) {
    if (k % 256) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    ActLayout L = cq_act_layout(w_dtype, k, rows);
    uint8_t *b = (uint8_t *)scratch;
    const int64_t spans = rows * (k / 256);
    const int64_t grid = (spans + 3) / 4;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (cq_is_kquant(w_dtype))
        hipLaunchKernelGGL(quantize_q8k_swiglu_kernel, dim3((unsigned)grid), dim3(256), 0, s, gate, up, gate_stride, up_stride, (int)(k / 256),
                           (int8_t *)(b + L.qs_off), (float *)(b + L.d_off), (int16_t *)(b + L.bs_off), spans);
    else
        hipLaunchKernelGGL(quantize_q80_swiglu_kernel, dim3((unsigned)grid), dim3(256), 0, s, gate, up, gate_stride, up_stride, (int)(k / 256),
                           (int8_t *)(b + L.qs_off), (float *)(b + L.d_off), spans);
    return (int)hipGetLastError();
}
