// Decode matvec for gfx950:  dst[b, row] = sum_k W[row, k] * x^[b, k]   (b < NB <= 8)
//
// W is streamed once from HBM in its GGUF block layout; x^ is the int8-quantized activation scratch
// written by the act-quant kernels (bit-identical to candle's CPU quantization), so the integer part
// of every dot product is exact and only the f32 summation order differs from
// k_quants::matmul (candle-core/src/quantized/k_quants.rs:2375-2492) and its vec_dot kernels
// (Q4_0 :294-311, Q8_0 :720-738, Q4_K :1460-1540, Q5_K :1714-1801, Q6_K :2035-2092).
//
// Work split: a row of W is cut into "units" — the bytes one lane consumes per step with 128-bit
// loads.  Lane l of a wave takes units l, l+64, ... of R consecutive rows, so the activation
// registers are reused across the R rows and the weight registers across the NB activation rows.
//   Q4_K / Q5_K: unit = one 16-byte slice of qs (8 per super-block) + the 16-byte block header
//   Q6_K       : unit = 16 `l` positions of one 128-element half (3 x 16 bytes, 4 per super-block)
//   Q4_0 / Q8_0: unit = one 32-element block
// Packed int8 dot products use v_dot4_i32_i8; wave64 butterflies reduce the per-lane partial sums.
#include "cq_device.h"
#include "cq_fmt.h"
#include "cq_launch.h"

namespace {

// ---------------------------------------------------------------------------------------------
// The kernel: 4 waves per workgroup, each wave owns R consecutive rows.
// ---------------------------------------------------------------------------------------------
template <int DT, int NB, int R>
__global__ __launch_bounds__(256) void matvec_kernel(const uint8_t *__restrict__ w, ActView av, void *__restrict__ dst,
                                                     int dst_dtype, int k, int n, int64_t stride_dst) {
    typedef Fmt<DT> F;
    const int lane = threadIdx.x & 63;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * R;
    if (row0 >= n) return;
    const int nblk = k / BlockInfo<DT>::elems;
    const int units = nblk * F::UPB;
    const int64_t row_bytes = (int64_t)nblk * BlockInfo<DT>::bytes;

    float acc[R][NB];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int b = 0; b < NB; b++) acc[r][b] = 0.0f;

    for (int u = lane; u < units; u += CQ_WAVE) {
        typename F::W wr[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            int64_t row = row0 + r < n ? row0 + r : n - 1;   // tail rows re-read the last row, never stored
            F::load_w(wr[r], w + row * row_bytes, u);
        }
        typename F::A ar[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) F::load_a(ar[b], av, b, k, u);
#pragma unroll
        for (int r = 0; r < R; r++) {
            typename F::P p;
            F::prep(p, wr[r], u);
#pragma unroll
            for (int b = 0; b < NB; b++) acc[r][b] = F::dot(p, ar[b], acc[r][b]);
        }
    }

#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int b = 0; b < NB; b++) {
            float v = wave_sum(acc[r][b]);
            if (lane == 0 && row0 + r < n) store_out(dst, dst_dtype, (int64_t)b * stride_dst + row0 + r, v);
        }
}

template <int DT, int NB>
int launch_nb(const void *w, const ActView &av, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t stride_dst, hipStream_t s) {
    constexpr int R = NB <= 2 ? 2 : 1;
    int64_t grid = (n + 4 * R - 1) / (4 * R);
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    hipLaunchKernelGGL((matvec_kernel<DT, NB, R>), dim3((unsigned)grid), dim3(256), 0, s, (const uint8_t *)w, av, dst, dst_dtype,
                       (int)k, (int)n, stride_dst);
    return (int)hipGetLastError();
}

template <int DT>
int launch_dt(const void *w, const ActView &av, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst,
              hipStream_t s) {
    switch (rows) {
        case 1: return launch_nb<DT, 1>(w, av, dst, dst_dtype, k, n, stride_dst, s);
        case 2: return launch_nb<DT, 2>(w, av, dst, dst_dtype, k, n, stride_dst, s);
        case 3: return launch_nb<DT, 3>(w, av, dst, dst_dtype, k, n, stride_dst, s);
        case 4: return launch_nb<DT, 4>(w, av, dst, dst_dtype, k, n, stride_dst, s);
        case 5: return launch_nb<DT, 5>(w, av, dst, dst_dtype, k, n, stride_dst, s);
        case 6: return launch_nb<DT, 6>(w, av, dst, dst_dtype, k, n, stride_dst, s);
        case 7: return launch_nb<DT, 7>(w, av, dst, dst_dtype, k, n, stride_dst, s);
        case 8: return launch_nb<DT, 8>(w, av, dst, dst_dtype, k, n, stride_dst, s);
    }
    return CQ_ERR_RANGE;
}

}  // namespace

int cq_matvec_launch_av(int w_dtype, const void *w, const ActView &av, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows,
                        int64_t stride_dst, hipStream_t s) {
    if (n == 0 || rows == 0) return CQ_OK;
    switch (w_dtype) {
        case CQ_Q4_0: return launch_dt<CQ_Q4_0>(w, av, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q8_0: return launch_dt<CQ_Q8_0>(w, av, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q4K: return launch_dt<CQ_Q4K>(w, av, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q5K: return launch_dt<CQ_Q5K>(w, av, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q6K: return launch_dt<CQ_Q6K>(w, av, dst, dst_dtype, k, n, rows, stride_dst, s);
    }
    return CQ_ERR_DTYPE;
}

int cq_matvec_launch(int w_dtype, const void *w, const void *scratch, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows,
                     int64_t stride_dst, hipStream_t s) {
    return cq_matvec_launch_av(w_dtype, w, cq_act_view(scratch, w_dtype, k, rows), dst, dst_dtype, k, n, rows, stride_dst, s);
}
