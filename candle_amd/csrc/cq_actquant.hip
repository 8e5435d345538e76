// On-the-fly int8 activation quantization for gfx950, bit-identical to candle's CPU path:
//   Q8_K blocks (256 elements, f32 scale, 16-element sums) for K-quant weights
//     — BlockQ8K::from_float, candle-core/src/quantized/k_quants.rs:2320-2358
//   Q8_0 blocks (32 elements, f16 scale) for Q4_0 / Q8_0 weights
//     — BlockQ8_0::from_float, k_quants.rs:658-687
// f16 / bf16 activations are widened to f32 first, as k_quants::matmul_f16 does (k_quants.rs:2652-2686).
//
// One wave64 quantizes one 256-element span: each lane owns four consecutive elements (one 16-byte
// load, one 4-byte packed int8 store), reductions run over wave64 butterflies.
#include "cq_device.h"

namespace {

template <int XDT> __device__ __forceinline__ void load4(const void *x, int64_t idx, float v[4]);
template <> __device__ __forceinline__ void load4<CQ_F32>(const void *x, int64_t idx, float v[4]) {
    f32x4 t = *reinterpret_cast<const f32x4 *>((const float *)x + idx);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <> __device__ __forceinline__ void load4<CQ_F16>(const void *x, int64_t idx, float v[4]) {
    u32x2 t = *reinterpret_cast<const u32x2 *>((const uint16_t *)x + idx);
    v[0] = h2f(t.x); v[1] = h2f(t.x >> 16); v[2] = h2f(t.y); v[3] = h2f(t.y >> 16);
}
template <> __device__ __forceinline__ void load4<CQ_BF16>(const void *x, int64_t idx, float v[4]) {
    u32x2 t = *reinterpret_cast<const u32x2 *>((const uint16_t *)x + idx);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}

// Rust `v as i8` after f32::round: saturating, NaN -> 0.
__device__ __forceinline__ int round_sat_i8(float v) {
    float r = roundf(v);                 // half away from zero, like f32::round
    if (!(r == r)) return 0;
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int)r;
}

// ---- Q8_K: one wave per 256-element block ---------------------------------------------------
template <int XDT>
__global__ __launch_bounds__(256) void quantize_q8k_kernel(const void *__restrict__ x, int8_t *__restrict__ qs,
                                                           float *__restrict__ dout, int16_t *__restrict__ bsums,
                                                           int64_t n_blocks) {
    const int lane = threadIdx.x & 63;
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;
    float v[4];
    load4<XDT>(x, blk * 256 + lane * 4, v);

    // signed value of the first element with the largest magnitude (strict `<`: first one wins)
    float amax = 0.0f;
    int idx = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float a = fabsf(v[i]);
        if (amax < a) { amax = a; idx = i; }
    }
    float wmax = amax;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) wmax = fmaxf(wmax, __shfl_xor(wmax, o, CQ_WAVE));
    int cand = (amax == wmax && wmax != 0.0f) ? lane * 4 + idx : 256;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, CQ_WAVE));
    float mine = idx == 0 ? v[0] : idx == 1 ? v[1] : idx == 2 ? v[2] : v[3];
    float maxv = __shfl(mine, (cand >> 2) & 63, CQ_WAVE);

    uint32_t packed = 0;
    int lsum = 0;
    float d = 0.0f;
    if (wmax != 0.0f) {
        float iscale = -127.0f / maxv;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int q = round_sat_i8(iscale * v[i]);
            lsum += q;
            packed |= (uint32_t)(q & 0xff) << (8 * i);
        }
        d = 1.0f / iscale;
    }
    reinterpret_cast<uint32_t *>(qs)[blk * 64 + lane] = packed;
    // 16-element sums: four neighbouring lanes
    lsum += __shfl_xor(lsum, 1, CQ_WAVE);
    lsum += __shfl_xor(lsum, 2, CQ_WAVE);
    if ((lane & 3) == 0) bsums[blk * 16 + (lane >> 2)] = (int16_t)lsum;
    if (lane == 0) dout[blk] = d;
}

// ---- Q8_0: one wave per 8 blocks of 32 elements ---------------------------------------------
// `total` (= rows * k) is a multiple of 32 but not necessarily of 256: lanes past the end stay in
// the wave for the shuffles and neither load nor store.
template <int XDT>
__global__ __launch_bounds__(256) void quantize_q80_kernel(const void *__restrict__ x, int8_t *__restrict__ qs,
                                                           float *__restrict__ ds, int64_t total) {
    const int lane = threadIdx.x & 63;
    const int64_t span = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);   // 256 elements = 8 blocks
    const int64_t base = span * 256 + lane * 4;
    const bool valid = base < total;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (valid) load4<XDT>(x, base, v);
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    amax = fmaxf(amax, __shfl_xor(amax, 1, CQ_WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 2, CQ_WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 4, CQ_WAVE));
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint32_t packed = 0;
    int lsum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int q = round_sat_i8(v[i] * id);
        lsum += q;
        packed |= (uint32_t)(q & 0xff) << (8 * i);
    }
    lsum += __shfl_xor(lsum, 1, CQ_WAVE);
    lsum += __shfl_xor(lsum, 2, CQ_WAVE);
    lsum += __shfl_xor(lsum, 4, CQ_WAVE);
    if (!valid) return;
    reinterpret_cast<uint32_t *>(qs)[base >> 2] = packed;
    if ((lane & 7) == 0) {
        // the CPU path stores d as f16 and multiplies by f16::to_f32(d) in vec_dot
        float d16 = h2f(f2h_bits(d));
        u32x2 o;
        o.x = __float_as_uint(d16);
        o.y = (uint32_t)lsum;
        reinterpret_cast<u32x2 *>(ds)[base >> 5] = o;
    }
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
