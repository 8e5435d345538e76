// Wave-level activation quantizers, bit-identical to candle's CPU path:
//   Q8_K blocks (256 elements, f32 scale, 16-element sums) for K-quant weights
//     — BlockQ8K::from_float, candle-core/src/quantized/k_quants.rs:2320-2358
//   Q8_0 blocks (32 elements, f16 scale) for Q4_0 / Q8_0 weights
//     — BlockQ8_0::from_float, k_quants.rs:658-687
// f16 / bf16 activations are widened to f32 first, as k_quants::matmul_f16 does (k_quants.rs:2652-2686).
//
// One wave64 quantizes one 256-element span: each lane owns four consecutive elements (one 16-byte
// load, one packed 4-byte int8 store).  The output pointers may be global (the stand-alone kernels)
// or LDS (the matvec kernel quantizes its activations in place).
#pragma once
#include "cq_device.h"

template <int XDT> __device__ __forceinline__ void cq_load4(const void *x, int64_t idx, float v[4]);
template <> __device__ __forceinline__ void cq_load4<CQ_F32>(const void *x, int64_t idx, float v[4]) {
    f32x4 t = *reinterpret_cast<const f32x4 *>((const float *)x + idx);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <> __device__ __forceinline__ void cq_load4<CQ_F16>(const void *x, int64_t idx, float v[4]) {
    u32x2 t = *reinterpret_cast<const u32x2 *>((const uint16_t *)x + idx);
    v[0] = h2f(t.x); v[1] = h2f(t.x >> 16); v[2] = h2f(t.y); v[3] = h2f(t.y >> 16);
}
template <> __device__ __forceinline__ void cq_load4<CQ_BF16>(const void *x, int64_t idx, float v[4]) {
    u32x2 t = *reinterpret_cast<const u32x2 *>((const uint16_t *)x + idx);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}

// Rust `v as i8` after f32::round: saturating, NaN -> 0.
__device__ __forceinline__ int cq_round_sat_i8(float v) {
    float r = roundf(v);                 // half away from zero, like f32::round
    if (!(r == r)) return 0;
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int)r;
}

// Q8_K: the calling wave quantizes block `blk` (elements blk*256 .. +255 of x).
//   qs    int8  [.. 256 per block]      d  float [1 per block]      bsums int16 [16 per block]
//
// cq_quantize_q8k_vals takes the lane's four values already in registers, so a caller can issue the
// load early and overlap its latency with other work.
__device__ __forceinline__ void cq_quantize_q8k_vals(const float v[4], int64_t blk, int lane, int8_t *qs, float *dout, int16_t *bsums) {
    // signed value of the first element with the largest magnitude (strict `<`: the first one wins)
    float amax = 0.0f;
    int idx = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float a = fabsf(v[i]);
        if (amax < a) { amax = a; idx = i; }
    }
    const float wmax = wave_max_nonneg(amax);
    const int cand = wave_min_int((amax == wmax && wmax != 0.0f) ? lane * 4 + idx : 256);   // lowest index holding the max
    float mine = idx == 0 ? v[0] : idx == 1 ? v[1] : idx == 2 ? v[2] : v[3];
    float maxv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), (cand >> 2) & 63));

    uint32_t packed = 0;
    int lsum = 0;
    float d = 0.0f;
    if (wmax != 0.0f) {
        float iscale = -127.0f / maxv;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int q = cq_round_sat_i8(iscale * v[i]);
            lsum += q;
            packed |= (uint32_t)(q & 0xff) << (8 * i);
        }
        d = 1.0f / iscale;
    }
    reinterpret_cast<uint32_t *>(qs)[blk * 64 + lane] = packed;
    lsum = quad_sum(lsum);                   // 16-element sums: four neighbouring lanes
    if ((lane & 3) == 0) bsums[blk * 16 + (lane >> 2)] = (int16_t)lsum;
    if (lane == 0) dout[blk] = d;
}

template <int XDT>
__device__ __forceinline__ void cq_quantize_q8k_span(const void *x, int64_t blk, int lane, int8_t *qs, float *dout, int16_t *bsums) {
    float v[4];
    cq_load4<XDT>(x, blk * 256 + lane * 4, v);
    cq_quantize_q8k_vals(v, blk, lane, qs, dout, bsums);
}

// Q8_0: the calling wave quantizes the 256-element span `span` (8 blocks of 32).  `total` is the
// element count of x, a multiple of 32 but not necessarily of 256: lanes past the end stay in the
// wave for the shuffles and neither load nor store.
//   qs int8 [..]      ds {float d (f16-rounded), int32 sum} [1 per 32-element block]
//
// cq_quantize_q80_vals: the lane's four values (zeros when `valid` is false) are already in registers.
__device__ __forceinline__ void cq_quantize_q80_vals(const float v[4], bool valid, int64_t base, int lane, int8_t *qs, float *ds) {
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    amax = oct_max(amax);                    // a 32-element block = eight neighbouring lanes
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint32_t packed = 0;
    int lsum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int q = cq_round_sat_i8(v[i] * id);
        lsum += q;
        packed |= (uint32_t)(q & 0xff) << (8 * i);
    }
    lsum = oct_sum(lsum);
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
__device__ __forceinline__ void cq_quantize_q80_span(const void *x, int64_t span, int lane, int64_t total, int8_t *qs, float *ds) {
    const int64_t base = span * 256 + lane * 4;
    const bool valid = base < total;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (valid) cq_load4<XDT>(x, base, v);
    cq_quantize_q80_vals(v, valid, base, lane, qs, ds);
}

// silu(gate) * up computed on the fly (the expression of silu_mul_kernel) and quantized: the f32 product never exists in
// memory.  Row r of the product is gate[r * gate_stride + i] , up[r * up_stride + i], i < 256 kb.
__device__ __forceinline__ void cq_load_swiglu4(const float *gate, const float *up, int64_t gi, int64_t ui, float v[4]) {
    const f32x4 g = *reinterpret_cast<const f32x4 *>(gate + gi), u = *reinterpret_cast<const f32x4 *>(up + ui);
    v[0] = g.x / (1.0f + expf(-g.x)) * u.x;
    v[1] = g.y / (1.0f + expf(-g.y)) * u.y;
    v[2] = g.z / (1.0f + expf(-g.z)) * u.z;
    v[3] = g.w / (1.0f + expf(-g.w)) * u.w;
}
