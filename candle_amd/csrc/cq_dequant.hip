// Block dequantization (QTensor::dequantize / dequantize_f16) for gfx950.
//
// Each thread produces four consecutive output elements (one 16-byte f32 store or one 8-byte f16
// store), so a wave writes 1 KiB / 512 B of contiguous output; the kernel is write-bound
// (4 B out per 0.5-1.06 B in).  The arithmetic is the CPU to_float, evaluated in the same order:
//   Q4_0 k_quants.rs:219-239, Q8_0 :640-656, Q4_K :1667-1694, Q5_K :1962-1996, Q6_K :2247-2278,
//   Q8_K :2360-2371, and the formats that exist here only as storage (no matmul kernels): Q4_1 :392-412, Q5_0 :496-518,
//   Q5_1 :607-631, Q8_1 :801-816, Q2_K :1013-1049, Q3_K :1369-1421 (candle-core/src/quantized/k_quants.rs).
// All products are exactly representable in f32 (so a fused multiply-add rounds like the CPU's multiply then add), and
// results are bit-identical to the CPU.
#include "cq_device.h"

namespace {

// 6-bit scale / min of sub-block j from the 12 packed bytes (utils.rs:50-60).
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t *q, int &sc, int &m) {
    if (j < 4) {
        sc = q[j] & 63;
        m = q[j + 4] & 63;
    } else {
        sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
        m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

template <int DT> __device__ __forceinline__ void dequant4(const uint8_t *blk, int e, float out[4]);

template <> __device__ __forceinline__ void dequant4<CQ_Q4_0>(const uint8_t *blk, int e, float out[4]) {
    float d = h2f(ld_u<uint16_t>(blk));
    uint32_t q = ld_u<uint32_t>(blk + 2 + (e & 15));
    if (e >= 16) q >>= 4;
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = (float)((int)((q >> (8 * i)) & 0xF) - 8) * d;
}

template <> __device__ __forceinline__ void dequant4<CQ_Q8_0>(const uint8_t *blk, int e, float out[4]) {
    float d = h2f(ld_u<uint16_t>(blk));
    uint32_t q = ld_u<uint32_t>(blk + 2 + e);
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = (float)(int8_t)((q >> (8 * i)) & 0xFF) * d;
}

template <> __device__ __forceinline__ void dequant4<CQ_Q8K>(const uint8_t *blk, int e, float out[4]) {
    float d = ld_u<float>(blk);
    uint32_t q = ld_u<uint32_t>(blk + 4 + e);
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = d * (float)(int8_t)((q >> (8 * i)) & 0xFF);
}

template <> __device__ __forceinline__ void dequant4<CQ_Q4K>(const uint8_t *blk, int e, float out[4]) {
    uint32_t dm = ld_u<uint32_t>(blk);
    float d = h2f(dm), dmin = h2f(dm >> 16);
    int g = e >> 6, half = (e >> 5) & 1, l = e & 31;
    int sc, m;
    scale_min_k4(2 * g + half, blk + 4, sc, m);
    float d1 = d * (float)sc, m1 = dmin * (float)m;
    uint32_t q = ld_u<uint32_t>(blk + 16 + 32 * g + l);
    if (half) q >>= 4;
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = d1 * (float)((q >> (8 * i)) & 0xF) - m1;
}

template <> __device__ __forceinline__ void dequant4<CQ_Q5K>(const uint8_t *blk, int e, float out[4]) {
    uint32_t dm = ld_u<uint32_t>(blk);
    float d = h2f(dm), dmin = h2f(dm >> 16);
    int g = e >> 6, half = (e >> 5) & 1, l = e & 31;
    int sc, m;
    scale_min_k4(2 * g + half, blk + 4, sc, m);
    float d1 = d * (float)sc, m1 = dmin * (float)m;
    uint32_t qh = ld_u<uint32_t>(blk + 16 + l) >> (2 * g + half);
    uint32_t q = ld_u<uint32_t>(blk + 48 + 32 * g + l);
    if (half) q >>= 4;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float to_add = ((qh >> (8 * i)) & 1) ? 16.0f : 0.0f;
        out[i] = d1 * ((float)((q >> (8 * i)) & 0xF) + to_add) - m1;
    }
}

template <> __device__ __forceinline__ void dequant4<CQ_Q6K>(const uint8_t *blk, int e, float out[4]) {
    float d = h2f(ld_u<uint16_t>(blk + 208));
    int h = e >> 7, r = e & 127, quarter = r >> 5, l = r & 31;
    const uint8_t *ql = blk + 64 * h, *qh = blk + 128 + 32 * h;
    int sc = (int)(int8_t)blk[192 + 8 * h + (l >> 4) + 2 * quarter];
    uint32_t lo = ld_u<uint32_t>(ql + l + ((quarter & 1) ? 32 : 0));
    if (quarter >= 2) lo >>= 4;
    uint32_t hi = ld_u<uint32_t>(qh + l) >> (2 * quarter);
    float ds = d * (float)sc;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int q = (int)(((lo >> (8 * i)) & 0xF) | (((hi >> (8 * i)) & 3) << 4)) - 32;
        out[i] = ds * (float)q;
    }
}

template <> __device__ __forceinline__ void dequant4<CQ_Q4_1>(const uint8_t *blk, int e, float out[4]) {
    uint32_t dm = ld_u<uint32_t>(blk);
    float d = h2f(dm), m = h2f(dm >> 16);
    uint32_t q = ld_u<uint32_t>(blk + 4 + (e & 15));
    if (e >= 16) q >>= 4;
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = (float)((q >> (8 * i)) & 0xF) * d + m;
}

// Q5_0 / Q5_1: bit j of the little-endian u32 qh is the fifth bit of element j (both halves of the block)
template <> __device__ __forceinline__ void dequant4<CQ_Q5_0>(const uint8_t *blk, int e, float out[4]) {
    float d = h2f(ld_u<uint16_t>(blk));
    uint32_t qh = ld_u<uint32_t>(blk + 2) >> e;
    uint32_t q = ld_u<uint32_t>(blk + 6 + (e & 15));
    if (e >= 16) q >>= 4;
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = (float)((int)(((q >> (8 * i)) & 0xF) | (((qh >> i) & 1) << 4)) - 16) * d;
}

template <> __device__ __forceinline__ void dequant4<CQ_Q5_1>(const uint8_t *blk, int e, float out[4]) {
    uint32_t dm = ld_u<uint32_t>(blk);
    float d = h2f(dm), m = h2f(dm >> 16);
    uint32_t qh = ld_u<uint32_t>(blk + 4) >> e;
    uint32_t q = ld_u<uint32_t>(blk + 8 + (e & 15));
    if (e >= 16) q >>= 4;
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = (float)(((q >> (8 * i)) & 0xF) | (((qh >> i) & 1) << 4)) * d + m;
}

template <> __device__ __forceinline__ void dequant4<CQ_Q8_1>(const uint8_t *blk, int e, float out[4]) {
    float d = h2f(ld_u<uint16_t>(blk));
    uint32_t q = ld_u<uint32_t>(blk + 4 + e);
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = (float)(int8_t)((q >> (8 * i)) & 0xFF) * d;
}

// Q2_K / Q3_K: element e = 128 h + 32 j + l holds bits [2 j, 2 j + 2) of qs[32 h + l]; its scale is number 8 h + 2 j + l / 16
template <> __device__ __forceinline__ void dequant4<CQ_Q2K>(const uint8_t *blk, int e, float out[4]) {
    uint32_t dm = ld_u<uint32_t>(blk + 80);
    float d = h2f(dm), dmin = h2f(dm >> 16);
    int h = e >> 7, j = (e >> 5) & 3, l = e & 31;
    uint32_t sc = blk[8 * h + 2 * j + (l >> 4)];
    float dl = d * (float)(sc & 0xF), ml = dmin * (float)(sc >> 4);
    uint32_t q = ld_u<uint32_t>(blk + 16 + 32 * h + l) >> (2 * j);
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = dl * (float)((q >> (8 * i)) & 3) - ml;
}

template <> __device__ __forceinline__ void dequant4<CQ_Q3K>(const uint8_t *blk, int e, float out[4]) {
    float d_all = h2f(ld_u<uint16_t>(blk + 108));
    int h = e >> 7, j = (e >> 5) & 3, l = e & 31;
    // 6-bit scale number is: low four bits in scales[is % 8] (low nibble for is < 8, high nibble otherwise), top two bits in
    // scales[8 + is % 4] at bit 2 (is / 4); stored with an offset of 32
    int is = 8 * h + 2 * j + (l >> 4);
    const uint8_t *sc = blk + 96;
    int lo = is < 8 ? (sc[is] & 0xF) : (sc[is - 8] >> 4);
    int hi = (sc[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
    float dl = d_all * ((float)(int8_t)(lo | (hi << 4)) - 32.0f);
    uint32_t q = ld_u<uint32_t>(blk + 32 + 32 * h + l) >> (2 * j);
    uint32_t hm = ld_u<uint32_t>(blk + l) >> (4 * h + j);          // hmask bit set: no -4
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = dl * (float)((int)((q >> (8 * i)) & 3) - (((hm >> (8 * i)) & 1) ? 0 : 4));
}

template <int DT, bool F16OUT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t *__restrict__ blocks, void *__restrict__ out, int64_t n_quads) {
    constexpr int E = BlockInfo<DT>::elems, B = BlockInfo<DT>::bytes;
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_quads) return;
    int64_t elem = t * 4;
    int64_t ib = elem / E;
    int e = (int)(elem - ib * E);
    float v[4];
    dequant4<DT>(blocks + ib * B, e, v);
    if (F16OUT) {
        u32x2 o;
        o.x = (uint32_t)f2h_bits(v[0]) | ((uint32_t)f2h_bits(v[1]) << 16);
        o.y = (uint32_t)f2h_bits(v[2]) | ((uint32_t)f2h_bits(v[3]) << 16);
        reinterpret_cast<u32x2 *>(out)[t] = o;
    } else {
        f32x4 o = {v[0], v[1], v[2], v[3]};
        reinterpret_cast<f32x4 *>(out)[t] = o;
    }
}

// QTensor::embedding: output row r is row ids[r] of the [rows, hidden] block matrix, dequantized (mod.rs:449-473).  An id
// outside [0, rows) gives a row of zeros (the CPU path reports an error instead; the host wrapper checks the ids).
template <int DT>
__global__ __launch_bounds__(256) void embedding_rows_kernel(const uint8_t *__restrict__ blocks, const uint32_t *__restrict__ ids,
                                                             float *__restrict__ out, int64_t n_quads, int quads_per_row, int rows) {
    constexpr int E = BlockInfo<DT>::elems, B = BlockInfo<DT>::bytes;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= n_quads) return;
    const int64_t r = t / quads_per_row;
    const int64_t col = (t - r * quads_per_row) * 4;
    const uint32_t id = ids[r];
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (id < (uint32_t)rows) {
        const int64_t elem = (int64_t)id * quads_per_row * 4 + col;
        const int64_t ib = elem / E;
        dequant4<DT>(blocks + ib * B, (int)(elem - ib * E), v);
    }
    reinterpret_cast<f32x4 *>(out)[t] = f32x4{v[0], v[1], v[2], v[3]};
}

template <int DT> int launch_embedding(const void *blocks, const uint32_t *ids, float *out, int64_t n_ids, int64_t rows, int64_t hidden, hipStream_t s) {
    const int64_t quads = n_ids * (hidden / 4);
    if (quads == 0) return CQ_OK;
    const int64_t grid = (quads + 255) / 256;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    hipLaunchKernelGGL((embedding_rows_kernel<DT>), dim3((unsigned)grid), dim3(256), 0, s, (const uint8_t *)blocks, ids, out, quads, (int)(hidden / 4),
                       (int)rows);
    return (int)hipGetLastError();
}

template <int DT> int launch_dequant(const void *blocks, void *out, int64_t elems, int out_dtype, hipStream_t s) {
    int64_t quads = elems / 4;
    if (quads == 0) return CQ_OK;
    int64_t grid = (quads + 255) / 256;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (out_dtype == CQ_F16)
        hipLaunchKernelGGL((dequant_kernel<DT, true>), dim3((unsigned)grid), dim3(256), 0, s, (const uint8_t *)blocks, out, quads);
    else
        hipLaunchKernelGGL((dequant_kernel<DT, false>), dim3((unsigned)grid), dim3(256), 0, s, (const uint8_t *)blocks, out, quads);
    return (int)hipGetLastError();
}

}  // namespace

int cq_dequantize_launch(int dtype, const void *blocks, void *out, int64_t elems, int out_dtype, hipStream_t s) {
    switch (dtype) {
        case CQ_Q4_0: return launch_dequant<CQ_Q4_0>(blocks, out, elems, out_dtype, s);
        case CQ_Q8_0: return launch_dequant<CQ_Q8_0>(blocks, out, elems, out_dtype, s);
        case CQ_Q4K: return launch_dequant<CQ_Q4K>(blocks, out, elems, out_dtype, s);
        case CQ_Q5K: return launch_dequant<CQ_Q5K>(blocks, out, elems, out_dtype, s);
        case CQ_Q6K: return launch_dequant<CQ_Q6K>(blocks, out, elems, out_dtype, s);
        case CQ_Q8K: return launch_dequant<CQ_Q8K>(blocks, out, elems, out_dtype, s);
        case CQ_Q4_1: return launch_dequant<CQ_Q4_1>(blocks, out, elems, out_dtype, s);
        case CQ_Q5_0: return launch_dequant<CQ_Q5_0>(blocks, out, elems, out_dtype, s);
        case CQ_Q5_1: return launch_dequant<CQ_Q5_1>(blocks, out, elems, out_dtype, s);
        case CQ_Q8_1: return launch_dequant<CQ_Q8_1>(blocks, out, elems, out_dtype, s);
        case CQ_Q2K: return launch_dequant<CQ_Q2K>(blocks, out, elems, out_dtype, s);
        case CQ_Q3K: return launch_dequant<CQ_Q3K>(blocks, out, elems, out_dtype, s);
    }
    return CQ_ERR_DTYPE;
}

int cq_embedding_launch(int dtype, const void *blocks, const uint32_t *ids, float *out, int64_t n_ids, int64_t rows, int64_t hidden, hipStream_t s) {
    switch (dtype) {
#define CQ_EMB(DT) case DT: return launch_embedding<DT>(blocks, ids, out, n_ids, rows, hidden, s);
        CQ_EMB(CQ_Q4_0) CQ_EMB(CQ_Q4_1) CQ_EMB(CQ_Q5_0) CQ_EMB(CQ_Q5_1) CQ_EMB(CQ_Q8_0) CQ_EMB(CQ_Q8_1)
        CQ_EMB(CQ_Q2K) CQ_EMB(CQ_Q3K) CQ_EMB(CQ_Q4K) CQ_EMB(CQ_Q5K) CQ_EMB(CQ_Q6K) CQ_EMB(CQ_Q8K)
#undef CQ_EMB
    }
    return CQ_ERR_DTYPE;
}
