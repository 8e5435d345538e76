// Weight quantization on the device (QTensor::quantize for a device tensor).
//
// candle's CUDA backend round-trips through the host for this (candle-core/src/quantized/cuda.rs:704-725:
// copy to host, GgmlType::from_float, copy back).  Here one GPU thread runs the scalar from_float
// arithmetic of one block, in the reference's evaluation order and with IEEE division / no
// contraction, so the bytes are the ones the CPU produces:
//   Q4_0 k_quants.rs:241-277, Q8_0 :658-687, Q4_K :1542-1600, Q5_K :1804-1877, Q6_K :2094-2164,
//   Q8_K :2320-2358; helpers utils.rs:1-3 (nearest_int), :62-224 (make_qx_quants), :227-284 (make_qkx1_quants).
// It is a load-time operation; blocks are independent, so the grid is simply one thread per block.
#include "cq_device.h"
#include "cq_launch.h"

namespace {

// ---- Rust cast semantics: saturating, NaN -> 0 ------------------------------------------------
__device__ __forceinline__ int f2i_sat(float v) {
    if (!(v == v)) return 0;
    if (v >= 2147483648.0f) return 2147483647;
    if (v <= -2147483648.0f) return (int)0x80000000;
    return (int)v;
}
__device__ __forceinline__ int nearest_int(float v) { return f2i_sat(roundf(v)); }
__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }
__device__ __forceinline__ uint32_t f2u8_sat(float v) {
    if (!(v == v) || v <= 0.0f) return 0;
    if (v >= 255.0f) return 255;
    return (uint32_t)v;
}
__device__ __forceinline__ int f2i8_sat(float v) {
    if (!(v == v)) return 0;
    if (v <= -128.0f) return -128;
    if (v >= 127.0f) return 127;
    return (int)v;
}
// f32::max / f32::min ignore a NaN operand, like fmaxf / fminf.
__device__ __forceinline__ int total_key(float f) {   // f32::total_cmp order
    int b = __float_as_int(f);
    return b ^ (int)(((uint32_t)(b >> 31)) >> 1);
}

// utils.rs:227-284
__device__ void make_qkx1(int nmax, int ntry, const float *x, float &scale_out, float &min_out) {
    uint8_t l[32];
    for (int i = 0; i < 32; i++) l[i] = 0;
    float mn = x[0], mx = x[0];
    for (int i = 1; i < 32; i++) {
        if (total_key(x[i]) < total_key(mn)) mn = x[i];
        if (total_key(x[i]) >= total_key(mx)) mx = x[i];
    }
    if (mx == mn) { scale_out = 0.0f; min_out = 0.0f; return; }
    if (!(mn < 0.0f)) mn = 0.0f;
    float iscale = (float)nmax / (mx - mn);
    float scale = 1.0f / iscale;
    for (int t = 0; t < ntry; t++) {
        float sumlx = 0.0f;
        int suml2 = 0;
        bool did_change = false;
        for (int i = 0; i < 32; i++) {
            int li = clampi(nearest_int(iscale * (x[i] - mn)), 0, nmax);
            if ((uint8_t)li != l[i]) { l[i] = (uint8_t)li; did_change = true; }
            sumlx += (x[i] - mn) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.0f;
        for (int i = 0; i < 32; i++) sum += x[i] - scale * (float)l[i];
        mn = sum / 32.0f;
        if (mn > 0.0f) mn = 0.0f;
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    scale_out = scale;
    min_out = -mn;
}

// utils.rs:62-224 with rmse_type = 1 and no external weights (the only form Q6_K uses): w = x*x
__device__ float make_qx_rmse1(int n, int nmax, const float *x, int8_t *ls) {
    float mx = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; mx = x[i]; }
    }
    if (amax == 0.0f) {
        for (int i = 0; i < n; i++) ls[i] = 0;
        return 0.0f;
    }
    float iscale = -(float)nmax / mx;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int l = clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1);
        ls[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        float lf = (float)l;
        sumlx += w * x[i] * lf;
        suml2 += w * lf * lf;
    }
    float scale = sumlx / suml2;
    float best = scale * sumlx;
    for (int itry = 0; itry < 3; itry++) {
        float is2 = 1.0f / scale;
        float slx = 0.0f, sl2 = 0.0f;
        bool changed = false;
        for (int i = 0; i < n; i++) {
            int l = clampi(nearest_int(is2 * x[i]), -nmax, nmax - 1);
            if (l + nmax != (int)ls[i]) changed = true;
            float w = x[i] * x[i];
            float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
        for (int i = 0; i < n; i++) {
            int l = nearest_int(is2 * x[i]);
            ls[i] = (int8_t)(nmax + clampi(l, -nmax, nmax - 1));
        }
        sumlx = slx;
        suml2 = sl2;
        scale = sumlx / suml2;
        best = scale * sumlx;
    }
    for (int itry = 0; itry < 5; itry++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            float w = x[i] * x[i];
            int l = (int)ls[i] - nmax;
            float slx = sumlx - w * x[i] * (float)l;
            if (slx > 0.0f) {
                float sl2 = suml2 - w * (float)l * (float)l;
                int new_l = clampi(nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1);
                if (new_l != l) {
                    slx += w * x[i] * (float)new_l;
                    sl2 += w * (float)new_l * (float)new_l;
                    if (sl2 > 0.0f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                        ls[i] = (int8_t)(nmax + new_l);
                        sumlx = slx;
                        suml2 = sl2;
                        scale = sumlx / suml2;
                        best = scale * sumlx;
                        n_changed++;
                    }
                }
            }
        }
        if (n_changed == 0) break;
    }
    return scale;
}

// ---- per-format block quantizers ----------------------------------------------------------------
template <int DT> __device__ void quantize_block(const float *x, uint8_t *blk);

template <> __device__ void quantize_block<CQ_Q4_0>(const float *x, uint8_t *blk) {
    float amax = 0.0f, mx = 0.0f;
    for (int j = 0; j < 32; j++)
        if (amax < fabsf(x[j])) { amax = fabsf(x[j]); mx = x[j]; }
    float d = mx / -8.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    st_u<uint16_t>(blk, f2h_bits(d));
    for (int j = 0; j < 16; j++) {
        uint32_t a = min(15u, f2u8_sat(x[j] * id + 8.5f));
        uint32_t b = min(15u, f2u8_sat(x[16 + j] * id + 8.5f));
        blk[2 + j] = (uint8_t)(a | (b << 4));
    }
}

template <> __device__ void quantize_block<CQ_Q8_0>(const float *x, uint8_t *blk) {
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(x[j]));
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    st_u<uint16_t>(blk, f2h_bits(d));
    for (int j = 0; j < 32; j++) blk[2 + j] = (uint8_t)(int8_t)f2i8_sat(roundf(x[j] * id));
}

template <> __device__ void quantize_block<CQ_Q8K>(const float *x, uint8_t *blk) {
    float mx = 0.0f, amax = 0.0f;
    for (int j = 0; j < 256; j++)
        if (amax < fabsf(x[j])) { amax = fabsf(x[j]); mx = x[j]; }
    if (amax == 0.0f) {
        for (int j = 0; j < 292; j++) blk[j] = 0;   // d = 0, qs = 0; bsums written as zeros
        return;
    }
    float iscale = -127.0f / mx;
    for (int j = 0; j < 16; j++) {
        int sum = 0;
        for (int ii = 0; ii < 16; ii++) {
            float v = roundf(iscale * x[16 * j + ii]);
            v = fminf(fmaxf(v, -128.0f), 127.0f);     // clamp keeps NaN, the cast below maps it to 0
            int q = f2i8_sat(v);
            blk[4 + 16 * j + ii] = (uint8_t)(int8_t)q;
            sum += q;
        }
        st_u<int16_t>(blk + 260 + 2 * j, (int16_t)sum);
    }
    st_u<float>(blk, 1.0f / iscale);
}

// sub-block scales / mins and their 6-bit packing, shared by Q4_K and Q5_K (k_quants.rs:1544-1576)
__device__ void kquant_scales(const float *x, int nmax, uint8_t *blk) {
    float scales[8], mins[8];
    for (int j = 0; j < 8; j++) make_qkx1(nmax, 5, x + 32 * j, scales[j], mins[j]);
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; j++) {
        max_scale = fmaxf(scales[j], max_scale);
        max_min = fmaxf(mins[j], max_min);
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint8_t sc[12];
    for (int j = 0; j < 12; j++) sc[j] = 0;
    for (int j = 0; j < 8; j++) {
        uint8_t ls = (uint8_t)min(nearest_int(inv_scale * scales[j]), 63);
        uint8_t lm = (uint8_t)min(nearest_int(inv_min * mins[j]), 63);
        if (j < 4) {
            sc[j] = ls;
            sc[j + 4] = lm;
        } else {
            sc[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            sc[j - 4] |= (uint8_t)((ls >> 4) << 6);
            sc[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    st_u<uint16_t>(blk, f2h_bits(max_scale / 63.0f));
    st_u<uint16_t>(blk + 2, f2h_bits(max_min / 63.0f));
    for (int j = 0; j < 12; j++) blk[4 + j] = sc[j];
}

__device__ __forceinline__ void k4_scale_min(int j, const uint8_t *q, int &sc, int &m) {   // utils.rs:50-60
    if (j < 4) {
        sc = q[j] & 63;
        m = q[j + 4] & 63;
    } else {
        sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
        m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

// quantized level of element e (0..255) of a Q4_K / Q5_K block whose header is already written
__device__ __forceinline__ int k45_level(const float *x, const uint8_t *blk, float d, float dmin, int e, int qmax) {
    int sc, m;
    k4_scale_min(e >> 5, blk + 4, sc, m);
    float ds = d * (float)sc;
    if (ds == 0.0f) return 0;
    float dm = dmin * (float)m;
    return clampi(nearest_int((x[e] + dm) / ds), 0, qmax);
}

template <> __device__ void quantize_block<CQ_Q4K>(const float *x, uint8_t *blk) {
    kquant_scales(x, 15, blk);
    float d = h2f(ld_u<uint16_t>(blk)), dmin = h2f(ld_u<uint16_t>(blk + 2));
    for (int g = 0; g < 4; g++)
        for (int l = 0; l < 32; l++) {
            int a = k45_level(x, blk, d, dmin, 64 * g + l, 15);
            int b = k45_level(x, blk, d, dmin, 64 * g + 32 + l, 15);
            blk[16 + 32 * g + l] = (uint8_t)(a | (b << 4));
        }
}

template <> __device__ void quantize_block<CQ_Q5K>(const float *x, uint8_t *blk) {
    kquant_scales(x, 31, blk);
    float d = h2f(ld_u<uint16_t>(blk)), dmin = h2f(ld_u<uint16_t>(blk + 2));
    for (int l = 0; l < 32; l++) {
        uint32_t qh = 0;
        for (int g = 0; g < 4; g++) {
            int a = k45_level(x, blk, d, dmin, 64 * g + l, 31);
            int b = k45_level(x, blk, d, dmin, 64 * g + 32 + l, 31);
            if (a > 15) { a -= 16; qh |= 1u << (2 * g); }
            if (b > 15) { b -= 16; qh |= 2u << (2 * g); }
            blk[48 + 32 * g + l] = (uint8_t)(a | (b << 4));
        }
        blk[16 + l] = (uint8_t)qh;
    }
}

template <> __device__ void quantize_block<CQ_Q6K>(const float *x, uint8_t *blk) {
    int8_t l[256];
    float scales[16];
    float max_scale = 0.0f, max_abs_scale = 0.0f;
    for (int ib = 0; ib < 16; ib++) {
        float scale = make_qx_rmse1(16, 32, x + 16 * ib, l + 16 * ib);
        scales[ib] = scale;
        float a = fabsf(scale);
        if (a > max_abs_scale) { max_abs_scale = a; max_scale = scale; }
    }
    float iscale = -128.0f / max_scale;          // no zero guard in the reference either
    uint16_t dbits = f2h_bits(1.0f / iscale);
    float d = h2f(dbits);
    st_u<uint16_t>(blk + 208, dbits);
    for (int j = 0; j < 16; j++) {
        int s = min(nearest_int(iscale * scales[j]), 127);
        int8_t s8 = (int8_t)s;
        blk[192 + j] = (uint8_t)s8;
        float dj = d * (float)s8;
        if (dj == 0.0f) continue;
        for (int ii = 0; ii < 16; ii++) {
            int ll = clampi(nearest_int(x[16 * j + ii] / dj), -32, 31);
            l[16 * j + ii] = (int8_t)(ll + 32);
        }
    }
    for (int h = 0; h < 2; h++)
        for (int li = 0; li < 32; li++) {
            int j = 128 * h + li;
            int q1 = l[j] & 0xF, q2 = l[j + 32] & 0xF, q3 = l[j + 64] & 0xF, q4 = l[j + 96] & 0xF;
            blk[64 * h + li] = (uint8_t)(q1 | (q3 << 4));
            blk[64 * h + li + 32] = (uint8_t)(q2 | (q4 << 4));
            blk[128 + 32 * h + li] = (uint8_t)((l[j] >> 4) | ((l[j + 32] >> 4) << 2) | ((l[j + 64] >> 4) << 4) | ((l[j + 96] >> 4) << 6));
        }
}

template <int DT>
__global__ __launch_bounds__(64) void quantize_kernel(const float *__restrict__ x, uint8_t *__restrict__ blocks, int64_t n_blocks) {
    int64_t b = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (b >= n_blocks) return;
    quantize_block<DT>(x + b * BlockInfo<DT>::elems, blocks + b * BlockInfo<DT>::bytes);
}

template <int DT> int launch_quantize(const float *x, void *blocks, int64_t elems, hipStream_t s) {
    int64_t nb = elems / BlockInfo<DT>::elems;
    int64_t grid = (nb + 63) / 64;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    hipLaunchKernelGGL((quantize_kernel<DT>), dim3((unsigned)grid), dim3(64), 0, s, x, (uint8_t *)blocks, nb);
    return (int)hipGetLastError();
}

}  // namespace

int cq_quantize_launch(int dtype, const float *x, void *blocks, int64_t elems, hipStream_t s) {
    if (elems == 0) return CQ_OK;
    switch (dtype) {
        case CQ_Q4_0: return launch_quantize<CQ_Q4_0>(x, blocks, elems, s);
        case CQ_Q8_0: return launch_quantize<CQ_Q8_0>(x, blocks, elems, s);
        case CQ_Q4K: return launch_quantize<CQ_Q4K>(x, blocks, elems, s);
        case CQ_Q5K: return launch_quantize<CQ_Q5K>(x, blocks, elems, s);
        case CQ_Q6K: return launch_quantize<CQ_Q6K>(x, blocks, elems, s);
        case CQ_Q8K: return launch_quantize<CQ_Q8K>(x, blocks, elems, s);
    }
    return CQ_ERR_DTYPE;
}
