// Weight quantization on the device (QTensor::quantize for a device tensor).
//
// candle's CUDA backend round-trips through the host for this (candle-core/src/quantized/cuda.rs:704-725:
// copy to host, GgmlType::from_float, copy back).  Here one GPU thread runs the scalar from_float
// arithmetic of one block, in the reference's evaluation order and with IEEE division / no
// contraction, so the bytes are the ones the CPU produces:
//   Q4_0 k_quants.rs:241-277, Q8_0 :658-687, Q4_K :1542-1600, Q5_K :1804-1877, Q6_K :2094-2164,
//   Q8_K :2320-2358, Q4_1 :353-389, Q5_0 :457-493, Q5_1 :564-604, Q8_1 :770-799, Q2_K :891-953, Q3_K :1190-1269; helpers utils.rs:1-3 (nearest_int), :62-224 (make_qx_quants), :227-284 (make_qkx1_quants).
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
__device__ void make_qkx1(int nmax, int ntry, const float *x, float &scale_out, float &min_out, int n = 32) {
    uint8_t l[32];
    for (int i = 0; i < n; i++) l[i] = 0;
    float mn = x[0], mx = x[0];
    for (int i = 1; i < n; i++) {
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
        for (int i = 0; i < n; i++) {
            int li = clampi(nearest_int(iscale * (x[i] - mn)), 0, nmax);
            if ((uint8_t)li != l[i]) { l[i] = (uint8_t)li; did_change = true; }
            sumlx += (x[i] - mn) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.0f;
        for (int i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];
        mn = sum / (float)n;
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

// ---- Q4_1 :353-389, Q5_0 :457-493, Q5_1 :564-604, Q8_1 :770-799, Q2_K :891-953, Q3_K :1190-1269 ----
// f32::min / f32::max return the other operand when one is NaN, like fminf / fmaxf.
template <> __device__ void quantize_block<CQ_Q4_1>(const float *x, uint8_t *blk) {
    float mn = INFINITY, mx = -INFINITY;
    for (int j = 0; j < 32; j++) { mn = fminf(x[j], mn); mx = fmaxf(x[j], mx); }
    float d = (mx - mn) / 15.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    st_u<uint16_t>(blk, f2h_bits(d));
    st_u<uint16_t>(blk + 2, f2h_bits(mn));
    for (int j = 0; j < 16; j++) {
        uint32_t a = min(15u, f2u8_sat((x[j] - mn) * id + 0.5f));
        uint32_t b = min(15u, f2u8_sat((x[16 + j] - mn) * id + 0.5f));
        blk[4 + j] = (uint8_t)(a | (b << 4));
    }
}

template <> __device__ void quantize_block<CQ_Q5_0>(const float *x, uint8_t *blk) {
    float amax = 0.0f, mx = 0.0f;
    for (int j = 0; j < 32; j++)
        if (amax < fabsf(x[j])) { amax = fabsf(x[j]); mx = x[j]; }
    float d = mx / -16.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    st_u<uint16_t>(blk, f2h_bits(d));
    uint32_t qh = 0;
    for (int j = 0; j < 16; j++) {
        // `(v + 16.5) as i8`, then the smaller of it and 31, then `as u8`: a negative value keeps its low bits
        uint32_t a = (uint32_t)(uint8_t)min(f2i8_sat(x[j] * id + 16.5f), 31);
        uint32_t b = (uint32_t)(uint8_t)min(f2i8_sat(x[16 + j] * id + 16.5f), 31);
        blk[6 + j] = (uint8_t)((a & 0x0f) | ((b & 0x0f) << 4));
        qh |= ((a & 0x10) >> 4) << j;
        qh |= ((b & 0x10) >> 4) << (j + 16);
    }
    st_u<uint32_t>(blk + 2, qh);
}

template <> __device__ void quantize_block<CQ_Q5_1>(const float *x, uint8_t *blk) {
    float mn = INFINITY, mx = -INFINITY;
    for (int j = 0; j < 32; j++) { mn = fminf(x[j], mn); mx = fmaxf(x[j], mx); }
    float d = (mx - mn) / 31.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    st_u<uint16_t>(blk, f2h_bits(d));
    st_u<uint16_t>(blk + 2, f2h_bits(mn));
    uint32_t qh = 0;
    for (int j = 0; j < 16; j++) {
        uint32_t a = f2u8_sat((x[j] - mn) * id + 0.5f);
        uint32_t b = f2u8_sat((x[16 + j] - mn) * id + 0.5f);
        blk[8 + j] = (uint8_t)((a & 0x0f) | ((b & 0x0f) << 4));
        qh |= ((a & 0x10) >> 4) << j;
        qh |= ((b & 0x10) >> 4) << (j + 16);
    }
    st_u<uint32_t>(blk + 4, qh);
}

template <> __device__ void quantize_block<CQ_Q8_1>(const float *x, uint8_t *blk) {
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(x[j]));
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    const uint16_t dbits = f2h_bits(d);
    st_u<uint16_t>(blk, dbits);
    int sum = 0;
    for (int j = 0; j < 32; j++) {
        int q = f2i8_sat(roundf(x[j] * id));
        blk[4 + j] = (uint8_t)(int8_t)q;
        sum += q;
    }
    // f16(sum) * d as a product of two f16 values: computed in f32, rounded back to f16
    st_u<uint16_t>(blk + 2, f2h_bits(h2f(f2h_bits((float)sum)) * h2f(dbits)));
}

template <> __device__ void quantize_block<CQ_Q2K>(const float *x, uint8_t *blk) {
    float scales[16], mins[16];
    for (int j = 0; j < 16; j++) make_qkx1(3, 5, x + 16 * j, scales[j], mins[j], 16);
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 16; j++) {
        max_scale = fmaxf(scales[j], max_scale);
        max_min = fmaxf(mins[j], max_min);
    }
    uint8_t sc[16];
    uint16_t dbits = f2h_bits(0.0f), mbits = f2h_bits(0.0f);
    if (max_scale > 0.0f) {
        float iscale = 15.0f / max_scale;
        for (int j = 0; j < 16; j++) sc[j] = (uint8_t)nearest_int(iscale * scales[j]);      // `as u8` of an i32: low byte
        dbits = f2h_bits(max_scale / 15.0f);
    } else {
        for (int j = 0; j < 16; j++) sc[j] = 0;
    }
    if (max_min > 0.0f) {
        float iscale = 15.0f / max_min;
        for (int j = 0; j < 16; j++) sc[j] |= (uint8_t)((uint8_t)nearest_int(iscale * mins[j]) << 4);
        mbits = f2h_bits(max_min / 15.0f);
    }
    for (int j = 0; j < 16; j++) blk[j] = sc[j];
    st_u<uint16_t>(blk + 80, dbits);
    st_u<uint16_t>(blk + 82, mbits);
    const float dall = h2f(dbits), dmin = h2f(mbits);
    // level of element e
    auto level = [&](int e) -> uint32_t {
        const int j = e >> 4;
        const float d = dall * (float)(sc[j] & 0xf);
        if (d == 0.0f) return 0u;
        const float dm = dmin * (float)(sc[j] >> 4);
        return (uint32_t)clampi(nearest_int((x[e] + dm) / d), 0, 3);
    };
    for (int j = 0; j < 256; j += 128)
        for (int l = 0; l < 32; l++)
            blk[16 + j / 4 + l] = (uint8_t)(level(j + l) | (level(j + l + 32) << 2) | (level(j + l + 64) << 4) | (level(j + l + 96) << 6));
}

// utils.rs:287-352 with do_rmse = true: the scale (the levels are not used by the caller)
__device__ float make_q3_rmse(const float *x, int n, int nmax) {
    int8_t l[16];
    float mx = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; mx = x[i]; }
    }
    if (amax == 0.0f) return 0.0f;
    float iscale = -(float)nmax / mx;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int li = clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1);
        l[i] = (int8_t)li;
        float w = x[i] * x[i];
        sumlx += w * x[i] * (float)li;
        suml2 += w * (float)(li * li);
    }
    for (int t = 0; t < 5; t++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            float w = x[i] * x[i];
            float slx = sumlx - w * x[i] * (float)l[i];
            if (slx > 0.0f) {
                float sl2 = suml2 - w * (float)((int)l[i] * (int)l[i]);
                int new_l = clampi(nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1);
                if (new_l != (int)l[i]) {
                    slx += w * x[i] * (float)new_l;
                    sl2 += w * (float)(new_l * new_l);
                    if (sl2 > 0.0f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                        l[i] = (int8_t)new_l;
                        sumlx = slx;
                        suml2 = sl2;
                        n_changed++;
                    }
                }
            }
        }
        if (n_changed == 0) break;
    }
    return sumlx / suml2;
}

template <> __device__ void quantize_block<CQ_Q3K>(const float *x, uint8_t *blk) {
    float scales[16];
    for (int j = 0; j < 16; j++) scales[j] = make_q3_rmse(x + 16 * j, 16, 4);
    float max_scale = 0.0f;
    for (int j = 0; j < 16; j++)
        if (fabsf(scales[j]) > fabsf(max_scale)) max_scale = scales[j];
    uint8_t sc[12];
    for (int j = 0; j < 12; j++) sc[j] = 0;
    uint16_t dbits = f2h_bits(0.0f);
    if (max_scale != 0.0f) {
        float iscale = -32.0f / max_scale;
        for (int j = 0; j < 16; j++) {
            int lv = clampi(nearest_int(iscale * scales[j]), -32, 31) + 32;
            if (j < 8) sc[j] = (uint8_t)(lv & 0xf);
            else sc[j - 8] |= (uint8_t)((lv & 0xf) << 4);
            lv >>= 4;
            sc[j % 4 + 8] |= (uint8_t)(lv << (2 * (j / 4)));
        }
        dbits = f2h_bits(1.0f / iscale);
    }
    for (int j = 0; j < 12; j++) blk[96 + j] = sc[j];
    st_u<uint16_t>(blk + 108, dbits);
    const float dall = h2f(dbits);
    // level 0..7 of element e
    auto level = [&](int e) -> int {
        const int j = e >> 4;
        const int s4 = j < 8 ? (sc[j] & 0xf) : (sc[j - 8] >> 4);
        const int s6 = (int)(int8_t)(s4 | (((sc[8 + j % 4] >> (2 * (j / 4))) & 3) << 4)) - 32;
        const float d = dall * (float)s6;
        if (d == 0.0f) return 0;
        return clampi(nearest_int(x[e] / d), -4, 3) + 4;
    };
    // hmask byte m holds bit b = the high bit of element 32 b + m; qs byte 32 h + v the low two bits of elements
    // 128 h + v + {0, 32, 64, 96}
    for (int m = 0; m < 32; m++) {
        uint32_t hb = 0;
        uint32_t lo[8];
        for (int b = 0; b < 8; b++) {
            const int lv = level(32 * b + m);
            if (lv > 3) hb |= 1u << b;
            lo[b] = (uint32_t)(lv & 3);
        }
        blk[m] = (uint8_t)hb;
        blk[32 + m] = (uint8_t)(lo[0] | (lo[1] << 2) | (lo[2] << 4) | (lo[3] << 6));
        blk[64 + m] = (uint8_t)(lo[4] | (lo[5] << 2) | (lo[6] << 4) | (lo[7] << 6));
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
        case CQ_Q4_1: return launch_quantize<CQ_Q4_1>(x, blocks, elems, s);
        case CQ_Q5_0: return launch_quantize<CQ_Q5_0>(x, blocks, elems, s);
        case CQ_Q5_1: return launch_quantize<CQ_Q5_1>(x, blocks, elems, s);
        case CQ_Q8_1: return launch_quantize<CQ_Q8_1>(x, blocks, elems, s);
        case CQ_Q2K: return launch_quantize<CQ_Q2K>(x, blocks, elems, s);
        case CQ_Q3K: return launch_quantize<CQ_Q3K>(x, blocks, elems, s);
    }
    return CQ_ERR_DTYPE;
}
