/*
 * CPU oracle for the GGUF quantized-matmul path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic of candle's CPU quantized path so
 * that the HIP kernels can be checked against it.  It is never linked into, imported by, or
 * called from the shipped library: only tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py may load it.
 *
 * Every function cites the reference source it follows (paths relative to the candle tree):
 *   k_quants.rs = candle-core/src/quantized/k_quants.rs
 *   utils.rs    = candle-core/src/quantized/utils.rs
 *   mod.rs      = candle-core/src/quantized/mod.rs
 *
 * Rust semantics that the restatement keeps:
 *   - f32::round is half-away-from-zero; `as` float->int casts saturate and map NaN to 0;
 *   - half::f16::from_f32 is round-to-nearest-even, to_f32 is exact;
 *   - no fused multiply-add and no re-association (build with -ffp-contract=off, no fast-math);
 *   - "first maximum wins" selection loops use a strict `<`.
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   to_float / from_float / vec_dot / matmul for Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, Q8_K are pinned
 *   by the reference's own known-answer vectors (candle-core/tests/quantized_tests.rs) plus
 *   closed-form and brute-force checks.  The MoE functions have no reference CPU counterpart
 *   (mod.rs:776-782 panics off-GPU); they are a composition of the pinned matmul and are pinned
 *   by brute force against per-pair matmul calls.
 *   to_float / from_float for Q4_1, Q5_0, Q5_1, Q2_K, Q3_K are pinned by the reference's quantize -> dequantize vectors for
 *   those formats (quantized_tests.rs:379-474, 751-844) and its error bounds; Q8_1 (no vector in the reference) by its
 *   closed form (the Q8_0 quantizer plus s = d * sum).  vec_dot / matmul for Q4_1, Q5_0, Q5_1, Q2_K, Q3_K are pinned by
 *   the reference's dot-product error ceilings (quantized_tests.rs:1101-1191), its seeded matmul values for Q2_K and
 *   Q3_K (:1331-1381), and the identity vec_dot(w, a) == sum(to_float(w) * to_float(a)) evaluated in f64 with the
 *   pinned to_float functions (random blocks, every bit of qs / qh / hmask / scales exercised).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256
#define K_SCALE_SIZE 12
#define QK4_0 32
#define QK8_0 32

/* GGUF type codes, mod.rs:300-342 */
enum {
    CQ_F32 = 0, CQ_F16 = 1, CQ_Q4_0 = 2, CQ_Q4_1 = 3, CQ_Q5_0 = 6, CQ_Q5_1 = 7, CQ_Q8_0 = 8,
    CQ_Q8_1 = 9, CQ_Q2K = 10, CQ_Q3K = 11, CQ_Q4K = 12, CQ_Q5K = 13, CQ_Q6K = 14, CQ_Q8K = 15,
    CQ_BF16 = 30
};

/* ---- block layouts, k_quants.rs:77-190 (repr(C), little-endian, no padding) ---- */
#pragma pack(push, 1)
typedef struct { uint16_t d; uint8_t qs[QK4_0 / 2]; } block_q4_0;                     /* 18 B */
typedef struct { uint16_t d; int8_t qs[QK8_0]; } block_q8_0;                          /* 34 B */
typedef struct { uint16_t d, m; uint8_t qs[16]; } block_q4_1;                           /* 20 B */
typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; } block_q5_0;               /* 22 B */
typedef struct { uint16_t d, m; uint8_t qh[4]; uint8_t qs[16]; } block_q5_1;            /* 24 B */
typedef struct { uint16_t d, s; int8_t qs[32]; } block_q8_1;                            /* 36 B */
typedef struct { uint8_t scales[QK_K / 16]; uint8_t qs[QK_K / 4]; uint16_t d, dmin; } block_q2_K;   /* 84 B */
typedef struct { uint8_t hmask[QK_K / 8]; uint8_t qs[QK_K / 4]; uint8_t scales[12]; uint16_t d; } block_q3_K; /* 110 B */
typedef struct { uint16_t d, dmin; uint8_t scales[K_SCALE_SIZE]; uint8_t qs[QK_K / 2]; } block_q4_K; /* 144 B */
typedef struct { uint16_t d, dmin; uint8_t scales[K_SCALE_SIZE]; uint8_t qh[QK_K / 8]; uint8_t qs[QK_K / 2]; } block_q5_K; /* 176 B */
typedef struct { uint8_t ql[QK_K / 2]; uint8_t qh[QK_K / 4]; int8_t scales[QK_K / 16]; uint16_t d; } block_q6_K; /* 210 B */
typedef struct { float d; int8_t qs[QK_K]; int16_t bsums[QK_K / 16]; } block_q8_K;   /* 292 B */
#pragma pack(pop)

_Static_assert(sizeof(block_q4_0) == 18, "q4_0");
_Static_assert(sizeof(block_q8_0) == 34, "q8_0");
_Static_assert(sizeof(block_q4_1) == 20 && sizeof(block_q5_0) == 22 && sizeof(block_q5_1) == 24 && sizeof(block_q8_1) == 36, "32-element blocks");
_Static_assert(sizeof(block_q2_K) == 84 && sizeof(block_q3_K) == 110, "q2_K / q3_K");
_Static_assert(sizeof(block_q4_K) == 144, "q4_K");
_Static_assert(sizeof(block_q5_K) == 176, "q5_K");
_Static_assert(sizeof(block_q6_K) == 210, "q6_K");
_Static_assert(sizeof(block_q8_K) == 292, "q8_K");

/* ------------------------------------------------------------------------------------------
 * f16 <-> f32, the `half` crate's software conversion (round to nearest even; to_f32 exact).
 * Call sites in the reference: k_quants.rs:229,267,308 and every block's d/dmin field.
 * ---------------------------------------------------------------------------------------- */
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float cqo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t cqo_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = x & 0x80000000u;
    uint32_t exp = x & 0x7F800000u;
    uint32_t man = x & 0x007FFFFFu;
    if (exp == 0x7F800000u) {
        uint32_t nan_bit = man == 0 ? 0 : 0x0200u;
        return (uint16_t)((sign >> 16) | 0x7C00u | nan_bit | (man >> 13));
    }
    uint32_t half_sign = sign >> 16;
    int32_t unbiased_exp = (int32_t)(exp >> 23) - 127;
    int32_t half_exp = unbiased_exp + 15;
    if (half_exp >= 0x1F) return (uint16_t)(half_sign | 0x7C00u);
    if (half_exp <= 0) {
        if (14 - half_exp > 24) return (uint16_t)half_sign;
        man |= 0x00800000u;
        uint32_t half_man = man >> (14 - half_exp);
        uint32_t round_bit = 1u << (13 - half_exp);
        if ((man & round_bit) != 0 && (man & (3 * round_bit - 1)) != 0) half_man += 1;
        return (uint16_t)(half_sign | half_man);
    }
    uint32_t he = (uint32_t)half_exp << 10;
    uint32_t half_man = man >> 13;
    uint32_t round_bit = 0x00001000u;
    if ((man & round_bit) != 0 && (man & (3 * round_bit - 1)) != 0)
        return (uint16_t)((half_sign | he | half_man) + 1);
    return (uint16_t)(half_sign | he | half_man);
}

/* ---- Rust numeric casts ---- */
static inline int32_t sat_i32(float v) {           /* `v as i32` */
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}
static inline uint8_t sat_u8(float v) {            /* `v as u8` */
    if (v != v) return 0;
    if (v <= 0.0f) return 0;
    if (v >= 255.0f) return 255;
    return (uint8_t)v;
}
static inline int8_t sat_i8(float v) {             /* `v as i8` */
    if (v != v) return 0;
    if (v <= -128.0f) return -128;
    if (v >= 127.0f) return 127;
    return (int8_t)v;
}
/* utils.rs:1-3  nearest_int = v.round() as i32 (round half away from zero) */
static inline int32_t nearest_int(float v) { return sat_i32(roundf(v)); }
static inline int32_t clamp_i32(int32_t v, int32_t lo, int32_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* utils.rs:50-60 */
static inline void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* f32 total order (Rust total_cmp), used by make_qkx1_quants' min/max scan */
static inline int32_t total_key(float f) {
    int32_t b = (int32_t)f32_bits(f);
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

/* ------------------------------------------------------------------------------------------
 * utils.rs:227-284  make_qkx1_quants(nmax, ntry, x) -> (scale, -min)
 * ---------------------------------------------------------------------------------------- */
static void make_qkx1_quants(int32_t nmax, int ntry, const float *x, int n, float *scale_out, float *min_out) {
    uint8_t l[64];
    memset(l, 0, sizeof(l));
    float min = x[0], max = x[0];
    for (int i = 1; i < n; i++) {                       /* min_by: first minimum; max_by: last maximum */
        if (total_key(x[i]) < total_key(min)) min = x[i];
        if (total_key(x[i]) >= total_key(max)) max = x[i];
    }
    if (max == min) { *scale_out = 0.0f; *min_out = 0.0f; return; }
    if (!(min < 0.0f)) min = 0.0f;                      /* min = min.min(0.) */
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    for (int t = 0; t < ntry; t++) {
        float sumlx = 0.0f;
        int32_t suml2 = 0;
        int did_change = 0;
        for (int i = 0; i < n; i++) {
            int32_t li = clamp_i32(nearest_int(iscale * (x[i] - min)), 0, nmax);
            uint8_t cl = (uint8_t)li;
            if (cl != l[i]) { l[i] = cl; did_change = 1; }
            sumlx += (x[i] - min) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.0f;
        for (int i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];
        min = sum / (float)n;
        if (min > 0.0f) min = 0.0f;
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    *scale_out = scale;
    *min_out = -min;
}

/* ------------------------------------------------------------------------------------------
 * utils.rs:62-224  make_qx_quants(n, nmax, x, ls, rmse_type, qw)
 * ---------------------------------------------------------------------------------------- */
static float make_qx_quants(int n, int32_t nmax, const float *x, int8_t *ls, int rmse_type, const float *qw) {
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.0f) {
        for (int i = 0; i < n; i++) ls[i] = 0;
        return 0.0f;
    }
    float iscale = -(float)nmax / max;
    if (rmse_type == 0) {
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(iscale * x[i]);
            ls[i] = (int8_t)(nmax + clamp_i32(l, -nmax, nmax - 1));
        }
        return 1.0f / iscale;
    }
    int weight_type = rmse_type % 2;
#define QX_W(i) (qw ? qw[i] : (weight_type == 1 ? x[i] * x[i] : 1.0f))
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int32_t l = clamp_i32(nearest_int(iscale * x[i]), -nmax, nmax - 1);
        ls[i] = (int8_t)(l + nmax);
        float w = QX_W(i);
        float lf = (float)l;
        sumlx += w * x[i] * lf;
        suml2 += w * lf * lf;
    }
    float scale = sumlx / suml2;
    float best = scale * sumlx;
    for (int itry = 0; itry < 3; itry++) {
        float is2 = 1.0f / scale;
        float slx = 0.0f, sl2 = 0.0f;
        int changed = 0;
        for (int i = 0; i < n; i++) {
            int32_t l = clamp_i32(nearest_int(is2 * x[i]), -nmax, nmax - 1);
            if (l + nmax != (int32_t)ls[i]) changed = 1;
            float w = QX_W(i);
            float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(is2 * x[i]);
            ls[i] = (int8_t)(nmax + clamp_i32(l, -nmax, nmax - 1));
        }
        sumlx = slx;
        suml2 = sl2;
        scale = sumlx / suml2;
        best = scale * sumlx;
    }
    for (int itry = 0; itry < 5; itry++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            float w = QX_W(i);
            int32_t l = (int32_t)ls[i] - nmax;
            float slx = sumlx - w * x[i] * (float)l;
            if (slx > 0.0f) {
                float sl2 = suml2 - w * (float)l * (float)l;
                int32_t new_l = clamp_i32(nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1);
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
    if (rmse_type < 3) return scale;
    for (int is = -4; is < 4; is++) {
        if (is == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)is) / max;
        float slx = 0.0f, sl2 = 0.0f;
        for (int i = 0; i < n; i++) {
            int32_t l = clamp_i32(nearest_int(iscale * x[i]), -nmax, nmax - 1);
            float w = QX_W(i);
            float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (sl2 > 0.0f && slx * slx > best * sl2) {
            for (int i = 0; i < n; i++) {
                int32_t l = nearest_int(iscale * x[i]);
                ls[i] = (int8_t)(nmax + clamp_i32(l, -nmax, nmax - 1));
            }
            scale = slx / sl2;
            best = scale * slx;
        }
    }
#undef QX_W
    return scale;
}

/* ==========================================================================================
 * Q4_0   k_quants.rs:213-312
 * ======================================================================================== */
static void q4_0_to_float(const block_q4_0 *xs, float *ys, int64_t k) {     /* :219-239 */
    int64_t nb = k / QK4_0;
    for (int64_t i = 0; i < nb; i++) {
        float d = cqo_f16_to_f32(xs[i].d);
        for (int j = 0; j < QK4_0 / 2; j++) {
            int x0 = (int)(xs[i].qs[j] & 0x0F) - 8;
            int x1 = (int)(xs[i].qs[j] >> 4) - 8;
            ys[i * QK4_0 + j] = (float)x0 * d;
            ys[i * QK4_0 + j + QK4_0 / 2] = (float)x1 * d;
        }
    }
}

static void q4_0_from_float(const float *xs, block_q4_0 *ys, int64_t k) {   /* :241-277 */
    int64_t nb = k / QK4_0;
    for (int64_t i = 0; i < nb; i++) {
        const float *x = xs + i * QK4_0;
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < QK4_0; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        float d = max / -8.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = cqo_f32_to_f16(d);
        for (int j = 0; j < QK4_0 / 2; j++) {
            float x0 = x[j] * id;
            float x1 = x[QK4_0 / 2 + j] * id;
            uint8_t xi0 = sat_u8(x0 + 8.5f); if (xi0 > 15) xi0 = 15;
            uint8_t xi1 = sat_u8(x1 + 8.5f); if (xi1 > 15) xi1 = 15;
            ys[i].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}

static float q4_0_q8_0_vec_dot(int64_t n, const block_q4_0 *xs, const block_q8_0 *ys) { /* :294-311 */
    int64_t nb = n / QK8_0;
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        int32_t sum_i = 0;
        for (int j = 0; j < QK8_0 / 2; j++) {
            int32_t v0 = (int32_t)(xs[i].qs[j] & 0x0F) - 8;
            int32_t v1 = (int32_t)(xs[i].qs[j] >> 4) - 8;
            sum_i += v0 * (int32_t)ys[i].qs[j] + v1 * (int32_t)ys[i].qs[j + QK8_0 / 2];
        }
        sumf += (float)sum_i * cqo_f16_to_f32(xs[i].d) * cqo_f16_to_f32(ys[i].d);
    }
    return sumf;
}

/* ==========================================================================================
 * Q8_0   k_quants.rs:634-739
 * ======================================================================================== */
static void q8_0_to_float(const block_q8_0 *xs, float *ys, int64_t k) {     /* :640-656 */
    int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        float d = cqo_f16_to_f32(xs[i].d);
        for (int j = 0; j < QK8_0; j++) ys[i * QK8_0 + j] = (float)xs[i].qs[j] * d;
    }
}

static void q8_0_from_float(const float *xs, block_q8_0 *ys, int64_t k) {   /* :658-687 */
    int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        const float *x = xs + i * QK8_0;
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; j++) amax = fmaxf(amax, fabsf(x[j]));
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = cqo_f32_to_f16(d);
        for (int j = 0; j < QK8_0; j++) ys[i].qs[j] = sat_i8(roundf(x[j] * id));
    }
}

static float q8_0_q8_0_vec_dot(int64_t n, const block_q8_0 *xs, const block_q8_0 *ys) { /* :720-738 */
    int64_t nb = n / QK8_0;
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        int32_t sum_i = 0;
        for (int j = 0; j < QK8_0; j++) sum_i += (int32_t)xs[i].qs[j] * (int32_t)ys[i].qs[j];
        sumf += (float)sum_i * cqo_f16_to_f32(xs[i].d) * cqo_f16_to_f32(ys[i].d);
    }
    return sumf;
}

/* ==========================================================================================
 * Q8_K   k_quants.rs:2281-2372   (activation type of every K-quant)
 * ======================================================================================== */
static void q8_K_from_float(const float *xs, block_q8_K *ys, int64_t k) {   /* :2320-2358 */
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const float *x = xs + i * QK_K;
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        if (amax == 0.0f) {
            ys[i].d = 0.0f;
            memset(ys[i].qs, 0, QK_K);
            /* The reference leaves bsums untouched here (stale); they are multiplied by d = 0
             * everywhere they are used.  The oracle writes zeros so that the bytes are defined. */
            memset(ys[i].bsums, 0, sizeof(ys[i].bsums));
        } else {
            float iscale = -127.0f / max;
            for (int j = 0; j < QK_K; j++) {
                float v = roundf(iscale * x[j]);
                if (v < -128.0f) v = -128.0f;
                if (v > 127.0f) v = 127.0f;
                ys[i].qs[j] = sat_i8(v);
            }
            for (int j = 0; j < QK_K / 16; j++) {
                int32_t sum = 0;
                for (int ii = 0; ii < 16; ii++) sum += (int32_t)ys[i].qs[j * 16 + ii];
                ys[i].bsums[j] = (int16_t)sum;
            }
            ys[i].d = 1.0f / iscale;
        }
    }
}

static void q8_K_to_float(const block_q8_K *xs, float *ys, int64_t k) {     /* :2360-2371 */
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++)
        for (int j = 0; j < QK_K; j++) ys[i * QK_K + j] = xs[i].d * (float)xs[i].qs[j];
}

static float q8_K_q8_K_vec_dot(int64_t n, const block_q8_K *xs, const block_q8_K *ys) { /* :2300-2317 */
    int64_t nb = n / QK_K;
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        int32_t sum_i = 0;
        for (int j = 0; j < QK_K; j++) sum_i += (int32_t)xs[i].qs[j] * (int32_t)ys[i].qs[j];
        sumf += (float)sum_i * xs[i].d * ys[i].d;
    }
    return sumf;
}

/* ==========================================================================================
 * Q4_K   k_quants.rs:1424-1695
 * ======================================================================================== */
static void q4_K_to_float(const block_q4_K *xs, float *ys, int64_t k) {     /* :1667-1694 */
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const block_q4_K *b = &xs[i];
        float d = cqo_f16_to_f32(b->d);
        float min = cqo_f16_to_f32(b->dmin);
        float *y = ys + i * QK_K;
        int is = 0, yi = 0;
        for (int j = 0; j < QK_K; j += 64) {
            const uint8_t *q = b->qs + j / 2;
            uint8_t sc, m;
            get_scale_min_k4(is, b->scales, &sc, &m);
            float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, b->scales, &sc, &m);
            float d2 = d * (float)sc, m2 = min * (float)m;
            for (int l = 0; l < 32; l++) y[yi++] = d1 * (float)(q[l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) y[yi++] = d2 * (float)(q[l] >> 4) - m2;
            is += 2;
        }
    }
}

/* shared by Q4_K (:1542-1600) and Q5_K (:1804-1850): sub-block scales/mins and 6-bit packing */
static void kquant_scales_mins(const float *x, int32_t nmax, uint8_t *scales_out, uint16_t *d_out, uint16_t *dmin_out) {
    float mins[QK_K / 32], scales[QK_K / 32];
    for (int j = 0; j < QK_K / 32; j++) make_qkx1_quants(nmax, 5, x + 32 * j, 32, &scales[j], &mins[j]);
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < QK_K / 32; j++) {
        max_scale = fmaxf(scales[j], max_scale);
        max_min = fmaxf(mins[j], max_min);
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    memset(scales_out, 0, K_SCALE_SIZE);
    for (int j = 0; j < QK_K / 32; j++) {
        int32_t lsi = nearest_int(inv_scale * scales[j]); if (lsi > 63) lsi = 63;
        int32_t lmi = nearest_int(inv_min * mins[j]);     if (lmi > 63) lmi = 63;
        uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
        if (j < 4) {
            scales_out[j] = ls;
            scales_out[j + 4] = lm;
        } else {
            scales_out[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            scales_out[j - 4] |= (uint8_t)((ls >> 4) << 6);
            scales_out[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    *d_out = cqo_f32_to_f16(max_scale / 63.0f);
    *dmin_out = cqo_f32_to_f16(max_min / 63.0f);
}

static void q4_K_from_float(const float *xs, block_q4_K *ys, int64_t k) {   /* :1542-1600 */
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const float *x = xs + i * QK_K;
        block_q4_K *b = &ys[i];
        kquant_scales_mins(x, 15, b->scales, &b->d, &b->dmin);
        uint8_t l[QK_K];
        memset(l, 0, sizeof(l));
        for (int j = 0; j < QK_K / 32; j++) {
            uint8_t sc, m;
            get_scale_min_k4(j, b->scales, &sc, &m);
            float d = cqo_f16_to_f32(b->d) * (float)sc;
            if (d != 0.0f) {
                float dm = cqo_f16_to_f32(b->dmin) * (float)m;
                for (int ii = 0; ii < 32; ii++) {
                    int32_t lv = nearest_int((x[32 * j + ii] + dm) / d);
                    l[32 * j + ii] = (uint8_t)clamp_i32(lv, 0, 15);
                }
            }
        }
        for (int j = 0; j < QK_K; j += 64)
            for (int lv = 0; lv < 32; lv++)
                b->qs[(j / 64) * 32 + lv] = (uint8_t)(l[j + lv] | (l[j + lv + 32] << 4));
    }
}

/* k_quants.rs:1499-1509 / :1760-1770  unpack the 12 scale bytes into 8 scales + 8 mins */
static inline void unpack_scales_mins(const uint8_t *s, uint8_t *scales, uint8_t *mins) {
    const uint32_t KMASK1 = 0x3f3f3f3fu, KMASK2 = 0x0f0f0f0fu, KMASK3 = 0x03030303u;
    uint32_t utmp[4];
    memcpy(utmp, s, 12);
    utmp[3] = ((utmp[2] >> 4) & KMASK2) | (((utmp[1] >> 6) & KMASK3) << 4);
    uint32_t uaux = utmp[1] & KMASK1;
    utmp[1] = (utmp[2] & KMASK2) | (((utmp[0] >> 6) & KMASK3) << 4);
    utmp[2] = uaux;
    utmp[0] &= KMASK1;
    memcpy(scales, &utmp[0], 8);
    memcpy(mins, &utmp[2], 8);
}

/* common tail of the Q4_K / Q5_K dot product (:1511-1539, :1772-1800) given unpacked aux8 */
static inline void kquant45_accumulate(const int8_t *aux8, const uint8_t *scales12, const block_q8_K *y,
                                       float xd, float xdmin, float *sums, float *sumf) {
    uint8_t scales[8], mins[8];
    int16_t aux16[8];
    int32_t aux32[8];
    memset(aux32, 0, sizeof(aux32));
    unpack_scales_mins(scales12, scales, mins);
    int32_t sumi = 0;
    for (int j = 0; j < QK_K / 16; j++) sumi += (int32_t)y->bsums[j] * (int32_t)mins[j / 2];
    const int8_t *a = aux8;
    const int8_t *q8 = y->qs;
    for (int is = 0; is < 8; is++) {
        int32_t scale = (int32_t)scales[is];
        for (int r = 0; r < 4; r++) {
            for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
            for (int l = 0; l < 8; l++) aux32[l] += scale * (int32_t)aux16[l];
            q8 += 8;
            a += 8;
        }
    }
    float d = xd * y->d;
    for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
    float dmin = xdmin * y->d;
    *sumf -= dmin * (float)sumi;
}

static float q4_K_q8_K_vec_dot(int64_t n, const block_q4_K *xs, const block_q8_K *ys) { /* :1460-1540 */
    int64_t nb = n / QK_K;
    int8_t aux8[QK_K];
    float sums[8] = {0};
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t *q4 = xs[i].qs;
        int8_t *a = aux8;
        for (int j = 0; j < QK_K / 64; j++) {
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] & 0xF);
            a += 32;
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] >> 4);
            a += 32;
            q4 += 32;
        }
        kquant45_accumulate(aux8, xs[i].scales, &ys[i], cqo_f16_to_f32(xs[i].d), cqo_f16_to_f32(xs[i].dmin), sums, &sumf);
    }
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += sums[l];
    return sumf + s;
}

/* ==========================================================================================
 * Q5_K   k_quants.rs:1698-1997
 * ======================================================================================== */
static void q5_K_to_float(const block_q5_K *xs, float *ys, int64_t k) {     /* :1962-1996 */
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const block_q5_K *b = &xs[i];
        float d = cqo_f16_to_f32(b->d);
        float min = cqo_f16_to_f32(b->dmin);
        float *y = ys + i * QK_K;
        int is = 0, yi = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < QK_K; j += 64) {
            const uint8_t *ql = b->qs + j / 2;
            uint8_t sc, m;
            get_scale_min_k4(is, b->scales, &sc, &m);
            float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, b->scales, &sc, &m);
            float d2 = d * (float)sc, m2 = min * (float)m;
            for (int l = 0; l < 32; l++) {
                float to_add = (b->qh[l] & u1) ? 16.0f : 0.0f;
                y[yi++] = d1 * ((float)(ql[l] & 0xF) + to_add) - m1;
            }
            for (int l = 0; l < 32; l++) {
                float to_add = (b->qh[l] & u2) ? 16.0f : 0.0f;
                y[yi++] = d2 * ((float)(ql[l] >> 4) + to_add) - m2;
            }
            is += 2;
            u1 <<= 2;
            u2 <<= 2;
        }
    }
}

static void q5_K_from_float(const float *xs, block_q5_K *ys, int64_t k) {   /* :1804-1877 */
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const float *x = xs + i * QK_K;
        block_q5_K *b = &ys[i];
        kquant_scales_mins(x, 31, b->scales, &b->d, &b->dmin);
        uint8_t l[QK_K];
        memset(l, 0, sizeof(l));
        for (int j = 0; j < QK_K / 32; j++) {
            uint8_t sc, m;
            get_scale_min_k4(j, b->scales, &sc, &m);
            float d = cqo_f16_to_f32(b->d) * (float)sc;
            if (d == 0.0f) continue;
            float dm = cqo_f16_to_f32(b->dmin) * (float)m;
            for (int ii = 0; ii < 32; ii++) {
                int32_t ll = nearest_int((x[32 * j + ii] + dm) / d);
                l[32 * j + ii] = (uint8_t)clamp_i32(ll, 0, 31);
            }
        }
        memset(b->qh, 0, sizeof(b->qh));
        uint8_t m1 = 1, m2 = 2;
        for (int n = 0; n < QK_K; n += 64) {
            int offset = (n / 64) * 32;
            for (int j = 0; j < 32; j++) {
                uint8_t l1 = l[n + j];
                if (l1 > 15) { l1 -= 16; b->qh[j] |= m1; }
                uint8_t l2 = l[n + j + 32];
                if (l2 > 15) { l2 -= 16; b->qh[j] |= m2; }
                b->qs[offset + j] = (uint8_t)(l1 | (l2 << 4));
            }
            m1 <<= 2;
            m2 <<= 2;
        }
    }
}

static float q5_K_q8_K_vec_dot(int64_t n, const block_q5_K *xs, const block_q8_K *ys) { /* :1714-1801 */
    int64_t nb = n / QK_K;
    int8_t aux8[QK_K];
    float sums[8] = {0};
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        const uint8_t *q5 = xs[i].qs;
        const uint8_t *hm = xs[i].qh;
        int8_t *a = aux8;
        uint8_t m = 1;
        for (int j = 0; j < QK_K / 64; j++) {
            for (int l = 0; l < 32; l++) {
                a[l] = (int8_t)(q5[l] & 0xF);
                a[l] += (hm[l] & m) ? 16 : 0;
            }
            a += 32;
            m <<= 1;
            for (int l = 0; l < 32; l++) {
                a[l] = (int8_t)(q5[l] >> 4);
                a[l] += (hm[l] & m) ? 16 : 0;
            }
            a += 32;
            m <<= 1;
            q5 += 32;
        }
        kquant45_accumulate(aux8, xs[i].scales, &ys[i], cqo_f16_to_f32(xs[i].d), cqo_f16_to_f32(xs[i].dmin), sums, &sumf);
    }
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += sums[l];
    return sumf + s;
}

/* ==========================================================================================
 * Q6_K   k_quants.rs:1999-2279
 * ======================================================================================== */
static void q6_K_to_float(const block_q6_K *xs, float *ys, int64_t k) {     /* :2247-2278 */
    int64_t nb = k / QK_K;
    for (int64_t i = 0; i < nb; i++) {
        const block_q6_K *x = &xs[i];
        float d = cqo_f16_to_f32(x->d);
        for (int n = 0; n < QK_K; n += 128) {
            int idx = n / 128;
            float *y = ys + i * QK_K + n;
            const int8_t *sc = x->scales + 8 * idx;
            const uint8_t *ql = x->ql + 64 * idx;
            const uint8_t *qh = x->qh + 32 * idx;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int)(int8_t)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32;
                int q2 = (int)(int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int q3 = (int)(int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int q4 = (int)(int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l] = d * (float)sc[is] * (float)q1;
                y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                y[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
        }
    }
}

static void q6_K_from_float(const float *xs, block_q6_K *ys, int64_t k) {   /* :2094-2164 */
    int64_t nb = k / QK_K;
    int8_t l[QK_K];
    float scales[QK_K / 16];
    memset(l, 0, sizeof(l));
    for (int64_t i = 0; i < nb; i++) {
        const float *x = xs + i * QK_K;
        block_q6_K *y = &ys[i];
        float max_scale = 0.0f, max_abs_scale = 0.0f;
        for (int ib = 0; ib < QK_K / 16; ib++) {
            float scale = make_qx_quants(16, 32, x + 16 * ib, l + 16 * ib, 1, NULL);
            scales[ib] = scale;
            float abs_scale = fabsf(scale);
            if (abs_scale > max_abs_scale) { max_abs_scale = abs_scale; max_scale = scale; }
        }
        /* No zero guard in the reference: an all-zero super-block gives iscale = -inf and
         * d = f16(1/-inf) = -0.0; nearest_int(-inf * 0) = nearest_int(NaN) = 0. */
        float iscale = -128.0f / max_scale;
        y->d = cqo_f32_to_f16(1.0f / iscale);
        for (int j = 0; j < QK_K / 16; j++) {
            int32_t s = nearest_int(iscale * scales[j]);
            if (s > 127) s = 127;
            y->scales[j] = (int8_t)s;
        }
        for (int j = 0; j < QK_K / 16; j++) {
            float d = cqo_f16_to_f32(y->d) * (float)y->scales[j];
            if (d == 0.0f) continue;
            for (int ii = 0; ii < 16; ii++) {
                int32_t ll = clamp_i32(nearest_int(x[16 * j + ii] / d), -32, 31);
                l[16 * j + ii] = (int8_t)(ll + 32);
            }
        }
        uint8_t *ql = y->ql;
        uint8_t *qh = y->qh;
        for (int j = 0; j < QK_K; j += 128) {
            for (int li = 0; li < 32; li++) {
                int8_t q1 = l[j + li] & 0xF;
                int8_t q2 = l[j + li + 32] & 0xF;
                int8_t q3 = l[j + li + 64] & 0xF;
                int8_t q4 = l[j + li + 96] & 0xF;
                ql[li] = (uint8_t)(q1 | (q3 << 4));
                ql[li + 32] = (uint8_t)(q2 | (q4 << 4));
                qh[li] = (uint8_t)((l[j + li] >> 4) | ((l[j + li + 32] >> 4) << 2) |
                                   ((l[j + li + 64] >> 4) << 4) | ((l[j + li + 96] >> 4) << 6));
            }
            ql += 64;
            qh += 32;
        }
    }
}

static float q6_K_q8_K_vec_dot(int64_t n, const block_q6_K *xs, const block_q8_K *ys) { /* :2035-2092 */
    int64_t nb = n / QK_K;
    int8_t aux8[QK_K];
    int16_t aux16[8];
    float sums[8] = {0};
    float aux32[8];
    for (int64_t i = 0; i < nb; i++) {
        const block_q6_K *x = &xs[i];
        const block_q8_K *y = &ys[i];
        for (int l = 0; l < 8; l++) aux32[l] = 0.0f;
        for (int j = 0; j < QK_K; j += 128) {
            int8_t *a = aux8 + j;
            const uint8_t *q4 = x->ql + j / 2;
            const uint8_t *qh = x->qh + j / 4;
            for (int l = 0; l < 32; l++) {
                a[l] = (int8_t)((int32_t)((q4[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
                a[l + 32] = (int8_t)((int32_t)((q4[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
                a[l + 64] = (int8_t)((int32_t)((q4[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
                a[l + 96] = (int8_t)((int32_t)((q4[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            }
        }
        for (int j = 0; j < QK_K / 16; j++) {
            float scale = (float)x->scales[j];
            const int8_t *q8 = y->qs + 16 * j;
            const int8_t *a = aux8 + 16 * j;
            for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
            for (int l = 0; l < 8; l++) aux32[l] += scale * (float)aux16[l];
            q8 += 8;
            a += 8;
            for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
            for (int l = 0; l < 8; l++) aux32[l] += scale * (float)aux16[l];
        }
        float d = cqo_f16_to_f32(x->d) * y->d;
        for (int l = 0; l < 8; l++) sums[l] += aux32[l] * d;
    }
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += sums[l];
    return s;
}

/* ==========================================================================================
 * The remaining GgmlDType block formats: to_float / from_float only.
 * ======================================================================================== */
static inline uint32_t rd_u32le(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
static inline void wr_u32le(uint8_t *p, uint32_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); p[2] = (uint8_t)(v >> 16); p[3] = (uint8_t)(v >> 24); }
static inline float f32_min_rust(float a, float b) { return (a != a) ? b : ((b != b) ? a : (a < b ? a : b)); }   /* f32::min ignores NaN */
static inline float f32_max_rust(float a, float b) { return (a != a) ? b : ((b != b) ? a : (a > b ? a : b)); }

static void q4_1_from_float(const float *xs, block_q4_1 *ys, int64_t k) {   /* k_quants.rs:353-389 */
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float min = INFINITY, max = -INFINITY;
        for (int j = 0; j < 32; j++) { min = f32_min_rust(x[j], min); max = f32_max_rust(x[j], max); }
        float d = (max - min) / 15.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = cqo_f32_to_f16(d);
        ys[i].m = cqo_f32_to_f16(min);
        for (int j = 0; j < 16; j++) {
            float x0 = (x[j] - min) * id, x1 = (x[16 + j] - min) * id;
            uint8_t xi0 = sat_u8(x0 + 0.5f), xi1 = sat_u8(x1 + 0.5f);
            if (xi0 > 15) xi0 = 15;
            if (xi1 > 15) xi1 = 15;
            ys[i].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}
static void q4_1_to_float(const block_q4_1 *xs, float *ys, int64_t k) {     /* :392-412 */
    for (int64_t i = 0; i < k / 32; i++) {
        float d = cqo_f16_to_f32(xs[i].d), m = cqo_f16_to_f32(xs[i].m);
        for (int j = 0; j < 16; j++) {
            ys[i * 32 + j] = (float)(xs[i].qs[j] & 0x0F) * d + m;
            ys[i * 32 + j + 16] = (float)(xs[i].qs[j] >> 4) * d + m;
        }
    }
}

static void q5_0_from_float(const float *xs, block_q5_0 *ys, int64_t k) {   /* :457-493 */
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < 32; j++) if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        float d = max / -16.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = cqo_f32_to_f16(d);
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            float x0 = x[j] * id, x1 = x[j + 16] * id;
            int8_t a = sat_i8(x0 + 16.5f), b = sat_i8(x1 + 16.5f);
            uint8_t xi0 = (uint8_t)(a < 31 ? a : 31), xi1 = (uint8_t)(b < 31 ? b : 31);
            ys[i].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (((uint32_t)xi0 & 0x10) >> 4) << j;
            qh |= (((uint32_t)xi1 & 0x10) >> 4) << (j + 16);
        }
        wr_u32le(ys[i].qh, qh);
    }
}
static void q5_0_to_float(const block_q5_0 *xs, float *ys, int64_t k) {     /* :496-518 */
    for (int64_t i = 0; i < k / 32; i++) {
        float d = cqo_f16_to_f32(xs[i].d);
        uint32_t qh = rd_u32le(xs[i].qh);
        for (int j = 0; j < 16; j++) {
            uint8_t xh_0 = (uint8_t)(((qh >> j) << 4) & 0x10), xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
            int32_t x0 = (int32_t)((xs[i].qs[j] & 0x0F) | xh_0) - 16, x1 = (int32_t)((xs[i].qs[j] >> 4) | xh_1) - 16;
            ys[i * 32 + j] = (float)x0 * d;
            ys[i * 32 + j + 16] = (float)x1 * d;
        }
    }
}

static void q5_1_from_float(const float *xs, block_q5_1 *ys, int64_t k) {   /* :564-604 */
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float min = INFINITY, max = -INFINITY;
        for (int j = 0; j < 32; j++) { min = f32_min_rust(x[j], min); max = f32_max_rust(x[j], max); }
        float d = (max - min) / 31.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = cqo_f32_to_f16(d);
        ys[i].m = cqo_f32_to_f16(min);
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            float x0 = (x[j] - min) * id, x1 = (x[16 + j] - min) * id;
            uint8_t xi0 = sat_u8(x0 + 0.5f), xi1 = sat_u8(x1 + 0.5f);
            ys[i].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (((uint32_t)xi0 & 0x10) >> 4) << j;
            qh |= (((uint32_t)xi1 & 0x10) >> 4) << (j + 16);
        }
        wr_u32le(ys[i].qh, qh);
    }
}
static void q5_1_to_float(const block_q5_1 *xs, float *ys, int64_t k) {     /* :607-631 */
    for (int64_t i = 0; i < k / 32; i++) {
        float d = cqo_f16_to_f32(xs[i].d), m = cqo_f16_to_f32(xs[i].m);
        uint32_t qh = rd_u32le(xs[i].qh);
        for (int j = 0; j < 16; j++) {
            uint8_t xh_0 = (uint8_t)(((qh >> j) << 4) & 0x10), xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
            uint8_t x0 = (uint8_t)((xs[i].qs[j] & 0x0F) | xh_0), x1 = (uint8_t)((xs[i].qs[j] >> 4) | xh_1);
            ys[i * 32 + j] = (float)x0 * d + m;
            ys[i * 32 + j + 16] = (float)x1 * d + m;
        }
    }
}

static void q8_1_from_float(const float *xs, block_q8_1 *ys, int64_t k) {   /* :770-799 */
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) amax = f32_max_rust(amax, fabsf(x[j]));
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = cqo_f32_to_f16(d);
        int32_t sum = 0;
        for (int j = 0; j < 16; j++) {
            ys[i].qs[j] = sat_i8(roundf(x[j] * id));
            ys[i].qs[j + 16] = sat_i8(roundf(x[j + 16] * id));
            sum += (int32_t)ys[i].qs[j] + (int32_t)ys[i].qs[j + 16];
        }
        /* f16::from_f32(sum as f32) * ys.d: the product of two f16 values, computed in f32 and rounded back to f16 */
        ys[i].s = cqo_f32_to_f16(cqo_f16_to_f32(cqo_f32_to_f16((float)sum)) * cqo_f16_to_f32(ys[i].d));
    }
}
static void q8_1_to_float(const block_q8_1 *xs, float *ys, int64_t k) {     /* :801-816 */
    for (int64_t i = 0; i < k / 32; i++) {
        float d = cqo_f16_to_f32(xs[i].d);
        for (int j = 0; j < 32; j++) ys[i * 32 + j] = (float)xs[i].qs[j] * d;
    }
}

static void q2_K_from_float(const float *xs, block_q2_K *ys, int64_t k) {   /* :891-953 */
    const float Q4SCALE = 15.0f;
    for (int64_t b = 0; b < k / QK_K; b++) {
        const float *x = xs + b * QK_K;
        block_q2_K *blk = ys + b;
        float mins[16], scales[16];
        for (int j = 0; j < 16; j++) make_qkx1_quants(3, 5, x + 16 * j, 16, &scales[j], &mins[j]);
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 16; j++) { max_scale = f32_max_rust(scales[j], max_scale); max_min = f32_max_rust(mins[j], max_min); }
        if (max_scale > 0.0f) {
            float iscale = Q4SCALE / max_scale;
            for (int j = 0; j < 16; j++) blk->scales[j] = (uint8_t)nearest_int(iscale * scales[j]);
            blk->d = cqo_f32_to_f16(max_scale / Q4SCALE);
        } else {
            for (int j = 0; j < 16; j++) blk->scales[j] = 0;
            blk->d = cqo_f32_to_f16(0.0f);
        }
        if (max_min > 0.0f) {
            float iscale = Q4SCALE / max_min;
            for (int j = 0; j < 16; j++) blk->scales[j] |= (uint8_t)((uint8_t)nearest_int(iscale * mins[j]) << 4);
            blk->dmin = cqo_f32_to_f16(max_min / Q4SCALE);
        } else {
            blk->dmin = cqo_f32_to_f16(0.0f);
        }
        uint8_t big_l[QK_K];
        memset(big_l, 0, sizeof(big_l));
        for (int j = 0; j < 16; j++) {
            float d = cqo_f16_to_f32(blk->d) * (float)(blk->scales[j] & 0xF);
            if (d == 0.0f) continue;
            float dm = cqo_f16_to_f32(blk->dmin) * (float)(blk->scales[j] >> 4);
            for (int ii = 0; ii < 16; ii++) big_l[16 * j + ii] = (uint8_t)clamp_i32(nearest_int((x[16 * j + ii] + dm) / d), 0, 3);
        }
        for (int j = 0; j < QK_K; j += 128)
            for (int l = 0; l < 32; l++)
                blk->qs[j / 4 + l] = (uint8_t)(big_l[j + l] | (big_l[j + l + 32] << 2) | (big_l[j + l + 64] << 4) | (big_l[j + l + 96] << 6));
    }
}
static void q2_K_to_float(const block_q2_K *xs, float *ys, int64_t k) {     /* :1013-1049 */
    for (int64_t b = 0; b < k / QK_K; b++) {
        const block_q2_K *blk = xs + b;
        float *y = ys + b * QK_K;
        float d = cqo_f16_to_f32(blk->d), min = cqo_f16_to_f32(blk->dmin);
        int is = 0;
        for (int h = 0; h < 2; h++) {
            const uint8_t *qs = blk->qs + 32 * h;
            int yi = 128 * h;
            for (int shift = 0; shift < 8; shift += 2) {
                for (int half = 0; half < 2; half++) {
                    uint8_t sc = blk->scales[is++];
                    float dl = d * (float)(sc & 0xF), ml = min * (float)(sc >> 4);
                    for (int l = 0; l < 16; l++) y[yi++] = dl * (float)((qs[16 * half + l] >> shift) & 3) - ml;
                }
            }
        }
    }
}

/* utils.rs:287-352 make_q3_quants(x, nmax, do_rmse = true) -> scale (the levels are not used by the caller) */
static float make_q3_quants(const float *x, int n, int32_t nmax) {
    int8_t l[64];
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) { float ax = fabsf(x[i]); if (ax > amax) { amax = ax; max = x[i]; } }
    if (amax == 0.0f) return 0.0f;
    float iscale = -(float)nmax / max;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int32_t li = clamp_i32(sat_i32(roundf(iscale * x[i])), -nmax, nmax - 1);
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
                float sl2 = suml2 - w * (float)((int32_t)l[i] * (int32_t)l[i]);
                int32_t new_l = clamp_i32(sat_i32(roundf(x[i] * sl2 / slx)), -nmax, nmax - 1);
                if (new_l != (int32_t)l[i]) {
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

static void q3_K_from_float(const float *xs, block_q3_K *ys, int64_t k) {   /* :1190-1269 */
    for (int64_t b = 0; b < k / QK_K; b++) {
        const float *x = xs + b * QK_K;
        block_q3_K *blk = ys + b;
        float scales[16];
        for (int j = 0; j < 16; j++) scales[j] = make_q3_quants(x + 16 * j, 16, 4);
        float max_scale = 0.0f;
        for (int j = 0; j < 16; j++) if (fabsf(scales[j]) > fabsf(max_scale)) max_scale = scales[j];
        memset(blk->scales, 0, sizeof(blk->scales));
        if (max_scale != 0.0f) {
            float iscale = -32.0f / max_scale;
            for (int j = 0; j < 16; j++) {
                int32_t l_val = clamp_i32(nearest_int(iscale * scales[j]), -32, 31) + 32;
                if (j < 8) blk->scales[j] = (uint8_t)(l_val & 0xF);
                else blk->scales[j - 8] |= (uint8_t)((l_val & 0xF) << 4);
                l_val >>= 4;
                blk->scales[j % 4 + 8] |= (uint8_t)(l_val << (2 * (j / 4)));
            }
            blk->d = cqo_f32_to_f16(1.0f / iscale);
        } else {
            blk->d = cqo_f32_to_f16(0.0f);
        }
        int8_t l[QK_K];
        memset(l, 0, sizeof(l));
        for (int j = 0; j < 16; j++) {
            uint8_t sc = j < 8 ? (blk->scales[j] & 0xF) : (blk->scales[j - 8] >> 4);
            int8_t scs = (int8_t)((int8_t)(sc | (((blk->scales[8 + j % 4] >> (2 * (j / 4))) & 3) << 4)) - 32);
            float d = cqo_f16_to_f32(blk->d) * (float)scs;
            if (d != 0.0f)
                for (int ii = 0; ii < 16; ii++) l[16 * j + ii] = (int8_t)(clamp_i32(nearest_int(x[16 * j + ii] / d), -4, 3) + 4);
        }
        memset(blk->hmask, 0, sizeof(blk->hmask));
        int m = 0;
        uint8_t hm = 1;
        for (int i = 0; i < QK_K; i++) {
            if (l[i] > 3) { blk->hmask[m] |= hm; l[i] -= 4; }
            if (++m == QK_K / 8) { m = 0; hm <<= 1; }
        }
        for (int j = 0; j < QK_K; j += 128)
            for (int v = 0; v < 32; v++)
                blk->qs[j / 4 + v] = (uint8_t)(l[j + v] | (l[j + v + 32] << 2) | (l[j + v + 64] << 4) | (l[j + v + 96] << 6));
    }
}
static void q3_K_to_float(const block_q3_K *xs, float *ys, int64_t k) {     /* :1369-1421 */
    const uint32_t KMASK1 = 0x03030303u, KMASK2 = 0x0f0f0f0fu;
    for (int64_t b = 0; b < k / QK_K; b++) {
        const block_q3_K *blk = xs + b;
        float *y = ys + b * QK_K;
        uint32_t aux[4];
        aux[0] = rd_u32le(blk->scales); aux[1] = rd_u32le(blk->scales + 4); aux[2] = rd_u32le(blk->scales + 8);
        uint32_t tmp = aux[2];
        aux[2] = ((aux[0] >> 4) & KMASK2) | (((tmp >> 4) & KMASK1) << 4);
        aux[3] = ((aux[1] >> 4) & KMASK2) | (((tmp >> 6) & KMASK1) << 4);
        aux[0] = (aux[0] & KMASK2) | ((tmp & KMASK1) << 4);
        aux[1] = (aux[1] & KMASK2) | (((tmp >> 2) & KMASK1) << 4);
        int8_t scales[16];
        for (int i = 0; i < 16; i++) scales[i] = (int8_t)((aux[i / 4] >> (8 * (i % 4))) & 0xff);
        float d_all = cqo_f16_to_f32(blk->d);
        uint8_t m = 1;
        int is = 0;
        for (int h = 0; h < 2; h++) {
            const uint8_t *qs = blk->qs + 32 * h;
            for (int shift = 0; shift < 8; shift += 2) {
                for (int si = 0; si < 2; si++) {
                    float dl = d_all * ((float)scales[is++] - 32.0f);
                    for (int i = 0; i < 16; i++) {
                        int8_t q = (int8_t)((qs[i + 16 * si] >> shift) & 3);
                        int8_t v = (int8_t)(q - ((blk->hmask[i + 16 * si] & m) == 0 ? 4 : 0));
                        y[128 * h + 16 * (shift) + 16 * si + i] = dl * (float)v;       /* shift / 2 * 32 + 16 si + i */
                    }
                }
                m <<= 1;
            }
        }
    }
}

/* ==========================================================================================
 * vec_dot of the remaining formats against their VecDotType (Q8_1, Q8_0, Q8_1, Q8_K, Q8_K)
 * ======================================================================================== */
static float q4_1_q8_1_vec_dot(int64_t n, const block_q4_1 *xs, const block_q8_1 *ys) { /* k_quants.rs:323-351 */
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / 32; i++) {
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            int32_t v0 = xs[i].qs[j] & 0x0F, v1 = xs[i].qs[j] >> 4;
            sumi += v0 * (int32_t)ys[i].qs[j] + v1 * (int32_t)ys[i].qs[j + 16];
        }
        float t = (float)sumi * cqo_f16_to_f32(xs[i].d) * cqo_f16_to_f32(ys[i].d);
        float u = cqo_f16_to_f32(xs[i].m) * cqo_f16_to_f32(ys[i].s);
        sumf += t + u;
    }
    return sumf;
}

static float q5_0_q8_0_vec_dot(int64_t n, const block_q5_0 *xs, const block_q8_0 *ys) { /* :434-455 */
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / 32; i++) {
        uint32_t qh = rd_u32le(xs[i].qh);
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            int32_t xh_0 = (int32_t)(uint8_t)(((qh & (1u << j)) >> j) << 4);
            int32_t xh_1 = (int32_t)(uint8_t)((qh & (1u << (j + 16))) >> (j + 12));
            int32_t x0 = ((xs[i].qs[j] & 0x0F) | xh_0) - 16;
            int32_t x1 = ((xs[i].qs[j] >> 4) | xh_1) - 16;
            sumi += x0 * (int32_t)ys[i].qs[j] + x1 * (int32_t)ys[i].qs[j + 16];
        }
        sumf += (float)sumi * cqo_f16_to_f32(xs[i].d) * cqo_f16_to_f32(ys[i].d);
    }
    return sumf;
}

static float q5_1_q8_1_vec_dot(int64_t n, const block_q5_1 *xs, const block_q8_1 *ys) { /* :530-562 */
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / 32; i++) {
        uint32_t qh = rd_u32le(xs[i].qh);
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            int32_t xh_0 = (int32_t)(((qh >> j) << 4) & 0x10);
            int32_t xh_1 = (int32_t)((qh >> (j + 12)) & 0x10);
            int32_t x0 = (xs[i].qs[j] & 0xF) | xh_0;
            int32_t x1 = (xs[i].qs[j] >> 4) | xh_1;
            sumi += x0 * (int32_t)ys[i].qs[j] + x1 * (int32_t)ys[i].qs[j + 16];
        }
        float t = (float)sumi * cqo_f16_to_f32(xs[i].d) * cqo_f16_to_f32(ys[i].d);
        float u = cqo_f16_to_f32(xs[i].m) * cqo_f16_to_f32(ys[i].s);
        sumf += t + u;
    }
    return sumf;
}

static float q2_K_q8_K_vec_dot(int64_t n, const block_q2_K *xs, const block_q8_K *ys) { /* :838-886 */
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / QK_K; i++) {
        const block_q2_K *x = xs + i;
        const block_q8_K *y = ys + i;
        const uint8_t *q2 = x->qs;
        const int8_t *q8 = y->qs;
        int32_t summs = 0;
        for (int j = 0; j < 16; j++) summs += (int32_t)y->bsums[j] * (int32_t)(x->scales[j] >> 4);
        float dall = y->d * cqo_f16_to_f32(x->d);
        float dmin = y->d * cqo_f16_to_f32(x->dmin);
        int32_t isum = 0;
        int is = 0;
        for (int h = 0; h < QK_K / 128; h++) {
            for (int shift = 0; shift < 8; shift += 2) {
                for (int half = 0; half < 2; half++) {
                    int32_t d = x->scales[is++] & 0xF;
                    int32_t isuml = 0;
                    for (int l = 16 * half; l < 16 * half + 16; l++) isuml += (int32_t)q8[l] * (int32_t)((q2[l] >> shift) & 3);
                    isum += d * isuml;
                }
                q8 += 32;
            }
            q2 += 32;
        }
        sumf += dall * (float)isum - dmin * (float)summs;
    }
    return sumf;
}

static float q3_K_q8_K_vec_dot(int64_t n, const block_q3_K *xs, const block_q8_K *ys) { /* :1068-1187 */
    const uint32_t KMASK1 = 0x03030303u, KMASK2 = 0x0f0f0f0fu;
    int8_t aux8[QK_K];
    int16_t aux16[8];
    float sums[8] = {0};
    int32_t aux32[8];
    for (int64_t i = 0; i < n / QK_K; i++) {
        const block_q3_K *x = xs + i;
        const block_q8_K *y = ys + i;
        const uint8_t *q3 = x->qs;
        const int8_t *q8 = y->qs;
        memset(aux32, 0, sizeof(aux32));
        int8_t *a = aux8;
        uint8_t m = 1;
        for (int h = 0; h < QK_K / 128; h++) {
            for (int shift = 0; shift < 8; shift += 2) {
                for (int l = 0; l < 32; l++) {
                    int8_t v = (int8_t)((q3[l] >> shift) & 3);
                    a[l] = (int8_t)(v - ((x->hmask[l] & m) != 0 ? 0 : 4));
                }
                a += 32;
                m <<= 1;
            }
            q3 += 32;
        }
        a = aux8;
        uint32_t auxs[4];
        auxs[0] = rd_u32le(x->scales); auxs[1] = rd_u32le(x->scales + 4); auxs[2] = rd_u32le(x->scales + 8);
        uint32_t tmp = auxs[2];
        auxs[2] = ((auxs[0] >> 4) & KMASK2) | (((tmp >> 4) & KMASK1) << 4);
        auxs[3] = ((auxs[1] >> 4) & KMASK2) | (((tmp >> 6) & KMASK1) << 4);
        auxs[0] = (auxs[0] & KMASK2) | ((tmp & KMASK1) << 4);
        auxs[1] = (auxs[1] & KMASK2) | (((tmp >> 2) & KMASK1) << 4);
        for (int j = 0; j < 16; j++) {
            int32_t scale = (int32_t)(int8_t)((auxs[j / 4] >> (8 * (j % 4))) & 0xff) - 32;
            for (int r = 0; r < 2; r++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * (int32_t)aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        float d = cqo_f16_to_f32(x->d) * y->d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
    }
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += sums[l];
    return s;
}

/* ==========================================================================================
 * dtype dispatch (mod.rs:386-421 type_size/block_size) and the exported entry points
 * ======================================================================================== */
int64_t cqo_block_size(int dtype) {
    switch (dtype) {
        case CQ_Q4_0: case CQ_Q8_0: case CQ_Q4_1: case CQ_Q5_0: case CQ_Q5_1: case CQ_Q8_1: return 32;
        case CQ_Q4K: case CQ_Q5K: case CQ_Q6K: case CQ_Q8K: case CQ_Q2K: case CQ_Q3K: return QK_K;
        default: return 0;
    }
}

int64_t cqo_type_size(int dtype) {
    switch (dtype) {
        case CQ_Q4_0: return sizeof(block_q4_0);
        case CQ_Q8_0: return sizeof(block_q8_0);
        case CQ_Q4K: return sizeof(block_q4_K);
        case CQ_Q5K: return sizeof(block_q5_K);
        case CQ_Q6K: return sizeof(block_q6_K);
        case CQ_Q8K: return sizeof(block_q8_K);
        case CQ_Q4_1: return sizeof(block_q4_1);
        case CQ_Q5_0: return sizeof(block_q5_0);
        case CQ_Q5_1: return sizeof(block_q5_1);
        case CQ_Q8_1: return sizeof(block_q8_1);
        case CQ_Q2K: return sizeof(block_q2_K);
        case CQ_Q3K: return sizeof(block_q3_K);
        default: return 0;
    }
}

/* the activation ("VecDotType") block type for a weight type: k_quants.rs:216,637,1427,1701,2002,2284 */
int cqo_vec_dot_type(int dtype) {
    switch (dtype) {
        case CQ_Q4_0: case CQ_Q8_0: case CQ_Q5_0: return CQ_Q8_0;
        case CQ_Q4_1: case CQ_Q5_1: return CQ_Q8_1;                               /* :317,524 */
        case CQ_Q2K: case CQ_Q3K: case CQ_Q4K: case CQ_Q5K: case CQ_Q6K: case CQ_Q8K: return CQ_Q8K;   /* :822,1055 */
        default: return -1;
    }
}

/* GgmlType::to_float: blocks -> k floats.  Returns 0, or -1 for an unsupported dtype / bad k. */
int cqo_to_float(int dtype, const void *blocks, float *ys, int64_t k) {
    int64_t bs = cqo_block_size(dtype);
    if (bs == 0 || k % bs != 0) return -1;
    switch (dtype) {
        case CQ_Q4_0: q4_0_to_float((const block_q4_0 *)blocks, ys, k); return 0;
        case CQ_Q8_0: q8_0_to_float((const block_q8_0 *)blocks, ys, k); return 0;
        case CQ_Q4K: q4_K_to_float((const block_q4_K *)blocks, ys, k); return 0;
        case CQ_Q5K: q5_K_to_float((const block_q5_K *)blocks, ys, k); return 0;
        case CQ_Q6K: q6_K_to_float((const block_q6_K *)blocks, ys, k); return 0;
        case CQ_Q8K: q8_K_to_float((const block_q8_K *)blocks, ys, k); return 0;
        case CQ_Q4_1: q4_1_to_float((const block_q4_1 *)blocks, ys, k); return 0;
        case CQ_Q5_0: q5_0_to_float((const block_q5_0 *)blocks, ys, k); return 0;
        case CQ_Q5_1: q5_1_to_float((const block_q5_1 *)blocks, ys, k); return 0;
        case CQ_Q8_1: q8_1_to_float((const block_q8_1 *)blocks, ys, k); return 0;
        case CQ_Q2K: q2_K_to_float((const block_q2_K *)blocks, ys, k); return 0;
        case CQ_Q3K: q3_K_to_float((const block_q3_K *)blocks, ys, k); return 0;
    }
    return -1;
}

/* GgmlType::from_float: k floats -> blocks. */
int cqo_from_float(int dtype, const float *xs, void *blocks, int64_t k) {
    int64_t bs = cqo_block_size(dtype);
    if (bs == 0 || k % bs != 0) return -1;
    switch (dtype) {
        case CQ_Q4_0: q4_0_from_float(xs, (block_q4_0 *)blocks, k); return 0;
        case CQ_Q8_0: q8_0_from_float(xs, (block_q8_0 *)blocks, k); return 0;
        case CQ_Q4K: q4_K_from_float(xs, (block_q4_K *)blocks, k); return 0;
        case CQ_Q5K: q5_K_from_float(xs, (block_q5_K *)blocks, k); return 0;
        case CQ_Q6K: q6_K_from_float(xs, (block_q6_K *)blocks, k); return 0;
        case CQ_Q8K: q8_K_from_float(xs, (block_q8_K *)blocks, k); return 0;
        case CQ_Q4_1: q4_1_from_float(xs, (block_q4_1 *)blocks, k); return 0;
        case CQ_Q5_0: q5_0_from_float(xs, (block_q5_0 *)blocks, k); return 0;
        case CQ_Q5_1: q5_1_from_float(xs, (block_q5_1 *)blocks, k); return 0;
        case CQ_Q8_1: q8_1_from_float(xs, (block_q8_1 *)blocks, k); return 0;
        case CQ_Q2K: q2_K_from_float(xs, (block_q2_K *)blocks, k); return 0;
        case CQ_Q3K: q3_K_from_float(xs, (block_q3_K *)blocks, k); return 0;
    }
    return -1;
}

/* GgmlType::vec_dot_unopt(n, xs, ys): xs in `dtype`, ys in its VecDotType. */
int cqo_vec_dot(int dtype, int64_t n, const void *xs, const void *ys, float *out) {
    int64_t bs = cqo_block_size(dtype);
    if (bs == 0 || n % bs != 0) return -1;
    switch (dtype) {
        case CQ_Q4_0: *out = q4_0_q8_0_vec_dot(n, (const block_q4_0 *)xs, (const block_q8_0 *)ys); return 0;
        case CQ_Q8_0: *out = q8_0_q8_0_vec_dot(n, (const block_q8_0 *)xs, (const block_q8_0 *)ys); return 0;
        case CQ_Q4K: *out = q4_K_q8_K_vec_dot(n, (const block_q4_K *)xs, (const block_q8_K *)ys); return 0;
        case CQ_Q5K: *out = q5_K_q8_K_vec_dot(n, (const block_q5_K *)xs, (const block_q8_K *)ys); return 0;
        case CQ_Q6K: *out = q6_K_q8_K_vec_dot(n, (const block_q6_K *)xs, (const block_q8_K *)ys); return 0;
        case CQ_Q8K: *out = q8_K_q8_K_vec_dot(n, (const block_q8_K *)xs, (const block_q8_K *)ys); return 0;
        case CQ_Q4_1: *out = q4_1_q8_1_vec_dot(n, (const block_q4_1 *)xs, (const block_q8_1 *)ys); return 0;
        case CQ_Q5_0: *out = q5_0_q8_0_vec_dot(n, (const block_q5_0 *)xs, (const block_q8_0 *)ys); return 0;
        case CQ_Q5_1: *out = q5_1_q8_1_vec_dot(n, (const block_q5_1 *)xs, (const block_q8_1 *)ys); return 0;
        case CQ_Q2K: *out = q2_K_q8_K_vec_dot(n, (const block_q2_K *)xs, (const block_q8_K *)ys); return 0;
        case CQ_Q3K: *out = q3_K_q8_K_vec_dot(n, (const block_q3_K *)xs, (const block_q8_K *)ys); return 0;
    }
    return -1;
}

/*
 * k_quants.rs:2375-2492  matmul((m,k,n), lhs f32 [m,k], rhs_t blocks [n, k/blk]) -> dst f32 [m,n].
 * Each lhs row is quantized to the weight type's VecDotType, then every (row, column) is one
 * vec_dot.  The reference's split of columns over worker threads does not change any value.
 */
int cqo_matmul(int dtype, int64_t m, int64_t k, int64_t n, const float *lhs, const void *rhs_t, float *dst) {
    int64_t bs = cqo_block_size(dtype);
    int vdt = cqo_vec_dot_type(dtype);
    if (bs == 0 || vdt < 0 || k % bs != 0) return -1;
    int64_t k_in_blocks = k / bs;
    int64_t w_row_bytes = k_in_blocks * cqo_type_size(dtype);
    int64_t a_row_bytes = k_in_blocks * cqo_type_size(vdt);
    uint8_t *lhs_b = (uint8_t *)malloc((size_t)(m * a_row_bytes) + 8);
    if (!lhs_b) return -2;
    for (int64_t r = 0; r < m; r++) cqo_from_float(vdt, lhs + r * k, lhs_b + r * a_row_bytes, k);
    for (int64_t r = 0; r < m; r++)
        for (int64_t c = 0; c < n; c++)
            cqo_vec_dot(dtype, k, (const uint8_t *)rhs_t + c * w_row_bytes, lhs_b + r * a_row_bytes, &dst[r * n + c]);
    free(lhs_b);
    return 0;
}

/*
 * QTensor::indexed_moe_forward (mod.rs:758-784; GPU-only in the reference, semantics from
 * candle-core/src/quantized/cuda.rs:505-584 and candle-kernels/src/quantized.cu:4670-4760):
 *   w [E, n, k] blocks, x [batch, input_dim1 (= topk or 1), k] f32, ids [batch, topk] u32
 *   out[b, t, :] = W[ids[b,t]] . x[b, (input_dim1 == 1 ? 0 : t), :]
 * The expert stride is n*k elements of `dtype` (the reference kernel's "/QK_K" stride is a bug for
 * 32-element block types and is not reproduced).  Restated as one CPU matmul per (b, t) pair.
 */
int cqo_indexed_moe_forward(int dtype, const void *w, const float *x, const uint32_t *ids, float *out,
                            int64_t num_experts, int64_t n, int64_t k, int64_t batch, int64_t topk, int64_t input_dim1) {
    int64_t bs = cqo_block_size(dtype);
    if (bs == 0 || k % bs != 0) return -1;
    if (input_dim1 != 1 && input_dim1 != topk) return -1;
    int64_t expert_bytes = n * (k / bs) * cqo_type_size(dtype);
    for (int64_t b = 0; b < batch; b++)
        for (int64_t t = 0; t < topk; t++) {
            int64_t task = b * topk + t;
            uint32_t e = ids[task];
            if ((int64_t)e >= num_experts) return -3;
            int64_t in_row = input_dim1 == 1 ? b : task;
            int rc = cqo_matmul(dtype, 1, k, n, x + in_row * k, (const uint8_t *)w + (int64_t)e * expert_bytes, out + task * n);
            if (rc) return rc;
        }
    return 0;
}

/*
 * candle_nn::moe::moe_gemm_gguf decode semantics (candle-nn/src/moe.rs:169-337,
 * candle-kernels/src/moe/moe_gguf.cu:55-132):
 *   for m in 0..size_m: tok = sorted_token_ids[m]; e = expert_ids[m]
 *     in_row = topk_weights ? tok : tok / topk;  scale = topk_weights ? topk_weights[tok] : 1
 *     out[tok, :] = scale * (W[e] . x[in_row, :])        (pairs with e outside [0,E) are skipped)
 * with the activation row quantized as the CPU path does (the GPU reference uses q8_1 instead).
 */
int cqo_moe_gemm_gguf(int dtype, const float *x, const void *w, const int32_t *sorted_token_ids,
                      const int32_t *expert_ids, const float *topk_weights, float *out,
                      int64_t num_experts, int64_t topk, int64_t size_m, int64_t n, int64_t k) {
    int64_t bs = cqo_block_size(dtype);
    if (bs == 0 || k % bs != 0) return -1;
    int64_t expert_bytes = n * (k / bs) * cqo_type_size(dtype);
    for (int64_t m = 0; m < size_m; m++) {
        int32_t tok = sorted_token_ids[m];
        int32_t e = expert_ids[m];
        if (e < 0 || e >= num_experts) continue;
        int64_t in_row = topk_weights ? tok : tok / topk;
        float scale = topk_weights ? topk_weights[tok] : 1.0f;
        float *o = out + (int64_t)tok * n;
        int rc = cqo_matmul(dtype, 1, k, n, x + in_row * k, (const uint8_t *)w + (int64_t)e * expert_bytes, o);
        if (rc) return rc;
        for (int64_t c = 0; c < n; c++) o[c] = o[c] * scale;
    }
    return 0;
}
