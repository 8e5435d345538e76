/*
 * Timed CPU baseline (TEST / BENCH INFRASTRUCTURE ONLY; never linked into the shipped library).
 *
 * candle on x86 is built with target-cpu=native (.cargo/config.toml:2), so QMatMul::forward runs
 * the AVX2 vec_dot kernels of candle-core/src/quantized/avx.rs and splits output columns over a
 * thread pool (k_quants.rs:2429-2469).  This file restates that configuration in C so bench.py can
 * time "what candle's CPU path does" on the GPU box's host cores: activation rows are quantized
 * with the scalar from_float of cq_oracle.c (included below, same translation unit), each dot
 * product follows the arithmetic of the matching avx.rs kernel, and columns are split over pthreads
 * with rows processed serially, as the reference does.
 *
 *   Q4_0 x Q8_0  avx.rs:50-68      Q8_0 x Q8_0  avx.rs:71-87     Q6_K x Q8_K  avx.rs:131-216
 *   Q4_K x Q8_K  avx.rs:443-525    Q5_K x Q8_K  avx.rs:528-638
 *
 * Results differ from the scalar oracle only in f32 summation order (checked in tests/).
 */
#include <immintrin.h>
#include <pthread.h>

#include "cq_oracle.c"

static inline float hsum8(__m256 x) {
    __m128 r = _mm_add_ps(_mm256_extractf128_ps(x, 1), _mm256_castps256_ps128(x));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_movehdup_ps(r));
    return _mm_cvtss_f32(r);
}

/* sum over groups of 4 of (signed x) * (signed y), as 8 floats */
static inline __m256 mul_sum_i8_pairs_float(__m256i x, __m256i y) {
    __m256i ax = _mm256_sign_epi8(x, x);
    __m256i sy = _mm256_sign_epi8(y, x);
    __m256i dot = _mm256_maddubs_epi16(ax, sy);
    return _mm256_cvtepi32_ps(_mm256_madd_epi16(_mm256_set1_epi16(1), dot));
}

static float fast_q4_0(int64_t n, const block_q4_0 *x, const block_q8_0 *y) {
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < n / 32; i++) {
        __m256 d = _mm256_set1_ps(cqo_f16_to_f32(x[i].d) * cqo_f16_to_f32(y[i].d));
        __m128i t = _mm_loadu_si128((const __m128i *)x[i].qs);
        __m256i b = _mm256_insertf128_si256(_mm256_castsi128_si256(t), _mm_srli_epi16(t, 4), 1);
        b = _mm256_sub_epi8(_mm256_and_si256(_mm256_set1_epi8(0xF), b), _mm256_set1_epi8(8));
        __m256i q8 = _mm256_loadu_si256((const __m256i *)y[i].qs);
        acc = _mm256_fmadd_ps(d, mul_sum_i8_pairs_float(b, q8), acc);
    }
    return hsum8(acc);
}

static float fast_q8_0(int64_t n, const block_q8_0 *x, const block_q8_0 *y) {
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < n / 32; i++) {
        __m256 d = _mm256_set1_ps(cqo_f16_to_f32(x[i].d) * cqo_f16_to_f32(y[i].d));
        __m256i a = _mm256_loadu_si256((const __m256i *)x[i].qs);
        __m256i b = _mm256_loadu_si256((const __m256i *)y[i].qs);
        acc = _mm256_fmadd_ps(d, mul_sum_i8_pairs_float(a, b), acc);
    }
    return hsum8(acc);
}

/* 16 x i16: scales (low 8) and mins (high 8) of a Q4_K / Q5_K block */
static inline __m256i k45_mins_and_scales(const uint8_t *s12) {
    uint8_t sc[8], mn[8];
    unpack_scales_mins(s12, sc, mn);
    __m128i v = _mm_set_epi64x(*(const int64_t *)mn, *(const int64_t *)sc);
    return _mm256_cvtepu8_epi16(v);
}

static inline __m256i k4_shuffle(int i) {   /* broadcast 16-bit scale i over a 128-bit lane pair */
    return _mm256_set1_epi16((short)((2 * i) | ((2 * i + 1) << 8)));
}

static float fast_q4_K(int64_t n, const block_q4_K *x, const block_q8_K *y) {
    const __m256i m4 = _mm256_set1_epi8(0xF);
    __m256 acc = _mm256_setzero_ps();
    __m128 acc_m = _mm_setzero_ps();
    for (int64_t i = 0; i < n / QK_K; i++) {
        float d = y[i].d * cqo_f16_to_f32(x[i].d);
        float dmin = -y[i].d * cqo_f16_to_f32(x[i].dmin);
        __m256i ms = k45_mins_and_scales(x[i].scales);
        __m256i q8sums = _mm256_loadu_si256((const __m256i *)y[i].bsums);
        __m128i q8s = _mm_hadd_epi16(_mm256_extracti128_si256(q8sums, 0), _mm256_extracti128_si256(q8sums, 1));
        __m128i prod = _mm_madd_epi16(_mm256_extracti128_si256(ms, 1), q8s);
        acc_m = _mm_fmadd_ps(_mm_set1_ps(dmin), _mm_cvtepi32_ps(prod), acc_m);
        __m128i sc128 = _mm256_extracti128_si256(ms, 0);
        __m256i scales = _mm256_insertf128_si256(_mm256_castsi128_si256(sc128), sc128, 1);
        const uint8_t *q4 = x[i].qs;
        const int8_t *q8 = y[i].qs;
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < QK_K / 64; j++) {
            __m256i scale_l = _mm256_shuffle_epi8(scales, k4_shuffle(2 * j));
            __m256i scale_h = _mm256_shuffle_epi8(scales, k4_shuffle(2 * j + 1));
            __m256i q4bits = _mm256_loadu_si256((const __m256i *)q4); q4 += 32;
            __m256i q4l = _mm256_and_si256(q4bits, m4);
            __m256i q4h = _mm256_and_si256(_mm256_srli_epi16(q4bits, 4), m4);
            __m256i q8l = _mm256_loadu_si256((const __m256i *)q8); q8 += 32;
            sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(scale_l, _mm256_maddubs_epi16(q4l, q8l)));
            __m256i q8h = _mm256_loadu_si256((const __m256i *)q8); q8 += 32;
            sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(scale_h, _mm256_maddubs_epi16(q4h, q8h)));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    acc_m = _mm_add_ps(acc_m, _mm_movehl_ps(acc_m, acc_m));
    acc_m = _mm_add_ss(acc_m, _mm_movehdup_ps(acc_m));
    return hsum8(acc) + _mm_cvtss_f32(acc_m);
}

static float fast_q5_K(int64_t n, const block_q5_K *x, const block_q8_K *y) {
    const __m256i m4 = _mm256_set1_epi8(0xF);
    __m256 acc = _mm256_setzero_ps();
    float summs = 0.0f;
    for (int64_t i = 0; i < n / QK_K; i++) {
        float d = y[i].d * cqo_f16_to_f32(x[i].d);
        float dmin = -y[i].d * cqo_f16_to_f32(x[i].dmin);
        __m256i ms = k45_mins_and_scales(x[i].scales);
        __m256i q8sums = _mm256_loadu_si256((const __m256i *)y[i].bsums);
        __m128i q8s = _mm_hadd_epi16(_mm256_extracti128_si256(q8sums, 0), _mm256_extracti128_si256(q8sums, 1));
        __m128i prod = _mm_madd_epi16(_mm256_extracti128_si256(ms, 1), q8s);
        __m128i hs = _mm_hadd_epi32(_mm_hadd_epi32(prod, _mm_setzero_si128()), _mm_setzero_si128());
        summs += dmin * (float)_mm_extract_epi32(hs, 0);
        __m128i sc128 = _mm256_extracti128_si256(ms, 0);
        __m256i scales = _mm256_insertf128_si256(_mm256_castsi128_si256(sc128), sc128, 1);
        __m256i hbits = _mm256_loadu_si256((const __m256i *)x[i].qh);
        const uint8_t *q5 = x[i].qs;
        const int8_t *q8 = y[i].qs;
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < QK_K / 64; j++) {
            __m256i scale_0 = _mm256_shuffle_epi8(scales, k4_shuffle(2 * j));
            __m256i scale_1 = _mm256_shuffle_epi8(scales, k4_shuffle(2 * j + 1));
            __m256i q5bits = _mm256_loadu_si256((const __m256i *)q5); q5 += 32;
            __m256i h0 = _mm256_and_si256(_mm256_srl_epi16(hbits, _mm_cvtsi32_si128(2 * j)), _mm256_set1_epi8(1));
            __m256i h1 = _mm256_and_si256(_mm256_srl_epi16(hbits, _mm_cvtsi32_si128(2 * j + 1)), _mm256_set1_epi8(1));
            __m256i q5_0 = _mm256_add_epi8(_mm256_and_si256(q5bits, m4), _mm256_slli_epi16(h0, 4));
            __m256i q5_1 = _mm256_add_epi8(_mm256_and_si256(_mm256_srli_epi16(q5bits, 4), m4), _mm256_slli_epi16(h1, 4));
            __m256i q8_0 = _mm256_loadu_si256((const __m256i *)q8); q8 += 32;
            __m256i q8_1 = _mm256_loadu_si256((const __m256i *)q8); q8 += 32;
            __m256i p0 = _mm256_madd_epi16(scale_0, _mm256_maddubs_epi16(q5_0, q8_0));
            __m256i p1 = _mm256_madd_epi16(scale_1, _mm256_maddubs_epi16(q5_1, q8_1));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p0, p1));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum8(acc) + summs;
}

static float fast_q6_K(int64_t n, const block_q6_K *x, const block_q8_K *y) {
    const __m256i m4 = _mm256_set1_epi8(0xF), m2 = _mm256_set1_epi8(3), m32s = _mm256_set1_epi8(32);
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < n / QK_K; i++) {
        float d = y[i].d * cqo_f16_to_f32(x[i].d);
        const uint8_t *q4 = x[i].ql, *qh = x[i].qh;
        const int8_t *q8 = y[i].qs;
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < QK_K / 128; j++) {
            __m256i sc[4];
            for (int q = 0; q < 4; q++) {   /* 16 x i16: scale 8j+2q for the low 128 bits, 8j+2q+1 for the high */
                __m128i lo = _mm_set1_epi16((short)x[i].scales[8 * j + 2 * q]);
                __m128i hi = _mm_set1_epi16((short)x[i].scales[8 * j + 2 * q + 1]);
                sc[q] = _mm256_insertf128_si256(_mm256_castsi128_si256(lo), hi, 1);
            }
            __m256i b1 = _mm256_loadu_si256((const __m256i *)q4); q4 += 32;
            __m256i b2 = _mm256_loadu_si256((const __m256i *)q4); q4 += 32;
            __m256i bh = _mm256_loadu_si256((const __m256i *)qh); qh += 32;
            __m256i h0 = _mm256_slli_epi16(_mm256_and_si256(bh, m2), 4);
            __m256i h1 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(bh, 2), m2), 4);
            __m256i h2 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(bh, 4), m2), 4);
            __m256i h3 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(bh, 6), m2), 4);
            __m256i v[4];
            v[0] = _mm256_or_si256(_mm256_and_si256(b1, m4), h0);
            v[1] = _mm256_or_si256(_mm256_and_si256(b2, m4), h1);
            v[2] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(b1, 4), m4), h2);
            v[3] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(b2, 4), m4), h3);
            for (int q = 0; q < 4; q++) {
                __m256i a = _mm256_loadu_si256((const __m256i *)q8); q8 += 32;
                __m256i p = _mm256_sub_epi16(_mm256_maddubs_epi16(v[q], a), _mm256_maddubs_epi16(m32s, a));
                sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(sc[q], p));
            }
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum8(acc);
}

static float fast_vec_dot(int dtype, int64_t k, const void *w, const void *a) {
    switch (dtype) {
        case CQ_Q4_0: return fast_q4_0(k, (const block_q4_0 *)w, (const block_q8_0 *)a);
        case CQ_Q8_0: return fast_q8_0(k, (const block_q8_0 *)w, (const block_q8_0 *)a);
        case CQ_Q4K: return fast_q4_K(k, (const block_q4_K *)w, (const block_q8_K *)a);
        case CQ_Q5K: return fast_q5_K(k, (const block_q5_K *)w, (const block_q8_K *)a);
        case CQ_Q6K: return fast_q6_K(k, (const block_q6_K *)w, (const block_q8_K *)a);
    }
    return 0.0f;
}

typedef struct {
    int dtype;
    int64_t m, k, n, col0, col1, w_row_bytes, a_row_bytes;
    const uint8_t *w, *a;
    float *dst;
} fast_job;

static void *fast_worker(void *arg) {
    fast_job *j = (fast_job *)arg;
    for (int64_t r = 0; r < j->m; r++)               /* rows serial, as in k_quants.rs:2438 */
        for (int64_t c = j->col0; c < j->col1; c++)
            j->dst[r * j->n + c] = fast_vec_dot(j->dtype, j->k, j->w + c * j->w_row_bytes, j->a + r * j->a_row_bytes);
    return NULL;
}

/* k_quants::matmul with AVX2 dot products and `threads` workers over column ranges. */
int cqf_matmul(int dtype, int64_t m, int64_t k, int64_t n, const float *lhs, const void *rhs_t, float *dst, int threads) {
    int64_t bs = cqo_block_size(dtype);
    int vdt = cqo_vec_dot_type(dtype);
    if (bs == 0 || vdt < 0 || dtype == CQ_Q8K || k % bs != 0) return -1;
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    int64_t k_in_blocks = k / bs;
    int64_t a_row_bytes = k_in_blocks * cqo_type_size(vdt);
    uint8_t *lhs_b = (uint8_t *)malloc((size_t)(m * a_row_bytes) + 64);
    if (!lhs_b) return -2;
    for (int64_t r = 0; r < m; r++) cqo_from_float(vdt, lhs + r * k, lhs_b + r * a_row_bytes, k);
    fast_job jobs[256];
    pthread_t tids[256];
    int64_t per = (n + threads - 1) / threads;
    int n_jobs = 0;
    for (int t = 0; t < threads; t++) {
        int64_t c0 = t * per, c1 = c0 + per < n ? c0 + per : n;
        if (c0 >= c1) break;
        fast_job jb = {dtype, m, k, n, c0, c1, k_in_blocks * cqo_type_size(dtype), a_row_bytes, (const uint8_t *)rhs_t, lhs_b, dst};
        jobs[n_jobs++] = jb;
    }
    for (int t = 0; t + 1 < n_jobs; t++) pthread_create(&tids[t], NULL, fast_worker, &jobs[t]);
    if (n_jobs > 0) fast_worker(&jobs[n_jobs - 1]);     /* the calling thread is a worker too */
    for (int t = 0; t + 1 < n_jobs; t++) pthread_join(tids[t], NULL);
    free(lhs_b);
    return 0;
}
