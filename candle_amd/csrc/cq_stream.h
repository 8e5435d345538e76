// Streaming decode matvec for Q4_K / Q5_K / Q6_K / Q4_0 / Q8_0 weights and one f32 activation row:
// dst[row] = sum_k W[row, k] * x^[k].  For Q4_0 / Q8_0 a "super-block" below is eight consecutive 32-element blocks.
//
// The weights of a tensor are one contiguous stream of super-blocks (rows follow each other without gaps).  A wave
// step is a run of that stream — 64 super-blocks when a row has a power of two of them, else one row — copied
// HBM -> LDS as it lies in memory by buffer loads that write LDS directly (16 bytes per lane, whole cache lines
// per instruction, no registers in between).  Each lane then reads ITS OWN super-block out of LDS and does the
// whole block: the 6-bit scales and mins are decoded four at a time, the eight sub-block dots are plain
// v_dot4_i32_i8 chains, and only the lanes of one row are added up (DPP, log2(lanes per row) steps).  Per weight
// row this is about half the vector instructions of the four-lanes-per-super-block kernel (qmv_kernel), where every
// lane decodes its own pair of scales and every row pays a six-step wave reduction.
//
// Why LDS copies and not register loads: vector loads are issued in order and block the wave's instruction stream
// while the memory pipeline is full, so loads requested ahead of time delay the arithmetic queued behind them.
// A copy into LDS needs no destination registers and no instruction after it until the data is used; the wave
// asks for its next step as soon as it has moved the current block from LDS to registers, before the arithmetic.
//
// Same arithmetic contract as qmv_kernel: activations quantized to Q8_K exactly like BlockQ8K::from_float
// (candle-core/src/quantized/k_quants.rs:2320-2358), integer dots exact, one f32 scaling per super-block
// (vec_dot Q4_K x Q8_K k_quants.rs:1460-1540, Q5_K :1714-1801, Q6_K :2035-2092); Q4_0 / Q8_0 rows take Q8_0 activation
// blocks like BlockQ8_0::from_float (k_quants.rs:658-687) and the per-block sums of their vec_dot (:294-311, 720-738),
// in block order; only the f32 summation order of the K-quant rows differs.
#pragma once
#include "cq_actquant.h"
#include "cq_device.h"

namespace {

typedef __attribute__((address_space(3))) void cq_lds_void;

// Quantized activations in LDS: per 256-element span 272 bytes of int8 (256 + 16: the sixteen lanes of a row read
// sixteen different spans at once, a stride of 256 bytes would put them all on the same banks) and a 64-byte record
//   f32 d | 12 bytes unused | u8 bl[8] | i8 bh[8] | u8 bl16[16] | i8 bh16[16]
// with  sum of 32-element sub-block j = 128 * bh[j] + bl[j]  and  sum of 16-element group g = 128 * bh16[g] + bl16[g],
// 0 <= bl < 128 (the sums split into two int8 halves, so that sum_j coefficient_j * sum_j is a few dot4).  The 16-element
// sums are written for Q6_K only, whose scales cover 16 elements.  Q8_0 activations (for Q4_0 / Q8_0 weights) have a scale
// per 32 elements: their record keeps the eight f32 scales in the last 32 bytes and the 32-element sums where they are.
constexpr int QS_ACT_STRIDE = 272;
constexpr int QS_AUX_STRIDE = 64;
template <int MAXB> struct StreamAct {
    static constexpr int AUX_OFF = (MAXB + 1) * QS_ACT_STRIDE;                     // one more span: the dump for waves without a span
    static constexpr int BYTES = AUX_OFF + (MAXB + 1) * QS_AUX_STRIDE;
};
// what a lane keeps of its span's record besides d
struct QsAux { u32x4 s32, bl16, bh16; };

__device__ __forceinline__ uint32_t qs_wave_umax(uint32_t v) {
    // unsigned max through DPP (fused into v_max_u32_dpp); non-negative floats order like their bit patterns
#define CQ_S(ctrl, rm, bc) v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, ctrl, rm, 0xf, bc))
    CQ_S(0x111, 0xf, true); CQ_S(0x112, 0xf, true); CQ_S(0x114, 0xf, true); CQ_S(0x118, 0xf, true);
    CQ_S(0x142, 0xa, false); CQ_S(0x143, 0xc, false);
#undef CQ_S
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// f32::round (half away from zero) followed by Rust's `as i8` (saturating, NaN -> 0) in five instructions.  Adding the largest
// float below one half, with the sign of x, carries exactly the values whose fraction is at least one half to the next
// integer: the sum is rounded to nearest, a fraction of one half ends within a quarter of an ulp of that integer and a
// smaller fraction at least an ulp of x below it (checked against trunc / compare / add on every float of magnitude
// 2^-8 .. 2^25).  v_cvt_i32_f32 truncates, saturates and turns NaN into 0.
__device__ __forceinline__ int qs_round_i8(float x) {
    const float t = x + __builtin_copysignf(0.49999997f, x);
    int q;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(q) : "v"(t));
    return min(max(q, -128), 127);
}
// four values in [-128, 127] -> four bytes
__device__ __forceinline__ uint32_t qs_pack4(const int (&q)[4]) {
    return __builtin_amdgcn_perm((uint32_t)q[1], (uint32_t)q[0], 0x0c0c0400u) | __builtin_amdgcn_perm((uint32_t)q[3], (uint32_t)q[2], 0x04000c0cu);
}

// One wave quantizes 256-element spans (lane l holds elements 4l .. 4l+3 of each) into the LDS layout above, in three
// parts so that a wave with several spans pays for one division sequence: the largest magnitude of each span; the
// scales of all spans, span j in lane j; the values.
// BlockQ8K::from_float takes the FIRST element of largest magnitude, with its sign, for the scale; here the scale always
// comes from the magnitude: with the other sign d and every q flip together and every product d * q is the same value,
// so no result of the matvec depends on it.  NaN / Inf inputs follow the CPU arithmetic (round, saturating cast, NaN -> 0).
__device__ __forceinline__ uint32_t qs_span_umax(const float v[4]) {
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    amax = amax == amax ? amax : 0.0f;                // four NaNs: the CPU's `amax < |x|` never takes a NaN either
    return qs_wave_umax(__float_as_uint(amax));
}
// iscale = -127 / max and d = 1 / iscale (both 0 for an all-zero span) of NS spans whose maxima are wave-uniform
template <int NS>
__device__ __forceinline__ void qs_span_scales(const uint32_t (&wmax)[NS], int lane, float (&iscale)[NS], float (&d)[NS]) {
    uint32_t m = wmax[NS - 1];
#pragma unroll
    for (int j = 0; j < NS - 1; j++) asm("v_writelane_b32 %0, %1, %2" : "+v"(m) : "s"(wmax[j]), "i"(j));
    float is = -127.0f / __uint_as_float(m);
    float dd = 1.0f / is;
    is = m != 0 ? is : 0.0f;
    dd = m != 0 ? dd : 0.0f;
#pragma unroll
    for (int j = 0; j < NS; j++) {
        iscale[j] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, is), j));
        d[j] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, dd), j));
    }
}
template <bool SUM16>
__device__ __forceinline__ void qs_span_store(const float v[4], float iscale, float d, int span, int lane, uint8_t *act, int aux_off) {
    int q[4];
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = qs_round_i8(iscale * v[i]);
    const uint32_t packed = qs_pack4(q);
    *(uint32_t *)(act + span * QS_ACT_STRIDE + lane * 4) = packed;
    int s = sdot4(packed, 0x01010101u, 0);
    uint8_t *aux = act + aux_off + span * QS_AUX_STRIDE;
    if (SUM16) {
        const int s16 = quad_sum(s);                  // sum of the 16-element group, in all four lanes
        if ((lane & 3) == 0) {
            aux[32 + (lane >> 2)] = (uint8_t)(s16 & 127);
            aux[48 + (lane >> 2)] = (uint8_t)(s16 >> 7);
        }
    }
    s = oct_sum(s);                                   // sum of the 32-element sub-block, in all eight lanes
    if ((lane & 7) == 0) {
        aux[16 + (lane >> 3)] = (uint8_t)(s & 127);
        aux[24 + (lane >> 3)] = (uint8_t)(s >> 7);    // arithmetic shift: 128 * bh + bl == s for negative sums too
    }
    if (lane == 0) *(float *)aux = d;
}
// NS spans of one wave: values v[j] go to LDS span span0 + j * stride, or to span `dump` when that is not below `limit`
template <bool SUM16, int NS>
__device__ __forceinline__ void qs_quantize_spans(const float (&v)[NS][4], int span0, int stride, int limit, int dump, int lane, uint8_t *act,
                                                  int aux_off) {
    uint32_t wmax[NS];
    float iscale[NS], d[NS];
#pragma unroll
    for (int j = 0; j < NS; j++) wmax[j] = qs_span_umax(v[j]);
    qs_span_scales<NS>(wmax, lane, iscale, d);
#pragma unroll
    for (int j = 0; j < NS; j++) {
        const int span = span0 + j * stride;
        qs_span_store<SUM16>(v[j], iscale[j], d[j], span < limit ? span : dump, lane, act, aux_off);
    }
}

// The same span as eight Q8_0 blocks (cq_quantize_q80_vals, cq_actquant.h: BlockQ8_0::from_float with the f16-rounded scale).
__device__ __forceinline__ void qs_quantize_span_q80(const float v[4], int span, int lane, uint8_t *act, int aux_off) {
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    amax = oct_max(amax);                             // a 32-element block = eight neighbouring lanes
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    int q[4];
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = qs_round_i8(v[i] * id);
    const uint32_t packed = qs_pack4(q);
    *(uint32_t *)(act + span * QS_ACT_STRIDE + lane * 4) = packed;
    int s = oct_sum(sdot4(packed, 0x01010101u, 0));
    uint8_t *aux = act + aux_off + span * QS_AUX_STRIDE;
    if ((lane & 7) == 0) {
        aux[16 + (lane >> 3)] = (uint8_t)(s & 127);
        aux[24 + (lane >> 3)] = (uint8_t)(s >> 7);
        ((float *)(aux + 32))[lane >> 3] = h2f(f2h_bits(d));      // the CPU stores d as f16 and multiplies by its f32 value
    }
}

// ---- per-format work of one lane on one super-block held in LDS --------------------------------------------
template <int DT> struct StreamFmt;

// sum over 32 bytes (8 dwords) of low / high nibbles against two 32-element activation sub-blocks
__device__ __forceinline__ void qs_dot_pair_q4(const u32x4 q0, const u32x4 q1, const u32x4 a0, const u32x4 a1, const u32x4 a2, const u32x4 a3,
                                               int &dl, int &dh) {
    const uint32_t M4 = 0x0f0f0f0fu;
    dl = 0; dh = 0;
    dl = sdot4(q0.x & M4, a0.x, dl); dl = sdot4(q0.y & M4, a0.y, dl); dl = sdot4(q0.z & M4, a0.z, dl); dl = sdot4(q0.w & M4, a0.w, dl);
    dl = sdot4(q1.x & M4, a1.x, dl); dl = sdot4(q1.y & M4, a1.y, dl); dl = sdot4(q1.z & M4, a1.z, dl); dl = sdot4(q1.w & M4, a1.w, dl);
    // high nibbles without a shift: (q ^ 0x80) & 0xf0 is the int8 value 16 * (hi - 8) (one v_bitop3_b32), so the chain
    // sums 16 * (hi - 8) * a; the caller adds 8 * sum(a) back through the sub-block sums
#define CQ_HI(v) (((v) ^ 0x80808080u) & 0xf0f0f0f0u)
    dh = sdot4(CQ_HI(q0.x), a2.x, dh); dh = sdot4(CQ_HI(q0.y), a2.y, dh); dh = sdot4(CQ_HI(q0.z), a2.z, dh); dh = sdot4(CQ_HI(q0.w), a2.w, dh);
    dh = sdot4(CQ_HI(q1.x), a3.x, dh); dh = sdot4(CQ_HI(q1.y), a3.y, dh); dh = sdot4(CQ_HI(q1.z), a3.z, dh); dh = sdot4(CQ_HI(q1.w), a3.w, dh);
#undef CQ_HI
    dh >>= 4;                                          // exact: every term is a multiple of 16
}

// scales / mins of the eight sub-blocks, four to a dword (get_scale_min_k4, candle-core/src/quantized/utils.rs:50-60)
struct QsScales { uint32_t scA, scB, mA, mB; };
__device__ __forceinline__ QsScales qs_scales_k4(uint32_t u0, uint32_t u1, uint32_t u2) {
    QsScales s;
    s.scA = u0 & 0x3f3f3f3fu;
    s.mA = u1 & 0x3f3f3f3fu;
    s.scB = (u2 & 0x0f0f0f0fu) | ((u0 >> 2) & 0x30303030u);
    s.mB = ((u2 >> 4) & 0x0f0f0f0fu) | ((u1 >> 2) & 0x30303030u);
    return s;
}

// sum_j c_j * (128 * bh_j + bl_j) for the eight byte coefficients (cA: j = 0..3, cB: j = 4..7); aux = {blA, blB, bhA, bhB}
__device__ __forceinline__ int qs_dot_sums(uint32_t cA, uint32_t cB, const u32x4 aux) {
    return (sdot4(cB, aux.w, sdot4(cA, aux.z, 0)) << 7) + sdot4(cB, aux.y, sdot4(cA, aux.x, 0));
}

template <> struct StreamFmt<CQ_Q4K> {
    static constexpr int BB = 144;             // bytes of a super-block
    static constexpr int NLD = 9;              // 16-byte-per-lane loads that cover 64 super-blocks
    struct Blk { u32x4 hdr; u32x4 q[8]; };
    static __device__ __forceinline__ void read(Blk &b, const uint8_t *p) {
        b.hdr = *(const u32x4 *)p;
#pragma unroll
        for (int i = 0; i < 8; i++) b.q[i] = *(const u32x4 *)(p + 16 + 16 * i);
    }
    // a[16]: the lane's 256 int8 activations; d8 and aux: the span's record
    static __device__ __forceinline__ float dot(const Blk &b, const u32x4 (&a)[16], float d8, const QsAux &aux) {
        const u32x4 aux1 = aux.s32;
        int D[8];
#pragma unroll
        for (int g = 0; g < 4; g++) qs_dot_pair_q4(b.q[2 * g], b.q[2 * g + 1], a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3], D[2 * g], D[2 * g + 1]);
        const QsScales s = qs_scales_k4(b.hdr.y, b.hdr.z, b.hdr.w);
        int S = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            S += __mul24((int)((s.scA >> (8 * j)) & 0xff), D[j]);
            S += __mul24((int)((s.scB >> (8 * j)) & 0xff), D[4 + j]);
        }
        // the odd sub-blocks came out as sum (hi - 8) * a: add 8 * sc_j * sum_j(a)
        S += qs_dot_sums(s.scA & 0xff00ff00u, s.scB & 0xff00ff00u, aux1) << 3;
        const int M = qs_dot_sums(s.mA, s.mB, aux1);
        return d8 * (h2f(b.hdr.x) * (float)S - h2f(b.hdr.x >> 16) * (float)M);
    }
};

template <> struct StreamFmt<CQ_Q5K> {
    static constexpr int BB = 176;
    static constexpr int NLD = 11;
    struct Blk { u32x4 hdr; u32x4 h[2]; u32x4 q[8]; };
    static __device__ __forceinline__ void read(Blk &b, const uint8_t *p) {
        b.hdr = *(const u32x4 *)p;
        b.h[0] = *(const u32x4 *)(p + 16);
        b.h[1] = *(const u32x4 *)(p + 32);
#pragma unroll
        for (int i = 0; i < 8; i++) b.q[i] = *(const u32x4 *)(p + 48 + 16 * i);
    }
    static __device__ __forceinline__ float dot(const Blk &b, const u32x4 (&a)[16], float d8, const QsAux &aux) {
        const u32x4 aux1 = aux.s32;
        const uint32_t M4 = 0x0f0f0f0fu;
        const uint32_t h[8] = {b.h[0].x, b.h[0].y, b.h[0].z, b.h[0].w, b.h[1].x, b.h[1].y, b.h[1].z, b.h[1].w};
        int D[8];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            // bytes 32g .. 32g+31 of qs: low nibbles + bit 2g of qh -> sub-block 2g, high nibbles + bit 2g+1 -> sub-block 2g+1
            const uint32_t q[8] = {b.q[2 * g].x, b.q[2 * g].y, b.q[2 * g].z, b.q[2 * g].w, b.q[2 * g + 1].x, b.q[2 * g + 1].y, b.q[2 * g + 1].z, b.q[2 * g + 1].w};
            const uint32_t al[8] = {a[4 * g].x, a[4 * g].y, a[4 * g].z, a[4 * g].w, a[4 * g + 1].x, a[4 * g + 1].y, a[4 * g + 1].z, a[4 * g + 1].w};
            const uint32_t ah[8] = {a[4 * g + 2].x, a[4 * g + 2].y, a[4 * g + 2].z, a[4 * g + 2].w, a[4 * g + 3].x, a[4 * g + 3].y, a[4 * g + 3].z, a[4 * g + 3].w};
            int dl = 0, dh = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t hb = h[i] >> (2 * g);
                dl = sdot4((q[i] & M4) | ((hb & 0x01010101u) << 4), al[i], dl);
                dh = sdot4(((q[i] >> 4) & M4) | ((hb << 3) & 0x10101010u), ah[i], dh);
            }
            D[2 * g] = dl; D[2 * g + 1] = dh;
        }
        const QsScales s = qs_scales_k4(b.hdr.y, b.hdr.z, b.hdr.w);
        int S = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            S += __mul24((int)((s.scA >> (8 * j)) & 0xff), D[j]);
            S += __mul24((int)((s.scB >> (8 * j)) & 0xff), D[4 + j]);
        }
        const int M = qs_dot_sums(s.mA, s.mB, aux1);
        return d8 * (h2f(b.hdr.x) * (float)S - h2f(b.hdr.x >> 16) * (float)M);
    }
};

// Q6_K (210 bytes: ql[128] | qh[64] | int8 scales[16] | f16 d): super-blocks lie at 2-byte alignment in the stream, so a
// lane's block is read from LDS with unaligned 16-byte reads.  Element layout (k_quants.rs:2265-2274): for half h and
// l in [0, 32), byte ql[64h + l] holds elements 128h + l (low nibble) and 128h + 64 + l (high), byte ql[64h + 32 + l]
// elements 128h + 32 + l and 128h + 96 + l; qh[32h + l] carries bits 4-5 of those four in its four bit pairs; scale
// 8h + l / 16 + 2t belongs to the t-th of them.  Values are taken as unsigned 6-bit numbers; their offset of 32 goes
// through the 16-element activation sums:  sum_g sc_g * (dot_g - 32 * sum16_g).
template <> struct StreamFmt<CQ_Q6K> {
    static constexpr int BB = 210;
    static constexpr int NLD = 14;             // 64 x 210 = 13440 bytes
    struct Blk { u32x4 ql[8]; u32x4 qh[4]; u32x4 sc; uint32_t d; };
    // The block starts on an even byte of LDS.  A 16-byte LDS read from an address that is not a multiple of 16 takes
    // several passes (measured: the lanes' reads of a step took 1.5 us against 0.3 us for the 144 aligned bytes of Q4_K), so
    // the lane reads the 54 aligned dwords around its block and shifts them by its own 0 or 2 bytes.
    static __device__ __forceinline__ void read(Blk &b, const uint8_t *p) {
        const uint32_t sh = (uint32_t)(uintptr_t)p & 2u;
        const uint32_t *q = (const uint32_t *)(p - sh);
        uint32_t r[54];
#pragma unroll
        for (int i = 0; i < 54; i++) r[i] = q[i];
        auto dw = [&](int i) { return __builtin_amdgcn_alignbyte(r[i + 1], r[i], sh); };
#pragma unroll
        for (int i = 0; i < 8; i++) b.ql[i] = u32x4{dw(4 * i), dw(4 * i + 1), dw(4 * i + 2), dw(4 * i + 3)};
#pragma unroll
        for (int i = 0; i < 4; i++) b.qh[i] = u32x4{dw(32 + 4 * i), dw(33 + 4 * i), dw(34 + 4 * i), dw(35 + 4 * i)};
        b.sc = u32x4{dw(48), dw(49), dw(50), dw(51)};
        b.d = dw(52) & 0xffffu;
    }
    static __device__ __forceinline__ float dot(const Blk &b, const u32x4 (&a)[16], float d8, const QsAux &aux) {
        const uint32_t M4 = 0x0f0f0f0fu, M2 = 0x30303030u;
        const uint32_t scw[4] = {b.sc.x, b.sc.y, b.sc.z, b.sc.w};
        int S = 0;
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int is = 0; is < 2; is++) {
                int g0 = 0, g1 = 0, g2 = 0, g3 = 0;                 // groups 8h + is + {0, 2, 4, 6}
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int j = 4 * is + jj;                      // dword of the 32 `l` positions
                    const uint32_t qa = b.ql[4 * h + (j >> 2)][j & 3], qb = b.ql[4 * h + 2 + (j >> 2)][j & 3];
                    const uint32_t hh = b.qh[2 * h + (j >> 2)][j & 3];
                    g0 = sdot4((qa & M4) | ((hh << 4) & M2), a[8 * h + is][jj], g0);
                    g1 = sdot4((qb & M4) | ((hh << 2) & M2), a[8 * h + 2 + is][jj], g1);
                    g2 = sdot4(((qa >> 4) & M4) | (hh & M2), a[8 * h + 4 + is][jj], g2);
                    g3 = sdot4(((qb >> 4) & M4) | ((hh >> 2) & M2), a[8 * h + 6 + is][jj], g3);
                }
                // scale bytes 8h + is + 2t: byte (is + 2t) % 4 of dword 2h + (is + 2t) / 4
                const uint32_t w0 = scw[2 * h], w1 = scw[2 * h + 1];
                S += __mul24((int)(int8_t)(w0 >> (8 * is)), g0);
                S += __mul24((int)(int8_t)(w0 >> (8 * (is + 2))), g1);
                S += __mul24((int)(int8_t)(w1 >> (8 * is)), g2);
                S += __mul24((int)(int8_t)(w1 >> (8 * (is + 2))), g3);
            }
        }
        // sum_g sc_g * sum16_g with sum16 = 128 * bh16 + bl16 (scales are signed bytes, the halves small enough for int8)
        int C = 0, Ch = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            C = sdot4(scw[i], aux.bl16[i], C);
            Ch = sdot4(scw[i], aux.bh16[i], Ch);
        }
        S -= ((Ch << 7) + C) << 5;
        return (h2f(b.d) * d8) * (float)S;
    }
};

// ---- Q4_0 / Q8_0: eight blocks of 18 / 34 bytes per lane -------------------------------------------------------------
// The lane's 144 / 272 bytes start on 16 bytes; inside them block b starts at byte 18 b / 34 b, so the quants of the even
// blocks sit 2 bytes off the dword grid and are put back with one v_alignbyte_b32 per dword.  `aux.bl16 | aux.bh16` hold the
// eight f32 activation scales, `aux.s32` the eight block sums as (bl, bh).
__device__ __forceinline__ float qs_q0_scale(const QsAux &aux, int b) {
    return __uint_as_float(b < 4 ? aux.bl16[b] : aux.bh16[b - 4]);
}
// dword i of the payload that starts `off` bytes into the dword array r (off even, known at compile time)
template <int N> __device__ __forceinline__ uint32_t qs_dword_at(const uint32_t (&r)[N], int off) {
    const int w = off >> 2;
    return (off & 2) ? __builtin_amdgcn_alignbyte(r[w + 1 < N ? w + 1 : w], r[w], 2) : r[w];
}
template <int N> __device__ __forceinline__ uint32_t qs_half_at(const uint32_t (&r)[N], int off) {
    return (off & 2) ? r[off >> 2] >> 16 : r[off >> 2] & 0xffffu;
}

template <> struct StreamFmt<CQ_Q8_0> {
    static constexpr int BB = 272;             // eight blocks
    static constexpr int NLD = 17;
    struct Blk { uint32_t r[68]; };
    static __device__ __forceinline__ void read(Blk &b, const uint8_t *p) {
#pragma unroll
        for (int i = 0; i < 17; i++) {
            const u32x4 t = *(const u32x4 *)(p + 16 * i);
            b.r[4 * i] = t.x; b.r[4 * i + 1] = t.y; b.r[4 * i + 2] = t.z; b.r[4 * i + 3] = t.w;
        }
    }
    static __device__ __forceinline__ float dot(const Blk &b, const u32x4 (&a)[16], float, const QsAux &aux) {
        float sumf = 0.0f;
#pragma unroll
        for (int blk = 0; blk < 8; blk++) {
            int s = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) s = sdot4(qs_dword_at(b.r, 34 * blk + 2 + 4 * i), a[2 * blk + (i >> 2)][i & 3], s);
            sumf += (float)s * h2f(qs_half_at(b.r, 34 * blk)) * qs_q0_scale(aux, blk);
        }
        return sumf;
    }
};

template <> struct StreamFmt<CQ_Q4_0> {
    static constexpr int BB = 144;
    static constexpr int NLD = 9;
    struct Blk { uint32_t r[36]; };
    static __device__ __forceinline__ void read(Blk &b, const uint8_t *p) {
#pragma unroll
        for (int i = 0; i < 9; i++) {
            const u32x4 t = *(const u32x4 *)(p + 16 * i);
            b.r[4 * i] = t.x; b.r[4 * i + 1] = t.y; b.r[4 * i + 2] = t.z; b.r[4 * i + 3] = t.w;
        }
    }
    static __device__ __forceinline__ float dot(const Blk &b, const u32x4 (&a)[16], float, const QsAux &aux) {
        const uint32_t M4 = 0x0f0f0f0fu;
        float sumf = 0.0f;
#pragma unroll
        for (int blk = 0; blk < 8; blk++) {
            // sum((q - 8) * y) = sum(q * y) - 8 * sum(y); the block sum is 128 * bh + bl
            const uint32_t bl = (aux.s32[blk >> 2] >> (8 * (blk & 3))) & 0xffu;
            const int bh = (int)(int8_t)(aux.s32[2 + (blk >> 2)] >> (8 * (blk & 3)));
            int s = -8 * (128 * bh + (int)bl);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t q = qs_dword_at(b.r, 18 * blk + 2 + 4 * i);
                s = sdot4(q & M4, a[2 * blk][i], s);
                s = sdot4((q >> 4) & M4, a[2 * blk + 1][i], s);
            }
            sumf += (float)s * h2f(qs_half_at(b.r, 18 * blk)) * qs_q0_scale(aux, blk);
        }
        return sumf;
    }
};

// Geometry of one launch, computed on the host.
struct StreamGeom {
    int k, n;
    int bpr;              // super-blocks per row
    int lp_shift;         // log2(lanes per row): lanes per row = bpr rounded up to a power of two
    int step_rows;        // rows per wave step = 64 >> lp_shift
    int step_bytes;       // step_rows * bpr * BB
    int total_steps;      // ceil(n / step_rows)
    int dst_dtype;
    int64_t stride_dst;   // unused by one-row launches, kept for symmetry with QmvGeom
    int64_t w_bytes;      // n * bpr * BB
};

// sum over aligned groups of 1 << lp_shift lanes; the last lane of each group ends with the group's sum
__device__ __forceinline__ float qs_group_sum(float v, int lp_shift) {
#define CQ_A(ctrl, rm, bc) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, rm, 0xf, bc))
    if (lp_shift >= 1) CQ_A(0x111, 0xf, true);
    if (lp_shift >= 2) CQ_A(0x112, 0xf, true);
    if (lp_shift >= 3) CQ_A(0x114, 0xf, true);
    if (lp_shift >= 4) CQ_A(0x118, 0xf, true);
    if (lp_shift >= 5) CQ_A(0x142, 0xa, false);
    if (lp_shift >= 6) CQ_A(0x143, 0xc, false);
#undef CQ_A
    return v;
}

}  // namespace
