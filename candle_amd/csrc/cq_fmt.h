// Per-format "unit" decoding shared by the decode matvec and the expert-grouped MoE matvec.
//
// A row of W is cut into units — what one lane consumes per step with 128-bit loads:
//   Q4_K / Q5_K: one 64-element group g of a super-block (32 bytes of qs = two 16-byte loads, the
//                matching qh bytes for Q5_K) + the 16-byte block header; 4 lanes per super-block
//   Q6_K       : 16 `l` positions of one 128-element half (3 x 16 bytes); 4 lanes per super-block
//   Q4_0 / Q8_0: one 32-element block (also Q4_1, Q5_0, Q5_1)
//   Q2_K / Q3_K: the 16 bytes qs[32h + 16c, +16) of a super-block = 16 positions of the four 32-element quarters of
//                half h, the element set of a Q6_K unit; 4 lanes per super-block
// so a wave64 step covers 16 super-blocks (4096 elements) of a K-quant row or 64 blocks (2048
// elements) of a Q4_0 / Q8_0 row.  For each format Fmt<DT> gives the raw weight registers (W), the
// activation registers (A) and the dot product of one unit: exact integer arithmetic inside the
// unit, one f32 scaling at the end, following the CPU vec_dot of
// candle-core/src/quantized/k_quants.rs (Q4_0 :294-311, Q8_0 :720-738, Q4_K :1460-1540,
// Q5_K :1714-1801, Q6_K :2035-2092, Q4_1 :323-351, Q5_0 :434-455, Q5_1 :530-562, Q2_K :838-886, Q3_K :1068-1187).
#pragma once
#include "cq_device.h"

namespace {

template <int DT> struct Fmt;

// Pointers to one quantized activation row (global scratch or its LDS copy).
struct ActRow {
    const int8_t *qs;       // [k]
    const float *d;         // K-quants: [k/256];  Q4_0 / Q8_0: {d, sum} pairs [k/32][2]
    const int16_t *bsums;   // K-quants: [k/16]
};

__device__ __forceinline__ ActRow act_row(const int8_t *qs, const float *d, const int16_t *bsums, int w_dtype, int64_t b, int k) {
    ActRow r;
    r.qs = qs + b * k;
    if (cq_is_kquant(w_dtype)) {
        r.d = d + b * (k >> 8);
        r.bsums = bsums + b * (k >> 4);
    } else {
        r.d = d + 2 * b * (k >> 5);
        r.bsums = bsums;
    }
    return r;
}

// ---- Q4_K / Q5_K common parts -------------------------------------------------------------------
struct AK45 {   // activations of one 64-element group
    u32x4 a0, a1, a2, a3;   // elements 0..15, 16..31 (sub-block 2g) and 32..47, 48..63 (sub-block 2g+1)
    float d8;
    int bs_lo, bs_hi;       // sums of the two 32-element sub-blocks
};

__device__ __forceinline__ void load_act_k45(AK45 &a, const ActRow &ar, int u) {
    const int8_t *q = ar.qs + u * 64;
    a.a0 = *reinterpret_cast<const u32x4 *>(q);
    a.a1 = *reinterpret_cast<const u32x4 *>(q + 16);
    a.a2 = *reinterpret_cast<const u32x4 *>(q + 32);
    a.a3 = *reinterpret_cast<const u32x4 *>(q + 48);
    a.d8 = ar.d[u >> 2];
    u32x2 bs = *reinterpret_cast<const u32x2 *>(ar.bsums + u * 4);   // four 16-element sums
    a.bs_lo = (int)(int16_t)(bs.x & 0xffff) + (int)(int16_t)(bs.x >> 16);
    a.bs_hi = (int)(int16_t)(bs.y & 0xffff) + (int)(int16_t)(bs.y >> 16);
}

// 6-bit scales / mins of sub-blocks 2g and 2g+1 as bytes [sc_lo, sc_hi, m_lo, m_hi]
// (get_scale_min_k4, candle-core/src/quantized/utils.rs:50-60, as two byte permutes).
__device__ __forceinline__ uint32_t k4_scale_min(uint32_t u0, uint32_t u1, uint32_t u2, int g) {
    // v_perm_b32(hi, lo, sel): selector bytes 0-3 pick from lo, 4-7 from hi
    const uint32_t sel = (g & 1) ? 0x07060302u : 0x05040100u;        // [lo.b(2p), lo.b(2p+1), hi.b(2p), hi.b(2p+1)]
    uint32_t A = __builtin_amdgcn_perm(u1, u0, sel);                 // [u0.b, u0.b', u1.b, u1.b']
    uint32_t B = __builtin_amdgcn_perm(u2 >> 4, u2, sel) & 0x0f0f0f0fu;
    const uint32_t lo = A & 0x3f3f3f3fu, hi = B | ((A >> 2) & 0x30303030u);
    const uint32_t m = 0u - (uint32_t)(g >> 1);        // all ones for g >= 2: a bit blend, not a divergent branch
    return (lo & ~m) | (hi & m);
}

__device__ __forceinline__ float finish_k45(uint32_t hdr0, uint32_t sm, int dl, int dh, const AK45 &a) {
    int S = __mul24((int)(sm & 0xff), dl) + __mul24((int)((sm >> 8) & 0xff), dh);
    int M = __mul24((int)((sm >> 16) & 0xff), a.bs_lo) + __mul24((int)(sm >> 24), a.bs_hi);
    float d = h2f(hdr0), dmin = h2f(hdr0 >> 16);
    return a.d8 * (d * (float)S - dmin * (float)M);
}

template <> struct Fmt<CQ_Q4K> {
    static constexpr int UE = 64, UPB = 4;
    struct W { u32x4 hdr, q0, q1; };
    typedef AK45 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (u >> 2) * 144;
        w.hdr = *reinterpret_cast<const u32x4 *>(blk);
        w.q0 = *reinterpret_cast<const u32x4 *>(blk + 16 + 32 * (u & 3));
        w.q1 = *reinterpret_cast<const u32x4 *>(blk + 32 + 32 * (u & 3));
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { load_act_k45(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int u) {
        uint32_t sm = k4_scale_min(w.hdr.y, w.hdr.z, w.hdr.w, u & 3);
        const uint32_t M4 = 0x0f0f0f0fu;
        int dl = 0, dh = 0;
        dl = sdot4(w.q0.x & M4, a.a0.x, dl); dl = sdot4(w.q0.y & M4, a.a0.y, dl);
        dl = sdot4(w.q0.z & M4, a.a0.z, dl); dl = sdot4(w.q0.w & M4, a.a0.w, dl);
        dl = sdot4(w.q1.x & M4, a.a1.x, dl); dl = sdot4(w.q1.y & M4, a.a1.y, dl);
        dl = sdot4(w.q1.z & M4, a.a1.z, dl); dl = sdot4(w.q1.w & M4, a.a1.w, dl);
        dh = sdot4((w.q0.x >> 4) & M4, a.a2.x, dh); dh = sdot4((w.q0.y >> 4) & M4, a.a2.y, dh);
        dh = sdot4((w.q0.z >> 4) & M4, a.a2.z, dh); dh = sdot4((w.q0.w >> 4) & M4, a.a2.w, dh);
        dh = sdot4((w.q1.x >> 4) & M4, a.a3.x, dh); dh = sdot4((w.q1.y >> 4) & M4, a.a3.y, dh);
        dh = sdot4((w.q1.z >> 4) & M4, a.a3.z, dh); dh = sdot4((w.q1.w >> 4) & M4, a.a3.w, dh);
        return finish_k45(w.hdr.x, sm, dl, dh, a);
    }
};

template <> struct Fmt<CQ_Q5K> {
    static constexpr int UE = 64, UPB = 4;
    struct W { u32x4 hdr, h0, h1, q0, q1; };
    typedef AK45 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (u >> 2) * 176;
        w.hdr = *reinterpret_cast<const u32x4 *>(blk);
        w.h0 = *reinterpret_cast<const u32x4 *>(blk + 16);          // qh[0..15]
        w.h1 = *reinterpret_cast<const u32x4 *>(blk + 32);          // qh[16..31]
        w.q0 = *reinterpret_cast<const u32x4 *>(blk + 48 + 32 * (u & 3));
        w.q1 = *reinterpret_cast<const u32x4 *>(blk + 64 + 32 * (u & 3));
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { load_act_k45(a, ar, u); }
    // one dword of qs + its qh dword -> unsigned 5-bit values of sub-block 2g (lo) and 2g+1 (hi)
    static __device__ __forceinline__ void unpack(uint32_t q, uint32_t h, int g, uint32_t &lo, uint32_t &hi) {
        uint32_t hb = h >> (2 * g);
        lo = (q & 0x0f0f0f0fu) | ((hb & 0x01010101u) << 4);
        hi = ((q >> 4) & 0x0f0f0f0fu) | ((hb << 3) & 0x10101010u);
    }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int u) {
        const int g = u & 3;
        uint32_t sm = k4_scale_min(w.hdr.y, w.hdr.z, w.hdr.w, g);
        const uint32_t q[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
        const uint32_t h[8] = {w.h0.x, w.h0.y, w.h0.z, w.h0.w, w.h1.x, w.h1.y, w.h1.z, w.h1.w};
        const uint32_t al[8] = {a.a0.x, a.a0.y, a.a0.z, a.a0.w, a.a1.x, a.a1.y, a.a1.z, a.a1.w};
        const uint32_t ah[8] = {a.a2.x, a.a2.y, a.a2.z, a.a2.w, a.a3.x, a.a3.y, a.a3.z, a.a3.w};
        int dl = 0, dh = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t lo, hi;
            unpack(q[i], h[i], g, lo, hi);
            dl = sdot4(lo, al[i], dl);
            dh = sdot4(hi, ah[i], dh);
        }
        return finish_k45(w.hdr.x, sm, dl, dh, a);
    }
};

template <> struct Fmt<CQ_Q6K> {
    static constexpr int UE = 64, UPB = 4;
    struct W { u32x4 qa, qb, qh; u32x2 sc; uint32_t d; };
    struct A { u32x4 a[4]; int bs[4]; float d8; };
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (u >> 2) * 210;
        int h = (u >> 1) & 1, c = u & 1;
        w.qa = ld_u<u32x4>(blk + 64 * h + 16 * c);          // ql[l], l = 16c..16c+15 of this half
        w.qb = ld_u<u32x4>(blk + 64 * h + 32 + 16 * c);     // ql[l + 32]
        w.qh = ld_u<u32x4>(blk + 128 + 32 * h + 16 * c);    // qh[l]
        w.sc = ld_u<u32x2>(blk + 192 + 8 * h);              // the 8 scales of this half
        w.d = ld_u<uint16_t>(blk + 208);
    }
    // unit (h, c) covers elements 128h + 32i + 16c + [0,16) for the four quarters i (k_quants.rs:2265-2274)
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) {
        int sb = u >> 2, h = (u >> 1) & 1, c = u & 1;
        const int8_t *q = ar.qs + sb * 256 + 128 * h + 16 * c;
#pragma unroll
        for (int i = 0; i < 4; i++) a.a[i] = *reinterpret_cast<const u32x4 *>(q + 32 * i);
        // 16-element sums of quarters 0..3 at index 8h + 2i + c
        u32x4 bs = *reinterpret_cast<const u32x4 *>(ar.bsums + sb * 16 + 8 * h);
        const uint32_t b4[4] = {bs.x, bs.y, bs.z, bs.w};
#pragma unroll
        for (int i = 0; i < 4; i++) a.bs[i] = (int)(int16_t)((b4[i] >> (16 * c)) & 0xffff);
        a.d8 = ar.d[sb];
    }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int u) {
        const int c = u & 1;
        // quarter i uses scale index c + 2i of the half
        uint32_t s0 = w.sc.x >> (8 * c), s1 = w.sc.y >> (8 * c);
        const int sc[4] = {(int)(int8_t)(s0 & 0xff), (int)(int8_t)((s0 >> 16) & 0xff), (int)(int8_t)(s1 & 0xff), (int)(int8_t)((s1 >> 16) & 0xff)};
        const uint32_t qa[4] = {w.qa.x, w.qa.y, w.qa.z, w.qa.w};
        const uint32_t qb[4] = {w.qb.x, w.qb.y, w.qb.z, w.qb.w};
        const uint32_t qh[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
        // unsigned 6-bit values; the -32 offset is applied through the 16-element sums
        int dq[4] = {-32 * a.bs[0], -32 * a.bs[1], -32 * a.bs[2], -32 * a.bs[3]};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t A0[4] = {a.a[0].x, a.a[0].y, a.a[0].z, a.a[0].w};
            const uint32_t A1[4] = {a.a[1].x, a.a[1].y, a.a[1].z, a.a[1].w};
            const uint32_t A2[4] = {a.a[2].x, a.a[2].y, a.a[2].z, a.a[2].w};
            const uint32_t A3[4] = {a.a[3].x, a.a[3].y, a.a[3].z, a.a[3].w};
            dq[0] = sdot4((qa[j] & 0x0f0f0f0fu) | ((qh[j] << 4) & 0x30303030u), A0[j], dq[0]);
            dq[1] = sdot4((qb[j] & 0x0f0f0f0fu) | ((qh[j] << 2) & 0x30303030u), A1[j], dq[1]);
            dq[2] = sdot4(((qa[j] >> 4) & 0x0f0f0f0fu) | (qh[j] & 0x30303030u), A2[j], dq[2]);
            dq[3] = sdot4(((qb[j] >> 4) & 0x0f0f0f0fu) | ((qh[j] >> 2) & 0x30303030u), A3[j], dq[3]);
        }
        int S = __mul24(sc[0], dq[0]) + __mul24(sc[1], dq[1]) + __mul24(sc[2], dq[2]) + __mul24(sc[3], dq[3]);
        return (h2f(w.d) * a.d8) * (float)S;
    }
};

// Q6_K rows of more than one wave step: 8 lanes per super-block.  Lane j of a super-block takes the 16 bytes
// ql[16j, 16j + 16) — so one load instruction reads each super-block's ql as one 128-byte run, and a 14336-element
// row is exactly 7 full wave steps — plus the qh bytes of the same 16 `l` positions.
// j = 4h + 2p + c: low nibbles are elements 128h + 32p + 16c + [0, 16) (qh bits 2p, 2p + 1), high nibbles the
// elements 64 further on (qh bits 2p + 4, 2p + 5); k_quants.rs:2265-2274.
struct FmtQ6Narrow {
    static constexpr int UE = 32, UPB = 8;
    struct W { u32x4 ql, qh; u32x2 sc; uint32_t d; };
    struct A { u32x4 lo, hi; int bs_lo, bs_hi; float d8; };
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (u >> 3) * 210;
        const int j = u & 7, h = j >> 2, c = j & 1;
        w.ql = ld_u<u32x4>(blk + 16 * j);
        w.qh = ld_u<u32x4>(blk + 128 + 32 * h + 16 * c);
        w.sc = ld_u<u32x2>(blk + 192 + 8 * h);              // the 8 scales of this half
        w.d = ld_u<uint16_t>(blk + 208);
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) {
        const int sb = u >> 3, j = u & 7, h = j >> 2, idx = 8 * h + (j & 3);      // 16-element group of the low nibbles
        const int8_t *q = ar.qs + sb * 256 + 16 * idx;
        a.lo = *reinterpret_cast<const u32x4 *>(q);
        a.hi = *reinterpret_cast<const u32x4 *>(q + 64);
        a.bs_lo = ar.bsums[sb * 16 + idx];
        a.bs_hi = ar.bsums[sb * 16 + idx + 4];
        a.d8 = ar.d[sb];
    }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int u) {
        const int pc = u & 3, p = (u >> 1) & 1;
        const int s_lo = (int)(int8_t)((w.sc.x >> (8 * pc)) & 0xff), s_hi = (int)(int8_t)((w.sc.y >> (8 * pc)) & 0xff);
        const uint32_t ql[4] = {w.ql.x, w.ql.y, w.ql.z, w.ql.w};
        const uint32_t qh[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
        const uint32_t al[4] = {a.lo.x, a.lo.y, a.lo.z, a.lo.w};
        const uint32_t ah[4] = {a.hi.x, a.hi.y, a.hi.z, a.hi.w};
        // unsigned 6-bit values; the -32 offset is applied through the 16-element sums
        int dl = -32 * a.bs_lo, dh = -32 * a.bs_hi;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t hs = qh[i] >> (2 * p);
            dl = sdot4((ql[i] & 0x0f0f0f0fu) | ((hs << 4) & 0x30303030u), al[i], dl);
            dh = sdot4(((ql[i] >> 4) & 0x0f0f0f0fu) | (hs & 0x30303030u), ah[i], dh);
        }
        const int S = __mul24(s_lo, dl) + __mul24(s_hi, dh);
        return (h2f(w.d) * a.d8) * (float)S;
    }
};

// ---- Q2_K / Q3_K: unit (h, c) = qs bytes [32h + 16c, +16), i.e. elements 128h + 32i + 16c + [0,16) for the four
// quarters i (bit pairs 2i, 2i + 1 of each byte) with scale index 8h + 2i + c — the element set and activation
// registers of a Q6_K unit (k_quants.rs:1013-1049, 1369-1421).
template <> struct Fmt<CQ_Q2K> {
    static constexpr int UE = 64, UPB = 4;
    struct W { u32x4 qs; u32x2 sc; uint32_t dd; };
    typedef Fmt<CQ_Q6K>::A A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (u >> 2) * 84;
        w.qs = ld_u<u32x4>(blk + 16 + 16 * (u & 3));
        w.sc = ld_u<u32x2>(blk + 8 * ((u >> 1) & 1));       // the 8 scale / min bytes of this half
        w.dd = ld_u<uint32_t>(blk + 80);                     // d | dmin << 16
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { Fmt<CQ_Q6K>::load_a(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int u) {
        const int c = u & 1;
        const uint32_t s0 = w.sc.x >> (8 * c), s1 = w.sc.y >> (8 * c);
        const uint32_t scb[4] = {s0 & 0xff, (s0 >> 16) & 0xff, s1 & 0xff, (s1 >> 16) & 0xff};
        const uint32_t q[4] = {w.qs.x, w.qs.y, w.qs.z, w.qs.w};
        int isum = 0, summs = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t A4[4] = {a.a[i].x, a.a[i].y, a.a[i].z, a.a[i].w};
            int t = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) t = sdot4((q[j] >> (2 * i)) & 0x03030303u, A4[j], t);
            isum += __mul24((int)(scb[i] & 0xf), t);
            summs += __mul24((int)(scb[i] >> 4), a.bs[i]);
        }
        const float d = h2f(w.dd), dmin = h2f(w.dd >> 16);
        return a.d8 * (d * (float)isum - dmin * (float)summs);
    }
};

template <> struct Fmt<CQ_Q3K> {
    static constexpr int UE = 64, UPB = 4;
    struct W { u32x4 qs, hm; uint32_t s0, s1, s2, d; };
    typedef Fmt<CQ_Q6K>::A A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (u >> 2) * 110;
        w.hm = ld_u<u32x4>(blk + 16 * (u & 1));              // hmask[16c, +16)
        w.qs = ld_u<u32x4>(blk + 32 + 16 * (u & 3));
        w.s0 = ld_u<uint32_t>(blk + 96);
        w.s1 = ld_u<uint32_t>(blk + 100);
        w.s2 = ld_u<uint32_t>(blk + 104);
        w.d = ld_u<uint16_t>(blk + 108);
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { Fmt<CQ_Q6K>::load_a(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int u) {
        const int h = (u >> 1) & 1, c = u & 1;
        // the eight 6-bit scales of half h as two dwords of bytes (k_quants.rs:1148-1156): low nibbles from
        // scales[0..8) (half 0) or their high nibbles (half 1), bits 4-5 from the bit pairs of scales[8..12)
        const uint32_t t2 = w.s2 >> (4 * h);
        const uint32_t e0 = ((w.s0 >> (4 * h)) & 0x0f0f0f0fu) | ((t2 & 0x03030303u) << 4);
        const uint32_t e1 = ((w.s1 >> (4 * h)) & 0x0f0f0f0fu) | (((t2 >> 2) & 0x03030303u) << 4);
        const uint32_t x0 = e0 >> (8 * c), x1 = e1 >> (8 * c);
        const int sc[4] = {(int)(x0 & 0xff) - 32, (int)((x0 >> 16) & 0xff) - 32, (int)(x1 & 0xff) - 32, (int)((x1 >> 16) & 0xff) - 32};
        const uint32_t q[4] = {w.qs.x, w.qs.y, w.qs.z, w.qs.w};
        const uint32_t hm[4] = {w.hm.x >> (4 * h), w.hm.y >> (4 * h), w.hm.z >> (4 * h), w.hm.w >> (4 * h)};
        int S = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t A4[4] = {a.a[i].x, a.a[i].y, a.a[i].z, a.a[i].w};
            // value = (2 bits | hmask bit << 2) - 4: the -4 goes through the 16-element sum
            int t = -4 * a.bs[i];
#pragma unroll
            for (int j = 0; j < 4; j++) t = sdot4(((q[j] >> (2 * i)) & 0x03030303u) | (((hm[j] >> i) & 0x01010101u) << 2), A4[j], t);
            S += __mul24(sc[i], t);
        }
        return (h2f(w.d) * a.d8) * (float)S;
    }
};

// The unit decomposition a kernel instance uses: rows of one wave step (SINGLE) and register-blocked instances
// keep Fmt<DT>.
template <int DT, int NB, bool SINGLE> struct UnitFmt { typedef Fmt<DT> type; };
template <> struct UnitFmt<CQ_Q6K, 1, false> { typedef FmtQ6Narrow type; };

// ---- Q4_0 / Q8_0: one 32-element block per unit, Q8_0-quantized activations ------------------
struct A0 {
    u32x4 a0, a1;
    float d8;
    int s8;
};

__device__ __forceinline__ void load_act_q0(A0 &a, const ActRow &ar, int u) {
    const int8_t *q = ar.qs + u * 32;
    a.a0 = *reinterpret_cast<const u32x4 *>(q);
    a.a1 = *reinterpret_cast<const u32x4 *>(q + 16);
    u32x2 ds = *reinterpret_cast<const u32x2 *>(ar.d + 2 * u);
    a.d8 = __uint_as_float(ds.x);
    a.s8 = (int)ds.y;
}

// ---- blocks of 2 (mod 4) bytes: Q4_0 (18), Q5_0 (22), Q8_0 (34) --------------------------------
// Every other block of such a row starts on an odd halfword, and a 16-byte load from an address that is not a multiple
// of 4 costs the vector memory path about a quarter of its rate (measured: Q4_1 / Q5_1, the same blocks plus 2 bytes,
// stream at 3.8 / 4.2 TB/s where Q4_0 / Q5_0 reached 3.0 / 3.1).  A block of 4 j + 2 bytes is one halfword plus j whole
// dwords, so it is fetched as exactly that: at a block address that is a multiple of 4 the dwords come first and the
// halfword is the block's last two bytes; on an odd halfword the halfword is the block's first two bytes and the dwords
// start 2 bytes in.  Every load is naturally aligned and none touches a byte outside [block, block + size).  The
// halfword offset is undone in registers with one byte permute per dword.
template <typename T> __device__ __forceinline__ T ld_a4(const void *p) {
    struct __attribute__((packed, aligned(4))) W { T v; };
    return reinterpret_cast<const W *>(p)->v;
}
// Splits a block of (2 + dw_bytes) bytes at `p`: returns the address of its dword run, `hw` = the address of its lone
// halfword.  `sel` is the v_perm_b32 selector that rebuilds payload dword i (the payload starts 2 bytes into the
// block) from the dword pair (y[i + 1], y[i]) of the sequence y = {dword run, halfword}: bytes 2..5 of the pair when
// the run starts at the block, bytes 0..3 when it starts with the payload.
__device__ __forceinline__ const uint8_t *split_hw(const uint8_t *p, int dw_bytes, const uint8_t *&hw, uint32_t &sel) {
    const bool odd = ((uintptr_t)p & 2) != 0;
    sel = odd ? 0x03020100u : 0x05040302u;
    hw = p + (odd ? 0 : dw_bytes);
    return p + (odd ? 2 : 0);
}
__device__ __forceinline__ uint32_t ld_hw(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }
__device__ __forceinline__ uint32_t take_hw(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }
// the f16 scale at the start of the block: the low half of the first dword of the run, or the lone halfword
__device__ __forceinline__ uint32_t head_hw(uint32_t y0, uint32_t hw, uint32_t sel) { return (sel & 2u) ? y0 : hw; }

template <> struct Fmt<CQ_Q4_0> {
    static constexpr int UE = 32, UPB = 1;
    struct W { u32x4 x; uint32_t hw, sel; };
    typedef A0 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *hw;
        const uint8_t *a = split_hw(row + u * 18, 16, hw, w.sel);
        w.x = ld_a4<u32x4>(a);
        w.hw = ld_hw(hw);
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { load_act_q0(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int) {
        const uint32_t M4 = 0x0f0f0f0fu;
        const uint32_t q0 = take_hw(w.x.y, w.x.x, w.sel), q1 = take_hw(w.x.z, w.x.y, w.sel), q2 = take_hw(w.x.w, w.x.z, w.sel),
                       q3 = take_hw(w.hw, w.x.w, w.sel);
        int s = -8 * a.s8;    // sum((q - 8) * y) = sum(q * y) - 8 * sum(y)
        s = sdot4(q0 & M4, a.a0.x, s); s = sdot4(q1 & M4, a.a0.y, s);
        s = sdot4(q2 & M4, a.a0.z, s); s = sdot4(q3 & M4, a.a0.w, s);
        s = sdot4((q0 >> 4) & M4, a.a1.x, s); s = sdot4((q1 >> 4) & M4, a.a1.y, s);
        s = sdot4((q2 >> 4) & M4, a.a1.z, s); s = sdot4((q3 >> 4) & M4, a.a1.w, s);
        return (float)s * h2f(head_hw(w.x.x, w.hw, w.sel)) * a.d8;
    }
};

template <> struct Fmt<CQ_Q8_0> {
    static constexpr int UE = 32, UPB = 1;
    struct W { u32x4 x, y; uint32_t hw, sel; };
    typedef A0 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *hw;
        const uint8_t *a = split_hw(row + u * 34, 32, hw, w.sel);
        w.x = ld_a4<u32x4>(a);
        w.y = ld_a4<u32x4>(a + 16);
        w.hw = ld_hw(hw);
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { load_act_q0(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int) {
        int s = 0;
        s = sdot4(take_hw(w.x.y, w.x.x, w.sel), a.a0.x, s); s = sdot4(take_hw(w.x.z, w.x.y, w.sel), a.a0.y, s);
        s = sdot4(take_hw(w.x.w, w.x.z, w.sel), a.a0.z, s); s = sdot4(take_hw(w.y.x, w.x.w, w.sel), a.a0.w, s);
        s = sdot4(take_hw(w.y.y, w.y.x, w.sel), a.a1.x, s); s = sdot4(take_hw(w.y.z, w.y.y, w.sel), a.a1.y, s);
        s = sdot4(take_hw(w.y.w, w.y.z, w.sel), a.a1.z, s); s = sdot4(take_hw(w.hw, w.y.w, w.sel), a.a1.w, s);
        return (float)s * h2f(head_hw(w.x.x, w.hw, w.sel)) * a.d8;
    }
};

// ---- Q4_1 / Q5_0 / Q5_1: one 32-element block per unit, Q8_0 activation registers.  The CPU path quantizes the
// activations of Q4_1 / Q5_1 to Q8_1, whose qs and d are those of Q8_0 and whose s = f16(f16(sum) * d)
// (k_quants.rs:770-799) follows from the {d, sum} pair the Q8_0 scratch holds.
__device__ __forceinline__ float q8_1_s(const A0 &a) { return h2f(f2h_bits(h2f(f2h_bits((float)a.s8)) * a.d8)); }

// four bits -> bit 4 of four bytes
__device__ __forceinline__ uint32_t spread4_to_bit4(uint32_t b) { return (((b & 0xfu) * 0x00204081u) & 0x01010101u) << 4; }

template <> struct Fmt<CQ_Q4_1> {
    static constexpr int UE = 32, UPB = 1;
    struct W { u32x4 qs; uint32_t dm; };
    typedef A0 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + u * 20;
        w.dm = ld_u<uint32_t>(blk);                          // d | m << 16
        w.qs = ld_u<u32x4>(blk + 4);
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { load_act_q0(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int) {
        const uint32_t M4 = 0x0f0f0f0fu;
        int s = 0;
        s = sdot4(w.qs.x & M4, a.a0.x, s); s = sdot4(w.qs.y & M4, a.a0.y, s);
        s = sdot4(w.qs.z & M4, a.a0.z, s); s = sdot4(w.qs.w & M4, a.a0.w, s);
        s = sdot4((w.qs.x >> 4) & M4, a.a1.x, s); s = sdot4((w.qs.y >> 4) & M4, a.a1.y, s);
        s = sdot4((w.qs.z >> 4) & M4, a.a1.z, s); s = sdot4((w.qs.w >> 4) & M4, a.a1.w, s);
        return (float)s * h2f(w.dm) * a.d8 + h2f(w.dm >> 16) * q8_1_s(a);
    }
};

// unsigned 5-bit values of a Q5_0 / Q5_1 block: qh bit j belongs to element j (low nibbles), bit j + 16 to element j + 16
__device__ __forceinline__ int dot_q5(const u32x4 &qs, uint32_t qh, const A0 &a, int s) {
    const uint32_t M4 = 0x0f0f0f0fu;
    const uint32_t q[4] = {qs.x, qs.y, qs.z, qs.w};
    const uint32_t lo[4] = {a.a0.x, a.a0.y, a.a0.z, a.a0.w};
    const uint32_t hi[4] = {a.a1.x, a.a1.y, a.a1.z, a.a1.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        s = sdot4((q[i] & M4) | spread4_to_bit4(qh >> (4 * i)), lo[i], s);
        s = sdot4(((q[i] >> 4) & M4) | spread4_to_bit4(qh >> (16 + 4 * i)), hi[i], s);
    }
    return s;
}

template <> struct Fmt<CQ_Q5_0> {
    static constexpr int UE = 32, UPB = 1;
    struct W { u32x4 x; uint32_t z, hw, sel; };
    typedef A0 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *hw;
        const uint8_t *a = split_hw(row + u * 22, 20, hw, w.sel);     // 22-byte blocks: a halfword and five dwords, see Fmt<CQ_Q4_0>
        w.x = ld_a4<u32x4>(a);
        w.z = *reinterpret_cast<const uint32_t *>(a + 16);
        w.hw = ld_hw(hw);
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { load_act_q0(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int) {
        const uint32_t qh = take_hw(w.x.y, w.x.x, w.sel);
        const u32x4 qs = {take_hw(w.x.z, w.x.y, w.sel), take_hw(w.x.w, w.x.z, w.sel), take_hw(w.z, w.x.w, w.sel), take_hw(w.hw, w.z, w.sel)};
        const int s = dot_q5(qs, qh, a, -16 * a.s8);    // sum((q - 16) * y) = sum(q * y) - 16 * sum(y)
        return (float)s * h2f(head_hw(w.x.x, w.hw, w.sel)) * a.d8;
    }
};

template <> struct Fmt<CQ_Q5_1> {
    static constexpr int UE = 32, UPB = 1;
    struct W { u32x4 qs; uint32_t dm, qh; };
    typedef A0 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + u * 24;
        w.dm = ld_u<uint32_t>(blk);                          // d | m << 16
        w.qh = ld_u<uint32_t>(blk + 4);
        w.qs = ld_u<u32x4>(blk + 8);
    }
    static __device__ __forceinline__ void load_a(A &a, const ActRow &ar, int u) { load_act_q0(a, ar, u); }
    static __device__ __forceinline__ float dot(const W &w, const A &a, int) {
        const int s = dot_q5(w.qs, w.qh, a, 0);
        return (float)s * h2f(w.dm) * a.d8 + h2f(w.dm >> 16) * q8_1_s(a);
    }
};

// ---------------------------------------------------------------------------------------------
// wave64 sum through DPP row shifts and row broadcasts; the total ends up in lane 63.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
#define CQ_DPP(ctrl, rmask, bc) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, rmask, 0xf, bc))
    v += CQ_DPP(0x111, 0xf, true);     // row_shr:1
    v += CQ_DPP(0x112, 0xf, true);     // row_shr:2
    v += CQ_DPP(0x114, 0xf, true);     // row_shr:4
    v += CQ_DPP(0x118, 0xf, true);     // row_shr:8   -> lane 15 of each row holds the row sum
    v += CQ_DPP(0x142, 0xa, false);    // row_bcast:15 into rows 1 and 3
    v += CQ_DPP(0x143, 0xc, false);    // row_bcast:31 into rows 2 and 3 -> lane 63 holds the total
#undef CQ_DPP
    return v;
}

// Four wave sums at once: lane 60 + r ends with the sum of v[r] over the wave (r = 0..3).  Two transposing steps inside
// the quads leave lane class (lane & 3) = r holding row r's quad sums (one select pair and one DPP add per step instead of
// one DPP add per row), two row shifts collect the 16-lane rows, two cross-lane reads the four rows of the wave:
// 15 instructions for four rows where wave_sum_to_lane63 takes 6 (plus their wait states) per row.
__device__ __forceinline__ float wave_sum4_to_lanes60(float v0, float v1, float v2, float v3, int lane) {
#define CQ_DPP(x, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, 0xf, 0xf, true))
    const bool odd = lane & 1, up = lane & 2;
    const float a = (odd ? v1 : v0) + CQ_DPP((odd ? v0 : v1), CQ_DPP_QUAD_XOR1);     // even lanes: row 0 pairs, odd lanes: row 1 pairs
    const float b = (odd ? v3 : v2) + CQ_DPP((odd ? v2 : v3), CQ_DPP_QUAD_XOR1);     // rows 2 / 3
    float c = (up ? b : a) + CQ_DPP((up ? a : b), CQ_DPP_QUAD_XOR2);                 // lane & 3 = r: quad sum of row r
    c += CQ_DPP(c, CQ_DPP_ROW_SHR(4));
    c += CQ_DPP(c, CQ_DPP_ROW_SHR(8));                                               // lanes 12..15 of each 16-lane row: its sums
#undef CQ_DPP
    c += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, c)));
    c += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, c)));
    return c;
}

// ---------------------------------------------------------------------------------------------
// Output conversion (the CUDA backend keeps the activation dtype; the CPU f16 path rounds the f32
// dot product to f16, k_quants.rs:2680-2682).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void store_out(void *dst, int dst_dtype, int64_t idx, float v) {
    if (dst_dtype == CQ_F32) {
        ((float *)dst)[idx] = v;
    } else if (dst_dtype == CQ_F16) {
        ((uint16_t *)dst)[idx] = f2h_bits(v);
    } else {
        uint32_t b = __float_as_uint(v);   // bf16, round to nearest even, NaN kept quiet
        uint32_t r = (b & 0x7fffffffu) > 0x7f800000u ? (b | 0x00400000u) : b + 0x7fffu + ((b >> 16) & 1u);
        ((uint16_t *)dst)[idx] = (uint16_t)(r >> 16);
    }
}

}  // namespace
