// Per-format "unit" decoding shared by the decode matvec and the expert-grouped MoE matvec.
//
// A row of W is cut into units — the bytes one lane consumes per step with 128-bit loads:
//   Q4_K / Q5_K: one 16-byte slice of qs (8 per super-block) + the 16-byte block header
//   Q6_K       : 16 `l` positions of one 128-element half (3 x 16 bytes, 4 per super-block)
//   Q4_0 / Q8_0: one 32-element block
// For each format Fmt<DT> gives the raw weight registers (W), the decoded weights (P), the
// activation registers (A) and the exact integer dot product of one unit.
#pragma once
#include "cq_device.h"

namespace {

// ---------------------------------------------------------------------------------------------
// Per-format unit: weight registers (W), decoded weights (P), activation registers (A).
// ---------------------------------------------------------------------------------------------
template <int DT> struct Fmt;

// ---- shared by Q4_K and Q5_K: 6-bit scale/min pair of sub-blocks 2g and 2g+1 -----------------
// (vectorised form of get_scale_min_k4, k_quants.rs:1499-1509)
__device__ __forceinline__ void k4_scales(uint32_t u0, uint32_t u1, uint32_t u2, int g, int &sc_lo, int &sc_hi, int &m_lo, int &m_hi) {
    uint32_t sc4, m4;
    if (g < 2) {
        sc4 = u0 & 0x3f3f3f3fu;
        m4 = u1 & 0x3f3f3f3fu;
    } else {
        sc4 = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
        m4 = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
    }
    int sh = (g & 1) * 16;
    sc_lo = (sc4 >> sh) & 0xff;
    sc_hi = (sc4 >> (sh + 8)) & 0xff;
    m_lo = (m4 >> sh) & 0xff;
    m_hi = (m4 >> (sh + 8)) & 0xff;
}

struct AK45 {   // activations for one Q4_K / Q5_K unit
    u32x4 lo, hi;
    float d8;
    int bs_lo, bs_hi;
};

struct PK45 {   // decoded Q4_K / Q5_K unit
    uint32_t lo[4], hi[4];
    float d, dmin;
    int sc_lo, sc_hi, m_lo, m_hi;
};

__device__ __forceinline__ void load_act_k45(AK45 &a, const ActView &av, int64_t arow, int k, int u) {
    int sb = u >> 3, j = u & 7, g = j >> 1, o = 16 * (j & 1);
    const int8_t *q = av.qs + arow * k + sb * 256 + 64 * g + o;
    a.lo = *reinterpret_cast<const u32x4 *>(q);
    a.hi = *reinterpret_cast<const u32x4 *>(q + 32);
    a.d8 = av.d[arow * (k >> 8) + sb];
    const int16_t *bs = av.bsums + arow * (k >> 4) + sb * 16 + 4 * g + (j & 1);
    a.bs_lo = bs[0];
    a.bs_hi = bs[2];
}

__device__ __forceinline__ float dot_k45(const PK45 &p, const AK45 &a, float acc) {
    int dl = 0, dh = 0;
    dl = sdot4(p.lo[0], a.lo.x, dl); dl = sdot4(p.lo[1], a.lo.y, dl);
    dl = sdot4(p.lo[2], a.lo.z, dl); dl = sdot4(p.lo[3], a.lo.w, dl);
    dh = sdot4(p.hi[0], a.hi.x, dh); dh = sdot4(p.hi[1], a.hi.y, dh);
    dh = sdot4(p.hi[2], a.hi.z, dh); dh = sdot4(p.hi[3], a.hi.w, dh);
    int S = p.sc_lo * dl + p.sc_hi * dh;
    int M = p.m_lo * a.bs_lo + p.m_hi * a.bs_hi;
    acc = fmaf(p.d * a.d8, (float)S, acc);
    acc = fmaf(-(p.dmin * a.d8), (float)M, acc);
    return acc;
}

template <> struct Fmt<CQ_Q4K> {
    static constexpr int UPB = 8;
    struct W { u32x4 hdr, qs; };
    typedef PK45 P;
    typedef AK45 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (int64_t)(u >> 3) * 144;
        w.hdr = *reinterpret_cast<const u32x4 *>(blk);
        w.qs = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * (u & 7));
    }
    static __device__ __forceinline__ void prep(P &p, const W &w, int u) {
        p.d = h2f(w.hdr.x);
        p.dmin = h2f(w.hdr.x >> 16);
        k4_scales(w.hdr.y, w.hdr.z, w.hdr.w, (u & 7) >> 1, p.sc_lo, p.sc_hi, p.m_lo, p.m_hi);
        const uint32_t q[4] = {w.qs.x, w.qs.y, w.qs.z, w.qs.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            p.lo[i] = q[i] & 0x0f0f0f0fu;
            p.hi[i] = (q[i] >> 4) & 0x0f0f0f0fu;
        }
    }
    static __device__ __forceinline__ void load_a(A &a, const ActView &av, int64_t arow, int k, int u) { load_act_k45(a, av, arow, k, u); }
    static __device__ __forceinline__ float dot(const P &p, const A &a, float acc) { return dot_k45(p, a, acc); }
};

template <> struct Fmt<CQ_Q5K> {
    static constexpr int UPB = 8;
    struct W { u32x4 hdr, qh, qs; };
    typedef PK45 P;
    typedef AK45 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (int64_t)(u >> 3) * 176;
        int j = u & 7;
        w.hdr = *reinterpret_cast<const u32x4 *>(blk);
        w.qh = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * (j & 1));
        w.qs = *reinterpret_cast<const u32x4 *>(blk + 48 + 16 * j);
    }
    static __device__ __forceinline__ void prep(P &p, const W &w, int u) {
        int g = (u & 7) >> 1;
        p.d = h2f(w.hdr.x);
        p.dmin = h2f(w.hdr.x >> 16);
        k4_scales(w.hdr.y, w.hdr.z, w.hdr.w, g, p.sc_lo, p.sc_hi, p.m_lo, p.m_hi);
        const uint32_t q[4] = {w.qs.x, w.qs.y, w.qs.z, w.qs.w};
        const uint32_t h[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t hb = h[i] >> (2 * g);
            p.lo[i] = (q[i] & 0x0f0f0f0fu) | ((hb & 0x01010101u) << 4);
            p.hi[i] = ((q[i] >> 4) & 0x0f0f0f0fu) | (((hb >> 1) & 0x01010101u) << 4);
        }
    }
    static __device__ __forceinline__ void load_a(A &a, const ActView &av, int64_t arow, int k, int u) { load_act_k45(a, av, arow, k, u); }
    static __device__ __forceinline__ float dot(const P &p, const A &a, float acc) { return dot_k45(p, a, acc); }
};

template <> struct Fmt<CQ_Q6K> {
    static constexpr int UPB = 4;
    struct W { u32x4 qa, qb, qh; u32x2 sc; uint32_t d; };
    struct P { uint32_t q[4][4]; int sc[4]; float d; };
    struct A { u32x4 a[4]; int bs[4]; float d8; };
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (int64_t)(u >> 2) * 210;
        int h = (u >> 1) & 1, c = u & 1;
        w.qa = ld_u<u32x4>(blk + 64 * h + 16 * c);          // ql[l], l = 16c..16c+15 of this half
        w.qb = ld_u<u32x4>(blk + 64 * h + 32 + 16 * c);     // ql[l + 32]
        w.qh = ld_u<u32x4>(blk + 128 + 32 * h + 16 * c);    // qh[l]
        w.sc = ld_u<u32x2>(blk + 192 + 8 * h);              // the 8 scales of this half
        w.d = ld_u<uint16_t>(blk + 208);
    }
    static __device__ __forceinline__ void prep(P &p, const W &w, int u) {
        int c = u & 1;
        p.d = h2f(w.d);
        // quarter i of the half uses scale index c + 2i (k_quants.rs:2265-2274)
        uint32_t s0 = w.sc.x >> (8 * c), s1 = w.sc.y >> (8 * c);
        p.sc[0] = (int)(int8_t)(s0 & 0xff);
        p.sc[1] = (int)(int8_t)((s0 >> 16) & 0xff);
        p.sc[2] = (int)(int8_t)(s1 & 0xff);
        p.sc[3] = (int)(int8_t)((s1 >> 16) & 0xff);
        const uint32_t a[4] = {w.qa.x, w.qa.y, w.qa.z, w.qa.w};
        const uint32_t b[4] = {w.qb.x, w.qb.y, w.qb.z, w.qb.w};
        const uint32_t h[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {   // unsigned 6-bit values; the -32 is applied through bsums
            p.q[0][i] = (a[i] & 0x0f0f0f0fu) | ((h[i] & 0x03030303u) << 4);
            p.q[1][i] = (b[i] & 0x0f0f0f0fu) | (((h[i] >> 2) & 0x03030303u) << 4);
            p.q[2][i] = ((a[i] >> 4) & 0x0f0f0f0fu) | (((h[i] >> 4) & 0x03030303u) << 4);
            p.q[3][i] = ((b[i] >> 4) & 0x0f0f0f0fu) | (((h[i] >> 6) & 0x03030303u) << 4);
        }
    }
    static __device__ __forceinline__ void load_a(A &a, const ActView &av, int64_t arow, int k, int u) {
        int sb = u >> 2, h = (u >> 1) & 1, c = u & 1;
        const int8_t *q = av.qs + arow * k + sb * 256 + 128 * h + 16 * c;
#pragma unroll
        for (int i = 0; i < 4; i++) a.a[i] = *reinterpret_cast<const u32x4 *>(q + 32 * i);
        // 16-element sums of quarters 0..3 at index 8h + 2i + c
        u32x4 bs = *reinterpret_cast<const u32x4 *>(av.bsums + arow * (k >> 4) + sb * 16 + 8 * h);
        const uint32_t b4[4] = {bs.x, bs.y, bs.z, bs.w};
#pragma unroll
        for (int i = 0; i < 4; i++) a.bs[i] = (int)(int16_t)((b4[i] >> (16 * c)) & 0xffff);
        a.d8 = av.d[arow * (k >> 8) + sb];
    }
    static __device__ __forceinline__ float dot(const P &p, const A &a, float acc) {
        int S = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int dq = -32 * a.bs[i];
            dq = sdot4(p.q[i][0], a.a[i].x, dq); dq = sdot4(p.q[i][1], a.a[i].y, dq);
            dq = sdot4(p.q[i][2], a.a[i].z, dq); dq = sdot4(p.q[i][3], a.a[i].w, dq);
            S += p.sc[i] * dq;
        }
        return fmaf(p.d * a.d8, (float)S, acc);
    }
};

// ---- Q4_0 / Q8_0: one 32-element block per unit, Q8_0-quantized activations ------------------
struct A0 {
    u32x4 a0, a1;
    float d8;
    int s8;
};

__device__ __forceinline__ void load_act_q0(A0 &a, const ActView &av, int64_t arow, int k, int u) {
    const int8_t *q = av.qs + arow * k + u * 32;
    a.a0 = *reinterpret_cast<const u32x4 *>(q);
    a.a1 = *reinterpret_cast<const u32x4 *>(q + 16);
    u32x2 ds = *reinterpret_cast<const u32x2 *>(av.d + 2 * (arow * (k >> 5) + u));
    a.d8 = __uint_as_float(ds.x);
    a.s8 = (int)ds.y;
}

template <> struct Fmt<CQ_Q4_0> {
    static constexpr int UPB = 1;
    struct W { u32x4 qs; uint32_t d; };
    struct P { uint32_t lo[4], hi[4]; float d; };
    typedef A0 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (int64_t)u * 18;
        w.d = ld_u<uint16_t>(blk);
        w.qs = ld_u<u32x4>(blk + 2);
    }
    static __device__ __forceinline__ void prep(P &p, const W &w, int) {
        p.d = h2f(w.d);
        const uint32_t q[4] = {w.qs.x, w.qs.y, w.qs.z, w.qs.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            p.lo[i] = q[i] & 0x0f0f0f0fu;          // elements 4i..4i+3
            p.hi[i] = (q[i] >> 4) & 0x0f0f0f0fu;   // elements 16+4i..
        }
    }
    static __device__ __forceinline__ void load_a(A &a, const ActView &av, int64_t arow, int k, int u) { load_act_q0(a, av, arow, k, u); }
    static __device__ __forceinline__ float dot(const P &p, const A &a, float acc) {
        int s = -8 * a.s8;    // sum((q - 8) * y) = sum(q * y) - 8 * sum(y)
        s = sdot4(p.lo[0], a.a0.x, s); s = sdot4(p.lo[1], a.a0.y, s);
        s = sdot4(p.lo[2], a.a0.z, s); s = sdot4(p.lo[3], a.a0.w, s);
        s = sdot4(p.hi[0], a.a1.x, s); s = sdot4(p.hi[1], a.a1.y, s);
        s = sdot4(p.hi[2], a.a1.z, s); s = sdot4(p.hi[3], a.a1.w, s);
        return acc + (float)s * p.d * a.d8;
    }
};

template <> struct Fmt<CQ_Q8_0> {
    static constexpr int UPB = 1;
    struct W { u32x4 q0, q1; uint32_t d; };
    struct P { u32x4 q0, q1; float d; };
    typedef A0 A;
    static __device__ __forceinline__ void load_w(W &w, const uint8_t *row, int u) {
        const uint8_t *blk = row + (int64_t)u * 34;
        w.d = ld_u<uint16_t>(blk);
        w.q0 = ld_u<u32x4>(blk + 2);
        w.q1 = ld_u<u32x4>(blk + 18);
    }
    static __device__ __forceinline__ void prep(P &p, const W &w, int) {
        p.d = h2f(w.d);
        p.q0 = w.q0;
        p.q1 = w.q1;
    }
    static __device__ __forceinline__ void load_a(A &a, const ActView &av, int64_t arow, int k, int u) { load_act_q0(a, av, arow, k, u); }
    static __device__ __forceinline__ float dot(const P &p, const A &a, float acc) {
        int s = 0;
        s = sdot4(p.q0.x, a.a0.x, s); s = sdot4(p.q0.y, a.a0.y, s);
        s = sdot4(p.q0.z, a.a0.z, s); s = sdot4(p.q0.w, a.a0.w, s);
        s = sdot4(p.q1.x, a.a1.x, s); s = sdot4(p.q1.y, a.a1.y, s);
        s = sdot4(p.q1.z, a.a1.z, s); s = sdot4(p.q1.w, a.a1.w, s);
        return acc + (float)s * p.d * a.d8;
    }
};

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
