// Prefill matmul over pre-quantized activations for gfx950 (MFMA), and the f32 -> f16/bf16 output
// conversion.   dst[m, n] = sum_k x^[m, k] * W^[n, k]
//
// Counterpart of candle's tensor-core MMQ path (candle-core/src/quantized/fast_mmq.rs:253-400,
// candle-kernels/src/mmq_gguf/).  The arithmetic follows the CPU path instead of the CUDA one:
// activations are the Q8_K / Q8_0 quantization written by cq_quantize_act.
//
// Q5_K, Q6_K, Q2_K, Q3_K — integer-exact formulation on the f16 matrix cores (qmm_kernel):
//   per 256-element super-block kb      S[m,n] = sum_k q8[m,k] * (sc[n,sub(k)] * q[n,k])
//   operands are small integers held exactly in f16 (|q8| <= 128, |sc*q| <= 1953 for Q5_K),
//   products accumulate in f32, and once per super-block
//       acc[m,n] += d8[m,kb] * ( d[n,kb] * S[m,n] - dmin[n,kb] * M[m,n] ),
//       M[m,n] = sum_{j<16} bsums16[m,j] * min[n, group j]     (one extra K=16 MFMA; Q5_K: min of sub-block j / 2, Q2_K: of group j)
//   — the same integers the CPU vec_dot sums (k_quants.rs:1714-1801, 2035-2092).  For Q6_K
//   the product sc*(q-32) can reach 4096, beyond the exact-integer range of f16, so it is fed as two
//   terms: its f16 rounding and the exact remainder in {-1, 0, 1} (a second MFMA per k-slice).  This
//   matters: a 1e-4 perturbation of one matmul is amplified to ~1e-2 in a decoder's logits by the
//   activation quantizers downstream, an exact one is not.
// Q4_K — the same sums on the int8 matrix cores (qmm_q4k_i8_kernel, k_quants.rs:1460-1540): the 6-bit sub-block scale
//   is split into two 3-bit halves so that scale * weight fits int8; S is exact in int32.
// Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 — the per-32 sums of the CPU vec_dot (k_quants.rs:294-311, 720-738, 323-351,
//   434-455, 530-562) on the int8 matrix cores (qmm_q0_i8_kernel): one v_mfma_i32_32x32x32_i8 per 32-element block gives
//   the exact int32 sum of q8 * q (q - 8, q - 16 for Q4_0, Q5_0), and the vector units add
//   (float(S) * d[n, block]) * d8[m, block]  (+ m[n, block] * s[m, block] for Q4_1 / Q5_1)  block by block, in the CPU's order.
//
// Tiling: workgroup = 4 waves (2 x 2), block tile 128 (m) x 64 (n), wave tile 64 x 32 as 2 x 1 MFMA tiles of 32 x 32
// (128 x 128 / 64 x 64 for large Q4_0 / Q8_0 problems, 32 x 128 with the waves side by side for up to 32 rows).
// qmm_kernel advances K by 64 elements per LDS stage: the threads dequantize the weight tile and convert the 128 x 64 int8
// activation tile to f16 into one of two LDS copies (row stride padded to 144 bytes) while the MFMAs run on the other;
// raw bytes are requested two stages ahead into two register sets.
#include "cq_device.h"
#include "cq_fmt.h"
#include "cq_launch.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BK = 64;
constexpr int CQ_QMM_SMALL_ROWS = 32;      // up to here the 32-row block tile is used (measured, 14336 x 4096 Q4_K: 16 / 32 rows
                                           // 37 / 38 us against 62 us on the 128-row tile; 64 rows as two tiles 73 us)
constexpr int LDK = BK + 8;            // padded row stride in halves (144 bytes)

// ---- integer bytes -> f16 pairs ------------------------------------------------------------------
// bytes b0..b3 of `x` (values 0..255) -> two dwords of f16 pairs holding (1024 + b) exactly:
// the f16 bit pattern 0x6400 | b is 1024 + b for b < 1024.
__device__ __forceinline__ void bytes_to_h1024(uint32_t x, uint32_t &lo, uint32_t &hi) {
    lo = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);   // [b0, 0x64, b1, 0x64]
    hi = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);   // [b2, 0x64, b3, 0x64]
}
__device__ __forceinline__ uint32_t pk_fma(uint32_t a, uint32_t b, uint32_t c) {
    half2v r = __builtin_elementwise_fma(__builtin_bit_cast(half2v, a), __builtin_bit_cast(half2v, b), __builtin_bit_cast(half2v, c));
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_add(uint32_t a, uint32_t b) {
    half2v r = __builtin_bit_cast(half2v, a) + __builtin_bit_cast(half2v, b);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_mul(uint32_t a, uint32_t b) {
    half2v r = __builtin_bit_cast(half2v, a) * __builtin_bit_cast(half2v, b);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t h2_splat(float v) {          // v exactly representable in f16
    uint32_t h = f2h_bits(v);
    return h | (h << 16);
}

// 6-bit scale / min of sub-block j (utils.rs:50-60) from the 12 packed bytes held in three dwords
__device__ __forceinline__ void k4_sub_scale_min(uint32_t u0, uint32_t u1, uint32_t u2, int j, int &sc, int &mn) {
    int sh = 8 * (j & 3);
    if (j < 4) {
        sc = (u0 >> sh) & 63;
        mn = (u1 >> sh) & 63;
    } else {
        sc = ((u2 >> sh) & 0xF) | (((u0 >> sh) >> 6 & 3) << 4);
        mn = ((u2 >> sh) >> 4 & 0xF) | (((u1 >> sh) >> 6 & 3) << 4);
    }
}

// ---- per-format staging of NW = 32 or 16 consecutive weights of one row into NW / 2 dwords of f16 pairs -------
// A 64-element stage (kb, g) of a row is split between 64 / NW threads; thread `part` takes elements
// 256 kb + 64 g + NW part + [0, NW).  jh = the 32-element half of the stage these lie in, sx = which 16 of that half
// (NW = 16 only).  Raw<NW>: what the thread loads for them.
template <int DT> struct Stage;

template <> struct Stage<CQ_Q5K> {
    static constexpr bool HAS_MIN = true;
    static constexpr int TERMS = 1;
    template <int NW> struct Raw { u32x4 hdr, h[NW / 16], q[NW / 16]; };
    template <int NW> static __device__ __forceinline__ void load(Raw<NW> &r, const uint8_t *row, int kb, int g, int part) {
        const uint8_t *blk = row + (int64_t)kb * 176;
        const int sx = NW == 16 ? part & 1 : 0;
        r.hdr = *reinterpret_cast<const u32x4 *>(blk);
#pragma unroll
        for (int i = 0; i < NW / 16; i++) {
            r.h[i] = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * (sx + i));
            r.q[i] = *reinterpret_cast<const u32x4 *>(blk + 48 + 32 * g + 16 * (sx + i));
        }
    }
    template <int NW> static __device__ __forceinline__ void header(const Raw<NW> &r, float &d, float &dmin) {
        d = h2f(r.hdr.x);
        dmin = h2f(r.hdr.x >> 16);
    }
    // the mins of the 16-element groups 2 jp and 2 jp + 1 in bits 0-7 and 16-23: both the min of sub-block jp (utils.rs:50-60)
    template <int NW> static __device__ __forceinline__ uint32_t min_pair(const Raw<NW> &r, int jp) {
        const uint32_t m4 = jp >= 4 ? ((r.hdr.w >> 4) & 0x0f0f0f0fu) | ((r.hdr.z >> 2) & 0x30303030u) : r.hdr.z & 0x3f3f3f3fu;
        return ((m4 >> (8 * (jp & 3))) & 0xffu) * 0x00010001u;
    }
    template <int NW> static __device__ __forceinline__ void convert(const Raw<NW> &r, int g, int part, uint32_t out[NW / 2]) {
        const int jh = NW == 16 ? part >> 1 : part;
        int sc, mn;
        k4_sub_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * g + jh, sc, mn);
        const uint32_t s2 = h2_splat((float)sc), c2 = h2_splat(-1024.0f * (float)sc);
#pragma unroll
        for (int i = 0; i < NW / 4; i++) {
            const uint32_t hb = (r.h[i >> 2][i & 3] >> (2 * g + jh)) & 0x01010101u;
            const uint32_t v = ((r.q[i >> 2][i & 3] >> (4 * jh)) & 0x0f0f0f0fu) | (hb << 4);
            uint32_t lo, hi;
            bytes_to_h1024(v, lo, hi);
            out[2 * i] = pk_fma(lo, s2, c2);        // (1024 + q) * sc - 1024 * sc = sc * q, one exact rounding
            out[2 * i + 1] = pk_fma(hi, s2, c2);
        }
    }
};

template <> struct Stage<CQ_Q6K> {
    static constexpr bool HAS_MIN = false;
    static constexpr int TERMS = 2;      // sc * (q - 32) reaches 4096: f16 head + exact remainder in {-1, 0, 1}
    // 32-element half (g, jh) = elements 64g + 32jh + [0, 32): half h6 = g >> 1 of the block, quarter = 2*(g&1) + jh
    template <int NW> struct Raw { u32x4 l[NW / 16], h[NW / 16]; uint32_t sc, d; };
    template <int NW> static __device__ __forceinline__ void load(Raw<NW> &r, const uint8_t *row, int kb, int g, int part) {
        const uint8_t *blk = row + (int64_t)kb * 210;
        const int jh = NW == 16 ? part >> 1 : part, sx = NW == 16 ? part & 1 : 0;
        const int h6 = g >> 1, quarter = 2 * (g & 1) + jh;
        const uint8_t *ql = blk + 64 * h6 + ((quarter & 1) ? 32 : 0);   // ql[l] or ql[l + 32], l = 0..31
#pragma unroll
        for (int i = 0; i < NW / 16; i++) {
            r.l[i] = ld_u<u32x4>(ql + 16 * (sx + i));
            r.h[i] = ld_u<u32x4>(blk + 128 + 32 * h6 + 16 * (sx + i));
        }
        // scales of this quarter: index 8*h6 + 2*quarter + l / 16
        if (NW == 16) r.sc = blk[192 + 8 * h6 + 2 * quarter + sx];
        else r.sc = ld_u<uint16_t>(blk + 192 + 8 * h6 + 2 * quarter);
        r.d = ld_u<uint16_t>(blk + 208);
    }
    template <int NW> static __device__ __forceinline__ void header(const Raw<NW> &r, float &d, float &dmin) {
        d = h2f(r.d);
        dmin = 0.0f;
    }
    template <int NW> static __device__ __forceinline__ uint32_t min_pair(const Raw<NW> &, int) { return 0; }
    // out = f16(sc * (q - 32)) (rounds odd products above 2048 to even), rem = sc * (q - 32) - out exactly
    template <int NW>
    static __device__ __forceinline__ void convert2(const Raw<NW> &r, int g, int part, uint32_t out[NW / 2], uint32_t rem[NW / 2]) {
        const int jh = NW == 16 ? part >> 1 : part;
        const int quarter = 2 * (g & 1) + jh;
        const uint32_t sA = h2_splat((float)(int8_t)(r.sc & 0xff)), sB = h2_splat((float)(int8_t)((r.sc >> 8) & 0xff));
        const uint32_t off = h2_splat(-1056.0f);                       // -(1024 + 32)
#pragma unroll
        for (int i = 0; i < NW / 4; i++) {
            const uint32_t lw = r.l[i >> 2][i & 3], hw = r.h[i >> 2][i & 3];
            uint32_t lo4 = (lw >> (quarter >= 2 ? 4 : 0)) & 0x0f0f0f0fu;
            uint32_t hi2 = ((hw >> (2 * quarter)) & 0x03030303u) << 4;
            uint32_t lo, hi;
            bytes_to_h1024(lo4 | hi2, lo, hi);
            const uint32_t s2 = i < 4 ? sA : sB;                         // l / 16
            const uint32_t a = pk_add(lo, off), b = pk_add(hi, off);     // q - 32, exact
            const uint32_t pa = pk_mul(a, s2), pb = pk_mul(b, s2);
            out[2 * i] = pa;
            out[2 * i + 1] = pb;
            rem[2 * i] = pk_fma(a, s2, pa ^ 0x80008000u);                // exact product minus its f16 rounding
            rem[2 * i + 1] = pk_fma(b, s2, pb ^ 0x80008000u);
        }
    }
};

// Q2_K / Q3_K: element 128 h + 32 s + 16 c + i of a super-block is bit pair s of qs[32 h + 16 c + i] (Q3_K: plus bit 4 h + s of
// hmask[16 c + i]), its 16-element group is 8 h + 2 s + c (k_quants.rs:1013-1049, 1369-1421).  Stage (kb, g), 32-element half jh:
// h = g >> 1, s = 2 (g & 1) + jh.  Both products are small exact integers in f16: sc * q <= 45, (sc - 32) * (q - 4) within +-128.
template <> struct Stage<CQ_Q2K> {
    static constexpr bool HAS_MIN = true;
    static constexpr int TERMS = 1;
    template <int NW> struct Raw { u32x4 sc, q[NW / 16]; uint32_t dd; };
    template <int NW> static __device__ __forceinline__ void load(Raw<NW> &r, const uint8_t *row, int kb, int g, int part) {
        const uint8_t *blk = row + (int64_t)kb * 84;
        const int sx = NW == 16 ? part & 1 : 0;
        r.sc = ld_u<u32x4>(blk);
#pragma unroll
        for (int i = 0; i < NW / 16; i++) r.q[i] = ld_u<u32x4>(blk + 16 + 32 * (g >> 1) + 16 * (sx + i));
        r.dd = ld_u<uint32_t>(blk + 80);
    }
    template <int NW> static __device__ __forceinline__ void header(const Raw<NW> &r, float &d, float &dmin) {
        d = h2f(r.dd);
        dmin = h2f(r.dd >> 16);
    }
    // mins (high nibbles of the scale bytes) of the 16-element groups 2 jp and 2 jp + 1, in bits 0-7 and 16-23
    template <int NW> static __device__ __forceinline__ uint32_t min_pair(const Raw<NW> &r, int jp) {
        const uint32_t two = (r.sc[jp >> 1] >> (16 * (jp & 1))) & 0xffffu;      // scale bytes 2 jp, 2 jp + 1
        return ((two >> 4) & 0xfu) | ((two >> 12) << 16);
    }
    template <int NW> static __device__ __forceinline__ void convert(const Raw<NW> &r, int g, int part, uint32_t out[NW / 2]) {
        const int jh = NW == 16 ? part >> 1 : part, sx = NW == 16 ? part & 1 : 0;
        const int s = 2 * (g & 1) + jh, grp = 8 * (g >> 1) + 2 * s + sx;      // first 16-element group of this thread's weights
#pragma unroll
        for (int i = 0; i < NW / 4; i++) {
            const int gi = grp + (i >> 2);
            const float sc = (float)((r.sc[gi >> 2] >> (8 * (gi & 3))) & 0xfu);
            const uint32_t s2 = h2_splat(sc), c2 = h2_splat(-1024.0f * sc);
            uint32_t lo, hi;
            bytes_to_h1024((r.q[i >> 2][i & 3] >> (2 * s)) & 0x03030303u, lo, hi);
            out[2 * i] = pk_fma(lo, s2, c2);        // (1024 + q) * sc - 1024 * sc = sc * q, one exact rounding
            out[2 * i + 1] = pk_fma(hi, s2, c2);
        }
    }
};

template <> struct Stage<CQ_Q3K> {
    static constexpr bool HAS_MIN = false;
    static constexpr int TERMS = 1;
    template <int NW> struct Raw { u32x4 q[NW / 16], hm[NW / 16]; uint32_t s0, s1, s2, d; };
    template <int NW> static __device__ __forceinline__ void load(Raw<NW> &r, const uint8_t *row, int kb, int g, int part) {
        const uint8_t *blk = row + (int64_t)kb * 110;
        const int sx = NW == 16 ? part & 1 : 0;
#pragma unroll
        for (int i = 0; i < NW / 16; i++) {
            r.hm[i] = ld_u<u32x4>(blk + 16 * (sx + i));
            r.q[i] = ld_u<u32x4>(blk + 32 + 32 * (g >> 1) + 16 * (sx + i));
        }
        r.s0 = ld_u<uint32_t>(blk + 96);
        r.s1 = ld_u<uint32_t>(blk + 100);
        r.s2 = ld_u<uint32_t>(blk + 104);
        r.d = ld_u<uint16_t>(blk + 108);
    }
    template <int NW> static __device__ __forceinline__ void header(const Raw<NW> &r, float &d, float &dmin) {
        d = h2f(r.d);
        dmin = 0.0f;
    }
    template <int NW> static __device__ __forceinline__ uint32_t min_pair(const Raw<NW> &, int) { return 0; }
    template <int NW> static __device__ __forceinline__ void convert(const Raw<NW> &r, int g, int part, uint32_t out[NW / 2]) {
        const int jh = NW == 16 ? part >> 1 : part, sx = NW == 16 ? part & 1 : 0;
        const int h = g >> 1, s = 2 * (g & 1) + jh;
        // the eight 6-bit scales of half h, one per byte of (e0, e1) (k_quants.rs:1148-1156)
        const uint32_t t2 = r.s2 >> (4 * h);
        const uint32_t e0 = ((r.s0 >> (4 * h)) & 0x0f0f0f0fu) | ((t2 & 0x03030303u) << 4);
        const uint32_t e1 = ((r.s1 >> (4 * h)) & 0x0f0f0f0fu) | (((t2 >> 2) & 0x03030303u) << 4);
        const uint32_t off = h2_splat(-1028.0f);                               // -(1024 + 4)
#pragma unroll
        for (int i = 0; i < NW / 4; i++) {
            const int gi = 2 * s + sx + (i >> 2);                               // 16-element group within the half, 0..7
            const int sc = (int)(((gi < 4 ? e0 : e1) >> (8 * (gi & 3))) & 0xffu) - 32;
            const uint32_t s2 = h2_splat((float)sc);
            const uint32_t v = ((r.q[i >> 2][i & 3] >> (2 * s)) & 0x03030303u) | (((r.hm[i >> 2][i & 3] >> (4 * h + s)) & 0x01010101u) << 2);
            uint32_t lo, hi;
            bytes_to_h1024(v, lo, hi);
            out[2 * i] = pk_mul(pk_add(lo, off), s2);                           // (q - 4) * (sc - 32), exact
            out[2 * i + 1] = pk_mul(pk_add(hi, off), s2);
        }
    }
};

// 32 int8 activations -> 16 dwords of f16 pairs holding the same integers
__device__ __forceinline__ void act_convert(const u32x4 &a0, const u32x4 &a1, uint32_t out[16]) {
    const uint32_t off = 0xe480e480u;    // two f16 -1152.0
    const uint32_t q[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t lo, hi;
        bytes_to_h1024(q[i] ^ 0x80808080u, lo, hi);
        out[2 * i] = pk_add(lo, off);
        out[2 * i + 1] = pk_add(hi, off);
    }
}

// NH halves (NH / 2 dwords of f16 pairs) to a 16-byte aligned LDS address
template <int NH> __device__ __forceinline__ void lds_write_h(_Float16 *dstrow, const uint32_t *v) {
    u32x4 *p = reinterpret_cast<u32x4 *>(dstrow);
#pragma unroll
    for (int i = 0; i < NH / 8; i++) p[i] = u32x4{v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
}

// NJ = 32-column MFMA tiles per wave: block tile 128 x (64 * NJ).  NJ = 1 halves the accumulators so that two
// workgroups share a CU and one converts operands while the other feeds the matrix cores.
// MOE: blockIdx.x is a tile of the chunk table: up to BMT expert-sorted activation rows [first, first + count) of
// expert e; the weights are that expert's [n, k] matrix and output rows are scattered through pair_out with pair_scale.
// SM (experts with few rows each): the block tile is 32 (m) x 128 (n) (one workgroup per CU for a two-term format, whose
// two weight tiles fill the LDS), the four waves side by side along n, so that a
// 16-row expert fills half of its tiles instead of an eighth, and one workgroup converts twice the weight rows per stage.
template <int DT, int NJ, bool MOE = false, bool SM = false>
__global__ __launch_bounds__(256, NJ == 1 && !(SM && Stage<DT>::TERMS == 2) ? 2 : 1) void qmm_kernel(const uint8_t *__restrict__ w, ActView av, float *__restrict__ dst, int k,
                                                                     int n, int rows, int64_t stride_dst, MoeChunks mc, int64_t expert_bytes,
                                                                     int64_t split_stride) {
    typedef Stage<DT> S;
    static_assert(!SM || NJ == 1, "the small-m tile has one 32-column MFMA tile per wave");
    constexpr int BMT = SM ? 32 : BM, MI = SM ? 1 : 2;             // rows of the block tile, 32-row MFMA tiles per wave
    constexpr int BN = SM ? 128 : 64 * NJ, WN = 32 * NJ;
    // every LDS array exists twice: while the matrix cores work on one stage, the threads convert the next one into
    // the other copy (one barrier per stage); the per-super-block arrays alternate with the super-block
    constexpr int NMIN = S::HAS_MIN ? 24 : 0;
    __shared__ __align__(16) _Float16 As[2][BMT * LDK];
    __shared__ __align__(16) _Float16 Bs[2][BN * LDK];
    __shared__ __align__(16) _Float16 Bs2[2][S::TERMS == 2 ? BN * LDK : 8];   // exact remainders of a two-term format
    __shared__ __align__(16) _Float16 Am[2][BMT * NMIN + 8];   // bsums16 of the super-block, as f16 (row stride 24 halves)
    __shared__ __align__(16) _Float16 Bm[2][BN * NMIN + 8];    // sub-block mins duplicated per 16-element group
    __shared__ float sD[2][BN], sDmin[2][BN], sD8[2][BMT];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = SM ? 0 : wv >> 1, wn = SM ? wv : wv & 1;
    int m0 = blockIdx.x * BMT;
    const int n0 = blockIdx.y * BN;
    if (MOE) {
        if ((int)blockIdx.x >= mc.n_chunks[0]) return;           // uniform over the workgroup
        m0 = mc.first[blockIdx.x];
        rows = m0 + mc.count[blockIdx.x];
        w += (int64_t)mc.expert[blockIdx.x] * expert_bytes;
    }
    // every thread stages NW = 64 / TPR weights of one row per stage (16 when the tile has 64 weight rows, else 32), so
    // that all waves carry the same conversion work and the loop body has no wave-dependent branch
    constexpr int TPR = 256 / BN, NW = 64 / TPR;
    static_assert(TPR == 2 || TPR == 4, "weight rows of the block tile");
    const bool astage = SM ? tid < 2 * BMT : true;               // threads that stage an activation row (wave-uniform)
    // split-K: blockIdx.z takes an equal share of the 256-element spans and writes its own partial plane
    const int nsb_all = k >> 8;
    const int kb0 = (int)(((int64_t)nsb_all * blockIdx.z) / gridDim.z), nsb = (int)(((int64_t)nsb_all * (blockIdx.z + 1)) / gridDim.z);
    dst += (int64_t)blockIdx.z * split_stride;
    const int64_t row_bytes = (int64_t)(k / BlockInfo<DT>::elems) * BlockInfo<DT>::bytes;

    // staging roles of this thread: activations (row r_l of the tile, 32-element half), weights (row r_w, part of NW)
    const int r_l = tid >> 1, half = tid & 1;
    const int r_w = tid / TPR, part = tid % TPR;
    const int wrow = min(n0 + r_w, n - 1);
    const int arow = min(m0 + (astage ? r_l : 0), rows - 1);
    const bool arow_ok = astage && m0 + r_l < rows;
    const uint32_t amask = arow_ok ? 0xffffffffu : 0u;
    const uint8_t *wrow_p = w + wrow * row_bytes;
    const int8_t *aq_p = av.qs + (int64_t)arow * k;

    f32x16 acc[MI][NJ], sb[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) { acc[i][j][e] = 0.0f; sb[i][j][e] = 0.0f; }

    // Raw bytes are requested two stages ahead (two register sets, chosen by the parity of the stage): one stage of
    // conversion + MFMA work is shorter than a trip to memory.  Stage (kb, g) covers k = 256 kb + 64 g + [0, 64).
    // Positions past the end of this split's range are clamped to its last super-block: what they load and convert
    // lands in LDS copies nobody reads.
    typedef typename S::template Raw<NW> WRaw;
    WRaw wraw2[2];
    u32x4 a02[2], a12[2], abs0 = u32x4{0, 0, 0, 0};
    float ad8[2] = {0.0f, 0.0f};
    auto load_stage = [&](int kb, int g, WRaw &wr, u32x4 &x0, u32x4 &x1, float &d8) {
        kb = min(kb, nsb - 1);
        S::template load<NW>(wr, wrow_p, kb, g, part);
        if (astage) {
            const int8_t *q = aq_p + kb * 256 + 64 * g + 32 * half;
            x0 = *reinterpret_cast<const u32x4 *>(q);
            x1 = *reinterpret_cast<const u32x4 *>(q + 16);
            if (g == 0) {
                d8 = av.d[(int64_t)arow * (k >> 8) + kb];
                if (S::HAS_MIN) abs0 = *reinterpret_cast<const u32x4 *>(av.bsums + (int64_t)arow * (k >> 4) + kb * 16 + 8 * half);
            }
        }
    };
    // what one thread contributes to the LDS image of a stage
    struct Conv {
        uint32_t w[NW / 2], w2[S::TERMS == 2 ? NW / 2 : 1], a[16];
        float d, dmin, d8;
        uint32_t mv[8 / TPR], bv[4];
    };
    auto convert_stage = [&](int g, const WRaw &wraw, const u32x4 &a0, const u32x4 &a1, float d8, Conv &c) {
        if constexpr (S::TERMS == 2) S::template convert2<NW>(wraw, g, part, c.w, c.w2);
        else S::template convert<NW>(wraw, g, part, c.w);
        if (astage) {
            act_convert(a0, a1, c.a);
#pragma unroll
            for (int i = 0; i < 16; i++) c.a[i] &= amask;        // rows past the end contribute zeros (no branch)
        }
        if (g == 0) {
            S::template header<NW>(wraw, c.d, c.dmin);
            c.d8 = arow_ok ? d8 : 0.0f;
            if (S::HAS_MIN) {
                // Bm[n][j] = min of the 16-element group j, this thread's share j = 2 ((8 / TPR) part + i) + {0, 1}; Am[m][j] = bsums16[j]
#pragma unroll
                for (int i = 0; i < 8 / TPR; i++)
                    c.mv[i] = pk_add(0x64006400u | S::template min_pair<NW>(wraw, (8 / TPR) * part + i), 0xe400e400u);   // (1024 + min) - 1024
                const uint32_t b4[4] = {abs0.x, abs0.y, abs0.z, abs0.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t lo = f2h_bits((float)(int16_t)(b4[i] & 0xffff)), hi = f2h_bits((float)(int16_t)(b4[i] >> 16));
                    c.bv[i] = arow_ok ? (lo | (hi << 16)) : 0u;
                }
            }
        }
    };
    // buf: LDS copy of the stage (its parity); hb: copy of the per-super-block arrays (parity of the super-block)
    auto store_stage = [&](int g, int buf, int hb, const Conv &c) {
        if constexpr (S::TERMS == 2) lds_write_h<NW>(Bs2[buf] + r_w * LDK + NW * part, c.w2);
        lds_write_h<NW>(Bs[buf] + r_w * LDK + NW * part, c.w);
        if (astage) lds_write_h<32>(As[buf] + r_l * LDK + 32 * half, c.a);
        if (g == 0) {
            // the threads of a row hold the same values: all of them write (no branch)
            sD[hb][r_w] = c.d; sDmin[hb][r_w] = c.dmin;
            if (astage) sD8[hb][r_l] = c.d8;
            if (S::HAS_MIN) {
                if constexpr (TPR == 2)
                    *reinterpret_cast<u32x4 *>(Bm[hb] + r_w * 24 + 8 * part) = u32x4{c.mv[0], c.mv[1], c.mv[2], c.mv[3]};
                else
                    *reinterpret_cast<uint2 *>(Bm[hb] + r_w * 24 + 4 * part) = uint2{c.mv[0], c.mv[1]};
                if (astage) *reinterpret_cast<u32x4 *>(Am[hb] + r_l * 24 + 8 * half) = u32x4{c.bv[0], c.bv[1], c.bv[2], c.bv[3]};
            }
        }
    };
    load_stage(kb0, 0, wraw2[0], a02[0], a12[0], ad8[0]);
    load_stage(kb0, 1, wraw2[1], a02[1], a12[1], ad8[1]);
    {
        Conv c;
        convert_stage(0, wraw2[0], a02[0], a12[0], ad8[0], c);
        store_stage(0, 0, kb0 & 1, c);
        load_stage(kb0, 2, wraw2[0], a02[0], a12[0], ad8[0]);
    }
    __syncthreads();

    for (int kb = kb0; kb < nsb; kb++) {
        const int hb = kb & 1;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            // ---- the next stage is converted in registers while the MFMAs of this one are in flight ----
            const int ng = (g + 1) & 3, nb = (g + 1) & 1;
            Conv c;
            convert_stage(ng, wraw2[nb], a02[nb], a12[nb], ad8[nb], c);
            // its register set is refilled with the stage two further on
            load_stage(g == 0 ? kb : kb + 1, (g + 3) & 3, wraw2[nb], a02[nb], a12[nb], ad8[nb]);
            // ---- 4 k-slices of 16: MI x NJ MFMA tiles per wave ----
            const _Float16 *Ab = As[g & 1], *Bb = Bs[g & 1], *Bb2 = Bs2[g & 1];
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                half8 af[MI], bf[NJ];
#pragma unroll
                for (int t = 0; t < MI; t++)
                    af[t] = *reinterpret_cast<const half8 *>(Ab + (wm * 64 + t * 32 + (lane & 31)) * LDK + ks * 16 + 8 * (lane >> 5));
#pragma unroll
                for (int t = 0; t < NJ; t++)
                    bf[t] = *reinterpret_cast<const half8 *>(Bb + (wn * WN + t * 32 + (lane & 31)) * LDK + ks * 16 + 8 * (lane >> 5));
#pragma unroll
                for (int i = 0; i < MI; i++)
#pragma unroll
                    for (int j = 0; j < NJ; j++) sb[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], sb[i][j], 0, 0, 0);
                if constexpr (S::TERMS == 2) {
#pragma unroll
                    for (int t = 0; t < NJ; t++)
                        bf[t] = *reinterpret_cast<const half8 *>(Bb2 + (wn * WN + t * 32 + (lane & 31)) * LDK + ks * 16 + 8 * (lane >> 5));
#pragma unroll
                    for (int i = 0; i < MI; i++)
#pragma unroll
                        for (int j = 0; j < NJ; j++) sb[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], sb[i][j], 0, 0, 0);
                }
            }
            store_stage(ng, nb, g == 3 ? hb ^ 1 : hb, c);
            if (g == 3) {
                // ---- end of the super-block: mins term and the f32 scales ----
                f32x16 mt[MI][NJ];
                if (S::HAS_MIN) {
                    half8 am[MI], bm[NJ];
#pragma unroll
                    for (int t = 0; t < MI; t++)
                        am[t] = *reinterpret_cast<const half8 *>(Am[hb] + (wm * 64 + t * 32 + (lane & 31)) * 24 + 8 * (lane >> 5));
#pragma unroll
                    for (int t = 0; t < NJ; t++)
                        bm[t] = *reinterpret_cast<const half8 *>(Bm[hb] + (wn * WN + t * 32 + (lane & 31)) * 24 + 8 * (lane >> 5));
#pragma unroll
                    for (int i = 0; i < MI; i++)
#pragma unroll
                        for (int j = 0; j < NJ; j++) {
                            f32x16 z;
#pragma unroll
                            for (int e = 0; e < 16; e++) z[e] = 0.0f;
                            mt[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(am[i], bm[j], z, 0, 0, 0);
                        }
                }
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    const int nl = wn * WN + j * 32 + (lane & 31);
                    const float d = sD[hb][nl], dmin = sDmin[hb][nl];
#pragma unroll
                    for (int i = 0; i < MI; i++) {
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            const int ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                            float t = d * sb[i][j][e];
                            if (S::HAS_MIN) t = fmaf(-dmin, mt[i][j][e], t);
                            acc[i][j][e] = fmaf(sD8[hb][ml], t, acc[i][j][e]);
                            sb[i][j][e] = 0.0f;
                        }
                    }
                }
            }
            __syncthreads();
        }
    }

    // ---- epilogue: C layout of the 32x32 tile: column = lane % 32, row = 8*(e/4) + 4*(lane/32) + e%4 ----
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int nn = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int mm = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                const float v = acc[i][j][e];
                if (mm < rows && nn < n) {
                    if (MOE) dst[(int64_t)mc.pair_out[mm] * stride_dst + nn] = v * mc.pair_scale[mm];
                    else dst[(int64_t)mm * stride_dst + nn] = v;
                }
            }
        }
}

// ---- Q4_K on the int8 matrix cores ----------------------------------------------------------------------------------
// The 6-bit sub-block scale is split as sc = 8 hi + lo (hi, lo < 8): lo * q and hi * q stay below 128, so they are int8
// operands, and     S[m,n] = sum_k q8[m,k] * sc * q[n,k] = 8 * sum_k q8 (hi q) + sum_k q8 (lo q)
// is two v_mfma_i32_32x32x32_i8 chains with exact int32 sums over the super-block — the integer the CPU vec_dot forms
// (k_quants.rs:1460-1540) — followed by the same f32 step as above: acc += d8 * (d * S - dmin * M).  Against the f16
// formulation: the activations go to LDS as the raw int8 (no conversion, half the bytes), four weights take one
// v_pk_mul_lo_u16 per term, and a k-slice of 32 needs as many LDS bytes as a k-slice of 16 did.
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_mul_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, (u16x2)(__builtin_bit_cast(u16x2, a) * __builtin_bit_cast(u16x2, b)));
}

// Same tiling and template parameters as qmm_kernel; a stage is 128 elements of k (half a super-block), held twice in
// LDS: while the matrix cores work on one copy the threads fill the other (one barrier per stage).  What goes through
// LDS is raw: the int8 activations, and the weight rows' packed nibbles and 16-byte headers as they lie in memory, both
// copied with fully used cache lines (8 lanes per 128-byte activation row, 4 per 64-byte weight row) because the
// address path of the vector cache, not the matrix cores, is what the tile loads saturate first.  Each lane then builds
// its own MFMA B operands: lane (n, kg) of a 32 x 32 x 32 MFMA wants 16 consecutive k of row n, which for Q4_K are the
// nibbles of one 16-byte piece — low nibbles for the even sub-block of a 64-element pair, high nibbles for the odd
// one — times the two halves of the sub-block scale.  16-byte pieces are XOR-swizzled inside their rows so that eight
// neighbouring lanes always touch eight different bank groups.
template <int NJ, bool MOE = false, bool SM = false>
__global__ __launch_bounds__(256, NJ == 1 ? 2 : 1) void qmm_q4k_i8_kernel(const uint8_t *__restrict__ w, ActView av, float *__restrict__ dst,
                                                                            int k, int n, int rows, int64_t stride_dst, MoeChunks mc,
                                                                            int64_t expert_bytes, int64_t split_stride) {
    static_assert(!SM || NJ == 1, "the small-m tile has one 32-column MFMA tile per wave");
    constexpr int BMT = SM ? 32 : BM, MI = SM ? 1 : 2;
    constexpr int BN = SM ? 128 : 64 * NJ, WN = 32 * NJ;
    constexpr int NA = BMT / 32, NB = BN / 64;                 // 16-byte pieces a thread copies per stage: activations, weights
    __shared__ __align__(16) int8_t As[2][BMT * 128];          // [row][8 pieces], piece p of row r at p ^ (r & 7)
    __shared__ __align__(16) uint8_t Bq[2][BN * 64];           // [row][4 pieces], piece p of row r at p ^ ((r >> 1) & 3)
    __shared__ __align__(16) uint8_t Bhd[2][BN * 16];          // block headers (d, dmin, scales), per super-block parity
    __shared__ __align__(16) _Float16 Am[2][BMT * 24];         // bsums16 of the super-block, as f16 (row stride 24 halves)
    __shared__ float sD8[2][BMT];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = SM ? 0 : wv >> 1, wn = SM ? wv : wv & 1;
    int m0 = blockIdx.x * BMT;
    const int n0 = blockIdx.y * BN;
    if (MOE) {
        if ((int)blockIdx.x >= mc.n_chunks[0]) return;           // uniform over the workgroup
        m0 = mc.first[blockIdx.x];
        rows = m0 + mc.count[blockIdx.x];
        w += (int64_t)mc.expert[blockIdx.x] * expert_bytes;
    }
    const int nsb_all = k >> 8;
    const int kb0 = (int)(((int64_t)nsb_all * blockIdx.z) / gridDim.z), nsb = (int)(((int64_t)nsb_all * (blockIdx.z + 1)) / gridDim.z);
    dst += (int64_t)blockIdx.z * split_stride;
    const int64_t row_bytes = (int64_t)(k / 256) * 144;

    // ---- copy roles.  Rows past the end of the tile are clamped to a valid row: an output row depends on its own
    // activation row only, and the rows past the end are not stored ----
    const int ra = tid >> 3, pa = tid & 7;                       // activations: piece pa of rows ra + 32 i
    const int rb = tid >> 2, pb = tid & 3;                       // weights: piece pb of rows rb + 64 i
    const int rh = tid & (BN - 1);                               // header of weight row rh
    const int rs = (tid >> 1) & (BMT - 1), half = tid & 1;       // d8 and eight of the sixteen bsums of activation row rs
    const int8_t *a_src[NA];
#pragma unroll
    for (int i = 0; i < NA; i++) a_src[i] = av.qs + (int64_t)min(m0 + ra + 32 * i, rows - 1) * k + 16 * pa;
    const uint8_t *b_src[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) b_src[i] = w + (int64_t)min(n0 + rb + 64 * i, n - 1) * row_bytes + 16 + 16 * pb;
    const uint8_t *h_src = w + (int64_t)min(n0 + rh, n - 1) * row_bytes;
    const int srow = min(m0 + rs, rows - 1);
    const int a_dst = ra * 128 + 16 * (pa ^ (ra & 7)), b_dst = rb * 64 + 16 * (pb ^ ((rb >> 1) & 3));
    // ---- MFMA operand roles ----
    const int kg = lane >> 5, swz_a = lane & 7, swz_b = (lane >> 1) & 3;

    f32x16 acc[MI][NJ];
    i32x16 sl[MI][NJ], sh[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) { acc[i][j][e] = 0.0f; sl[i][j][e] = 0; sh[i][j][e] = 0; }

    // registers of the stage in flight.  Stage (kb, s2) covers k = 256 kb + 128 s2 + [0, 128).  Positions past the end of
    // this split's range are clamped to its last super-block: what they bring lands in an LDS copy that nobody reads.
    u32x4 ga[NA], gb[NB], ghdr = u32x4{0, 0, 0, 0}, gbs = u32x4{0, 0, 0, 0};
    float gd8 = 0.0f;
    auto load_stage = [&](int kb, int s2) {
        kb = min(kb, nsb - 1);
#pragma unroll
        for (int i = 0; i < NA; i++) ga[i] = *reinterpret_cast<const u32x4 *>(a_src[i] + kb * 256 + 128 * s2);
#pragma unroll
        for (int i = 0; i < NB; i++) gb[i] = *reinterpret_cast<const u32x4 *>(b_src[i] + (int64_t)kb * 144 + 64 * s2);
        if (s2 == 0) {
            ghdr = *reinterpret_cast<const u32x4 *>(h_src + (int64_t)kb * 144);
            gd8 = av.d[(int64_t)srow * (k >> 8) + kb];
            gbs = *reinterpret_cast<const u32x4 *>(av.bsums + (int64_t)srow * (k >> 4) + kb * 16 + 8 * half);
        }
    };
    // buf: LDS copy of the stage (s2); hb: copy of the per-super-block arrays (parity of the super-block)
    auto store_stage = [&](int s2, int hb) {
#pragma unroll
        for (int i = 0; i < NA; i++) *reinterpret_cast<u32x4 *>(As[s2] + a_dst + 32 * 128 * i) = ga[i];
#pragma unroll
        for (int i = 0; i < NB; i++) *reinterpret_cast<u32x4 *>(Bq[s2] + b_dst + 64 * 64 * i) = gb[i];
        if (s2 == 0) {
            // threads that share a row write the same values
            *reinterpret_cast<u32x4 *>(Bhd[hb] + 16 * rh) = ghdr;
            sD8[hb][rs] = gd8;
            const uint32_t b4[4] = {gbs.x, gbs.y, gbs.z, gbs.w};
            u32x4 bv;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t lo = f2h_bits((float)(int16_t)(b4[i] & 0xffff)), hi = f2h_bits((float)(int16_t)(b4[i] >> 16));
                bv[i] = lo | (hi << 16);
            }
            *reinterpret_cast<u32x4 *>(Am[hb] + rs * 24 + 8 * half) = bv;
        }
    };
    load_stage(kb0, 0);
    store_stage(0, kb0 & 1);
    load_stage(kb0, 1);
    __syncthreads();

    for (int kb = kb0; kb < nsb; kb++) {
        const int hb = kb & 1;
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) {
            const int8_t *Ab = As[s2];
            const uint8_t *Bb = Bq[s2];
            u32x4 hdr[NJ];
#pragma unroll
            for (int t = 0; t < NJ; t++) hdr[t] = *reinterpret_cast<const u32x4 *>(Bhd[hb] + 16 * (wn * WN + t * 32 + (lane & 31)));
#pragma unroll
            for (int gg = 0; gg < 2; gg++) {
                const int g = 2 * s2 + gg;
                // ---- weights of sub-blocks 2 g (low nibbles) and 2 g + 1 (high nibbles) ----
                i32x4 bl[2][NJ], bh[2][NJ];
#pragma unroll
                for (int t = 0; t < NJ; t++) {
                    const u32x4 q = *reinterpret_cast<const u32x4 *>(Bb + (wn * WN + t * 32 + (lane & 31)) * 64 + 16 * ((2 * gg + kg) ^ swz_b));
                    const u32x4 h = hdr[t];
#pragma unroll
                    for (int ks = 0; ks < 2; ks++) {
                        // 6-bit scale of sub-block j = 2 g + ks (utils.rs:50-60); j < 4 exactly when g < 2
                        const int sft = 16 * (g & 1) + 8 * ks;
                        const uint32_t sc = g < 2 ? (h.y >> sft) & 63u : ((h.w >> sft) & 0xFu) | (((h.y >> sft) >> 2) & 0x30u);
                        const uint32_t lo2 = (sc & 7u) * 0x00010001u, hi2 = (sc >> 3) * 0x00010001u;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const uint32_t v = (ks ? q[i] >> 4 : q[i]) & 0x0f0f0f0fu;    // four weights, one per byte
                            bl[ks][t][i] = (int)pk_mul_u16(v, lo2);                         // bytes stay below 128: no carries
                            bh[ks][t][i] = (int)pk_mul_u16(v, hi2);
                        }
                    }
                }
                // ---- 2 k-slices of 32: MI x NJ tiles, two MFMA chains each ----
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    i32x4 af[MI];
#pragma unroll
                    for (int t = 0; t < MI; t++)
                        af[t] = *reinterpret_cast<const i32x4 *>(Ab + (wm * 64 + t * 32 + (lane & 31)) * 128 + 16 * ((4 * gg + 2 * ks + kg) ^ swz_a));
#pragma unroll
                    for (int i = 0; i < MI; i++)
#pragma unroll
                        for (int j = 0; j < NJ; j++) {
                            if (g == 0 && ks == 0) {                    // first slice of the super-block: the sums start from zero
                                i32x16 z;
#pragma unroll
                                for (int e = 0; e < 16; e++) z[e] = 0;
                                sl[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bl[ks][j], z, 0, 0, 0);
                                sh[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bh[ks][j], z, 0, 0, 0);
                            } else {
                                sl[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bl[ks][j], sl[i][j], 0, 0, 0);
                                sh[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bh[ks][j], sh[i][j], 0, 0, 0);
                            }
                        }
                }
            }
            // ---- the stage in flight goes to the other LDS copy; its registers take the stage after it ----
            store_stage(s2 ^ 1, s2 ? hb ^ 1 : hb);
            load_stage(kb + 1, s2);
            if (s2 == 1) {
                // ---- end of the super-block: mins term and the f32 scales ----
                half8 am[MI];
#pragma unroll
                for (int t = 0; t < MI; t++)
                    am[t] = *reinterpret_cast<const half8 *>(Am[hb] + (wm * 64 + t * 32 + (lane & 31)) * 24 + 8 * kg);
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    const u32x4 h = hdr[j];
                    const float d = h2f(h.x), dmin = h2f(h.x >> 16);
                    // B operand of the mins MFMA: element 2 i, 2 i + 1 of this lane = min of sub-block 4 kg + i, one per
                    // byte first (sub-blocks 0-3: low 6 bits of h.z; 4-7: high nibbles of h.w | top bits of h.z)
                    const uint32_t mine = kg ? ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u) : h.z & 0x3f3f3f3fu;
                    u32x4 mv;
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        mv[i] = pk_add((0x6400u | ((mine >> (8 * i)) & 0xffu)) * 0x00010001u, 0xe400e400u);   // (1024 + min) - 1024, twice
                    const half8 bm = __builtin_bit_cast(half8, mv);
#pragma unroll
                    for (int i = 0; i < MI; i++) {
                        f32x16 z;
#pragma unroll
                        for (int e = 0; e < 16; e++) z[e] = 0.0f;
                        const f32x16 mt = __builtin_amdgcn_mfma_f32_32x32x16_f16(am[i], bm, z, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            const int ml = wm * 64 + i * 32 + 8 * (e >> 2) + 4 * kg + (e & 3);
                            float t = d * (float)(8 * sh[i][j][e] + sl[i][j][e]);
                            t = fmaf(-dmin, mt[e], t);
                            acc[i][j][e] = fmaf(sD8[hb][ml], t, acc[i][j][e]);
                        }
                    }
                }
            }
            __syncthreads();
        }
    }

#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int nn = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int mm = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * kg + (e & 3);
                if (mm < rows && nn < n) {
                    if (MOE) dst[(int64_t)mc.pair_out[mm] * stride_dst + nn] = acc[i][j][e] * mc.pair_scale[mm];
                    else dst[(int64_t)mm * stride_dst + nn] = acc[i][j][e];
                }
            }
        }
}

// ---- Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 on the int8 matrix cores --------------------------------------------------------
// Same tiling and template parameters as above.  Both operands carry an f16 scale per 32 elements, so a 32 x 32 x 32 int8
// MFMA is exactly one block: its int32 result S is the sum the CPU vec_dot forms for that block (k_quants.rs:294-311,
// 720-738, 323-351, 434-455, 530-562), and each lane folds its 16 results into the f32 accumulators as
// (float(S) * d[n]) * d8[m], plus m[n] * s[m] for the formats with a block minimum (s = the Q8_1 block sum, k_quants.rs:770-799),
// block after block in k order like the CPU loop.  That scaling is three or four vector instructions per result and
// bounds the kernel; the matrix cores idle most of the time.  A stage is 128 elements of k (four blocks), held twice in
// LDS (one barrier per stage): the int8 activations as in the Q4_K kernel, the four d8 (and s) per activation row, and
// the weight rows' four blocks as they lie in memory (72 .. 136 contiguous bytes per row), copied in 8-byte pieces by
// neighbouring lanes so that a load instruction touches a handful of cache lines, not one per lane.  Lane (n, kg) of the
// B operand wants 16 consecutive k of row n: the 16 quant bytes of the block (4- and 5-bit formats: low nibbles for
// kg = 0, high nibbles for kg = 1, plus 16 bits of qh) or one half of its 32 (Q8_0), read from LDS at the block's own
// 2-byte alignment.  Needs 8-byte aligned weights (row lengths are multiples of 256 elements, so every row and stage
// then starts on 8 bytes).
//   nibble q -> int8 (q - 8) on four bytes at once: (x + 0x78787878) ^ 0x80808080 (no carries: x < 16 per byte);
//   5-bit q -> (q - 16): (x + 0x70707070) ^ 0x80808080.
template <int DT> struct Q0Info;
template <> struct Q0Info<CQ_Q4_0> { static constexpr int QS = 2, QH = -1, MIN = -1; static constexpr uint32_t BIAS = 0x78787878u; };
template <> struct Q0Info<CQ_Q8_0> { static constexpr int QS = 2, QH = -1, MIN = -1; static constexpr uint32_t BIAS = 0; };
template <> struct Q0Info<CQ_Q4_1> { static constexpr int QS = 4, QH = -1, MIN = 2; static constexpr uint32_t BIAS = 0; };
template <> struct Q0Info<CQ_Q5_0> { static constexpr int QS = 6, QH = 2, MIN = -1; static constexpr uint32_t BIAS = 0x70707070u; };
template <> struct Q0Info<CQ_Q5_1> { static constexpr int QS = 8, QH = 4, MIN = 2; static constexpr uint32_t BIAS = 0; };
// MOE: blockIdx.x is a tile of the chunk table, as in the kernels above.
template <int DT, int NJ, bool MOE = false, bool SM = false>
__global__ __launch_bounds__(256, NJ == 1 ? 2 : 1) void qmm_q0_i8_kernel(const uint8_t *__restrict__ w, ActView av, float *__restrict__ dst,
                                                                           int k, int n, int rows, int64_t stride_dst, MoeChunks mc,
                                                                           int64_t expert_bytes, int64_t split_stride) {
    typedef Q0Info<DT> QI;                                      // byte offsets of qs / qh / the block minimum (-1: none)
    static_assert(!SM || NJ == 1, "the small-m tile has one 32-column MFMA tile per wave");
    constexpr int BB = BlockInfo<DT>::bytes;
    constexpr bool HAS_MIN = QI::MIN >= 0;
    constexpr int BMT = SM ? 32 : BM, MI = SM ? 1 : 2;
    constexpr int BN = SM ? 128 : 64 * NJ, WN = 32 * NJ;
    constexpr int NA = BMT / 32;                                // 16-byte activation pieces a thread copies per stage
    constexpr int RS = 4 * BB, PPR = RS / 8;                    // bytes and 8-byte pieces of a weight row per stage
    constexpr int NBP = (BN * PPR + 255) / 256;                 // weight pieces a thread copies per stage (the last round is partial)
    __shared__ __align__(16) int8_t As[2][BMT * 128];           // [row][8 pieces], piece p of row r at p ^ (r & 7)
    __shared__ __align__(16) uint8_t Bq[2][BN * RS];            // [row][four blocks]
    __shared__ __align__(16) float sD8[2][4][BMT];              // d8 of the stage's four blocks
    __shared__ __align__(16) float sS8[2][HAS_MIN ? 4 : 1][HAS_MIN ? BMT : 4];   // their Q8_1 sums s = f16(f16(sum) * d8)

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = SM ? 0 : wv >> 1, wn = SM ? wv : wv & 1;
    int m0 = blockIdx.x * BMT;
    const int n0 = blockIdx.y * BN;
    if (MOE) {
        if ((int)blockIdx.x >= mc.n_chunks[0]) return;           // uniform over the workgroup
        m0 = mc.first[blockIdx.x];
        rows = m0 + mc.count[blockIdx.x];
        w += (int64_t)mc.expert[blockIdx.x] * expert_bytes;
    }
    // split-K over spans of 256 elements, like the other kernels; a stage is half a span
    const int nsb_all = k >> 8;
    const int st0 = 2 * (int)(((int64_t)nsb_all * blockIdx.z) / gridDim.z), st1 = 2 * (int)(((int64_t)nsb_all * (blockIdx.z + 1)) / gridDim.z);
    dst += (int64_t)blockIdx.z * split_stride;
    const int64_t row_bytes = (int64_t)(k >> 5) * BB;
    const int kg = lane >> 5, swz_a = lane & 7;

    // ---- copy roles.  Rows past the end of the tile are clamped to a valid row: an output row depends on its own
    // activation row only, and the rows past the end are not stored ----
    const int ra = tid >> 3, pa = tid & 7;                       // activations: piece pa of rows ra + 32 i
    const int rs = (tid >> 1) & (BMT - 1), half = tid & 1;       // d8 of blocks 2 half, 2 half + 1 of activation row rs
    const int8_t *a_src[NA];
#pragma unroll
    for (int i = 0; i < NA; i++) a_src[i] = av.qs + (int64_t)min(m0 + ra + 32 * i, rows - 1) * k + 16 * pa;
    const float *d_src = av.d + 2 * ((int64_t)min(m0 + rs, rows - 1) * (k >> 5) + 2 * half);
    const int a_dst = ra * 128 + 16 * (pa ^ (ra & 7));
    // weights: piece (tid + 256 i) of the tile's BN x PPR pieces, row-major; pieces past the end repeat the last one
    const uint8_t *b_src[NBP];
    int b_dst[NBP];
#pragma unroll
    for (int i = 0; i < NBP; i++) {
        const int p = min(tid + 256 * i, BN * PPR - 1), r = p / PPR, c = p - r * PPR;
        b_src[i] = w + (int64_t)min(n0 + r, n - 1) * row_bytes + 8 * c;
        b_dst[i] = r * RS + 8 * c;
    }
    // MFMA operand roles: this lane's weight row of tile j, and where its 16 quant bytes sit inside a block
    const int q_off = DT == CQ_Q8_0 ? QI::QS + 16 * kg : QI::QS;

    f32x16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // registers of the stage in flight.  Positions past the end of the split's range are clamped to its last stage: what
    // they bring lands in an LDS copy that nobody reads.
    u32x4 ga[NA], gds = u32x4{0, 0, 0, 0};
    u32x2 gb[NBP];
    auto load_stage = [&](int st) {
        st = min(st, st1 - 1);
#pragma unroll
        for (int i = 0; i < NA; i++) ga[i] = *reinterpret_cast<const u32x4 *>(a_src[i] + st * 128);
        gds = *reinterpret_cast<const u32x4 *>(d_src + 8 * st);         // {d, sum} pairs of two blocks
#pragma unroll
        for (int i = 0; i < NBP; i++) gb[i] = *reinterpret_cast<const u32x2 *>(b_src[i] + (int64_t)st * RS);
    };
    auto store_stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NA; i++) *reinterpret_cast<u32x4 *>(As[buf] + a_dst + 32 * 128 * i) = ga[i];
#pragma unroll
        for (int i = 0; i < NBP; i++) *reinterpret_cast<u32x2 *>(Bq[buf] + b_dst[i]) = gb[i];     // repeated pieces rewrite the same bytes
        // threads that share a row write the same values
        sD8[buf][2 * half][rs] = __uint_as_float(gds.x);
        sD8[buf][2 * half + 1][rs] = __uint_as_float(gds.z);
        if constexpr (HAS_MIN) {
            sS8[buf][2 * half][rs] = h2f(f2h_bits(h2f(f2h_bits((float)(int)gds.y)) * __uint_as_float(gds.x)));
            sS8[buf][2 * half + 1][rs] = h2f(f2h_bits(h2f(f2h_bits((float)(int)gds.w)) * __uint_as_float(gds.z)));
        }
    };
    load_stage(st0);
    store_stage(st0 & 1);
    __syncthreads();

    for (int st = st0; st < st1; st++) {
        const int buf = st & 1;
        load_stage(st + 1);
        const int8_t *Ab = As[buf];
        const uint8_t *Bb = Bq[buf];
#pragma unroll
        for (int b = 0; b < 4; b++) {
            i32x4 bop[NJ];
            float dw[NJ], mw[NJ];
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const uint8_t *blk = Bb + (wn * WN + j * 32 + (lane & 31)) * RS + b * BB;
                const u32x4 q = ld_u<u32x4>(blk + q_off);
                uint32_t qh = 0;
                if constexpr (QI::QH >= 0) qh = ld_u<uint32_t>(blk + QI::QH) >> (16 * kg);     // bit i: fifth bit of this lane's element i
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t v = q[i];
                    if constexpr (DT != CQ_Q8_0) v = (v >> (4 * kg)) & 0x0f0f0f0fu;
                    if constexpr (QI::QH >= 0) v |= spread4_to_bit4(qh >> (4 * i));
                    if constexpr (QI::BIAS != 0) v = (v + QI::BIAS) ^ 0x80808080u;
                    bop[j][i] = (int)v;
                }
                dw[j] = h2f(ld_u<uint16_t>(blk));
                mw[j] = HAS_MIN ? h2f(ld_u<uint16_t>(blk + (HAS_MIN ? QI::MIN : 0))) : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < MI; i++) {
                const int rl = wm * 64 + i * 32;
                const i32x4 af = *reinterpret_cast<const i32x4 *>(Ab + (rl + (lane & 31)) * 128 + 16 * ((2 * b + kg) ^ swz_a));
                f32x4 d8[4], s8[4];
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    d8[q4] = *reinterpret_cast<const f32x4 *>(&sD8[buf][b][rl + 8 * q4 + 4 * kg]);
                    if constexpr (HAS_MIN) s8[q4] = *reinterpret_cast<const f32x4 *>(&sS8[buf][b][rl + 8 * q4 + 4 * kg]);
                }
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    i32x16 z;
#pragma unroll
                    for (int e = 0; e < 16; e++) z[e] = 0;
                    const i32x16 sI = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bop[j], z, 0, 0, 0);
#pragma unroll
                    for (int e = 0; e < 16; e++) {
                        float t = fmaf((float)sI[e] * dw[j], d8[e >> 2][e & 3], acc[i][j][e]);
                        if constexpr (HAS_MIN) t = fmaf(mw[j], s8[e >> 2][e & 3], t);
                        acc[i][j][e] = t;
                    }
                }
            }
        }
        store_stage(buf ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int nn = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int mm = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * kg + (e & 3);
                if (mm < rows && nn < n) {
                    if (MOE) dst[(int64_t)mc.pair_out[mm] * stride_dst + nn] = acc[i][j][e] * mc.pair_scale[mm];
                    else dst[(int64_t)mm * stride_dst + nn] = acc[i][j][e];
                }
            }
        }
}

// dst[m, n] = sum over the split planes, in split order (deterministic); n % 4 == 0 whenever split-K is chosen
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ part, float *__restrict__ dst, int splits, int64_t n,
                                                            int64_t stride_dst, int64_t count) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= count) return;
    f32x4 a = *reinterpret_cast<const f32x4 *>(part + i);
    for (int sI = 1; sI < splits; sI++) {
        const f32x4 b = *reinterpret_cast<const f32x4 *>(part + sI * count + i);
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    const int64_t r = i / n, c = i - r * n;
    float *o = dst + r * stride_dst + c;
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}

typedef void (*QmmFn)(const uint8_t *, ActView, float *, int, int, int, int64_t, MoeChunks, int64_t, int64_t);
// the kernel of a format and tile shape: Q4_K and the 32-element formats run on the int8 matrix cores, the others on the f16 ones
template <int DT, int NJ, bool MOE, bool SM>
QmmFn qmm_fn() {
    if constexpr (DT == CQ_Q4K) return qmm_q4k_i8_kernel<NJ, MOE, SM>;
    else if constexpr (DT == CQ_Q4_0 || DT == CQ_Q8_0 || DT == CQ_Q4_1 || DT == CQ_Q5_0 || DT == CQ_Q5_1)
        return qmm_q0_i8_kernel<DT, NJ, MOE, SM>;
    else return qmm_kernel<DT, NJ, MOE, SM>;
}

template <int DT>
int launch_qmm(const void *w, const ActView &av, float *dst, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, hipStream_t s,
               float *split_ws) {
    // 128 x 64 tiles (two workgroups per CU) everywhere except Q4_0 / Q8_0 problems whose grid of 128 x 128 tiles still
    // covers the chip (one workgroup per CU, half the weight-operand builds per activation row).  For the int8 kernel the
    // two tile shapes are within 10 % of each other (measured in TFLOP/s at 2048 rows, 128 x 128 against 128 x 64 tiles:
    // Q4_0 14336 x 4096 440 / 500, Q4_0 4096 x 14336 461 / 439, Q8_0 14336 x 4096 460 / 447; 512 rows 360 / 351).
    const bool wide = !cq_is_kquant(DT) && ((rows + 127) / 128) * ((n + 127) / 128) >= 384;
    // a few dozen activation rows (batched decode): 32 x 128 tiles, so that the matrix cores and the activation staging
    // are not spent on 128-row tiles that are mostly padding
    const bool small = rows <= CQ_QMM_SMALL_ROWS;
    const int bn = wide || small ? 128 : 64, bm = small ? 32 : BM;
    const int splits = split_ws ? cq_qmm_splits(k, n, rows) : 1;
    dim3 grid((unsigned)((rows + bm - 1) / bm), (unsigned)((n + bn - 1) / bn), (unsigned)splits);
    if (grid.y > 65535) return CQ_ERR_RANGE;
    const MoeChunks none{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0};
    // with split-K every split writes a contiguous [rows, n] plane of the workspace; a second kernel adds them in order
    float *out = splits > 1 ? split_ws : dst;
    const int64_t ld = splits > 1 ? n : stride_dst, plane = splits > 1 ? rows * n : 0;
    if (small)
        hipLaunchKernelGGL((qmm_fn<DT, 1, false, true>()), grid, dim3(256), 0, s, (const uint8_t *)w, av, out, (int)k, (int)n, (int)rows, ld, none,
                           (int64_t)0, plane);
    else if (wide)
        hipLaunchKernelGGL((qmm_fn<DT, 2, false, false>()), grid, dim3(256), 0, s, (const uint8_t *)w, av, out, (int)k, (int)n, (int)rows, ld, none, (int64_t)0,
                           plane);
    else
        hipLaunchKernelGGL((qmm_fn<DT, 1, false, false>()), grid, dim3(256), 0, s, (const uint8_t *)w, av, out, (int)k, (int)n, (int)rows, ld, none, (int64_t)0,
                           plane);
    int rc = (int)hipGetLastError();
    if (rc || splits == 1) return rc;
    const int64_t count = rows * n;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((count / 4 + 255) / 256)), dim3(256), 0, s, (const float *)split_ws, dst, splits, n,
                       stride_dst, count);
    return (int)hipGetLastError();
}

__global__ __launch_bounds__(256) void convert_f32_kernel(const float *__restrict__ src, void *__restrict__ dst, int dst_dtype, int64_t count) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    float v = src[i];
    if (dst_dtype == CQ_F16) {
        ((uint16_t *)dst)[i] = f2h_bits(v);
    } else {
        uint32_t b = __float_as_uint(v);
        uint32_t r = (b & 0x7fffffffu) > 0x7f800000u ? (b | 0x00400000u) : b + 0x7fffu + ((b >> 16) & 1u);
        ((uint16_t *)dst)[i] = (uint16_t)(r >> 16);
    }
}

}  // namespace

int cq_convert_f32_launch(const float *src, void *dst, int dst_dtype, int64_t count, hipStream_t s) {
    if (count == 0) return CQ_OK;
    if (dst_dtype != CQ_F16 && dst_dtype != CQ_BF16) return CQ_ERR_DTYPE;
    int64_t grid = (count + 255) / 256;
    if (grid > 0x7fffffffLL) return CQ_ERR_RANGE;
    hipLaunchKernelGGL(convert_f32_kernel, dim3((unsigned)grid), dim3(256), 0, s, src, dst, dst_dtype, count);
    return (int)hipGetLastError();
}

namespace {
template <int DT>
int launch_qmm_moe(const void *w, const ActView &av, float *out, const MoeChunks &mc, int64_t k, int64_t n, int tile_rows, hipStream_t s) {
    const int bn = tile_rows == 32 ? 128 : 64;
    dim3 grid((unsigned)mc.max_chunks, (unsigned)((n + bn - 1) / bn));
    if (grid.y > 65535) return CQ_ERR_RANGE;
    const int64_t expert_bytes = n * (k / BlockInfo<DT>::elems) * BlockInfo<DT>::bytes;
    if (tile_rows == 32)
        hipLaunchKernelGGL((qmm_fn<DT, 1, true, true>()), grid, dim3(256), 0, s, (const uint8_t *)w, av, out, (int)k, (int)n, 0, n, mc,
                           expert_bytes, (int64_t)0);
    else
        hipLaunchKernelGGL((qmm_fn<DT, 1, true, false>()), grid, dim3(256), 0, s, (const uint8_t *)w, av, out, (int)k, (int)n, 0, n, mc, expert_bytes,
                           (int64_t)0);
    return (int)hipGetLastError();
}

}  // namespace

// tile_rows: rows of one chunk of the table, CQ_MOE_TILE_SMALL (32) or CQ_MOE_TILE_LARGE (128)
int cq_matmul_moe_launch(int w_dtype, const void *w, const void *scratch, int64_t rows_alloc, float *out, const MoeChunks &mc, int64_t k, int64_t n,
                         int tile_rows, hipStream_t s) {
    if (mc.max_chunks == 0 || n == 0) return CQ_OK;
    if (k % 256) return CQ_ERR_SHAPE;
    if (tile_rows != CQ_MOE_TILE_SMALL && tile_rows != CQ_MOE_TILE_LARGE) return CQ_ERR_RANGE;
    ActView av = cq_act_view(scratch, w_dtype, k, rows_alloc);
    switch (w_dtype) {
        case CQ_Q4_0: return launch_qmm_moe<CQ_Q4_0>(w, av, out, mc, k, n, tile_rows, s);
        case CQ_Q8_0: return launch_qmm_moe<CQ_Q8_0>(w, av, out, mc, k, n, tile_rows, s);
        case CQ_Q4K: return launch_qmm_moe<CQ_Q4K>(w, av, out, mc, k, n, tile_rows, s);
        case CQ_Q5K: return launch_qmm_moe<CQ_Q5K>(w, av, out, mc, k, n, tile_rows, s);
        case CQ_Q6K: return launch_qmm_moe<CQ_Q6K>(w, av, out, mc, k, n, tile_rows, s);
        case CQ_Q2K: return launch_qmm_moe<CQ_Q2K>(w, av, out, mc, k, n, tile_rows, s);
        case CQ_Q3K: return launch_qmm_moe<CQ_Q3K>(w, av, out, mc, k, n, tile_rows, s);
    }
    return CQ_ERR_DTYPE;
}

// k is a multiple of 256 for the MFMA kernel (always true for K-quants); Q4_0 / Q8_0 rows whose length
// is only a multiple of 32, and very small problems, go through the row-chunked matvec instead.
// Small grids (few activation rows or few weight rows) split K so that about 512 workgroups exist.  1 = no split.
int cq_qmm_splits(int64_t k, int64_t n, int64_t rows) {
    if (k % 256 || n % 4 || rows < 1) return 1;
    const int64_t base = rows <= CQ_QMM_SMALL_ROWS ? ((rows + 31) / 32) * ((n + 127) / 128) : ((rows + BM - 1) / BM) * ((n + 63) / 64);
    const int64_t nsb = k / 256;
    // about two workgroups per CU: one converts operands while the other feeds the matrix cores (measured against a target
    // of one per CU: Q6_K 4096 x 14336 at 128 / 256 / 512 rows 69 / 131 / 248 -> 57 / 105 / 200 us, Q4_K 4096 x 4096 at 512
    // rows 67 -> 54 us; three per CU is no better)
    const int64_t target = 512;
    if (base >= target * 3 / 4 || nsb < 8) return 1;
    int64_t sp = (target + base - 1) / base;
    if (sp > 8) sp = 8;
    if (sp > nsb / 4) sp = nsb / 4;
    return sp < 2 ? 1 : (int)sp;
}

// Which row counts go to the matrix cores: everything beyond the matvec kernel's 8 rows, and for Q4_K, whose int8 kernel is
// the faster one, from 6 rows (measured, Q4_K 14336 x 4096 / 4096 x 14336 in us: matvec at 4 / 5 / 6 / 8 rows 19.4 / 21.6 /
// 23.4 / 27.5 and 18.3 / 20.8 / 23.6 / 29.9, the 32-row MFMA tile 20.7 and 22.3 at any of them, 21.3 / 23.0 at 16 / 32 rows).
constexpr int CQ_Q4K_MFMA_MIN_ROWS = 6;
bool cq_use_mfma(int w_dtype, int64_t rows, int64_t k) {
    if (k % 256 || !cq_has_mfma(w_dtype)) return false;
    return rows > CQ_MATVEC_MAX_ROWS || (w_dtype == CQ_Q4K && rows >= CQ_Q4K_MFMA_MIN_ROWS);
}

int cq_matmul_launch(int w_dtype, const void *w, const void *scratch, float *dst, int64_t k, int64_t n, int64_t rows,
                     int64_t stride_dst, hipStream_t s, float *split_ws) {
    ActView av = cq_act_view(scratch, w_dtype, k, rows);
    // the matrix-core kernel of the 32-element formats copies weight rows in 8-byte pieces; weights at another alignment
    // take the loop below
    const bool q0_unaligned = !cq_is_kquant(w_dtype) && ((uintptr_t)w & 7) != 0;
    if (cq_use_mfma(w_dtype, rows, k) && !q0_unaligned) {
        switch (w_dtype) {
            case CQ_Q4_0: return launch_qmm<CQ_Q4_0>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q8_0: return launch_qmm<CQ_Q8_0>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q4_1: return launch_qmm<CQ_Q4_1>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q5_0: return launch_qmm<CQ_Q5_0>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q5_1: return launch_qmm<CQ_Q5_1>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q4K: return launch_qmm<CQ_Q4K>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q5K: return launch_qmm<CQ_Q5K>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q6K: return launch_qmm<CQ_Q6K>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q2K: return launch_qmm<CQ_Q2K>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
            case CQ_Q3K: return launch_qmm<CQ_Q3K>(w, av, dst, k, n, rows, stride_dst, s, split_ws);
        }
        return CQ_ERR_DTYPE;
    }
    for (int64_t r0 = 0; r0 < rows; r0 += CQ_MATVEC_MAX_ROWS) {
        int64_t nb = rows - r0 < CQ_MATVEC_MAX_ROWS ? rows - r0 : CQ_MATVEC_MAX_ROWS;
        ActView c = cq_act_view_rows(av, w_dtype, k, r0);
        int rc = cq_matvec_launch_av(w_dtype, w, c, dst + r0 * stride_dst, CQ_F32, k, n, nb, stride_dst, s);
        if (rc) return rc;
    }
    return CQ_OK;
}
