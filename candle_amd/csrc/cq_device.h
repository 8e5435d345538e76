// Shared device-side definitions for the gfx950 GGUF quantized-matmul kernels:
// block geometry, unaligned vector loads, f16 helpers, wave64 reductions and the layout of the
// quantized-activation scratch buffer.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "../../include/candle_hip_quant.h"

#define CQ_QK_K 256
#define CQ_WAVE 64

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// GGUF block sizes in bytes (candle-core/src/quantized/k_quants.rs:77-190).
template <int DT> struct BlockInfo;
template <> struct BlockInfo<CQ_Q4_0> { static constexpr int elems = 32, bytes = 18; };
template <> struct BlockInfo<CQ_Q8_0> { static constexpr int elems = 32, bytes = 34; };
template <> struct BlockInfo<CQ_Q4K> { static constexpr int elems = 256, bytes = 144; };
template <> struct BlockInfo<CQ_Q5K> { static constexpr int elems = 256, bytes = 176; };
template <> struct BlockInfo<CQ_Q6K> { static constexpr int elems = 256, bytes = 210; };
template <> struct BlockInfo<CQ_Q8K> { static constexpr int elems = 256, bytes = 292; };
template <> struct BlockInfo<CQ_Q4_1> { static constexpr int elems = 32, bytes = 20; };
template <> struct BlockInfo<CQ_Q5_0> { static constexpr int elems = 32, bytes = 22; };
template <> struct BlockInfo<CQ_Q5_1> { static constexpr int elems = 32, bytes = 24; };
template <> struct BlockInfo<CQ_Q8_1> { static constexpr int elems = 32, bytes = 36; };
template <> struct BlockInfo<CQ_Q2K> { static constexpr int elems = 256, bytes = 84; };
template <> struct BlockInfo<CQ_Q3K> { static constexpr int elems = 256, bytes = 110; };

// formats whose activations are quantized to Q8_K (the others: Q8_0 blocks, read as Q8_1 where the weight format asks for it)
__host__ __device__ inline bool cq_is_kquant(int dt) {
    return dt == CQ_Q4K || dt == CQ_Q5K || dt == CQ_Q6K || dt == CQ_Q8K || dt == CQ_Q2K || dt == CQ_Q3K;
}
// formats with a matrix-core kernel (cq_matmul.hip): every QMatMul weight format
__host__ __device__ constexpr bool cq_has_mfma(int dt) {
    return dt == CQ_Q4_0 || dt == CQ_Q8_0 || dt == CQ_Q4K || dt == CQ_Q5K || dt == CQ_Q6K || dt == CQ_Q2K || dt == CQ_Q3K || dt == CQ_Q4_1 ||
           dt == CQ_Q5_0 || dt == CQ_Q5_1;
}
// formats with every fused instance of the decode matvec (f16 / bf16 activations, decoder prologues and epilogues)
__host__ __device__ constexpr bool cq_full_matvec(int dt) { return dt == CQ_Q4_0 || dt == CQ_Q8_0 || dt == CQ_Q4K || dt == CQ_Q5K || dt == CQ_Q6K; }
__host__ __device__ inline bool cq_is_q0(int dt) { return dt == CQ_Q4_0 || dt == CQ_Q8_0; }

// Global loads from addresses that are only 2-byte aligned (Q6_K, Q8_0 and Q4_0 blocks): gfx950
// serves these with one global_load_dword[x2|x4].
template <typename T> __device__ __forceinline__ T ld_u(const void *p) {
    struct __attribute__((packed, aligned(2))) W { T v; };
    return reinterpret_cast<const W *>(p)->v;
}
template <typename T> __device__ __forceinline__ void st_u(void *p, T v) {
    struct __attribute__((packed, aligned(2))) W { T v; };
    reinterpret_cast<W *>(p)->v = v;
}

// f16 bit pattern -> f32 (exact, subnormals included).
__device__ __forceinline__ float h2f(uint32_t bits16) {
    return __half2float(__ushort_as_half((unsigned short)(bits16 & 0xffffu)));
}
// f32 -> f16 bit pattern, round to nearest even.  The conversion is issued as an opaque
// v_cvt_f16_f32 on the finished f32 value: left to the compiler, `f16(a * b)` becomes
// v_fma_mixlo_f16(a, b, +0), which turns a -0.0 product into +0.0.
__device__ __forceinline__ uint16_t f2h_bits(float f) {
    uint32_t r;
    asm("v_cvt_f16_f32 %0, %1" : "=v"(r) : "v"(f));
    return (uint16_t)(r & 0xffffu);
}

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// ---- DPP cross-lane helpers (a few cycles each; ds_bpermute-based shuffles cost a round trip through
// the LDS crossbar per step, which dominates short dependent chains) --------------------------------
#define CQ_DPP_QUAD_XOR1 0xB1     // quad_perm [1,0,3,2]
#define CQ_DPP_QUAD_XOR2 0x4E     // quad_perm [2,3,0,1]
#define CQ_DPP_ROW_SHR(n) (0x110 + (n))
#define CQ_DPP_ROW_HALF_MIRROR 0x141
#define CQ_DPP_ROW_BCAST15 0x142
#define CQ_DPP_ROW_BCAST31 0x143

// max over the wave of a non-negative float, returned in every lane (through a scalar register)
__device__ __forceinline__ float wave_max_nonneg(float v) {
#define CQ_MX(ctrl, rmask, bc) v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), ctrl, rmask, 0xf, bc)))
    CQ_MX(CQ_DPP_ROW_SHR(1), 0xf, false);
    CQ_MX(CQ_DPP_ROW_SHR(2), 0xf, false);
    CQ_MX(CQ_DPP_ROW_SHR(4), 0xf, false);
    CQ_MX(CQ_DPP_ROW_SHR(8), 0xf, false);      // lane 15 of each row: row max
    CQ_MX(CQ_DPP_ROW_BCAST15, 0xa, false);
    CQ_MX(CQ_DPP_ROW_BCAST31, 0xc, false);     // lane 63: wave max
#undef CQ_MX
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// min over the wave of an int, returned in every lane
__device__ __forceinline__ int wave_min_int(int v) {
#define CQ_MN(ctrl, rmask) v = min(v, __builtin_amdgcn_update_dpp(v, v, ctrl, rmask, 0xf, false))
    CQ_MN(CQ_DPP_ROW_SHR(1), 0xf);
    CQ_MN(CQ_DPP_ROW_SHR(2), 0xf);
    CQ_MN(CQ_DPP_ROW_SHR(4), 0xf);
    CQ_MN(CQ_DPP_ROW_SHR(8), 0xf);
    CQ_MN(CQ_DPP_ROW_BCAST15, 0xa);
    CQ_MN(CQ_DPP_ROW_BCAST31, 0xc);
#undef CQ_MN
    return __builtin_amdgcn_readlane(v, 63);
}

// sums / maxima over aligned groups of 4 and 8 lanes, result in every lane of the group
__device__ __forceinline__ int quad_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, CQ_DPP_QUAD_XOR1, 0xf, 0xf, true);
    v += __builtin_amdgcn_update_dpp(0, v, CQ_DPP_QUAD_XOR2, 0xf, 0xf, true);
    return v;
}
__device__ __forceinline__ int oct_sum(int v) {
    v = quad_sum(v);
    v += __builtin_amdgcn_update_dpp(0, v, CQ_DPP_ROW_HALF_MIRROR, 0xf, 0xf, true);
    return v;
}
__device__ __forceinline__ float oct_max(float v) {
#define CQ_MX(ctrl) v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true)))
    CQ_MX(CQ_DPP_QUAD_XOR1);
    CQ_MX(CQ_DPP_QUAD_XOR2);
    CQ_MX(CQ_DPP_ROW_HALF_MIRROR);
#undef CQ_MX
    return v;
}

// wave64 sum; every lane ends with the total (through a scalar register).  DPP row shifts and row broadcasts: six
// VALU steps, where a butterfly of __shfl_xor is six trips through the LDS crossbar.
__device__ __forceinline__ float wave_sum(float v) {
#define CQ_AD(ctrl, rmask, bc) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, rmask, 0xf, bc))
    CQ_AD(CQ_DPP_ROW_SHR(1), 0xf, true);
    CQ_AD(CQ_DPP_ROW_SHR(2), 0xf, true);
    CQ_AD(CQ_DPP_ROW_SHR(4), 0xf, true);
    CQ_AD(CQ_DPP_ROW_SHR(8), 0xf, true);      // lane 15 of each row: row sum
    CQ_AD(CQ_DPP_ROW_BCAST15, 0xa, false);
    CQ_AD(CQ_DPP_ROW_BCAST31, 0xc, false);    // lane 63: wave sum
#undef CQ_AD
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// wave64 maximum of any float, in every lane
__device__ __forceinline__ float wave_max(float v) {
#define CQ_MX(ctrl, rmask) v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), ctrl, rmask, 0xf, false)))
    CQ_MX(CQ_DPP_ROW_SHR(1), 0xf);
    CQ_MX(CQ_DPP_ROW_SHR(2), 0xf);
    CQ_MX(CQ_DPP_ROW_SHR(4), 0xf);
    CQ_MX(CQ_DPP_ROW_SHR(8), 0xf);
    CQ_MX(CQ_DPP_ROW_BCAST15, 0xa);
    CQ_MX(CQ_DPP_ROW_BCAST31, 0xc);
#undef CQ_MX
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// ---------------------------------------------------------------------------------------------
// Quantized-activation scratch (written by the act-quant kernels, read by matvec / matmul / MoE).
//   K-quant weights : int8 qs[rows][k] | float d[rows][k/256] | int16 bsums[rows][k/16]
//   Q4_0 / Q8_0     : int8 qs[rows][k] | {float d; int32 sum;} ds[rows][k/32]
// Sections start on 256-byte boundaries.
// ---------------------------------------------------------------------------------------------
struct ActLayout {
    int64_t qs_off, d_off, bs_off, total;
};

__host__ __device__ inline int64_t cq_align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

__host__ __device__ inline ActLayout cq_act_layout(int w_dtype, int64_t k, int64_t rows) {
    ActLayout L;
    L.qs_off = 0;
    L.d_off = cq_align256(rows * k);
    if (cq_is_kquant(w_dtype)) {
        L.bs_off = L.d_off + cq_align256(rows * (k / 256) * 4);
        L.total = L.bs_off + cq_align256(rows * (k / 16) * 2);
    } else {
        L.bs_off = L.d_off;
        L.total = L.d_off + cq_align256(rows * (k / 32) * 8);
    }
    return L;
}

struct ActView {            // resolved pointers for one scratch buffer
    const int8_t *qs;       // [rows][k]
    const float *d;         // K-quants: [rows][k/256];  Q4_0/Q8_0: interleaved {d, sum} pairs [rows][k/32][2]
    const int16_t *bsums;   // K-quants only: [rows][k/16]
};

__host__ __device__ inline ActView cq_act_view(const void *scratch, int w_dtype, int64_t k, int64_t rows) {
    ActLayout L = cq_act_layout(w_dtype, k, rows);
    const uint8_t *b = (const uint8_t *)scratch;
    ActView v;
    v.qs = (const int8_t *)(b + L.qs_off);
    v.d = (const float *)(b + L.d_off);
    v.bsums = (const int16_t *)(b + L.bs_off);
    return v;
}

// The same view starting at activation row r0.
__host__ __device__ inline ActView cq_act_view_rows(const ActView &av, int w_dtype, int64_t k, int64_t r0) {
    ActView v = av;
    v.qs = av.qs + r0 * k;
    if (cq_is_kquant(w_dtype)) {
        v.d = av.d + r0 * (k / 256);
        v.bsums = av.bsums + r0 * (k / 16);
    } else {
        v.d = av.d + 2 * r0 * (k / 32);
    }
    return v;
}
