// Batched decode matvec on the int8 matrix cores:  dst[b, row] = sum_k W[row, k] * x^[b, k]  for 3 .. 16 activation rows,
// Q4_K weights, the weights read once at streaming speed.
//
// The single-row kernels pay per activation row for every dot product (v_dot4 on the vector ALU), and the prefill tiles pay
// per WEIGHT for folding the sub-block scales into the matrix operands — worth it when hundreds of rows share a weight tile,
// not for a handful.  With at most 16 rows the cheap side is the OUTPUT: one v_mfma_i32_16x16x32_i8 is exactly one
// 32-element sub-block of 16 weight rows against 16 activation rows, its int32 result is the sub-block dot the CPU forms
// (k_quants.rs:1460-1540, BlockQ4K x BlockQ8K), and the 6-bit sub-block scale is applied to the 4 results a lane holds
// (two vector instructions per result).  A weight costs a quarter of a vector instruction per nibble (one AND per four),
// whatever the number of rows.
//
// Work split.  A workgroup takes blocks of 16 weight rows (block m = blockIdx.x, + gridDim.x, ...).  Its 8 waves split K:
// wave w owns the super-block columns [w * CPW, (w + 1) * CPW) of every row, and keeps the int8 activations of those columns,
// for all rows of the batch, in registers as matrix operands for the whole kernel (lane (c, kg): 8 consecutive values of
// batch row c per sub-block), so the only stream is the weights: a block of 16 rows is one contiguous piece of the tensor,
// which the waves copy HBM -> LDS together, one KB per instruction (buffer loads that write LDS directly; each wave copying
// only its own columns, 16 short runs per tile, was tried first: those instructions take five times as long to issue), into
// a ring of tiles, two blocks ahead.  The partial sums of the 8 waves meet in LDS once per block and are added in wave order.
//
// The activations are quantized like BlockQ8K::from_float (up to a common sign of a span's values and scale, which no product
// sees) by a small kernel of this file, or by the waves of the main kernel for up to 8 rows, which leaves them laid out
// as the matrix operands the waves load.
//
// The same formulation serves MoE calls with hundreds of pairs: every expert a batched matvec over its own pairs
// (qme_q4k_kernel at the end of this file).
//
// (-DCL_STAMPS compiles this file with per-wave s_memrealtime stamps and two extra entry points for a timeline of the launch;
// the library is built without it.)
#include <algorithm>
#include "cq_actquant.h"
#include "cq_device.h"
#include "cq_fmt.h"
#include "cq_launch.h"
#include "cq_stream.h"

#ifdef CL_STAMPS
#define QB_STAMP(i) do { if ((threadIdx.x & 63) == 0) qb_stamp_lds[threadIdx.x >> 6][(i)] = (uint32_t)__builtin_amdgcn_s_memrealtime(); } while (0)
static uint32_t *qb_stamps_dev = nullptr;
extern "C" void qb_set_stamps(uint32_t *p) { qb_stamps_dev = p; }
#else
#define QB_STAMP(i) do { } while (0)
#endif

namespace {

#ifdef CL_STAMPS
__shared__ uint32_t qb_stamp_lds[8][16];
#endif

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef long i64x2 __attribute__((ext_vector_type(2)));

constexpr int QB_NW = 8;
constexpr int QB_BB = 144;                        // bytes of a Q4_K super-block
// Q5_K is Q4_K with a fifth bit per weight: the same 16-byte header (d, dmin, 6-bit scales and minima), then qh[32] (bit j of
// byte l: the fifth bit of element l of sub-block j), then the nibbles.  The kernels of this file take both (template flag Q5):
// the fifth bits of a lane's eight elements of all eight sub-blocks are one 8-byte read, and a sub-block's operand is
// nibbles | (bits << 4), values 0 .. 31.
template <bool Q5> struct QbW { static constexpr int BB = Q5 ? 176 : 144, QS = Q5 ? 48 : 16; };
__host__ __device__ constexpr int qb_bb(bool q5) { return q5 ? 176 : 144; }
constexpr int QB_RED_BYTES = QB_NW * 64 * 16;     // the waves' partial results of one block of rows
constexpr int QB_LDS_BYTES = 160 * 1024;
// A tile (16 rows of up to 8 * CPW super-blocks) is copied by whole instructions of 64 lanes x 16 bytes, each wave the same number:
// it occupies a multiple of 8 KB.
constexpr int qb_tile_instr(int cpw, int bb = QB_BB) { return (16 * 8 * cpw * bb + 8 * 1024 - 1) / (8 * 1024); }       // copy instructions per wave and tile
// In LDS every KB of a tile is followed by 16 unused bytes: a row is 9 * 16 * (super-blocks per row) bytes, for rows of 16
// super-blocks a multiple of all 64 banks, and the 16 lanes that read the same bytes of 16 different rows would meet on one bank.
constexpr int QB_KB = 1024 + 16;
// a tile of a block of `block_bytes`: its KBs, and one more that takes the zeros of the copy instructions beyond the block
__host__ __device__ constexpr int qb_tile_bytes(int block_bytes) { return ((block_bytes + 1023) / 1024 + 1) * QB_KB; }

// ---- the activations, quantized like BlockQ8K::from_float and laid out as this kernel's matrix operands ----
// For super-block column s of the row length, 16 batch slots (rows beyond the batch are zeros):
//   operands [s][g < 4][kg < 4][slot c < 16][16 bytes]         values 8 kg .. 8 kg + 7 of sub-blocks 2 g and 2 g + 1 of column s of
//                                                              row c: what lane (c, kg) feeds the matrix core against the low and
//                                                              the high nibbles of weight bytes 32 g + 8 kg .. + 7; one 16-byte
//                                                              load per lane, 1 KB contiguous per wave;
//   records  [s][c] { u8 bl[8], i8 bh[8] (sum of sub-block j = 128 * bh_j + bl_j), f32 d, 12 bytes unused }
// Batch row b sits in operand slot 4 (b % 4) + b / 4 (the map is its own inverse): a lane's result r of lane group kg then belongs
// to batch row 4 r + kg, and a batch of `rows` rows needs only the first ceil(rows / 4) of a lane's four results worked out (the
// scaling of a result is most of the kernels' vector work).
__host__ __device__ constexpr int qb_slot(int b) { return 4 * (b & 3) + (b >> 2); }
constexpr int QB_OP_COL_BYTES = 8 * 4 * 16 * 8;       // 4096
constexpr int QB_REC_BYTES = 32;
__host__ __device__ inline int64_t qb_operand_bytes(int64_t bpr) { return bpr * (QB_OP_COL_BYTES + 16 * QB_REC_BYTES); }

// where the lane's dword of a span goes inside one column of operands laid out [g < 4][kg < 4][slot < SLOTS][16 bytes]:
// elements 4 lane .. + 3 are values 4 (lane % 8) .. + 3 of sub-block lane / 8: lane group kg = (lane % 8) / 2, dword lane % 2
__device__ __forceinline__ int qb_operand_dword(int lane, int c, int slots) {
    return (((lane >> 4) * 4 + ((lane & 7) >> 1)) * slots + c) * 16 + 8 * ((lane >> 3) & 1) + 4 * (lane & 1);
}

// XDT < 0: the rows are silu(x[c]) * up[c], rows of f32 with strides of their own (a feed-forward's w2 over several rows)
template <int XDT>
__global__ __launch_bounds__(256) void qb_quantize_kernel(const void *__restrict__ x, const float *__restrict__ up, int64_t x_stride, int64_t up_stride,
                                                          uint8_t *__restrict__ op, int bpr, int rows) {
    const int span = (int)blockIdx.x * 4 + ((int)threadIdx.x >> 6);          // span = s * 16 + c
    if (span >= bpr * 16) return;
    const int lane = threadIdx.x & 63, s = span >> 4, slot = span & 15, c = qb_slot(slot);      // c: the batch row of this slot
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (c < rows) {
        if constexpr (XDT < 0) cq_load_swiglu4((const float *)x, up, c * x_stride + s * 256 + lane * 4, c * up_stride + s * 256 + lane * 4, v);
        else cq_load4<XDT>(x, c * x_stride + s * 256 + lane * 4, v);
    }
    // the streaming kernel's span quantizer (cq_stream.h: where the first largest magnitude is negative the int8 values and the scale
    // come out with the other sign than BlockQ8K::from_float gives them, and every product is the same)
    const float vv[1][4] = {{v[0], v[1], v[2], v[3]}};
    const uint32_t wmax[1] = {qs_span_umax(vv[0])};
    float iscale[1], d[1];
    qs_span_scales<1>(wmax, lane, iscale, d);
    int q[4];
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = qs_round_i8(iscale[0] * v[i]);
    const uint32_t packed = qs_pack4(q);
    uint8_t *colp = op + (int64_t)s * QB_OP_COL_BYTES;
    *(uint32_t *)(colp + qb_operand_dword(lane, slot, 16)) = packed;
    const int s32 = oct_sum(sdot4(packed, 0x01010101u, 0));       // the sum of the 32-element sub-block, in its eight lanes
    uint8_t *rec = op + (int64_t)bpr * QB_OP_COL_BYTES + (int64_t)span * QB_REC_BYTES;
    if ((lane & 7) == 0) { rec[lane >> 3] = (uint8_t)(s32 & 127); rec[8 + (lane >> 3)] = (uint8_t)(s32 >> 7); }
    if (lane == 0) *(float *)(rec + 16) = d[0];
}

// FQ > 0: `op` is not the operand buffer but the f32 activations themselves, [rows == FQ][256 bpr], and every wave quantizes
// the spans of its own columns while the first tiles are on their way (all 64 lanes on one span at a time, the int8 values
// turned into matrix operands through the LDS of the last tile of the ring, which the weights need only later).  The same
// results as from qb_quantize_kernel's operands, bit for bit (where the first largest magnitude of a span is negative the
// int8 values and the scale both come out with the other sign, as in the streaming kernel, and their products are the same).  Every workgroup repeats the work, which pays while it hides behind the
// first tile's latency: up to 8 rows.  (The row count is a template parameter: with the spans behind run-time conditions
// the compiler cannot interleave their dependent chains, and a span costs 0.67 us instead of a third of that.)
constexpr int QB_FQ_MAX_SPANS = 16;                // spans (columns x rows) a wave quantizes itself at most; beyond, the separate kernel is ahead
constexpr int QB_FQ_REC = 32;                      // bytes of a staged record {u8 bl[8], u8 bh[8], f32 d, unused}
__host__ __device__ constexpr int qb_fq_col_bytes(int fq) { return fq * 256 + fq * QB_FQ_REC; }      // operands + records of one column
// NR: results per lane that the batch needs, ceil(rows / 4) (a template parameter: behind a run-time bound every result is a basic
// block of its own, and 16 rows lose 0.7 us)
template <int CPW, int DEPTH, int FQ, int NR = (FQ + 3) / 4, bool Q5 = false>
__global__ __launch_bounds__(QB_NW * 64) void qmb_q4k_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ op, void *__restrict__ dst, int n, int bpr,
                                                              int rows, int dst_dtype, int64_t stride_dst
#ifdef CL_STAMPS
                                                              , uint32_t *stamps
#endif
                                                              ) {
    constexpr int BB = QbW<Q5>::BB, QS = QbW<Q5>::QS;
    constexpr int NIW = qb_tile_instr(CPW, BB);   // copy instructions per wave and tile (those beyond the block copy nothing)
    static_assert((DEPTH - 1) * NIW <= 63 && DEPTH >= 2, "counted waits");
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int bx = blockIdx.x, gx = gridDim.x;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, kg = lane >> 4;
    // wave w takes columns w, w + 8, w + 16: waves w and w + 4 share a SIMD, and where the columns do not fill all waves evenly (12 or 20
    // super-blocks per row) every SIMD gets the same number of them, which contiguous columns per wave do not give
    const int ncols = max(0, min(CPW, (bpr - wv + QB_NW - 1) / QB_NW));
    const int RS = bpr * BB;                   // bytes of a row, in memory and in a tile
    const int block_bytes = 16 * RS;
    const int nkb = (block_bytes + 1023) >> 10;   // KBs of a tile
    const int TILE = qb_tile_bytes(block_bytes);
    float *red = (float *)(lds + DEPTH * TILE);                              // [8 waves][64 lanes][4]

    // ---- the weight stream ----
    const int nsteps = (n + 15) >> 4;
    const int64_t w_bytes = (int64_t)n * RS;
    // instruction t of wave w copies KB number t * 8 + w of the block
    auto issue = [&](int i) {
        const int m = bx + i * gx;
        const bool live = m < nsteps;
        const int64_t off = live ? (int64_t)m * block_bytes : 0;
        const int64_t left = w_bytes - off;
        const int bytes = live ? (int)(left < block_bytes ? left : block_bytes) : 0;      // an absent block: a descriptor of zero bytes
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(w + off), 0, bytes, 0x00020000);
        uint8_t *tile = lds + (i % DEPTH) * TILE;
#pragma unroll
        for (int t = 0; t < NIW; t++) {
            const int kb = min(t * QB_NW + wv, nkb);             // KB number nkb: beyond the block, nothing read, zeros into the spare KB
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (cq_lds_void *)(tile + kb * QB_KB), 16, lane * 16, kb * 1024, 0, 0);
        }
    };
    long A[CPW][8];
    u32x4 aux[CPW][4];                            // {bl 0-3, bl 4-7, bh 0-3, bh 4-7} of slot 4 kg + r (batch row 4 r + kg): sub-block sum j = 128 * bh_j + bl_j
    float d8[CPW][4];
    if constexpr (FQ > 0) {
        // ---- the wave quantizes the activations of its columns itself ----
        // Vector loads complete in order: the activations are asked for before the weights, or they would wait for them.
        const float *x = (const float *)op;
        constexpr int NSP = CPW * FQ;              // the wave's spans: (column ci, batch row r) = span ci * FQ + r
        float xv[NSP][4];
#pragma unroll
        for (int ci = 0; ci < CPW; ci++) {
            const int col = min(wv + QB_NW * ci, bpr - 1);
#pragma unroll
            for (int r = 0; r < FQ; r++) {
                const f32x4 t = *(const f32x4 *)(x + ((int64_t)r * bpr + col) * 256 + lane * 4);
                xv[ci * FQ + r][0] = t.x; xv[ci * FQ + r][1] = t.y; xv[ci * FQ + r][2] = t.z; xv[ci * FQ + r][3] = t.w;
            }
        }
        asm volatile("" ::: "memory");
        issue(0);
        asm volatile("" ::: "memory");
        QB_STAMP(0);
        uint8_t *stage = lds + (DEPTH - 1) * TILE + wv * (CPW * qb_fq_col_bytes(FQ));        // this wave's part of the ring's last tile
        // the streaming kernel's span quantizer (cq_stream.h): the largest magnitudes, one division sequence for all spans, the values
        uint32_t wmax[NSP];
        float iscale[NSP], dsp[NSP];
        // (the six cross-lane steps of all spans side by side: a span's chain alone waits two cycles between steps)
#pragma unroll
        for (int j = 0; j < NSP; j++) {
            float amax = fmaxf(fmaxf(fabsf(xv[j][0]), fabsf(xv[j][1])), fmaxf(fabsf(xv[j][2]), fabsf(xv[j][3])));
            amax = amax == amax ? amax : 0.0f;
            wmax[j] = __float_as_uint(amax);
        }
#define QB_S(ctrl, rm, bc)                                                                                                    \
    _Pragma("unroll") for (int j = 0; j < NSP; j++)                                                                           \
        wmax[j] = max(wmax[j], (uint32_t)__builtin_amdgcn_update_dpp(0, (int)wmax[j], ctrl, rm, 0xf, bc));                    \
    __builtin_amdgcn_sched_barrier(0);
        QB_S(0x111, 0xf, true) QB_S(0x112, 0xf, true) QB_S(0x114, 0xf, true) QB_S(0x118, 0xf, true) QB_S(0x142, 0xa, false) QB_S(0x143, 0xc, false)
#undef QB_S
#pragma unroll
        for (int j = 0; j < NSP; j++) wmax[j] = (uint32_t)__builtin_amdgcn_readlane((int)wmax[j], 63);
        qs_span_scales<NSP>(wmax, lane, iscale, dsp);
        QB_STAMP(14);
        // (the second tile is asked for a little after the first, as in the kernel without the quantizer: asked for together, the
        // first tiles of the late workgroups queue behind the second tiles of the early ones and the launch starts 0.5 us later)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 1; i < DEPTH - 1; i++) issue(i);
        asm volatile("" ::: "memory");
#pragma unroll
        for (int ci = 0; ci < CPW; ci++) {
            uint8_t *colp = stage + ci * qb_fq_col_bytes(FQ), *recs = colp + FQ * 256;
#pragma unroll
            for (int r = 0; r < FQ; r++) {
                const int j = ci * FQ + r;
                int q[4];
#pragma unroll
                for (int i = 0; i < 4; i++) q[i] = qs_round_i8(iscale[j] * xv[j][i]);
                const uint32_t packed = qs_pack4(q);
                *(uint32_t *)(colp + qb_operand_dword(lane, r, FQ)) = packed;
                const int s32 = oct_sum(sdot4(packed, 0x01010101u, 0));       // the sum of the 32-element sub-block, in its eight lanes
                uint8_t *rec = recs + r * QB_FQ_REC;
                // (the eight lanes of a sub-block write the same bytes, every lane the same scale: cheaper than masking lanes off)
                rec[lane >> 3] = (uint8_t)(s32 & 127);
                rec[8 + (lane >> 3)] = (uint8_t)(s32 >> 7);
                *(float *)(rec + 16) = dsp[j];
            }
        }
        // (the wave reads back what it wrote itself: LDS takes a wave's accesses in order)
#pragma unroll
        for (int ci = 0; ci < CPW; ci++) {
            const uint8_t *colp = stage + ci * qb_fq_col_bytes(FQ), *recs = colp + FQ * 256;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                // (staged by batch row; slot c of the operand is batch row qb_slot(c))
                const i64x2 v = qb_slot(c) < FQ ? *(const i64x2 *)(colp + ((g * 4 + kg) * FQ + qb_slot(c)) * 16) : i64x2{0, 0};
                A[ci][2 * g] = v.x; A[ci][2 * g + 1] = v.y;
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint8_t *rec = recs + min(4 * r + kg, FQ - 1) * QB_FQ_REC;         // (results of batch rows beyond the last are not stored)
                aux[ci][r] = *(const u32x4 *)rec;
                d8[ci][r] = *(const float *)(rec + 16);
            }
        }
        // everything is in registers before the wave passes the first barrier, behind which the last tile is asked for
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else {
    issue(0);                                     // the first tile is on its way before anything else is asked for
    asm volatile("" ::: "memory");

    // ---- the wave's activations, in registers for the whole kernel ----
    // The activations are the FIRST matrix operand (lane (c, kg): values 8 kg .. 8 kg + 7 of each sub-block of batch row c) and
    // the weights the second, so a lane's four results belong to ONE weight row (row c of the block: one header to decode per
    // column) and to the slots 4 kg + r (batch rows 4 r + kg), whose block sums and scales it keeps as well.
    QB_STAMP(0);
    // (a wave's load of one operand is 512 contiguous bytes; the four lane groups read four records)
#pragma unroll
    for (int ci = 0; ci < CPW; ci++) {
        const int col = min(wv + QB_NW * ci, bpr - 1);
        const uint8_t *colp = op + (int64_t)col * QB_OP_COL_BYTES + lane * 16;         // lane = kg * 16 + c
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const i64x2 v = qb_slot(c) < rows ? *(const i64x2 *)(colp + g * 1024) : i64x2{0, 0};    // (slots beyond the batch hold zeros)
            A[ci][2 * g] = v.x; A[ci][2 * g + 1] = v.y;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint8_t *rec = op + (int64_t)bpr * QB_OP_COL_BYTES + (int64_t)(col * 16 + 4 * kg + r) * QB_REC_BYTES;
            aux[ci][r] = *(const u32x4 *)rec;
            d8[ci][r] = *(const float *)(rec + 16);
        }
    }
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 1; i < DEPTH - 1; i++) issue(i);
    }
    const int my = bx < nsteps ? (nsteps - bx + gx - 1) / gx : 0;
    QB_STAMP(1);
    for (int i = 0; i < my; i++) {
        // tile i has landed when this wave's copies of it have (at most the later tiles' outstanding) and every other wave's too
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 2) * NIW) : "memory");
        asm volatile("s_barrier" ::: "memory");
        // (behind this barrier every wave has also finished the sums of block i - 1: `red` may be written again, and tile
        // i - 1 is free, which is where tile i + 2 goes)
        issue(i + DEPTH - 1);
        const uint8_t *tile = lds + (i % DEPTH) * TILE;
        if (i < 4) QB_STAMP(2 + 3 * i);
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ci = 0; ci < CPW; ci++) {
            if (ci < ncols) {
                const int o = c * RS + (wv + QB_NW * ci) * BB;                  // weight row c of the block, this column's super-block
                auto at = [&](int off) { return tile + off + (off >> 10) * 16; };      // byte `off` of the block in the padded tile
                const u32x4 hdr = *(const u32x4 *)at(o);
                i32x4 cl[4], ch[4];
                long qh = 0;
                if constexpr (Q5) qh = *(const long *)at(o + 16 + 8 * kg);       // fifth bits of elements 8kg .. 8kg + 7, bit j: sub-block j
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    // bytes 32g + 8kg .. + 7 of qs: low nibbles = sub-block 2g, high nibbles = sub-block 2g + 1
                    const long qa = *(const long *)at(o + QS + 32 * g + 8 * kg);
                    long lo = qa & 0x0f0f0f0f0f0f0f0fl, hi = (qa >> 4) & 0x0f0f0f0f0f0f0f0fl;
                    if constexpr (Q5) {
                        lo |= ((qh >> (2 * g)) & 0x0101010101010101l) << 4;
                        hi |= ((qh >> (2 * g + 1)) & 0x0101010101010101l) << 4;
                    }
                    const i32x4 z = {0, 0, 0, 0};
                    cl[g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(A[ci][2 * g], lo, z, 0, 0, 0);
                    ch[g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(A[ci][2 * g + 1], hi, z, 0, 0, 0);
                }
                const QsScales s = qs_scales_k4(hdr.y, hdr.z, hdr.w);
                int sc[8];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    sc[j] = (int)((s.scA >> (8 * j)) & 0xff);
                    sc[4 + j] = (int)((s.scB >> (8 * j)) & 0xff);
                }
                const float dw = h2f(hdr.x), dm = h2f(hdr.x >> 16);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (r < NR) {                                     // result r belongs to batch rows 4 r .. 4 r + 3
                        int S = 0;
#pragma unroll
                        for (int g = 0; g < 4; g++) S += __mul24(sc[2 * g], cl[g][r]) + __mul24(sc[2 * g + 1], ch[g][r]);
                        const int M = qs_dot_sums(s.mA, s.mB, aux[ci][r]);
                        acc[r] += d8[ci][r] * (dw * (float)S - dm * (float)M);
                    }
                }
            }
        }
        if (i < 4) QB_STAMP(3 + 3 * i);
        // ---- the eight K-slices of the block meet in LDS and are added in wave order ----
        *(f32x4 *)(red + (wv * 64 + lane) * 4) = f32x4{acc[0], acc[1], acc[2], acc[3]};
        // (barriers without the fence of __syncthreads(): the fence would wait for the copies in flight)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (tid < 256) {
            const int l2 = tid & 63, r = tid >> 6;
            float v = 0.0f;
#pragma unroll
            for (int w2 = 0; w2 < QB_NW; w2++) v += red[(w2 * 64 + l2) * 4 + r];
            const int m = bx + i * gx;
            const int row = m * 16 + (l2 & 15), br = 4 * r + (l2 >> 4);
            if (row < n && br < rows) store_out(dst, dst_dtype, (int64_t)br * stride_dst + row, v);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");          // the sums have left LDS before this wave reaches the next barrier
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");               // no copy may land in LDS after the workgroup has left
#ifdef CL_STAMPS
    QB_STAMP(15);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (tid < 128 && stamps) stamps[(bx * 8 + tid / 16) * 16 + tid % 16] = qb_stamp_lds[tid / 16][tid % 16];
#endif
}

// ---- rows of more than 24 super-blocks ------------------------------------------------------------------------------------
// The activations of a whole row no longer fit the registers of eight waves next to their block sums, and a block of 16 such
// rows no longer fits LDS three times.  So a row block is taken in Q column chunks of cpp <= 16 super-blocks (tile = 16 rows x
// one chunk, gathered by the copy instructions from 16 row segments), wave w owns columns 2 w, 2 w + 1 of EVERY chunk and
// keeps their int8 operands in registers (Q x 2 x 16 registers), and the per-row records (block sums, scale) wait in LDS.
// The accumulators run across the chunks of a block; everything else is the kernel above.
template <int Q, int NR, bool Q5 = false>
__global__ __launch_bounds__(QB_NW * 64) void qmb_q4k_long_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ op, void *__restrict__ dst, int n,
                                                                   int bpr, int rows, int dst_dtype, int64_t stride_dst, int cpp
#ifdef CL_STAMPS
                                                                   , uint32_t *stamps
#endif
                                                                   ) {
    constexpr int CPW = 2, DEPTH = 3;
    constexpr int BB = QbW<Q5>::BB, QS = QbW<Q5>::QS;
    constexpr int NIW = qb_tile_instr(CPW, BB);
    static_assert((DEPTH - 1) * NIW <= 63, "counted waits");
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int bx = blockIdx.x, gx = gridDim.x;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, kg = lane >> 4;
    // inside a chunk wave w takes columns w and w + 8 (a short last chunk is spread over all waves, and over the SIMDs evenly)
    const int RS = bpr * BB;                   // bytes of a row in memory
    const int block_bytes = 16 * RS;
    const int TILE = qb_tile_bytes(16 * cpp * BB);
    const int last_cols = bpr - (Q - 1) * cpp;    // columns of the last chunk (1 .. cpp)
    float *red = (float *)(lds + DEPTH * TILE);                              // [8 waves][64 lanes][4]
    uint8_t *recs = (uint8_t *)red + QB_RED_BYTES;                           // [bpr][16 batch slots] records

    const int nsteps = (n + 15) >> 4;
    const int64_t w_bytes = (int64_t)n * RS;
    const int my = bx < nsteps ? (nsteps - bx + gx - 1) / gx : 0;
    const int ntiles = my * Q;
    // instruction t of wave w copies KB number t * 8 + w of the tile; where in the block (less the chunk's first column) its
    // lane's 16 bytes come from, for a full chunk and for the last one:
    int voff_full[NIW], voff_last[NIW];
#pragma unroll
    for (int t = 0; t < NIW; t++) {
        const int tb = (t * QB_NW + wv) * 1024 + lane * 16;
        const int rf = tb / (cpp * BB), rl = tb / (last_cols * BB);
        voff_full[t] = rf < 16 ? rf * RS + (tb - rf * cpp * BB) : block_bytes;            // beyond the tile: out of range, zeros
        voff_last[t] = rl < 16 ? rl * RS + (tb - rl * last_cols * BB) : block_bytes;
    }
    // (Every workgroup takes the chunks in the same order.  Rotating the order by workgroup, so that the launch reads all column
    // ranges of the tensor at any moment instead of the same quarter of every row, was measured a third slower.)
    auto issue = [&](int tau) {
        const int i = tau / Q, q = tau - i * Q;
        const int m = bx + i * gx;
        const bool live = tau < ntiles;
        const int pc = q == Q - 1 ? last_cols : cpp;
        const int64_t off = live ? (int64_t)m * block_bytes + q * cpp * BB : 0;
        const int64_t left = w_bytes - off;
        const int bytes = live ? (int)(left < block_bytes ? left : block_bytes) : 0;      // an absent tile: a descriptor of zero bytes
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(w + off), 0, bytes, 0x00020000);
        uint8_t *tile = lds + (tau % DEPTH) * TILE;
        const int nkb = (16 * pc * BB + 1023) >> 10;
#pragma unroll
        for (int t = 0; t < NIW; t++) {
            const int kb = min(t * QB_NW + wv, nkb);             // KB number nkb: beyond the tile, nothing read, zeros into the spare KB
            const int vo = q == Q - 1 ? voff_last[t] : voff_full[t];
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (cq_lds_void *)(tile + kb * QB_KB), 16, vo, 0, 0, 0);
        }
    };
    issue(0);
    asm volatile("" ::: "memory");
    QB_STAMP(0);
    // the operands into registers, the records (32 bytes per (column, batch slot), at most 4 pieces of 16 bytes per thread)
    // through registers into LDS; the second tile is asked for before anything here is waited for
    // (of the first chunk only: the operands of chunk q + 1 are asked for while chunk q of the first block is worked on --
    // all of them up front would keep the load path busy for 6 us before the second tile could be asked for)
    long A[Q][CPW][8];
    auto load_operands = [&](int q) {
#pragma unroll
        for (int ci = 0; ci < CPW; ci++) {
            const int col = min(q * cpp + wv + QB_NW * ci, bpr - 1);
            const uint8_t *colp = op + (int64_t)col * QB_OP_COL_BYTES + lane * 16;     // lane = kg * 16 + c
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const i64x2 v = qb_slot(c) < rows ? *(const i64x2 *)(colp + g * 1024) : i64x2{0, 0};    // (slots beyond the batch hold zeros)
                A[q][ci][2 * g] = v.x; A[q][ci][2 * g + 1] = v.y;
            }
        }
    };
    load_operands(0);
    const int npieces = bpr * 16 * (QB_REC_BYTES / 16);
    u32x4 rv[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
        rv[j] = *(const u32x4 *)(op + (int64_t)bpr * QB_OP_COL_BYTES + (int64_t)min(tid + j * QB_NW * 64, npieces - 1) * 16);
    asm volatile("" ::: "memory");
    issue(1);
#pragma unroll
    for (int j = 0; j < 4; j++)
        if (tid + j * QB_NW * 64 < npieces) *(u32x4 *)(recs + (tid + j * QB_NW * 64) * 16) = rv[j];
    QB_STAMP(1);
    for (int i = 0; i < my; i++) {
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const int tau = i * Q + q;
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 2) * NIW) : "memory");
            // (lgkmcnt: the first time round, this wave's records are in LDS before anyone passes the barrier)
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            // (in front of the copies: waiting for these operands, one chunk on, then waits for nothing younger than tile tau + 1)
            if (q + 1 < Q && i == 0) load_operands(q + 1 < Q ? q + 1 : 0);
            asm volatile("" ::: "memory");
            issue(tau + DEPTH - 1);
            const uint8_t *tile = lds + (tau % DEPTH) * TILE;
            if (tau < 4) QB_STAMP(2 + 3 * tau);
            const int pc = q == Q - 1 ? last_cols : cpp;
            const int TRS = pc * BB;
#pragma unroll
            for (int ci = 0; ci < CPW; ci++) {
                if (wv + QB_NW * ci < pc) {
                    const int o = c * TRS + (wv + QB_NW * ci) * BB;                 // weight row c of the block, this column's super-block
                    auto at = [&](int off) { return tile + off + (off >> 10) * 16; };      // byte `off` of the tile in its padded form
                    const u32x4 hdr = *(const u32x4 *)at(o);
                    i32x4 cl[4], ch[4];
                    long qh = 0;
                    if constexpr (Q5) qh = *(const long *)at(o + 16 + 8 * kg);
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const long qa = *(const long *)at(o + QS + 32 * g + 8 * kg);
                        long lo = qa & 0x0f0f0f0f0f0f0f0fl, hi = (qa >> 4) & 0x0f0f0f0f0f0f0f0fl;
                        if constexpr (Q5) {
                            lo |= ((qh >> (2 * g)) & 0x0101010101010101l) << 4;
                            hi |= ((qh >> (2 * g + 1)) & 0x0101010101010101l) << 4;
                        }
                        const i32x4 z = {0, 0, 0, 0};
                        cl[g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(A[q][ci][2 * g], lo, z, 0, 0, 0);
                        ch[g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(A[q][ci][2 * g + 1], hi, z, 0, 0, 0);
                    }
                    const QsScales s = qs_scales_k4(hdr.y, hdr.z, hdr.w);
                    int sc[8];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        sc[j] = (int)((s.scA >> (8 * j)) & 0xff);
                        sc[4 + j] = (int)((s.scB >> (8 * j)) & 0xff);
                    }
                    const float dw = h2f(hdr.x), dm = h2f(hdr.x >> 16);
                    const uint8_t *rec = recs + ((q * cpp + wv + QB_NW * ci) * 16 + 4 * kg) * QB_REC_BYTES;
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        if (r < NR) {                                     // result r belongs to batch rows 4 r .. 4 r + 3
                            int S = 0;
#pragma unroll
                            for (int g = 0; g < 4; g++) S += __mul24(sc[2 * g], cl[g][r]) + __mul24(sc[2 * g + 1], ch[g][r]);
                            const u32x4 aux = *(const u32x4 *)(rec + r * QB_REC_BYTES);
                            const float d8 = *(const float *)(rec + r * QB_REC_BYTES + 16);
                            const int M = qs_dot_sums(s.mA, s.mB, aux);
                            acc[r] += d8 * (dw * (float)S - dm * (float)M);
                        }
                    }
                }
            }
            if (tau < 4) QB_STAMP(3 + 3 * tau);
        }
        // ---- the eight K-slices of the block meet in LDS and are added in wave order ----
        *(f32x4 *)(red + (wv * 64 + lane) * 4) = f32x4{acc[0], acc[1], acc[2], acc[3]};
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (tid < 256) {
            const int l2 = tid & 63, r = tid >> 6;
            float v = 0.0f;
#pragma unroll
            for (int w2 = 0; w2 < QB_NW; w2++) v += red[(w2 * 64 + l2) * 4 + r];
            const int m = bx + i * gx;
            const int row = m * 16 + (l2 & 15), br = 4 * r + (l2 >> 4);
            if (row < n && br < rows) store_out(dst, dst_dtype, (int64_t)br * stride_dst + row, v);
        }
        // (the sums have left LDS before this wave passes the next barrier, behind which `red` is written again only after
        // a whole block's chunks: the barrier at the top of the next chunk orders the reads above before those writes)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");               // no copy may land in LDS after the workgroup has left
#ifdef CL_STAMPS
    QB_STAMP(15);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (tid < 128 && stamps) stamps[(bx * 8 + tid / 16) * 16 + tid % 16] = qb_stamp_lds[tid / 16][tid % 16];
#endif
}

// LDS of the chunked-row kernel: three tiles of a chunk, the partial results, the records of a whole row of operands
constexpr size_t qb_long_lds(int64_t bpr, int cpp, int bb) { return (size_t)3 * qb_tile_bytes(16 * cpp * bb) + QB_RED_BYTES + (size_t)bpr * 16 * QB_REC_BYTES; }
template <int Q, int NR, bool Q5>
int launch_qmb_long_r(const void *w, const uint8_t *op, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, int cpp,
                      hipStream_t s) {
    const int64_t bpr = k / 256;
    const size_t lds_bytes = qb_long_lds(bpr, cpp, qb_bb(Q5));
    if (lds_bytes > (size_t)QB_LDS_BYTES - 1024) return CQ_ERR_RANGE;
    auto kern = qmb_q4k_long_kernel<Q, NR, Q5>;
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
    const int64_t nsteps = (n + 15) / 16;
    // every workgroup the same number of blocks where that is possible with at most one workgroup per CU (896 blocks: 224 x 4)
    const unsigned grid = (unsigned)(nsteps < 256 ? nsteps : (nsteps + (nsteps + 255) / 256 - 1) / ((nsteps + 255) / 256));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(QB_NW * 64), lds_bytes, s, (const uint8_t *)w, op, dst, (int)n, (int)bpr, (int)rows, dst_dtype, stride_dst,
                       cpp
#ifdef CL_STAMPS
                       , qb_stamps_dev
#endif
    );
    return (int)hipGetLastError();
}

template <int Q, bool Q5>
int launch_qmb_long(const void *w, const uint8_t *op, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, int cpp,
                    hipStream_t s) {
    switch ((rows + 3) / 4) {
        case 1: return launch_qmb_long_r<Q, 1, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, cpp, s);
        case 2: return launch_qmb_long_r<Q, 2, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, cpp, s);
        case 3: return launch_qmb_long_r<Q, 3, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, cpp, s);
        default: return launch_qmb_long_r<Q, 4, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, cpp, s);
    }
}

template <int CPW, int DEPTH, int FQ, int NR, bool Q5>
int launch_qmb_dr(const void *w, const uint8_t *op, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, size_t lds_bytes,
                  hipStream_t s) {
    auto kern = qmb_q4k_kernel<CPW, DEPTH, FQ, NR, Q5>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    const int64_t nsteps = (n + 15) / 16;
    // every workgroup the same number of blocks where that is possible with at most one workgroup per CU (896 blocks: 224 x 4)
    const unsigned grid = (unsigned)(nsteps < 256 ? nsteps : (nsteps + (nsteps + 255) / 256 - 1) / ((nsteps + 255) / 256));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(QB_NW * 64), lds_bytes, s, (const uint8_t *)w, op, dst, (int)n, (int)(k / 256), (int)rows, dst_dtype,
                       stride_dst
#ifdef CL_STAMPS
                       , qb_stamps_dev
#endif
    );
    return (int)hipGetLastError();
}
template <int CPW, int DEPTH, bool Q5, int FQ = 0>
int launch_qmb_d(const void *w, const uint8_t *op, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, size_t lds_bytes,
                 hipStream_t s) {
    if constexpr (FQ > 0) return launch_qmb_dr<CPW, DEPTH, FQ, (FQ + 3) / 4, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, lds_bytes, s);
    switch ((rows + 3) / 4) {
        case 1: return launch_qmb_dr<CPW, DEPTH, 0, 1, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, lds_bytes, s);
        case 2: return launch_qmb_dr<CPW, DEPTH, 0, 2, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, lds_bytes, s);
        case 3: return launch_qmb_dr<CPW, DEPTH, 0, 3, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, lds_bytes, s);
        default: return launch_qmb_dr<CPW, DEPTH, 0, 4, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, lds_bytes, s);
    }
}
// Three tiles where LDS holds them (the one being worked on and two on their way), else two.  (Four were measured slower:
// with three tiles asked for at the start the first one lands 1 us later, and the steady state gains nothing.)
// fq: `op` holds the f32 activations (see the kernel); the caller has checked qb_fused_rows
template <int CPW, bool Q5>
int launch_qmb(const void *w, const uint8_t *op, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, int fq, hipStream_t s) {
    const int tile = qb_tile_bytes((int)(16 * (k / 256) * qb_bb(Q5)));
    const int fit = (QB_LDS_BYTES - QB_RED_BYTES - 1024) / tile;
#define QB_FQ_CASE(R)                                                                                                                           \
    case R:                                                                                                                                    \
        if constexpr (CPW * R <= QB_FQ_MAX_SPANS) {                                                                                            \
            if (fit >= 3) return launch_qmb_d<CPW, 3, Q5, R>(w, op, dst, dst_dtype, k, n, rows, stride_dst, (size_t)3 * tile + QB_RED_BYTES, s);  \
            if (fit == 2) return launch_qmb_d<CPW, 2, Q5, R>(w, op, dst, dst_dtype, k, n, rows, stride_dst, (size_t)2 * tile + QB_RED_BYTES, s);  \
        }                                                                                                                                      \
        return CQ_ERR_RANGE;
    switch (fq) {
        QB_FQ_CASE(3) QB_FQ_CASE(4) QB_FQ_CASE(5) QB_FQ_CASE(6) QB_FQ_CASE(7) QB_FQ_CASE(8)
        default: break;
    }
#undef QB_FQ_CASE
    if (fit >= 3) return launch_qmb_d<CPW, 3, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, (size_t)3 * tile + QB_RED_BYTES, s);
    if (fit == 2) return launch_qmb_d<CPW, 2, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, (size_t)2 * tile + QB_RED_BYTES, s);
    return CQ_ERR_RANGE;
}


// ---- the expert-grouped form (MoE with hundreds of pairs) -----------------------------------------------------------------
// Every expert hit by at most a few dozen pairs is a batched matvec of its own: its pairs are the batch rows (sets of 16, two
// sets held in registers per pass over the weights), its matrix the weight stream.  What bounds such a launch is how evenly the
// experts' bytes are spread over the CUs (a CU streams about 20 KB per us through the copy-to-LDS path): workgroup
// (part, expert, tensor) takes a contiguous range of the expert's row tiles, with parts x experts x tensors a multiple of the
// CU count where the shape allows, and leaves at once when the expert has no pair.
//
// Short rows.  With fewer than eight super-blocks per row the waves do not all get a column: CW waves (a power of two) share a
// block of 16 rows, wave w taking columns (w / NRB) * CPW .. of row block w % NRB of a tile of NRB = 8 / CW row blocks.
//
// Operands.  Tile (expert e, set s) — pairs offsets[e] + 16 s .. of the expert-sorted pair list — lives at tile index
// offsets[e] / 16 + e + s (unique and below n_pairs / 16 + experts without a scan over the experts), laid out like one column
// set of the dense kernel: [column][g][kg][slot][16 bytes], then [column][slot] records.
// Pair b of a set sits in operand slot 4 (b % 4) + b / 4: a lane's result r of lane group kg then belongs to pair 4 r + kg, and a
// set of `cnt` pairs needs only the first ceil(cnt / 4) of a lane's four results worked out (the scaling of a result is most of
// the kernel's vector work, and most sets are far from full).
__host__ __device__ constexpr int qme_slot(int b) { return qb_slot(b); }
constexpr int QME_TILE_COL_BYTES = QB_OP_COL_BYTES + 16 * QB_REC_BYTES;          // 4608 bytes of a tile per super-block column
__host__ __device__ inline int64_t qme_operand_tiles(int64_t n_pairs, int64_t num_experts) { return n_pairs / 16 + num_experts + 1; }

// workgroup (chunk of the grouping pass, column): one wave per pair of the chunk (16 sorted pairs of one expert at most) quantizes
// the pair's 256 values of the column, gathered through row_map, into the chunk's operand tile — the streaming kernel's span
// quantizer (cq_stream.h: where the first largest magnitude is negative the int8 values and the scale come out with the other
// sign than BlockQ8K::from_float gives them, and every product is the same).  SW: the rows are silu(x[row]) * up[row], and the
// pair's scale is scale_in[row] (the down projection after gate / up: one row per pair).  The kernel is a chain of four memory
// trips (chunk, row index, values, store); a wave that takes several columns in turn makes it longer, not shorter.
template <bool SW>
__global__ __launch_bounds__(1024) void qme_quantize_kernel(const float *__restrict__ x, const float *__restrict__ up, const int *__restrict__ row_map,
                                                            const float *__restrict__ scale_in, float *__restrict__ scale_out,
                                                            const int *__restrict__ chunks, int max_chunks, const int *__restrict__ offsets,
                                                            uint8_t *__restrict__ op, int bpr, int64_t x_stride, int64_t up_stride) {
    const int ci = blockIdx.x, col = blockIdx.y;
    const int lane = threadIdx.x & 63, c = threadIdx.x >> 6;
    int tile;
    int64_t row;
    int first = 16 * ci;
    if (chunks) {
        // (the four words of the chunk in one trip: entries behind the last chunk hold anything and are not used)
        const int n_chunks = chunks[0], e = chunks[1 + ci], count = chunks[1 + 2 * max_chunks + ci];
        first = chunks[1 + max_chunks + ci];
        if (ci >= n_chunks || c >= count) return;
        const int seg0 = offsets[e];
        tile = (seg0 >> 4) + e + ((first - seg0) >> 4);
        row = row_map[first + c];
    } else {
        // one matrix, the rows as they are (max_chunks: the number of rows): chunk ci is rows 16 ci .. of tile ci
        if (first + c >= max_chunks) return;
        tile = ci;
        row = first + c;
    }
    uint8_t *tp = op + (int64_t)tile * bpr * QME_TILE_COL_BYTES;
    if (SW && scale_out && col == 0 && lane == 0) scale_out[first + c] = scale_in[row];
    float v[1][4];
    if constexpr (SW) cq_load_swiglu4(x, up, row * x_stride + col * 256 + lane * 4, row * up_stride + col * 256 + lane * 4, v[0]);
    else cq_load4<CQ_F32>(x, row * x_stride + col * 256 + lane * 4, v[0]);
    const uint32_t wmax[1] = {qs_span_umax(v[0])};
    float iscale[1], d[1];
    qs_span_scales<1>(wmax, lane, iscale, d);
    int q[4];
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = qs_round_i8(iscale[0] * v[0][i]);
    const uint32_t packed = qs_pack4(q);
    const int slot = qme_slot(c);
    *(uint32_t *)(tp + col * QB_OP_COL_BYTES + qb_operand_dword(lane, slot, 16)) = packed;
    const int s32 = oct_sum(sdot4(packed, 0x01010101u, 0));
    uint8_t *rec = tp + bpr * QB_OP_COL_BYTES + (col * 16 + slot) * QB_REC_BYTES;
    if ((lane & 7) == 0) { rec[lane >> 3] = (uint8_t)(s32 & 127); rec[8 + (lane >> 3)] = (uint8_t)(s32 >> 7); }
    if (lane == 0) *(float *)(rec + 16) = d[0];
}

#ifdef CL_STAMPS
__device__ uint32_t *qme_stamps;
#endif
struct QmeArgs {
    const uint8_t *w[2];          // [experts][n][bpr] super-blocks each
    float *out[2];                // [pairs][n]
    const uint8_t *op;
    const int *offsets;           // [experts + 1]: expert e's pairs are offsets[e] .. offsets[e + 1] of the sorted list
    const int *pair_out;          // output row of a sorted pair
    const float *pair_scale;      // and the factor on its results
    int n, bpr, parts;
    int dense_rows;               // > 0: one matrix and rows 0 .. dense_rows - 1 as its pairs (no offsets, output row = pair, factor 1)
    int *extra;                   // n | two counters | (expert, pass)[n]: the passes beyond an expert's first; NULL: every workgroup runs all passes of its expert
    int extra_slot;               // which of the two counters this launch counts with
    int extra_parts;              // parts per expert and tensor that a listed pass is cut into (a multiple of parts: finer than a workgroup's own share)
};
constexpr int QME_NS = 2;         // sets of 16 pairs per pass over the weights
constexpr int QME_MAX_AVG_PAIRS = 64;   // pairs per expert on average up to which a call takes this form
constexpr int QME_DEPTH = 4;      // tiles of the ring where LDS holds them

template <int CW, int CPW, int DEPTH, bool Q5 = false>
__global__ __launch_bounds__(QB_NW * 64) void qme_q4k_kernel(const QmeArgs a) {
    constexpr int BB = QbW<Q5>::BB, QS = QbW<Q5>::QS;
    constexpr int NRB = QB_NW / CW;                                        // row blocks of a tile
    constexpr int NIW = (16 * NRB * CW * CPW * BB + 8 * 1024 - 1) / (8 * 1024);      // copy instructions per wave and tile
    static_assert((DEPTH - 1) * NIW <= 63 && DEPTH >= 2, "counted waits");
    extern __shared__ __align__(16) uint8_t lds[];
    int e = blockIdx.y;
    QB_STAMP(0);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, kg = lane >> 4;
    // wave w: row block w % NRB, column group w / NRB.  Waves w and w + 4 share a SIMD, and where the last column group holds fewer
    // columns (rows of 3 super-blocks: two columns and one) every SIMD then gets a heavy and a light wave instead of two of a kind.
    const int rb = wv % NRB, col0 = (wv / NRB) * CPW;
    const int n = a.n, bpr = a.bpr;
    const int ncols = max(0, min(CPW, bpr - col0));
    const int RS = bpr * BB;
    const int block_bytes = 16 * NRB * RS;
    const int nkb = (block_bytes + 1023) >> 10;
    const int TILE = qb_tile_bytes(block_bytes);
    float *red = (float *)(lds + DEPTH * TILE);                            // [2][sets][8 waves][64 lanes][4]
    constexpr int REC_KB = (CW * CPW * 16 * QB_REC_BYTES + 1023) / 1024;   // KBs of the records of one set (at most CW * CPW columns)
    uint8_t *recs = lds + DEPTH * TILE + 2 * QME_NS * QB_RED_BYTES;        // [sets][REC_KB KB], one spare KB
    const int ntiles = (n + 16 * NRB - 1) / (16 * NRB);
    const int64_t w_bytes = (int64_t)n * RS;
    // what the workgroup works on: expert e, tensor, tiles t0 .. t0 + my - 1 of the expert's matrix (its own share first; then, where
    // a list of further passes exists, whatever it draws from that list)
    const uint8_t *w;
    float *out;
    int t0, my;
    auto place = [&](int ee, int tensor, int part, int nparts) {
        e = ee;
        w = a.w[tensor] + (int64_t)ee * n * RS;
        out = a.out[tensor];
        t0 = (int)((int64_t)part * ntiles / nparts);
        my = (int)((int64_t)(part + 1) * ntiles / nparts) - t0;
    };
    place(blockIdx.y, blockIdx.z, blockIdx.x, a.parts);
    __shared__ int drawn;
    int seq = 0;                                                           // tiles asked for so far, over all passes: the ring slot
    auto issue = [&](int i) {                                              // tile t0 + i of this pass (nothing beyond the range)
        const bool live = i < my;
        const int64_t off = live ? (int64_t)(t0 + i) * block_bytes : 0;
        const int64_t left = w_bytes - off;
        const int bytes = live ? (int)(left < block_bytes ? left : block_bytes) : 0;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(w + off), 0, bytes, 0x00020000);
        uint8_t *tile = lds + (seq % DEPTH) * TILE;
        seq++;
#pragma unroll
        for (int t = 0; t < NIW; t++) {
            const int kb = min(t * QB_NW + wv, nkb);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (cq_lds_void *)(tile + kb * QB_KB), 16, lane * 16, kb * 1024, 0, 0);
        }
    };
    // The first tile is asked for before the expert's pair range is known (a memory trip): where the weights are does not
    // depend on it.  An expert without pairs waits for those copies and leaves.
    issue(0);
    asm volatile("" ::: "memory");
    int seg0 = a.dense_rows ? 0 : a.offsets[e], seg1 = a.dense_rows ? a.dense_rows : a.offsets[e + 1];
    const int n_extra = a.extra ? a.extra[0] : 0;
    // one pass over tiles t0 .. of expert e's matrix against sets sg, sg + 1 of its pairs; issued0: the first tile is on its way
    auto run_pass = [&](const int sg, const bool issued0) {
        const int nsets = (seg1 - seg0 + 15) >> 4;
        // (a pass starts behind the barrier that ended the one before: every tile of the ring is free)
        const int sets_here = min(QME_NS, nsets - sg);
        // The records of the pass (block sums and scales of every pair and column) go to LDS by copy instructions ahead of the
        // first tile, whose wait covers them: loaded by every lane from memory they were 2/3 of the wave's operand requests,
        // sixteen lanes asking for the same 20 bytes, and the waves took 4 us to get their requests out.
#pragma unroll
        for (int t = 0; t < (QME_NS * REC_KB + QB_NW - 1) / QB_NW; t++) {
            const int j = t * QB_NW + wv, st = j / REC_KB, piece = j - st * REC_KB;
            const bool live = st < sets_here;
            const int tile = (seg0 >> 4) + e + sg + (live ? st : 0);
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(a.op + (int64_t)tile * bpr * QME_TILE_COL_BYTES + bpr * QB_OP_COL_BYTES), 0, live ? bpr * 16 * QB_REC_BYTES : 0, 0x00020000);
            // (a copy for a set that does not exist carries no bytes and writes zeros: into a spare KB behind the records)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (cq_lds_void *)(recs + (live ? st * REC_KB + piece : QME_NS * REC_KB) * 1024), 16, lane * 16,
                                                     piece * 1024, 0, 0);
        }
        if (!issued0) issue(0);
        asm volatile("" ::: "memory");
        int rounds[QME_NS];                                                // results per lane a set needs: ceil(pairs / 4)
#pragma unroll
        for (int st = 0; st < QME_NS; st++) rounds[st] = (min(16, max(0, seg1 - seg0 - (sg + st) * 16)) + 3) >> 2;
        long A[QME_NS][CPW][8];
        long Abl[QME_NS][CPW], Abh[QME_NS][CPW];          // the block sums of slot c (sum j = 128 * bh_j + bl_j) as matrix operands: lane group 0 only
        float d8[QME_NS][CPW][4];
#pragma unroll
        for (int st = 0; st < QME_NS; st++) {
            const int cnt = min(16, seg1 - seg0 - (sg + st) * 16);         // pairs of this set (<= 0: the set does not exist)
            const int tile = (seg0 >> 4) + e + min(sg + st, nsets - 1);
            const uint8_t *tp = a.op + (int64_t)tile * bpr * QME_TILE_COL_BYTES;
#pragma unroll
            for (int ci = 0; ci < CPW; ci++) {
                const int col = min(col0 + ci, bpr - 1);
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const i64x2 v = qme_slot(c) < cnt ? *(const i64x2 *)(tp + col * QB_OP_COL_BYTES + g * 1024 + lane * 16) : i64x2{0, 0};
                    A[st][ci][2 * g] = v.x; A[st][ci][2 * g + 1] = v.y;
                }
            }
        }
        // the pair this thread stores at the end of every tile: set tid / 256, result r of lane group l2 / 16 = pair 4 r + l2 / 16
        const int oset = tid >> 8, ol2 = tid & 63, orr = (tid >> 6) & 3;
        const int opos = seg0 + (sg + oset) * 16 + 4 * orr + (ol2 >> 4);
        const bool ovalid = opos < seg1;
        const int64_t orow = !ovalid ? 0 : a.dense_rows ? opos : a.pair_out[opos];
        const float oscale = !ovalid ? 0.0f : a.dense_rows ? 1.0f : a.pair_scale[opos];
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 1; i < DEPTH - 1; i++) issue(i);
        // One barrier per tile: behind it tile i has landed for every wave, and every wave has left its partial results of tile
        // i - 1 in red[(i - 1) % 2], which 8 threads per result add up and store while the waves go on with tile i.
        QB_STAMP(1);
        for (int i = 0; i <= my; i++) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 2) * NIW) : "memory");
            if (i < 4) QB_STAMP(2 + 3 * i);
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            if (i < 4) QB_STAMP(3 + 3 * i);
            if (i == 0) {
                // the lane's records, now in LDS: slot 4 kg + r holds pair 4 r + kg
#pragma unroll
                for (int st = 0; st < QME_NS; st++) {
                    const int cnt = min(16, seg1 - seg0 - (sg + st) * 16);
#pragma unroll
                    for (int ci = 0; ci < CPW; ci++) {
                        const int col = min(col0 + ci, bpr - 1);
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            const uint8_t *rec = recs + min(st, sets_here - 1) * (REC_KB * 1024) + (col * 16 + 4 * kg + r) * QB_REC_BYTES;
                            const float td = *(const float *)(rec + 16);
                            d8[st][ci][r] = 4 * r + kg < cnt ? td : 0.0f;
                        }
                        const i64x2 sums = *(const i64x2 *)(recs + min(st, sets_here - 1) * (REC_KB * 1024) + (col * 16 + c) * QB_REC_BYTES);
                        const bool mine = kg == 0 && qme_slot(c) < cnt;
                        Abl[st][ci] = mine ? sums.x : 0;
                        Abh[st][ci] = mine ? sums.y : 0;
                    }
                }
            }
            if (i > 0 && ovalid) {
                const float *rd = red + ((i - 1) & 1) * (QME_NS * QB_NW * 64 * 4);
#pragma unroll
                for (int g = 0; g < NRB; g++) {
                    float v = 0.0f;
#pragma unroll
                    for (int w2 = 0; w2 < CW; w2++) v += rd[((oset * QB_NW + w2 * NRB + g) * 64 + ol2) * 4 + orr];
                    const int row = ((t0 + i - 1) * NRB + g) * 16 + (ol2 & 15);
                    if (row < n) out[orow * n + row] = v * oscale;
                }
            }
            if (i == my) break;
            const uint8_t *tile = lds + ((seq - (DEPTH - 1)) % DEPTH) * TILE;       // tile i of this pass
            issue(i + DEPTH - 1);
            float acc[QME_NS][4];
#pragma unroll
            for (int st = 0; st < QME_NS; st++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[st][r] = 0.0f;
#pragma unroll
            for (int ci = 0; ci < CPW; ci++) {
                if (ci < ncols) {
                    const int o = (rb * 16 + c) * RS + (col0 + ci) * BB;
                    auto at = [&](int off) { return tile + off + (off >> 10) * 16; };
                    const u32x4 hdr = *(const u32x4 *)at(o);
                    long lo[4], hi[4];
                    long qh = 0;
                    if constexpr (Q5) qh = *(const long *)at(o + 16 + 8 * kg);       // fifth bits of elements 8kg .. 8kg + 7, bit j: sub-block j
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const long qa = *(const long *)at(o + QS + 32 * g + 8 * kg);
                        lo[g] = qa & 0x0f0f0f0f0f0f0f0fl; hi[g] = (qa >> 4) & 0x0f0f0f0f0f0f0f0fl;
                        if constexpr (Q5) {
                            lo[g] |= ((qh >> (2 * g)) & 0x0101010101010101l) << 4;
                            hi[g] |= ((qh >> (2 * g + 1)) & 0x0101010101010101l) << 4;
                        }
                    }
                    const QsScales s = qs_scales_k4(hdr.y, hdr.z, hdr.w);
                    int sc[8];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        sc[j] = (int)((s.scA >> (8 * j)) & 0xff);
                        sc[4 + j] = (int)((s.scB >> (8 * j)) & 0xff);
                    }
                    const float dw = h2f(hdr.x), dm = h2f(hdr.x >> 16);
                    // The minimum term sum_j m_j * (sub-block sum j of the pair) is a product of its own — the row's eight 6-bit
                    // minima against the pair's eight sums, split 128 * bh + bl into bytes — and goes to the matrix cores as
                    // well: two instructions per set and column instead of six vector instructions per result.
                    const long mins = kg == 0 ? (long)(((uint64_t)s.mB << 32) | s.mA) : 0;
#pragma unroll
                    for (int st = 0; st < QME_NS; st++) {
                        if (st >= sets_here) continue;
                        i32x4 cl[4], ch[4];
                        const i32x4 z = {0, 0, 0, 0};
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            cl[g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(A[st][ci][2 * g], lo[g], z, 0, 0, 0);
                            ch[g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(A[st][ci][2 * g + 1], hi[g], z, 0, 0, 0);
                        }
                        const i32x4 ml = __builtin_amdgcn_mfma_i32_16x16x32_i8(Abl[st][ci], mins, z, 0, 0, 0);
                        const i32x4 mh = __builtin_amdgcn_mfma_i32_16x16x32_i8(Abh[st][ci], mins, z, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            if (r < rounds[st]) {
                                int S = __mul24(sc[0], cl[0][r]);
                                S = __mul24(sc[1], ch[0][r]) + S;
#pragma unroll
                                for (int g = 1; g < 4; g++) {
                                    S = __mul24(sc[2 * g], cl[g][r]) + S;
                                    S = __mul24(sc[2 * g + 1], ch[g][r]) + S;
                                }
                                const int M = (mh[r] << 7) + ml[r];
                                acc[st][r] += d8[st][ci][r] * (dw * (float)S - dm * (float)M);
                            }
                        }
                    }
                }
            }
            if (i < 4) QB_STAMP(4 + 3 * i);
            float *rw = red + (i & 1) * (QME_NS * QB_NW * 64 * 4);
#pragma unroll
            for (int st = 0; st < QME_NS; st++)
                *(f32x4 *)(rw + ((st * QB_NW + wv) * 64 + lane) * 4) = f32x4{acc[st][0], acc[st][1], acc[st][2], acc[st][3]};
        }
        // the copies beyond the range carried no bytes, but they count: nothing may be outstanding when the next pass counts again
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    };
    if (seg0 >= seg1) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");           // (the first tile of an expert without pairs: wait, then nothing)
    } else if (a.extra) {
        run_pass(0, true);
    } else {
        for (int sg = 0; 16 * sg < seg1 - seg0; sg += QME_NS) run_pass(sg, sg == 0);
    }
    // Further passes of experts with more than 32 pairs: (expert, pass) items x tensors x parts, drawn from a counter by whichever
    // workgroup has finished what it had, in pieces finer than a workgroup's own share (a router is rarely balanced: with a static
    // split the launch would wait for the workgroups of its most loaded expert).  Every draw is one atomic; the loop ends with the first draw beyond the list.
    if (n_extra > 0) {
        const int per_item = a.extra_parts * (int)gridDim.z, total = n_extra * per_item;
        for (;;) {
            if (tid == 0) drawn = __hip_atomic_fetch_add(a.extra + 1 + a.extra_slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            const int idx = drawn;
            if (idx >= total) break;
            const int item = idx / per_item, rem = idx - item * per_item;
            place(a.extra[CQ_MOE_EXTRA_HEADER + 2 * item], rem / a.extra_parts, rem % a.extra_parts, a.extra_parts);
            seg0 = a.offsets[e];
            seg1 = a.offsets[e + 1];
            // (every wave has read `drawn` before any of them passes the first barrier of the pass, and thread 0 writes it again
            // only behind the last one)
            run_pass(a.extra[CQ_MOE_EXTRA_HEADER + 2 * item + 1] * QME_NS, false);
        }
    }
#ifdef CL_STAMPS
    QB_STAMP(15);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (tid < 128 && qme_stamps) qme_stamps[((blockIdx.y * gridDim.x + blockIdx.x) * 8 + tid / 16) * 16 + tid % 16] = qb_stamp_lds[tid / 16][tid % 16];
#endif
}

template <int CW, int CPW, int DEPTH, bool Q5>
int launch_qme_d(const QmeArgs &a, int64_t num_experts, int tensors, size_t lds_bytes, hipStream_t s) {
    auto kern = qme_q4k_kernel<CW, CPW, DEPTH, Q5>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)a.parts, (unsigned)num_experts, (unsigned)tensors), dim3(QB_NW * 64), lds_bytes, s, a);
    return (int)hipGetLastError();
}
template <int CW, int CPW, bool Q5>
int launch_qme(const QmeArgs &a, int64_t num_experts, int tensors, hipStream_t s) {
    const int tile = qb_tile_bytes(16 * (QB_NW / CW) * a.bpr * qb_bb(Q5));
    const int red = 2 * QME_NS * QB_RED_BYTES + (QME_NS * ((CW * CPW * 16 * QB_REC_BYTES + 1023) / 1024) + 1) * 1024;      // partial results, records
    const int fit = (QB_LDS_BYTES - red - 1024) / tile;
    if (fit >= QME_DEPTH) return launch_qme_d<CW, CPW, QME_DEPTH, Q5>(a, num_experts, tensors, (size_t)QME_DEPTH * tile + red, s);
    if (fit >= 3) return launch_qme_d<CW, CPW, 3, Q5>(a, num_experts, tensors, (size_t)3 * tile + red, s);
    if (fit == 2) return launch_qme_d<CW, CPW, 2, Q5>(a, num_experts, tensors, (size_t)2 * tile + red, s);
    return CQ_ERR_RANGE;
}

}  // namespace

// Does the batched matrix-core matvec take this call?  Q4_K or Q5_K, 3 .. 16 rows, rows of up to 64 super-blocks (k <= 16384:
// up to 24 with three columns per wave, beyond that in up to four column chunks, which is what a wave's registers hold of a
// row; Q5_K's larger tiles leave room for the records of up to 56 super-blocks beside them).
constexpr int QB_MAX_BPR = 64;        // (and 64 x 16 records of 32 bytes are 4 pieces of 16 bytes per thread)
static bool qb_weights(int w_dtype) { return w_dtype == CQ_Q4K || w_dtype == CQ_Q5K; }
// the chunked-row kernel's split of a row: chunks of at most 16 super-blocks, all about the same size
// Full chunks of 16 super-blocks and a shorter last one where LDS holds three such tiles beside the records (every wave then has two
// columns in all chunks but the last: with chunks of equal size, 14 for rows of 56 super-blocks, the eighth wave has none and its
// SIMD half the work of the others); else chunks of about the same size.
static int qb_long_cpp(int64_t bpr, int bb) {
    const int64_t chunks = (bpr + 2 * QB_NW - 1) / (2 * QB_NW);
    if (qb_long_lds(bpr, 2 * QB_NW, bb) <= (size_t)QB_LDS_BYTES - 1024) return 2 * QB_NW;
    return (int)((bpr + chunks - 1) / chunks);
}
static bool qb_row_fits(int w_dtype, int64_t bpr) {
    return bpr >= 1 && bpr <= QB_MAX_BPR && (bpr <= 3 * QB_NW || qb_long_lds(bpr, qb_long_cpp(bpr, qb_bb(w_dtype == CQ_Q5K)), qb_bb(w_dtype == CQ_Q5K)) <= (size_t)QB_LDS_BYTES - 1024);
}
bool cq_matvec_batch_takes(int w_dtype, const void *w, int64_t k, int64_t n, int64_t rows) {
    return qb_weights(w_dtype) && rows >= 3 && rows <= 16 && k % 256 == 0 && qb_row_fits(w_dtype, k / 256) && n >= 1 && n <= 0x7ffffff0 / 16 &&
           n * (k / 256) * qb_bb(w_dtype == CQ_Q5K) < 0x7fffffffLL && ((uintptr_t)w & 15) == 0;
}
// bytes of workspace the call needs (the activations as matrix operands); 0 when the shape can never take this path
int64_t cq_matvec_batch_workspace(int w_dtype, int64_t k, int64_t rows) {
    return qb_weights(w_dtype) && rows >= 3 && rows <= 16 && k % 256 == 0 && qb_row_fits(w_dtype, k / 256) ? cq_align256(qb_operand_bytes(k / 256)) : 0;
}

// Rows the main kernel quantizes itself (= rows), 0: the quantize kernel runs first.  Contiguous f32 rows of up to
// 24 super-blocks, at most 8 of them and at most QB_FQ_MAX_SPANS spans per wave, and the staged operands of the eight waves
// must fit one tile of the ring.
static int qb_fused_rows(int w_dtype, int x_dtype, const void *x, int64_t x_stride, int64_t k, int64_t rows) {
    const int64_t bpr = k / 256, cpw = (bpr + QB_NW - 1) / QB_NW;
    if (x_dtype != CQ_F32 || x_stride != k || bpr > 3 * QB_NW || rows > 8 || cpw * rows > QB_FQ_MAX_SPANS || ((uintptr_t)x & 15)) return 0;
    const int fq = (int)rows;
    const int tile = qb_tile_bytes((int)(16 * bpr * qb_bb(w_dtype == CQ_Q5K)));
    if ((QB_LDS_BYTES - QB_RED_BYTES - 1024) / tile < 2) return 0;
    return QB_NW * cpw * qb_fq_col_bytes(fq) <= tile ? fq : 0;
}

// QMatMul::forward for 3 .. 16 rows of x: one small kernel quantizes them into `workspace`, then the weights are read once.
// x_dtype < 0: the rows are silu(x) * up, f32, with row strides in floats (multiples of 4).
template <bool Q5>
static int qb_launch_w(int w_dtype, const void *w, const void *x, const float *up, int64_t x_stride, int64_t up_stride, int x_dtype, void *workspace,
                       void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, hipStream_t s) {
    if (!cq_matvec_batch_takes(w_dtype, w, k, n, rows)) return CQ_ERR_RANGE;
    const int bpr = (int)(k / 256);
    const int64_t cpw = (k / 256 + QB_NW - 1) / QB_NW;
    if (const int fq = qb_fused_rows(w_dtype, x_dtype, x, x_stride, k, rows)) {
        switch (cpw) {
            case 1: return launch_qmb<1, Q5>(w, (const uint8_t *)x, dst, dst_dtype, k, n, rows, stride_dst, fq, s);
            case 2: return launch_qmb<2, Q5>(w, (const uint8_t *)x, dst, dst_dtype, k, n, rows, stride_dst, fq, s);
            case 3: return launch_qmb<3, Q5>(w, (const uint8_t *)x, dst, dst_dtype, k, n, rows, stride_dst, fq, s);
            default: return CQ_ERR_RANGE;
        }
    }
    const unsigned qgrid = (unsigned)((bpr * 16 + 3) / 4);
    uint8_t *op = (uint8_t *)workspace;
    switch (x_dtype) {
        case -1: hipLaunchKernelGGL(qb_quantize_kernel<-1>, dim3(qgrid), dim3(256), 0, s, x, up, x_stride, up_stride, op, bpr, (int)rows); break;
        case CQ_F32: hipLaunchKernelGGL(qb_quantize_kernel<CQ_F32>, dim3(qgrid), dim3(256), 0, s, x, up, x_stride, up_stride, op, bpr, (int)rows); break;
        case CQ_F16: hipLaunchKernelGGL(qb_quantize_kernel<CQ_F16>, dim3(qgrid), dim3(256), 0, s, x, up, x_stride, up_stride, op, bpr, (int)rows); break;
        case CQ_BF16: hipLaunchKernelGGL(qb_quantize_kernel<CQ_BF16>, dim3(qgrid), dim3(256), 0, s, x, up, x_stride, up_stride, op, bpr, (int)rows); break;
        default: return CQ_ERR_DTYPE;
    }
    if (bpr > 3 * QB_NW) {
        const int chunks = (bpr + 2 * QB_NW - 1) / (2 * QB_NW), cpp = qb_long_cpp(bpr, qb_bb(Q5));
        switch (chunks) {
            case 2: return launch_qmb_long<2, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, cpp, s);
            case 3: return launch_qmb_long<3, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, cpp, s);
            case 4: return launch_qmb_long<4, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, cpp, s);
            default: return CQ_ERR_RANGE;
        }
    }
    switch (cpw) {
        case 1: return launch_qmb<1, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, 0, s);
        case 2: return launch_qmb<2, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, 0, s);
        case 3: return launch_qmb<3, Q5>(w, op, dst, dst_dtype, k, n, rows, stride_dst, 0, s);
        default: return CQ_ERR_RANGE;
    }
}
static int qb_launch(int w_dtype, const void *w, const void *x, const float *up, int64_t x_stride, int64_t up_stride, int x_dtype, void *workspace,
                     void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, hipStream_t s) {
    return w_dtype == CQ_Q5K ? qb_launch_w<true>(w_dtype, w, x, up, x_stride, up_stride, x_dtype, workspace, dst, dst_dtype, k, n, rows, stride_dst, s)
                             : qb_launch_w<false>(w_dtype, w, x, up, x_stride, up_stride, x_dtype, workspace, dst, dst_dtype, k, n, rows, stride_dst, s);
}
int cq_matvec_batch_launch(int w_dtype, const void *w, const void *x, int x_dtype, void *workspace, void *dst, int dst_dtype, int64_t k, int64_t n,
                           int64_t rows, int64_t stride_dst, hipStream_t s) {
    return qb_launch(w_dtype, w, x, nullptr, k, 0, x_dtype, workspace, dst, dst_dtype, k, n, rows, stride_dst, s);
}
int cq_matvec_batch_swiglu_launch(int w_dtype, const void *w, const float *gate, const float *up, int64_t gate_stride, int64_t up_stride, void *workspace,
                                  void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, hipStream_t s) {
    return qb_launch(w_dtype, w, gate, up, gate_stride, up_stride, -1, workspace, dst, dst_dtype, k, n, rows, stride_dst, s);
}

// ---- MoE: experts as batched matvecs (see qme_q4k_kernel) ----
// Q4_K or Q5_K experts of rows up to 16 super-blocks (two columns per wave: three do not fit the registers next to two operand sets),
// 16-byte aligned, and on average at most 64 pairs per expert: beyond that a pass over the weights per 32 pairs loses to the
// tiles that reuse a weight 32 or 128 times.
bool cq_moe_stream_shape(int w_dtype, int64_t num_experts, int64_t n_pairs, int64_t k, int64_t n) {
    return qb_weights(w_dtype) && k % 256 == 0 && k / 256 <= 2 * QB_NW && n >= 1 && n <= 0x7ffffff0 / 16 && num_experts >= 1 && num_experts <= 65535 &&
           n_pairs <= QME_MAX_AVG_PAIRS * num_experts && n * (k / 256) * qb_bb(w_dtype == CQ_Q5K) < 0x7fffffffLL;
}
bool cq_moe_stream_takes(int w_dtype, const void *w, const void *w_b, int64_t num_experts, int64_t n_pairs, int64_t k, int64_t n) {
    return cq_moe_stream_shape(w_dtype, num_experts, n_pairs, k, n) && ((uintptr_t)w & 15) == 0 && ((uintptr_t)w_b & 15) == 0;
}
int64_t cq_moe_stream_operand_bytes(int64_t num_experts, int64_t n_pairs, int64_t k) {
    return qme_operand_tiles(n_pairs, num_experts) * (k / 256) * QME_TILE_COL_BYTES;
}
// chunks: the grouping pass's table for chunks of 16 pairs (n | expert[max_chunks] | first[] | count[]).  up != nullptr: the rows are
// silu(x[row]) * up[row] and scale_out[i] = scale_in[row_map[i]].
int cq_moe_stream_quantize_launch(const float *x, const float *up, const int *row_map, const float *scale_in, float *scale_out, const int *chunks,
                                  int64_t max_chunks, int64_t num_experts, int64_t n_pairs, const int *offsets, void *op, int64_t k, hipStream_t s) {
    // chunks of 16 pairs: at most one partly filled chunk per expert (the table has room for chunks of 8)
    const int64_t grid = std::min<int64_t>(max_chunks, n_pairs / 16 + std::min(num_experts, n_pairs));
    if (up)
        hipLaunchKernelGGL(qme_quantize_kernel<true>, dim3((unsigned)grid, (unsigned)(k / 256)), dim3(1024), 0, s, x, up, row_map, scale_in, scale_out, chunks,
                           (int)max_chunks, offsets, (uint8_t *)op, (int)(k / 256), k, k);
    else
        hipLaunchKernelGGL(qme_quantize_kernel<false>, dim3((unsigned)grid, (unsigned)(k / 256)), dim3(1024), 0, s, x, up, row_map, scale_in, scale_out, chunks,
                           (int)max_chunks, offsets, (uint8_t *)op, (int)(k / 256), k, k);
    return (int)hipGetLastError();
}
static int qme_launch(QmeArgs &a, int w_dtype, int64_t num_experts, int tensors, hipStream_t s);
// out_a[pair_out[p]][:] = (W_a[expert of p] . x^[p]) * pair_scale[p] for every sorted pair p; the same for (w_b, out_b) when given
int cq_moe_stream_launch(int w_dtype, const void *w_a, const void *w_b, float *out_a, float *out_b, const void *op, const int *offsets, const int *pair_out,
                         const float *pair_scale, int *extra, int launch_slot, int64_t num_experts, int64_t k, int64_t n, hipStream_t s) {
    const int bpr = (int)(k / 256), tensors = w_b ? 2 : 1;
    QmeArgs a;
    a.w[0] = (const uint8_t *)w_a; a.w[1] = (const uint8_t *)w_b; a.out[0] = out_a; a.out[1] = out_b;
    a.op = (const uint8_t *)op; a.offsets = offsets; a.pair_out = pair_out; a.pair_scale = pair_scale; a.n = (int)n; a.bpr = bpr;
    a.dense_rows = 0; a.extra = extra; a.extra_slot = launch_slot;
    return qme_launch(a, w_dtype, num_experts, tensors, s);
}

// the launch geometry of the expert kernel: waves per row block, parts per expert and tensor
template <bool Q5>
static int qme_launch_w(QmeArgs &a, int64_t num_experts, int tensors, hipStream_t s) {
    const int bpr = a.bpr;
    const int64_t n = a.n;
    // waves that share a row block: the fewest (a power of two) with at most two columns each — large tiles: a tile costs about
    // a microsecond of barriers and latencies whatever it holds
    const int cw = bpr > 8 ? 8 : bpr > 4 ? 4 : bpr > 2 ? 2 : 1;
    const int64_t ntiles = (n + 16 * (QB_NW / cw) - 1) / (16 * (QB_NW / cw));
    // parts: experts x tensors x parts fills the CUs once or twice (all experts hit: the same bytes everywhere)
    int64_t parts = (256 + num_experts * tensors - 1) / (num_experts * tensors);
    if (parts > ntiles) parts = ntiles;
    // (every part the same number of tiles where that is possible: 896 tiles are 224 parts of 4, not 256 of 3 or 4)
    if (parts > 1) parts = (ntiles + (ntiles + parts - 1) / parts - 1) / ((ntiles + parts - 1) / parts);
    a.parts = (int)parts;
    // a listed pass in pieces of about eight tiles: short enough to spread over the workgroups that have finished, long enough for
    // the five microseconds until a piece's first tile is there
    const int64_t tiles_per_part = (ntiles + parts - 1) / parts;
    a.extra_parts = (int)(parts * std::max<int64_t>(1, tiles_per_part / 8));
    switch (cw) {
        case 8: return launch_qme<8, 2, Q5>(a, num_experts, tensors, s);
        case 4: return launch_qme<4, 2, Q5>(a, num_experts, tensors, s);
        case 2: return launch_qme<2, 2, Q5>(a, num_experts, tensors, s);
        default: return bpr == 2 ? launch_qme<1, 2, Q5>(a, num_experts, tensors, s) : launch_qme<1, 1, Q5>(a, num_experts, tensors, s);
    }
}
static int qme_launch(QmeArgs &a, int w_dtype, int64_t num_experts, int tensors, hipStream_t s) {
    return w_dtype == CQ_Q5K ? qme_launch_w<true>(a, num_experts, tensors, s) : qme_launch_w<false>(a, num_experts, tensors, s);
}

// ---- QMatMul::forward for 17 .. 64 rows: the matrix as the one expert of the kernel above, the rows as its pairs (two sets of 16
// per pass over the weights) ----
// (the 32-row / 128-row matrix-core tiles convert every weight for the rows of a tile: at these row counts that costs more than
// scaling the results)
bool cq_matvec_batch_mid_takes(int w_dtype, const void *w, const void *x, int x_dtype, int dst_dtype, int64_t k, int64_t n, int64_t rows) {
    return qb_weights(w_dtype) && x_dtype == CQ_F32 && dst_dtype == CQ_F32 && rows > 16 && rows <= 64 &&
           cq_moe_stream_takes(w_dtype, w, nullptr, 1, rows, k, n) && ((uintptr_t)x & 15) == 0;
}
int64_t cq_matvec_batch_mid_workspace(int w_dtype, int64_t k, int64_t rows) {
    return qb_weights(w_dtype) && rows > 16 && rows <= 64 && k % 256 == 0 && k / 256 <= 2 * QB_NW ? cq_align256(((rows + 15) / 16) * (k / 256) * QME_TILE_COL_BYTES) : 0;
}
// up != nullptr: the rows are silu(x[r]) * up[r], with row strides in floats
int cq_matvec_batch_mid_launch(int w_dtype, const void *w, const float *x, const float *up, int64_t x_stride, int64_t up_stride, void *workspace, float *dst,
                               int64_t k, int64_t n, int64_t rows, hipStream_t s) {
    const int bpr = (int)(k / 256);
    const dim3 grid((unsigned)((rows + 15) / 16), (unsigned)bpr);
    if (up)
        hipLaunchKernelGGL(qme_quantize_kernel<true>, grid, dim3(1024), 0, s, x, up, (const int *)nullptr, (const float *)nullptr, (float *)nullptr,
                           (const int *)nullptr, (int)rows, (const int *)nullptr, (uint8_t *)workspace, bpr, x_stride, up_stride);
    else
        hipLaunchKernelGGL(qme_quantize_kernel<false>, grid, dim3(1024), 0, s, x, up, (const int *)nullptr, (const float *)nullptr, (float *)nullptr,
                           (const int *)nullptr, (int)rows, (const int *)nullptr, (uint8_t *)workspace, bpr, x_stride, up_stride);
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    QmeArgs a;
    a.w[0] = (const uint8_t *)w; a.w[1] = nullptr; a.out[0] = dst; a.out[1] = nullptr;
    a.op = (const uint8_t *)workspace; a.offsets = nullptr; a.pair_out = nullptr; a.pair_scale = nullptr; a.n = (int)n; a.bpr = bpr;
    a.dense_rows = (int)rows; a.extra = nullptr; a.extra_slot = 0;
    return qme_launch(a, w_dtype, 1, 1, s);
}

#ifdef CL_STAMPS
extern "C" int qme_debug_launch(const void *w, float *out, const void *op, const int *offsets, const int *pout, const float *pscale, int64_t experts,
                                int64_t k, int64_t n, uint32_t *stamps, void *stream) {
    hipMemcpyToSymbol(HIP_SYMBOL(qme_stamps), &stamps, sizeof(stamps));
    return cq_moe_stream_launch(CQ_Q4K, w, nullptr, out, nullptr, op, offsets, pout, pscale, nullptr, 0, experts, k, n, (hipStream_t)stream);
}
extern "C" int qb_debug_launch(const void *w, const void *x, void *workspace, void *dst, int64_t k, int64_t n, int64_t rows, void *stream) {
    return cq_matvec_batch_launch(CQ_Q4K, w, x, CQ_F32, workspace, dst, CQ_F32, k, n, rows, n, (hipStream_t)stream);
}
#endif
