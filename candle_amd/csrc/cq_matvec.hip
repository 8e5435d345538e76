// Decode matvec for gfx950:  dst[b, row] = sum_k W[row, k] * x^[b, k]   (b < NB <= 8)
//
// W is streamed once from HBM in its GGUF block layout; x^ is the int8 quantization of the
// activations, bit-identical to candle's CPU quantization, so the integer part of every dot product is
// exact and only the f32 summation order differs from k_quants::matmul
// (candle-core/src/quantized/k_quants.rs:2375-2492).
//
// One kernel does the whole QMatMul::forward for a decode step:
//   1. every wave issues the 128-bit loads of its first row of W;
//   2. the workgroup quantizes the NB activation rows into LDS (Q8_K or Q8_0 blocks, one wave per
//      256-element span) — or copies an already quantized scratch buffer into LDS;
//   3. each wave walks its rows (row = first + wave, + waves, ...): lane l takes units l, l+64, ... of
//      the row (see cq_fmt.h), the next step's weights are in flight while the current one is reduced
//      with v_dot4_i32_i8, and a DPP wave reduction leaves the row result in lane 63.
// When a row is a single wave step (K = 4096 for K-quants) the activation registers are loaded from
// LDS once and reused for every row.
//
// The grid is one workgroup of up to 16 waves per CU (256 CUs): waves live long enough to amortize
// the activation quantization, and all of a CU's weight loads are in flight from the first cycle.
#include "cq_actquant.h"
#include "cq_device.h"
#include "cq_fmt.h"
#include "cq_launch.h"
#include "cq_stream.h"
#include "cq_stream_body.h"

namespace {

template <int DT, int NB, int SRC, bool SINGLE, int PRO, int EPI, bool PRE>
__device__ __forceinline__ void qmv_body(const uint8_t *__restrict__ w, const ActSrc &src, void *__restrict__ dst, const QmvGeom &g, const Fuse &fz,
                                         const int block, const int nblocks) {
    typedef typename UnitFmt<DT, NB, SINGLE>::type F;
    static_assert((PRO == PRO_NONE && (EPI == EPI_NONE || EPI == EPI_MOE)) || (NB == 1 && SRC == CQ_F32), "fusions are for one f32 row");
    static_assert(PRO != PRO_MERGE || (SINGLE && !PRE), "the merge prologue preloads one span per wave");
    static_assert(!pro_is_split(PRO) || !PRE, "the plane-merging prologue holds one span per wave");
    static_assert(EPI != EPI_SWIGLU || SINGLE, "the paired-row epilogue is written for rows of one wave step");
    constexpr bool FUSED = SRC != SRC_SCRATCH;
    constexpr bool RESID = epi_is_resid(EPI);
    constexpr int ME = EPI == EPI_RESID_SPLIT ? MAXP : 1;          // planes added to the residual row
    constexpr int XDT = FUSED ? SRC : CQ_F32;
    extern __shared__ __align__(16) uint8_t lds[];
    int8_t *lqs = (int8_t *)lds;
    float *ld = (float *)(lds + g.lds_d_off);
    int16_t *lbs = (int16_t *)(lds + g.lds_bs_off);

    const int k = g.k, n = g.n, dst_dtype = g.dst_dtype;
    const int64_t stride_dst = g.stride_dst;
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int nwaves = 1 << g.nw_shift;
    const int units = g.units;
    const int steps = g.steps;
    const int row_bytes = g.row_bytes;
    const int wave_stride = row_bytes << g.nw_shift;
    const int wg_row0 = block * g.rows_per_wg;
    const int wg_row1 = min(n, wg_row0 + g.rows_per_wg);

    // 0. The activation loads go out first.  Vector loads complete in order, so anything issued after
    //    the weight loads below could only be consumed once the (slow, HBM) weights have arrived.
    const int total = NB * k;                 // elements of x
    // fused: this wave's first XS 256-element spans (span wv, wv + nwaves, ...) are loaded up front; with
    // long rows (PRE) that is normally all of them, so no load -> use round trip is left in the prologue
    constexpr int XS = PRE ? 4 : 1;
    float xv[XS][4], av4[XS][4];              // av4: PRO: norm weight / up values of the same spans
#pragma unroll
    for (int j = 0; j < XS; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) { xv[j][e] = 0.0f; av4[j][e] = 0.0f; }
    const int xbase = wv * 256 + lane * 4;
    const int xstep = 256 << g.nw_shift;
    u32x4 c_qs = {0, 0, 0, 0};                // pre-quantized: first round of the scratch -> LDS copy
    u32x2 c_d = {0, 0};
    uint32_t c_bs = 0;
    float pp[NPART / 64] = {0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int MS = PRO == PRO_MERGE ? MAXS : 1;
    MergeRegs<MS> mg;
    constexpr int MP = PRO == PRO_NORM_SPLIT ? MAXP : 1;
    float pl[MP][4];
    if (FUSED && PRO == PRO_MERGE) {
        merge_load<MS>(fz, xbase, xbase < total, mg);
    } else if (FUSED) {
#pragma unroll
        for (int j = 0; j < XS; j++) {
            if (xbase + j * xstep < total) cq_load4<XDT>(src.x, xbase + j * xstep, xv[j]);
            if (PRO != PRO_NONE && xbase + j * xstep < total) cq_load4<CQ_F32>(fz.aux, xbase + j * xstep, av4[j]);
        }
        if (PRO == PRO_NORM) {
#pragma unroll
            for (int i = 0; i < NPART / 64; i++) pp[i] = fz.part_in[lane + 64 * i];
        }
        if (pro_is_split(PRO)) {
            // unconditional loads (a plane that is not there re-reads the last one and is zeroed when it is added):
            // branches here would make the compiler wait for these loads before it issues the weight loads
            const int xc = min(xbase, total - 4);
#pragma unroll
            for (int sI = 0; sI < MP; sI++) cq_load4<CQ_F32>(fz.planes, (int64_t)min(sI, fz.n_planes - 1) * k + xc, pl[sI]);
        }
    } else {
        if (tid < (total >> 4)) c_qs = ((const u32x4 *)src.av.qs)[tid];
        if (cq_is_kquant(DT)) {
            if (tid < NB * (k >> 8)) c_d.x = __float_as_uint(src.av.d[tid]);
            if (tid < (NB * (k >> 4)) >> 1) c_bs = ((const uint32_t *)src.av.bsums)[tid];
        } else {
            if (tid < NB * (k >> 5)) c_d = ((const u32x2 *)src.av.d)[tid];
        }
    }

    // 1. first weights in flight.  The load is unconditional (idle waves re-read the last row) so that
    //    the compiler can wait for the activation load alone and leave these in flight.
    const int wv_s = __builtin_amdgcn_readfirstlane(wv);
    int row = wg_row0 + wv_s;
    // rows this wave owns (the wave count is a power of two: a shift, not an integer division)
    const int my_rows = row < wg_row1 ? (wg_row1 - row + nwaves - 1) >> g.nw_shift : 0;
    const uint8_t *wp = w + (int64_t)min(row, n - 1) * (int64_t)row_bytes;
    const int u0 = min(lane, units - 1);
    typename F::W wa, wb;
    // PRE (rows of 2..4 wave steps, e.g. K = 14336): all steps of the wave's first row are issued here, so the
    // whole first row streams in behind the activation prologue instead of one step of it
    typename F::W pre[PRE ? 4 : 1];
    // BLOCKED (rows of one wave step, more than two activation rows): weight rows are taken RB at a time and held in
    // registers while each activation row is read from LDS once per block, not once per weight row
    constexpr bool BLOCKED = SINGLE && NB > 2;
    constexpr int RB = 4;
    typename F::W wA[BLOCKED ? RB : 1], wB[BLOCKED ? RB : 1];
    const int last_j = max(my_rows - 1, 0);
    if (PRE) {
#pragma unroll
        for (int i = 0; i < 4; i++) F::load_w(pre[i], wp, min(lane + 64 * i, units - 1));
    } else if (BLOCKED) {
#pragma unroll
        for (int r = 0; r < RB; r++) F::load_w(wA[r], wp + (int64_t)min(r, last_j) * wave_stride, u0);
    } else {
        F::load_w(wa, wp, u0);
    }

    // every load above is issued before the first wait below (the scheduler would otherwise sink some of the
    // weight loads behind the waits for the activation loads)
    if (pro_is_split(PRO)) __builtin_amdgcn_sched_barrier(0);

    // 2. activations -> LDS
    if (FUSED) {
        // The first span is peeled out of the loop on purpose: its values are already in xv, and as
        // straight-line code the compiler waits for that one load only (vmcnt = the weight loads still
        // in flight).  Inside a loop it would wait for everything, i.e. for the weights, and the
        // quantization latency would no longer hide behind the HBM fetch.
        const int spans = (total + 255) >> 8;
        float pm = 1.0f;
        if (PRO == PRO_NORM) {
            // fixed summation order: the same bits in every wave, workgroup and replay
            const float sum2 = wave_sum((pp[0] + pp[1]) + (pp[2] + pp[3]));
            pm = sqrtf(sum2 / (float)k + fz.eps);
        }
        if (PRO == PRO_MERGE) merge_reduce<MS>(mg, xbase < total, xv[0]);
        if (pro_is_split(PRO)) {
            // the merged row (absent planes are zeros) and sum(x^2) over the whole row in a fixed order: one span
            // per wave, so a workgroup-wide reduction is needed
#pragma unroll
            for (int sI = 0; sI < MP; sI++)
#pragma unroll
                for (int e = 0; e < 4; e++) xv[0][e] += (sI < fz.n_planes && xbase < total) ? pl[sI][e] : 0.0f;
            const float ss = wave_sum((xv[0][0] * xv[0][0] + xv[0][1] * xv[0][1]) + (xv[0][2] * xv[0][2] + xv[0][3] * xv[0][3]));
            float *red = (float *)(lds + g.lds_red_off);
            if (lane == 0) red[wv] = ss;
            if (wv == 0 && lane >= nwaves && lane < 16) red[lane] = 0.0f;        // slots of waves that do not exist
            __syncthreads();
            // four broadcast reads and a fixed order of additions (no loop over the wave count: each trip would
            // be a dependent LDS round trip)
            const f32x4 r0 = ((const f32x4 *)red)[0], r1 = ((const f32x4 *)red)[1], r2 = ((const f32x4 *)red)[2], r3 = ((const f32x4 *)red)[3];
            const float sum2 = ((((r0.x + r0.y) + (r0.z + r0.w)) + ((r1.x + r1.y) + (r1.z + r1.w))) +
                                (((r2.x + r2.y) + (r2.z + r2.w)) + ((r3.x + r3.y) + (r3.z + r3.w))));
            pm = sqrtf(sum2 / (float)k + fz.eps);
        }
#pragma unroll
        for (int j = 0; j < XS; j++) {
            const int span = wv_s + (j << g.nw_shift);
            if (PRO == PRO_NORM || PRO == PRO_SILU) pro_apply<PRO>(xv[j], av4[j], pm);
            if (pro_is_split(PRO)) pro_apply<PRO_NORM>(xv[j], av4[j], pm);
            if (span < spans) {
                if (cq_is_kquant(DT))
                    cq_quantize_q8k_vals(xv[j], span, lane, lqs, ld, lbs);
                else
                    cq_quantize_q80_vals(xv[j], xbase + j * xstep < total, xbase + j * xstep, lane, lqs, ld);
            }
        }
        for (int span = wv_s + XS * nwaves; span < spans; span += nwaves) {
            if (PRO == PRO_NONE) {
                if (cq_is_kquant(DT))
                    cq_quantize_q8k_span<XDT>(src.x, span, lane, lqs, ld, lbs);
                else
                    cq_quantize_q80_span<XDT>(src.x, span, lane, total, lqs, ld);
            } else {
                const int base = span * 256 + lane * 4;
                const bool ok = base < total;
                float v[4] = {0.0f, 0.0f, 0.0f, 0.0f}, a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                if (PRO == PRO_MERGE) {
                    // fewer waves than spans (a short weight matrix): later spans are merged here
                    MergeRegs<MS> mr;
                    merge_load<MS>(fz, base, ok, mr);
                    merge_reduce<MS>(mr, ok, v);
                } else {
                    if (ok) {
                        cq_load4<XDT>(src.x, base, v);
                        cq_load4<CQ_F32>(fz.aux, base, a);
                    }
                    pro_apply<PRO>(v, a, pm);
                }
                if (cq_is_kquant(DT))
                    cq_quantize_q8k_vals(v, span, lane, lqs, ld, lbs);
                else
                    cq_quantize_q80_vals(v, ok, base, lane, lqs, ld);
            }
        }
    } else {
        if (tid < (total >> 4)) ((u32x4 *)lqs)[tid] = c_qs;
        for (int i = tid + nthr; i < total >> 4; i += nthr) ((u32x4 *)lqs)[i] = ((const u32x4 *)src.av.qs)[i];
        if (cq_is_kquant(DT)) {
            if (tid < NB * (k >> 8)) ld[tid] = __uint_as_float(c_d.x);
            for (int i = tid + nthr; i < NB * (k >> 8); i += nthr) ld[i] = src.av.d[i];
            if (tid < (NB * (k >> 4)) >> 1) ((uint32_t *)lbs)[tid] = c_bs;
            for (int i = tid + nthr; i < (NB * (k >> 4)) >> 1; i += nthr) ((uint32_t *)lbs)[i] = ((const uint32_t *)src.av.bsums)[i];
        } else {
            if (tid < NB * (k >> 5)) ((u32x2 *)ld)[tid] = c_d;
            for (int i = tid + nthr; i < NB * (k >> 5); i += nthr) ((u32x2 *)ld)[i] = ((const u32x2 *)src.av.d)[i];
        }
    }
    __syncthreads();
    if (!RESID && my_rows == 0) return;
    float ssq = 0.0f;            // EPI_RESID: lane 63 accumulates residual^2 of this wave's rows
    // The residual value of a row (and, EPI_RESID_SPLIT, the plane values to add to it) is requested together with the
    // row's weights and travels behind them in the same in-order load queue.  Unconditional loads: a plane that is
    // not there re-reads the last one and counts as zero.
    auto load_res = [&](int r, float &rv, float (&pv)[ME]) {
        const int rc = min(r, n - 1);
        rv = fz.resid[rc];
        if (EPI == EPI_RESID_SPLIT) {
#pragma unroll
            for (int sI = 0; sI < ME; sI++) pv[sI] = fz.planes[(int64_t)min(sI, fz.n_planes - 1) * n + rc];
        }
    };
    auto merge_res = [&](float rv, const float (&pv)[ME]) {
        if (EPI == EPI_RESID_SPLIT) {
#pragma unroll
            for (int sI = 0; sI < ME; sI++) rv += sI < fz.n_planes ? pv[sI] : 0.0f;
        }
        return rv;
    };
    constexpr bool MOE_TAB = EPI == EPI_MOE && !(SINGLE && NB > 2);      // the blocked path reads them per b instead
    int64_t moe_off[MOE_TAB ? NB : 1];
    float moe_sc[MOE_TAB ? NB : 1];
    if (MOE_TAB) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const bool live = b < fz.nvalid;
            moe_off[b] = live ? (int64_t)fz.row_map[b] * stride_dst : -1;
            moe_sc[b] = live ? fz.row_scale[b] : 0.0f;
        }
    }

    ActRow ar[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) ar[b] = act_row(lqs, ld, lbs, DT, b, k);

    if (SINGLE) {
        // A row is one wave step: lane l always works on unit l.  With few activation rows their
        // registers are loaded from LDS once and reused for every row of W.
        constexpr bool CACHE = NB <= 2;
        const bool valid = lane < units;
        typename F::A areg[NB];
        if (CACHE) {
#pragma unroll
            for (int b = 0; b < NB; b++) F::load_a(areg[b], ar[b], u0);
        }
        auto one_row = [&](const typename F::W &cur, int r, float res) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                if (!CACHE) F::load_a(areg[b], ar[b], u0);
                float v = F::dot(cur, areg[b], u0);
                v = wave_sum_to_lane63(valid ? v : 0.0f);
                if (RESID) {
                    if (lane == 63) {
                        const float sres = res + v;                     // (x + residual), quantized_llama.rs:584,591
                        fz.resid[r] = sres;
                        ssq += sres * sres;
                    }
                } else if (EPI == EPI_MOE) {
                    if (lane == 63 && moe_off[MOE_TAB ? b : 0] >= 0) ((float *)dst)[moe_off[MOE_TAB ? b : 0] + r] = v * moe_sc[MOE_TAB ? b : 0];
                } else if (lane == 63) {
                    store_out(dst, dst_dtype, (int64_t)b * stride_dst + r, EPI == EPI_SCALE ? v * fz.eps : v);
                }
            }
        };
        if (BLOCKED) {
            auto load_block = [&](typename F::W (&wr)[BLOCKED ? RB : 1], int j0) {
#pragma unroll
                for (int r = 0; r < RB; r++) F::load_w(wr[BLOCKED ? r : 0], wp + (int64_t)min(j0 + r, last_j) * wave_stride, u0);
            };
            auto compute_block = [&](const typename F::W (&wr)[BLOCKED ? RB : 1], int j0) {
                // not unrolled over the activation rows: everything that depends on b is recomputed from b, so the
                // registers hold two blocks of weight rows and one activation unit, whatever NB is
#pragma unroll 1
                for (int b = 0; b < NB; b++) {
                    const ActRow arb = act_row(lqs, ld, lbs, DT, b, k);
                    F::load_a(areg[0], arb, u0);
                    int64_t off = (int64_t)b * stride_dst;
                    float sc = 1.0f;
                    if (EPI == EPI_MOE) {
                        const bool live = b < fz.nvalid;
                        off = live ? (int64_t)fz.row_map[live ? b : 0] * stride_dst : -1;
                        sc = live ? fz.row_scale[live ? b : 0] : 0.0f;
                    }
                    // the four rows of the block are reduced together: lane 60 + r ends with row r
                    static_assert(RB == 4, "wave_sum4_to_lanes60 reduces four rows");
                    float v4[RB];
#pragma unroll
                    for (int r = 0; r < RB; r++) {
                        const float v = F::dot(wr[BLOCKED ? r : 0], areg[0], u0);
                        v4[r] = valid ? v : 0.0f;
                    }
                    const float v = wave_sum4_to_lanes60(v4[0], v4[1], v4[2], v4[3], lane);
                    const int r = lane - 60;
                    if (r >= 0 && j0 + r < my_rows && off >= 0) {
                        const int rr = row + ((j0 + r) << g.nw_shift);
                        if (EPI == EPI_MOE) ((float *)dst)[off + rr] = v * sc;
                        else store_out(dst, dst_dtype, off + rr, v);
                    }
                }
            };
            for (int j = 0; j < my_rows; j += 2 * RB) {
                load_block(wB, j + RB);
                compute_block(wA, j);
                if (j + RB >= my_rows) break;
                load_block(wA, j + 2 * RB);
                compute_block(wB, j + RB);
            }
            return;
        }
        if (EPI == EPI_SWIGLU) {
            // wa = W1[row] (already in flight), wb = W3[row]; the next W1 row is requested before W3 is reduced
            for (int j = 0; j < my_rows; j++) {
                F::load_w(wb, wp + fz.pair_off, u0);
                float gate = F::dot(wa, areg[0], u0);
                gate = wave_sum_to_lane63(valid ? gate : 0.0f);
                const uint8_t *p1 = j + 1 < my_rows ? wp + wave_stride : wp;
                F::load_w(wa, p1, u0);
                float up = F::dot(wb, areg[0], u0);
                up = wave_sum_to_lane63(valid ? up : 0.0f);
                if (lane == 63) store_out(dst, dst_dtype, row, gate / (1.0f + expf(-gate)) * up);   // Mlp::forward, quantized_llama.rs:56-63
                row += nwaves;
                wp = p1;
            }
            return;
        }
        if constexpr (DT == CQ_Q6K && NB == 1 && (EPI == EPI_NONE || EPI == EPI_SCALE)) {
            // Q6_K plain rows: the same ping-pong, but the wave sums of four consecutive rows are formed together
            // (wave_sum4_to_lanes60) and lanes 60..63 store them at once.  Measured per format on 14336 x 4096: Q6_K
            // 12.86 -> 12.08 us, Q4_K 8.51 -> 8.59, Q3_K 9.27 -> 9.39: it pays for the longest dot only.
            for (int j = 0; j < my_rows; j += 4) {
                float v0 = 0.0f, v1 = 0.0f, v2 = 0.0f, v3 = 0.0f;
                const uint8_t *p1 = j + 1 < my_rows ? wp + wave_stride : wp;
                F::load_w(wb, p1, u0);
                v0 = F::dot(wa, areg[0], u0);
                wp = p1;
                if (j + 1 < my_rows) {
                    const uint8_t *p2 = j + 2 < my_rows ? p1 + wave_stride : p1;
                    F::load_w(wa, p2, u0);
                    v1 = F::dot(wb, areg[0], u0);
                    wp = p2;
                    if (j + 2 < my_rows) {
                        const uint8_t *p3 = j + 3 < my_rows ? p2 + wave_stride : p2;
                        F::load_w(wb, p3, u0);
                        v2 = F::dot(wa, areg[0], u0);
                        wp = p3;
                        if (j + 3 < my_rows) {
                            const uint8_t *p4 = j + 4 < my_rows ? p3 + wave_stride : p3;
                            F::load_w(wa, p4, u0);
                            v3 = F::dot(wb, areg[0], u0);
                            wp = p4;
                        }
                    }
                }
                const float c = wave_sum4_to_lanes60(valid ? v0 : 0.0f, valid ? v1 : 0.0f, valid ? v2 : 0.0f, valid ? v3 : 0.0f, lane);
                const int r = lane - 60;
                if (r >= 0 && j + r < my_rows) store_out(dst, dst_dtype, row + r * nwaves, EPI == EPI_SCALE ? c * fz.eps : c);
                row += 4 * nwaves;
            }
            return;
        }
        // ping-pong between wa and wb: the next row's loads are in flight while this one is reduced;
        // the prefetch past the last row re-reads it instead of branching around the load.  The residual
        // value of a row travels behind its weights in the same in-order load queue.
        float ra = 0.0f, rb = 0.0f, pa[ME], pb[ME];
        if (RESID) load_res(row, ra, pa);
        for (int j = 0; j < my_rows; j += 2) {
            const uint8_t *p1 = j + 1 < my_rows ? wp + wave_stride : wp;
            F::load_w(wb, p1, u0);
            if (RESID) load_res(row + nwaves, rb, pb);
            one_row(wa, row, merge_res(ra, pa));
            if (j + 1 >= my_rows) break;
            const uint8_t *p2 = j + 2 < my_rows ? p1 + wave_stride : p1;
            F::load_w(wa, p2, u0);
            if (RESID) load_res(row + 2 * nwaves, ra, pa);
            one_row(wb, row + nwaves, merge_res(rb, pb));
            row += 2 * nwaves;
            wp = p2;
        }
    } else {
        // General walk over (row, step), unrolled by two for the same ping-pong.
        typename F::A areg[NB];
        float acc[NB];
#pragma unroll
        for (int b = 0; b < NB; b++) acc[b] = 0.0f;
        int total_steps = my_rows * steps;
        int i = 0;
        float rcur = 0.0f, pcur[ME];
        if (RESID) load_res(row, rcur, pcur);
        auto finish_row = [&]() {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float r = wave_sum_to_lane63(acc[b]);
                if (RESID) {
                    if (lane == 63) {
                        const float sres = merge_res(rcur, pcur) + r;
                        fz.resid[row] = sres;
                        ssq += sres * sres;
                    }
                } else if (EPI == EPI_MOE) {
                    if (lane == 63 && moe_off[MOE_TAB ? b : 0] >= 0) ((float *)dst)[moe_off[MOE_TAB ? b : 0] + row] = r * moe_sc[MOE_TAB ? b : 0];
                } else if (lane == 63) {
                    store_out(dst, dst_dtype, (int64_t)b * stride_dst + row, EPI == EPI_SCALE ? r * fz.eps : r);
                }
                acc[b] = 0.0f;
            }
            row += nwaves;
            if (RESID) load_res(row, rcur, pcur);   // consumed a whole row of steps later
        };
        auto accumulate = [&](const typename F::W &cur, int step) {
            const int u = lane + 64 * step;
            const bool valid = u < units;
            const int uc = valid ? u : units - 1;
#pragma unroll
            for (int b = 0; b < NB; b++) {
                F::load_a(areg[b], ar[b], uc);
                float v = F::dot(cur, areg[b], uc);
                acc[b] += valid ? v : 0.0f;
            }
        };
        if (PRE) {
            if (my_rows > 0) {
#pragma unroll
                for (int st = 0; st < 4; st++)
                    if (st < steps) accumulate(pre[st], st);
                finish_row();
                wp += wave_stride;
                total_steps -= steps;
                if (total_steps > 0) F::load_w(wa, wp, u0);
            } else {
                total_steps = 0;
            }
        }
        auto one_step = [&](const typename F::W &cur, typename F::W &nxt, int t) {
            // next (row, step); past the end the last unit is re-read
            int ni = i + 1;
            const uint8_t *nwp = wp;
            if (ni == steps) { ni = 0; nwp = wp + wave_stride; }
            if (t + 1 >= total_steps) { ni = i; nwp = wp; }
            F::load_w(nxt, nwp, min(lane + 64 * ni, units - 1));
            accumulate(cur, i);
            if (i == steps - 1) finish_row();
            i = ni;
            wp = nwp;
        };
        for (int t = 0; t < total_steps; t += 2) {
            one_step(wa, wb, t);
            if (t + 1 >= total_steps) break;
            one_step(wb, wa, t + 1);
        }
    }
    if (RESID) {
        // the workgroup's partial of sum(residual^2), summed in a fixed order; block 0 clears the unused slots
        float *red = (float *)(lds + g.lds_red_off);
        if (lane == 63) red[wv] = ssq;
        __syncthreads();
        if (tid == 0) {
            float t = 0.0f;
            for (int i = 0; i < nwaves; i++) t += red[i];
            fz.part_out[block] = t;
        }
        if (block == 0)
            for (int i = nblocks + tid; i < NPART; i += nthr) fz.part_out[i] = 0.0f;
    }
}

// More than two activation rows keep blocks of weight rows in registers: workgroups of 8 waves (256 VGPRs per
// lane) instead of 16 (128).
template <int DT, int NB, int SRC, bool SINGLE, int PRO = PRO_NONE, int EPI = EPI_NONE, bool PRE = false>
__global__ __launch_bounds__(NB > 2 ? 512 : 1024) void qmv_kernel(const uint8_t *__restrict__ w, ActSrc src, void *__restrict__ dst, QmvGeom g, Fuse fz) {
    qmv_body<DT, NB, SRC, SINGLE, PRO, EPI, PRE>(w, src, dst, g, fz, blockIdx.x, gridDim.x);
}

// Two weight tensors of different K-quant formats over the same activation row in one launch (attention_wq|wk and
// attention_wv of a Q4_K_M file): workgroups [0, blocks_a) take tensor A, the rest tensor B.
template <int DTA, int DTB, bool SINGLE, int PRO>
__global__ __launch_bounds__(1024) void qmv2_kernel(const uint8_t *__restrict__ wa, const uint8_t *__restrict__ wb, ActSrc src, void *__restrict__ dsta,
                                                    void *__restrict__ dstb, QmvGeom ga, QmvGeom gb, Fuse fz, int blocks_a) {
    if ((int)blockIdx.x < blocks_a)
        qmv_body<DTA, 1, CQ_F32, SINGLE, PRO, EPI_NONE, false>(wa, src, dsta, ga, fz, blockIdx.x, blocks_a);
    else
        qmv_body<DTB, 1, CQ_F32, SINGLE, PRO, EPI_NONE, false>(wb, src, dstb, gb, fz, blockIdx.x - blocks_a, gridDim.x - blocks_a);
}

// Kernel arguments of the streaming kernel, packed: every pointer and scalar a (PRO, EPI) pair does not use is left
// out and the launch geometry is derived from (n, super-blocks per row) in the kernel.  What a kernel reads of its
// argument block should lie in the first 64 bytes: a read from the next 64 (explicit arguments, or the hidden ones
// behind them that gridDim / blockDim come from) is a second trip to memory before anything else can start
// (measured on the 33 MB matvec: 7.67 us per launch with 56 bytes of arguments, 7.96 us with 60).
__host__ __device__ constexpr int qs_groups(int total_steps) { return total_steps < 256 ? total_steps : 256; }
constexpr int qs_pro_ptrs(int pro) { return pro == PRO_NORM || pro == PRO_NORM_SPLIT ? 3 : pro == PRO_SILU ? 2 : 1; }
constexpr int qs_epi_ptrs(int epi) { return epi == EPI_RESID ? 2 : epi == EPI_RESID_SPLIT ? 3 : 1; }
constexpr bool qs_has_f(int pro, int epi) { return pro == PRO_NORM || pro == PRO_NORM_SPLIT || epi == EPI_SCALE; }
template <int PRO, int EPI> struct QsArgs {
    static constexpr int NP = 1 + qs_pro_ptrs(PRO) + qs_epi_ptrs(EPI);
    static constexpr int NI = 2 + (qs_has_f(PRO, EPI) ? 1 : 0) + (EPI == EPI_SWIGLU ? 1 : 0);
    const void *p[NP];     // w | PRO_NONE: x; NORM: x, norm weight, partial sums; SILU: x, up; MERGE: partials; NORM_SPLIT: x, norm weight, planes
                           //   | EPI_NONE / SCALE / SWIGLU: dst; RESID: residual, partial sums out; RESID_SPLIT: residual, partial sums out, planes
    int i[NI];             // n | bpr + (dst_dtype << 8) + (n_planes << 16) + (splits << 20) + (hd_shift << 26) | eps or scale | pair distance / 16
};

template <int DT, int PRO, int EPI>
QsArgs<PRO, EPI> qs_pack(const void *w, const float *x, void *dst, const StreamGeom &g, const Fuse &fz) {
    QsArgs<PRO, EPI> a;
    int np = 0;
    a.p[np++] = w;
    if (PRO != PRO_MERGE) a.p[np++] = x;
    if (PRO != PRO_NONE) a.p[np++] = fz.aux;
    if (PRO == PRO_NORM) a.p[np++] = fz.part_in;
    if (PRO == PRO_NORM_SPLIT) a.p[np++] = fz.planes;
    if (epi_is_resid(EPI)) {
        a.p[np++] = fz.resid;
        a.p[np++] = fz.part_out;
        if (EPI == EPI_RESID_SPLIT) a.p[np++] = fz.planes;
    } else {
        a.p[np++] = dst;
    }
    int ni = 0;
    a.i[ni++] = g.n;
    a.i[ni++] = g.bpr | (g.dst_dtype << 8) | (fz.n_planes << 16) | (fz.splits << 20) | (fz.hd_shift << 26);
    if (qs_has_f(PRO, EPI)) a.i[ni++] = __builtin_bit_cast(int, fz.eps);
    if (EPI == EPI_SWIGLU) a.i[ni++] = (int)(fz.pair_off / 16);
    return a;
}

template <int DT, int PRO, int EPI>
__device__ __forceinline__ void qs_unpack(const QsArgs<PRO, EPI> &a, const uint8_t *&w, const float *&x, void *&dst, StreamGeom &g, Fuse &fz) {
    int np = 0;
    w = qs_global<const uint8_t>(a.p[np++]);
    x = PRO != PRO_MERGE ? qs_global<const float>(a.p[np++]) : nullptr;
    fz.aux = PRO != PRO_NONE ? qs_global<const float>(a.p[np++]) : nullptr;
    fz.part_in = PRO == PRO_NORM ? qs_global<const float>(a.p[np++]) : nullptr;
    fz.planes = PRO == PRO_NORM_SPLIT ? qs_global<const float>(a.p[np++]) : nullptr;
    dst = nullptr; fz.resid = nullptr; fz.part_out = nullptr;
    if (epi_is_resid(EPI)) {
        fz.resid = qs_global<float>(a.p[np++]);
        fz.part_out = qs_global<float>(a.p[np++]);
        if (EPI == EPI_RESID_SPLIT) fz.planes = qs_global<const float>(a.p[np++]);
    } else {
        dst = qs_global<void>(a.p[np++]);
    }
    int ni = 0;
    const int n = a.i[ni++];
    const uint32_t meta = (uint32_t)a.i[ni++];
    fz.eps = qs_has_f(PRO, EPI) ? __builtin_bit_cast(float, a.i[ni++]) : 0.0f;
    fz.pair_off = EPI == EPI_SWIGLU ? (int64_t)a.i[ni++] * 16 : 0;
    fz.n_planes = (meta >> 16) & 15; fz.splits = (meta >> 20) & 63; fz.hd_shift = meta >> 26;
    fz.row_map = nullptr; fz.row_scale = nullptr; fz.nvalid = 0;
    const int bpr = meta & 255;
    g.k = bpr * 256; g.n = n; g.bpr = bpr;
    g.lp_shift = bpr > 1 ? 32 - __builtin_clz(bpr - 1) : 0;
    g.step_rows = 64 >> g.lp_shift;
    g.step_bytes = g.step_rows * bpr * StreamFmt<DT>::BB;
    g.total_steps = (n + g.step_rows - 1) >> (6 - g.lp_shift);
    g.dst_dtype = (meta >> 8) & 255; g.stride_dst = n;
    g.w_bytes = (int64_t)n * (bpr * StreamFmt<DT>::BB);
}

template <int DT, int XS, int MAXB, int PRO, int EPI, int MSP>
__global__ __launch_bounds__(QS_NW * 64) void qms_kernel(QsArgs<PRO, EPI> a) {
    const uint8_t *w; const float *x; void *dst; StreamGeom g; Fuse fz;
    qs_unpack<DT, PRO, EPI>(a, w, x, dst, g, fz);
    // the grid size is derived, not read: gridDim comes from the hidden arguments behind the explicit ones, and every
    // argument byte a kernel reads beyond the first 64 costs a second trip at its start
    qms_body<DT, QS_NW, XS, MAXB, PRO, EPI, MSP>(w, x, dst, g, fz, blockIdx.x, qs_groups(g.total_steps));
}

// The same kernel with its argument block handed over as fourteen 32-bit scalars (every block of at most 56 bytes): scalar
// arguments can be placed in SGPRs when the wave is launched (the build asks for that), and the kernel then starts without
// the trip to memory for its arguments.
#define CQ_DW14_PARAMS uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, uint32_t a4, uint32_t a5, uint32_t a6, uint32_t a7, uint32_t a8, \
                       uint32_t a9, uint32_t a10, uint32_t a11, uint32_t a12, uint32_t a13
#define CQ_DW14_LIST a0, a1, a2, a3, a4, a5, a6, a7, a8, a9, a10, a11, a12, a13
struct Dwords14 { uint32_t d[14]; };
template <typename A> Dwords14 to_dwords14(const A &a) {
    static_assert(sizeof(A) <= 56, "fourteen dwords");
    Dwords14 r{};
    __builtin_memcpy(r.d, &a, sizeof(A));
    return r;
}
template <typename A> __device__ __forceinline__ A from_dwords14(CQ_DW14_PARAMS) {
    const uint32_t d[14] = {CQ_DW14_LIST};
    A a;
    __builtin_memcpy(&a, d, sizeof(A));
    return a;
}
template <int DT, int XS, int MAXB, int PRO, int EPI, int MSP>
__global__ __launch_bounds__(QS_NW * 64) void qms_kernel_dw(CQ_DW14_PARAMS) {
    const QsArgs<PRO, EPI> a = from_dwords14<QsArgs<PRO, EPI>>(CQ_DW14_LIST);
    const uint8_t *w; const float *x; void *dst; StreamGeom g; Fuse fz;
    qs_unpack<DT, PRO, EPI>(a, w, x, dst, g, fz);
    qms_body<DT, QS_NW, XS, MAXB, PRO, EPI, MSP>(w, x, dst, g, fz, blockIdx.x, qs_groups(g.total_steps));
}

// ---- two activation rows on the streaming kernel -------------------------------------------------------------
// QMatMul::forward for two f32 rows (no prologue, no epilogue): the same stream of weight steps as qms_body; a lane keeps
// the 256 activations of its super-block for both rows and takes two dots from every block it reads.  The weights are
// read once, as for one row; what doubles is the activation prologue and the dot products.
struct QsRowsArgs {
    const uint8_t *w; const float *x; void *dst;
    int n;
    uint32_t meta;            // bpr | dst_dtype << 8
    int stride_dst;           // elements between the two output rows
};
template <int DT, int XS, int MAXB>
__global__ __launch_bounds__(QS_NW * 64) void qms_rows2_kernel(const uint8_t *a_w, const float *a_x, void *a_dst, int a_n, uint32_t a_meta, int a_stride_dst) {
    const QsRowsArgs a{a_w, a_x, a_dst, a_n, a_meta, a_stride_dst};       // scalar arguments: in SGPRs when the wave starts
    typedef StreamFmt<DT> SF;
    typedef StreamAct<MAXB> SA;
    constexpr int NB = 2, NW = QS_NW, PRE = 4, SLOT = SF::NLD * 1024;
    extern __shared__ __align__(16) uint8_t slots[];
    __shared__ __align__(16) uint8_t act[NB][SA::BYTES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = a.n, bpr = a.meta & 255, dst_dtype = (a.meta >> 8) & 255, k = bpr * 256;
    const int lp_shift = bpr > 1 ? 32 - __builtin_clz(bpr - 1) : 0;
    const int step_rows = 64 >> lp_shift, step_bytes = step_rows * bpr * SF::BB;
    const int total_steps = (n + step_rows - 1) >> (6 - lp_shift);
    const int64_t w_bytes = (int64_t)n * (bpr * SF::BB);
    const int block = blockIdx.x, nblocks = qs_groups(total_steps);

    // activation loads first, then the first copies of the wave's first step, then the quantization, then the rest
    f32x4 xt[NB][XS];
#pragma unroll
    for (int r = 0; r < NB; r++)
#pragma unroll
        for (int j = 0; j < XS; j++) xt[r][j] = *(const f32x4 *)(a.x + (int64_t)r * k + min(wv + j * NW, bpr - 1) * 256 + lane * 4);
    asm volatile("" ::: "memory");
    uint8_t *slot = slots + wv * SLOT;
    const int step0 = wv * nblocks + block, sstride = NW * nblocks;
    const int my = step0 < total_steps ? (total_steps - step0 + sstride - 1) / sstride : 0;
    auto issue = [&](int t, int j0, int j1) {
        const bool live = t < my;
        const int64_t off = (int64_t)(live ? step0 + t * sstride : 0) * step_bytes;
        const int64_t left = w_bytes - off;
        const int bytes = live ? (int)(left < step_bytes ? left : step_bytes) : 0;     // an absent step: a descriptor of zero bytes
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(a.w + off), 0, bytes, 0x00020000);
#pragma unroll
        for (int j = 0; j < SF::NLD; j++)
            if (j >= j0 && j < j1) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (cq_lds_void *)(slot + j * 1024), 16, lane * 16, j * 1024, 0, 0);
    };
    issue(0, 0, PRE);
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < NB; r++) {
        float xv[XS][4];
#pragma unroll
        for (int j = 0; j < XS; j++) { xv[j][0] = xt[r][j].x; xv[j][1] = xt[r][j].y; xv[j][2] = xt[r][j].z; xv[j][3] = xt[r][j].w; }
        qs_quantize<DT, XS>(xv, wv, NW, bpr, MAXB, lane, act[r], SA::AUX_OFF);
    }
    asm volatile("" ::: "memory");
    issue(0, PRE, SF::NLD);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");       // no fence: it would wait for the copies in flight

    const int lp = 1 << lp_shift;
    const int rin = lane >> lp_shift, sb = lane & (lp - 1);
    const bool valid_sb = sb < bpr;
    const int sbc = valid_sb ? sb : bpr - 1;
    u32x4 areg[NB][16];
    QsAux aux[NB];
    float d8[NB];
#pragma unroll
    for (int r = 0; r < NB; r++) {
#pragma unroll
        for (int i = 0; i < 16; i++) areg[r][i] = *(const u32x4 *)(act[r] + sbc * QS_ACT_STRIDE + 16 * i);
        const uint8_t *auxp = act[r] + SA::AUX_OFF + sbc * QS_AUX_STRIDE;
        d8[r] = __uint_as_float((*(const u32x4 *)auxp).x);
        aux[r].s32 = *(const u32x4 *)(auxp + 16);
        if constexpr (qs_wide_aux(DT)) {
            aux[r].bl16 = *(const u32x4 *)(auxp + 32);
            aux[r].bh16 = *(const u32x4 *)(auxp + 48);
        }
    }
    const int boff = (rin * bpr + sbc) * SF::BB;
    const bool last = sb == lp - 1;
    for (int t = 0; t < my; t++) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const int row = (step0 + t * sstride) * step_rows + rin;
        typename SF::Blk b0;
        SF::read(b0, slot + boff);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        issue(t + 1, 0, SF::NLD);
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r = 0; r < NB; r++) {
            float v = SF::dot(b0, areg[r], d8[r], aux[r]);
            v = qs_group_sum(valid_sb ? v : 0.0f, lp_shift);
            if (last && row < n) store_out(a.dst, dst_dtype, (int64_t)r * a.stride_dst + row, v);
        }
    }
}

// Two weight tensors over the same activation row in one launch, tensor A on the streaming body; tensor B on the
// streaming body as well (SB) or on qmv_body.  Workgroups [0, blocks_a) take tensor A.  NW waves per workgroup: 8, or
// 16 where qmv_body needs one wave per activation span (its plane-merging prologue).
// Arguments of the two-tensor launch, 60 bytes: tensor B and its output are given as distances from tensor A's.
struct Qs2Args {
    const uint8_t *wa; const float *x, *aux, *extra; float *dsta;      // extra: partial sums (PRO_NORM) or planes (PRO_NORM_SPLIT)
    int na, nb;
    uint32_t meta;            // bpr | blocks_a << 8 | blocks_b << 16 | n_planes << 24
    float eps;
    int wb_off16;             // (wb - wa) / 16
    int dstb_off;             // dstb - dsta, in floats
};
// The arguments are scalars, ordered by first use, so that the fourteen dwords placed in SGPRs at wave launch are the ones
// the first loads need; the output pointer, needed last, is read from the argument block.
template <int DTA, int DTB, int NW, int XS, int MAXB, bool SINGLE, int PRO, bool SB>
__global__ __launch_bounds__(NW * 64) void qms2_kernel(const uint8_t *a_wa, const float *a_x, const float *a_aux, const float *a_extra, int a_na, int a_nb,
                                                       uint32_t a_meta, int a_wb_off16, float a_eps, int a_dstb_off, float *a_dsta) {
    const Qs2Args a{a_wa, a_x, a_aux, a_extra, a_dsta, a_na, a_nb, a_meta, a_eps, a_wb_off16, a_dstb_off};
    const int blocks_a = (a.meta >> 8) & 255, blocks_b = (a.meta >> 16) & 255, bpr = a.meta & 255;
    Fuse fz{a.aux, PRO == PRO_NORM ? a.extra : nullptr, a.eps, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0, PRO == PRO_NORM_SPLIT ? a.extra : nullptr,
            (int)(a.meta >> 24)};
    const bool first = (int)blockIdx.x < blocks_a;
    if (first || SB) {
        const int n = first ? a.na : a.nb;
        StreamGeom g;
        g.k = bpr * 256; g.n = n; g.bpr = bpr;
        g.lp_shift = bpr > 1 ? 32 - __builtin_clz(bpr - 1) : 0;
        g.step_rows = 64 >> g.lp_shift;
        g.dst_dtype = CQ_F32; g.stride_dst = n;
        g.total_steps = (n + g.step_rows - 1) >> (6 - g.lp_shift);
        if (first) {
            g.step_bytes = g.step_rows * bpr * StreamFmt<DTA>::BB;
            g.w_bytes = (int64_t)n * (bpr * StreamFmt<DTA>::BB);
            qms_body<DTA, NW, XS, MAXB, PRO, EPI_NONE>(a.wa, a.x, a.dsta, g, fz, blockIdx.x, blocks_a);
        } else if constexpr (SB) {
            g.step_bytes = g.step_rows * bpr * StreamFmt<DTB>::BB;
            g.w_bytes = (int64_t)n * (bpr * StreamFmt<DTB>::BB);
            qms_body<DTB, NW, XS, MAXB, PRO, EPI_NONE>(a.wa + (int64_t)a.wb_off16 * 16, a.x, a.dsta + a.dstb_off, g, fz, blockIdx.x - blocks_a, blocks_b);
        }
    } else if constexpr (!SB) {
        // tensor B on qmv_body: its geometry as make_geom() lays it out for NW waves and blocks_b workgroups
        QmvGeom gb;
        const int k = bpr * 256, n = a.nb;
        const int rows_per_wg = (n + blocks_b - 1) / blocks_b;
        const ActLayout L = cq_act_layout(DTB, k, 1);
        gb.k = k; gb.n = n; gb.rows_per_wg = rows_per_wg;
        gb.units = k / UnitFmt<DTB, 1, SINGLE>::type::UE; gb.steps = (gb.units + 63) >> 6;
        gb.lds_d_off = (int)L.d_off; gb.lds_bs_off = (int)L.bs_off;
        gb.nw_shift = NW == 16 ? 4 : 3;
        gb.row_bytes = (k / BlockInfo<DTB>::elems) * BlockInfo<DTB>::bytes;
        gb.lds_red_off = (int)L.total;
        gb.dst_dtype = CQ_F32; gb.stride_dst = n;
        ActSrc src{a.x, ActView{nullptr, nullptr, nullptr}};
        qmv_body<DTB, 1, CQ_F32, SINGLE, PRO, EPI_NONE, false>(a.wa + (int64_t)a.wb_off16 * 16, src, a.dsta + a.dstb_off, gb, fz, blockIdx.x - blocks_a, blocks_b);
    }
}

template <int DT, int XS, int MAXB, int PRO, int EPI, int MSP = 1>
int launch_stream_xs(const void *w, const float *x, void *dst, const StreamGeom &g, hipStream_t s, const Fuse &fz) {
    const size_t lds_bytes = (size_t)QS_NW * StreamFmt<DT>::NLD * 1024;
    if (lds_bytes + StreamAct<MAXB>::BYTES + 256 > (size_t)LDS_BUDGET) return CQ_ERR_RANGE;
    const int groups = qs_groups(g.total_steps);
    if (fz.pair_off % 16 || fz.n_planes > 15 || fz.splits > 63 || g.dst_dtype > 255) return CQ_ERR_RANGE;
    const dim3 grid((unsigned)groups), block(64 * QS_NW);
    const QsArgs<PRO, EPI> a = qs_pack<DT, PRO, EPI>(w, x, dst, g, fz);
    if constexpr (sizeof(QsArgs<PRO, EPI>) <= 56) {
        auto kern = qms_kernel_dw<DT, XS, MAXB, PRO, EPI, MSP>;
        if (lds_bytes > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (e != hipSuccess) return (int)e;
        }
        const Dwords14 r = to_dwords14(a);
        hipLaunchKernelGGL(kern, grid, block, lds_bytes, s, r.d[0], r.d[1], r.d[2], r.d[3], r.d[4], r.d[5], r.d[6], r.d[7], r.d[8], r.d[9], r.d[10], r.d[11],
                           r.d[12], r.d[13]);
    } else {
        auto kern = qms_kernel<DT, XS, MAXB, PRO, EPI, MSP>;
        if (lds_bytes > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (e != hipSuccess) return (int)e;
        }
        hipLaunchKernelGGL(kern, grid, block, lds_bytes, s, a);
    }
    return (int)hipGetLastError();
}

// the merge prologue in the smallest capacity that holds the launch's splits
template <int DT, int XS, int EPI>
int launch_stream_merge(const void *w, void *dst, const StreamGeom &g, hipStream_t s, const Fuse &fz) {
    if (fz.splits <= 4) return launch_stream_xs<DT, XS, 16, PRO_MERGE, EPI, 4>(w, nullptr, dst, g, s, fz);
    if (fz.splits <= 8) return launch_stream_xs<DT, XS, 16, PRO_MERGE, EPI, 8>(w, nullptr, dst, g, s, fz);
    return launch_stream_xs<DT, XS, 16, PRO_MERGE, EPI, MAXS>(w, nullptr, dst, g, s, fz);
}

// CQ_ERR_RANGE: not a shape (or fusion) of the streaming kernel; the caller takes qmv_kernel
template <int DT, int PRO, int EPI>
int launch_stream(const void *w, const float *x, void *dst, int dst_dtype, int64_t k, int64_t n, hipStream_t s, const Fuse &fz) {
    if constexpr (!qs_streams(DT)) {
        return CQ_ERR_RANGE;
    } else {
        StreamGeom g;
        if (!stream_geom<DT>(g, k, n, dst_dtype)) return CQ_ERR_RANGE;
        if ((uintptr_t)w & 15) return CQ_ERR_RANGE;              // the copies into LDS move aligned 16-byte pieces
        if (epi_is_resid(EPI) && n > (int64_t)256 * 64 * 1024) return CQ_ERR_RANGE;
        const int bpr = g.bpr;
        if constexpr (PRO == PRO_MERGE) {
            // rows of up to 4096 elements (as in qmv_kernel): the merge holds two spans of partials per wave
            if (bpr > 16) return CQ_ERR_RANGE;
            if (bpr <= 8) return launch_stream_merge<DT, 1, EPI>(w, dst, g, s, fz);
            return launch_stream_merge<DT, 2, EPI>(w, dst, g, s, fz);
        } else if constexpr (EPI == EPI_SWIGLU) {
            if (bpr > 16) return CQ_ERR_RANGE;                 // the range of the paired-row launch of qmv_kernel
            if (bpr <= 8) return launch_stream_xs<DT, 1, 16, PRO, EPI>(w, x, dst, g, s, fz);
            return launch_stream_xs<DT, 2, 16, PRO, EPI>(w, x, dst, g, s, fz);
        } else {
            if (bpr <= 8) return launch_stream_xs<DT, 1, 16, PRO, EPI>(w, x, dst, g, s, fz);
            if (bpr <= 16) return launch_stream_xs<DT, 2, 16, PRO, EPI>(w, x, dst, g, s, fz);
            if (bpr <= 32) return launch_stream_xs<DT, 4, 64, PRO, EPI>(w, x, dst, g, s, fz);
            if (bpr <= 56) return launch_stream_xs<DT, 7, 64, PRO, EPI>(w, x, dst, g, s, fz);
            return launch_stream_xs<DT, 8, 64, PRO, EPI>(w, x, dst, g, s, fz);
        }
    }
}

template <int DT, int XS, int MAXB>
int launch_stream_rows2_xs(const void *w, const float *x, void *dst, const StreamGeom &g, int64_t stride_dst, hipStream_t s) {
    const size_t lds_bytes = (size_t)QS_NW * StreamFmt<DT>::NLD * 1024;
    if (lds_bytes + 2 * StreamAct<MAXB>::BYTES + 256 > (size_t)LDS_BUDGET) return CQ_ERR_RANGE;
    auto kern = qms_rows2_kernel<DT, XS, MAXB>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    if (stride_dst > 0x7fffffffLL || g.dst_dtype > 255) return CQ_ERR_RANGE;
    QsRowsArgs a{(const uint8_t *)w, x, dst, g.n, (uint32_t)g.bpr | ((uint32_t)g.dst_dtype << 8), (int)stride_dst};
    hipLaunchKernelGGL(kern, dim3((unsigned)qs_groups(g.total_steps)), dim3(64 * QS_NW), lds_bytes, s, a.w, a.x, a.dst, a.n, a.meta, a.stride_dst);
    return (int)hipGetLastError();
}

// two f32 rows; CQ_ERR_RANGE: not a shape of the streaming kernel
template <int DT>
int launch_stream_rows2(const void *w, const float *x, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t stride_dst, hipStream_t s) {
    StreamGeom g;
    if (!stream_geom<DT>(g, k, n, dst_dtype) || ((uintptr_t)w & 15)) return CQ_ERR_RANGE;
    if (g.bpr <= 8) return launch_stream_rows2_xs<DT, 1, 16>(w, x, dst, g, stride_dst, s);
    if (g.bpr <= 16) return launch_stream_rows2_xs<DT, 2, 16>(w, x, dst, g, stride_dst, s);
    if (g.bpr <= 32) return launch_stream_rows2_xs<DT, 4, 64>(w, x, dst, g, stride_dst, s);
    if (g.bpr <= 56) return launch_stream_rows2_xs<DT, 7, 64>(w, x, dst, g, stride_dst, s);
    return launch_stream_rows2_xs<DT, 8, 64>(w, x, dst, g, stride_dst, s);
}

// Geometry of one launch.  waves == 0: as many waves per workgroup (a power of two, at most 16) as still leave every
// wave a row when 256 workgroups are launched; otherwise the given wave count is used.
template <int DT, int NB>
int make_geom(QmvGeom &g, int64_t &groups, int &waves, int64_t k, int64_t n, int64_t stride_dst, int dst_dtype, int extra_lds, size_t &lds_bytes,
              int64_t max_groups = 256) {
    // units of the instance that will run: rows longer than one wave step of Fmt<DT> may use another decomposition
    const bool single = k / Fmt<DT>::UE <= 64;
    const int ue = single ? Fmt<DT>::UE : UnitFmt<DT, NB, false>::type::UE;
    if (waves == 0) {
        waves = NB > 2 ? 8 : 16;
        while (waves > 1 && n < 256 * (int64_t)waves) waves >>= 1;
    }
    groups = (n + waves - 1) / waves;
    if (groups > max_groups) groups = max_groups;
    int64_t rows_per_wg = (n + groups - 1) / groups;
    groups = (n + rows_per_wg - 1) / rows_per_wg;
    const ActLayout L = cq_act_layout(DT, k, NB);
    lds_bytes = (size_t)L.total + extra_lds;
    g.lds_red_off = (int)L.total;
    g.k = (int)k; g.n = (int)n; g.rows_per_wg = (int)rows_per_wg;
    g.units = (int)(k / ue); g.steps = (g.units + 63) >> 6;
    g.lds_d_off = (int)L.d_off; g.lds_bs_off = (int)L.bs_off;
    g.nw_shift = 0;
    while ((1 << g.nw_shift) < waves) g.nw_shift++;
    int64_t rb = (k / BlockInfo<DT>::elems) * BlockInfo<DT>::bytes;
    if (rb > 0x3fffffff) return CQ_ERR_RANGE;
    g.row_bytes = (int)rb;
    g.dst_dtype = dst_dtype; g.stride_dst = stride_dst;
    return CQ_OK;
}

// PRO_NORM_SPLIT: the smallest workgroup (a power of two of waves) that gives every 256-element span its own wave
inline int split_min_waves(int64_t k) {
    const int64_t spans = (k + 255) / 256;
    if (spans > 16) return 0;
    int w = 1;
    while (w < spans) w <<= 1;
    return w;
}

template <int DT, int NB, int SRC, bool SINGLE, int PRO = PRO_NONE, int EPI = EPI_NONE, bool PRE = false>
int launch_cfg(const void *w, const ActSrc &src, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t stride_dst, hipStream_t s,
               const Fuse &fz = Fuse{nullptr, nullptr, 0.0f, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0}) {
    QmvGeom g;
    int64_t groups;
    int waves = 0;
    size_t lds_bytes;
    constexpr int XL = epi_is_resid(EPI) || pro_is_split(PRO) ? 64 : 0;
    int rc = make_geom<DT, NB>(g, groups, waves, k, n, stride_dst, dst_dtype, XL, lds_bytes);
    if (rc) return rc;
    Fuse f2 = fz;
    if (pro_is_split(PRO)) {
        const int need = split_min_waves(k);                        // one span per wave
        if (need == 0) return CQ_ERR_RANGE;
        if (waves < need) {
            waves = need;
            if ((rc = make_geom<DT, NB>(g, groups, waves, k, n, stride_dst, dst_dtype, XL, lds_bytes))) return rc;
        }
    }
    auto kern = qmv_kernel<DT, NB, SRC, SINGLE, PRO, EPI, PRE>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)groups), dim3(64 * waves), lds_bytes, s, (const uint8_t *)w, src, dst, g, f2);
    return (int)hipGetLastError();
}

template <int DT, int NB, int SRC>
int launch_nb(const void *w, const ActSrc &src, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t stride_dst, hipStream_t s) {
    if (k / Fmt<DT>::UE <= 64) return launch_cfg<DT, NB, SRC, true>(w, src, dst, dst_dtype, k, n, stride_dst, s);
    if (NB == 1 && k / UnitFmt<DT, NB, false>::type::UE <= 256)
        return launch_cfg<DT, NB, SRC, false, PRO_NONE, EPI_NONE, NB == 1>(w, src, dst, dst_dtype, k, n, stride_dst, s);
    return launch_cfg<DT, NB, SRC, false>(w, src, dst, dst_dtype, k, n, stride_dst, s);
}

template <int DT, int SRC>
int launch_rows(const void *w, const ActSrc &src, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst,
                hipStream_t s) {
    // Q4_1, Q5_0, Q5_1, Q2_K, Q3_K have the fused instances QMatMul::forward uses (f32 activations, one or two rows);
    // everything else of theirs goes through the pre-quantized scratch.
    if constexpr (!cq_full_matvec(DT) && SRC != SRC_SCRATCH) {
        if constexpr (SRC == CQ_F32) {
            if (rows == 1) return launch_nb<DT, 1, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            if (rows == 2) return launch_nb<DT, 2, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
        }
        return CQ_ERR_RANGE;
    } else {
        switch (rows) {
            case 1: return launch_nb<DT, 1, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            case 2: return launch_nb<DT, 2, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            case 3: return launch_nb<DT, 3, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            case 4: return launch_nb<DT, 4, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            case 5: return launch_nb<DT, 5, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            case 6: return launch_nb<DT, 6, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            case 7: return launch_nb<DT, 7, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
            case 8: return launch_nb<DT, 8, SRC>(w, src, dst, dst_dtype, k, n, stride_dst, s);
        }
        return CQ_ERR_RANGE;
    }
}

template <int SRC>
int launch_dt(int w_dtype, const void *w, const ActSrc &src, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows,
              int64_t stride_dst, hipStream_t s) {
    switch (w_dtype) {
        case CQ_Q4_0: return launch_rows<CQ_Q4_0, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q8_0: return launch_rows<CQ_Q8_0, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q4K: return launch_rows<CQ_Q4K, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q5K: return launch_rows<CQ_Q5K, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q6K: return launch_rows<CQ_Q6K, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q4_1: return launch_rows<CQ_Q4_1, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q5_0: return launch_rows<CQ_Q5_0, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q5_1: return launch_rows<CQ_Q5_1, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q2K: return launch_rows<CQ_Q2K, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
        case CQ_Q3K: return launch_rows<CQ_Q3K, SRC>(w, src, dst, dst_dtype, k, n, rows, stride_dst, s);
    }
    return CQ_ERR_DTYPE;
}

// Activation rows are processed in groups whose quantized form fits in LDS (always all of them for
// the shapes of an 8B decoder; a very long k with 8 rows is split, each group streaming W once).
template <class Launch>
int for_row_groups(int w_dtype, int64_t k, int64_t rows, Launch launch) {
    int64_t per_row = cq_act_layout(w_dtype, k, 1).total;
    if (per_row > LDS_BUDGET) return CQ_ERR_RANGE;
    int64_t fit = rows;
    while (fit > 1 && cq_act_layout(w_dtype, k, fit).total > LDS_BUDGET) fit--;
    for (int64_t r0 = 0; r0 < rows; r0 += fit) {
        int rc = launch(r0, rows - r0 < fit ? rows - r0 : fit);
        if (rc) return rc;
    }
    return CQ_OK;
}

}  // namespace

int cq_matvec_launch_av(int w_dtype, const void *w, const ActView &av, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows,
                        int64_t stride_dst, hipStream_t s) {
    if (n == 0 || rows == 0) return CQ_OK;
    const int64_t esz = dst_dtype == CQ_F32 ? 4 : 2;
    return for_row_groups(w_dtype, k, rows, [&](int64_t r0, int64_t nb) {
        ActSrc src;
        src.x = nullptr;
        src.av = cq_act_view_rows(av, w_dtype, k, r0);
        return launch_dt<SRC_SCRATCH>(w_dtype, w, src, (uint8_t *)dst + r0 * stride_dst * esz, dst_dtype, k, n, nb, stride_dst, s);
    });
}

int cq_matvec_launch(int w_dtype, const void *w, const void *scratch, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows,
                     int64_t stride_dst, hipStream_t s) {
    return cq_matvec_launch_av(w_dtype, w, cq_act_view(scratch, w_dtype, k, rows), dst, dst_dtype, k, n, rows, stride_dst, s);
}

// QMatMul::forward for up to CQ_MATVEC_MAX_ROWS activation rows, activation quantization fused in.
int cq_matvec_fused_launch(int w_dtype, const void *w, const void *x, int x_dtype, void *dst, int dst_dtype, int64_t k, int64_t n,
                           int64_t rows, int64_t stride_dst, hipStream_t s) {
    if (n == 0 || rows == 0) return CQ_OK;
    if (rows == 1 && x_dtype == CQ_F32) {
        // one f32 row over Q4_K / Q5_K / Q6_K / Q4_0 / Q8_0 weights: the streaming kernel where it takes the shape
        const Fuse none{nullptr, nullptr, 0.0f, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0};
        int rc = CQ_ERR_RANGE;
        if (w_dtype == CQ_Q4K) rc = launch_stream<CQ_Q4K, PRO_NONE, EPI_NONE>(w, (const float *)x, dst, dst_dtype, k, n, s, none);
        if (w_dtype == CQ_Q5K) rc = launch_stream<CQ_Q5K, PRO_NONE, EPI_NONE>(w, (const float *)x, dst, dst_dtype, k, n, s, none);
        if (w_dtype == CQ_Q6K) rc = launch_stream<CQ_Q6K, PRO_NONE, EPI_NONE>(w, (const float *)x, dst, dst_dtype, k, n, s, none);
        if (w_dtype == CQ_Q4_0) rc = launch_stream<CQ_Q4_0, PRO_NONE, EPI_NONE>(w, (const float *)x, dst, dst_dtype, k, n, s, none);
        if (w_dtype == CQ_Q8_0) rc = launch_stream<CQ_Q8_0, PRO_NONE, EPI_NONE>(w, (const float *)x, dst, dst_dtype, k, n, s, none);
        if (rc != CQ_ERR_RANGE) return rc;
    }
    if (rows == 2 && x_dtype == CQ_F32) {
        // two f32 rows: both on one pass of the streaming kernel
        int rc = CQ_ERR_RANGE;
        if (w_dtype == CQ_Q4K) rc = launch_stream_rows2<CQ_Q4K>(w, (const float *)x, dst, dst_dtype, k, n, stride_dst, s);
        if (w_dtype == CQ_Q5K) rc = launch_stream_rows2<CQ_Q5K>(w, (const float *)x, dst, dst_dtype, k, n, stride_dst, s);
        if (w_dtype == CQ_Q6K) rc = launch_stream_rows2<CQ_Q6K>(w, (const float *)x, dst, dst_dtype, k, n, stride_dst, s);
        if (w_dtype == CQ_Q4_0) rc = launch_stream_rows2<CQ_Q4_0>(w, (const float *)x, dst, dst_dtype, k, n, stride_dst, s);
        if (w_dtype == CQ_Q8_0) rc = launch_stream_rows2<CQ_Q8_0>(w, (const float *)x, dst, dst_dtype, k, n, stride_dst, s);
        if (rc != CQ_ERR_RANGE) return rc;
    }
    const int64_t xsz = x_dtype == CQ_F32 ? 4 : 2, esz = dst_dtype == CQ_F32 ? 4 : 2;
    return for_row_groups(w_dtype, k, rows, [&](int64_t r0, int64_t nb) {
        ActSrc src;
        src.x = (const uint8_t *)x + r0 * k * xsz;
        src.av = ActView{nullptr, nullptr, nullptr};
        void *d = (uint8_t *)dst + r0 * stride_dst * esz;
        switch (x_dtype) {
            case CQ_F32: return launch_dt<CQ_F32>(w_dtype, w, src, d, dst_dtype, k, n, nb, stride_dst, s);
            case CQ_F16: return launch_dt<CQ_F16>(w_dtype, w, src, d, dst_dtype, k, n, nb, stride_dst, s);
            case CQ_BF16: return launch_dt<CQ_BF16>(w_dtype, w, src, d, dst_dtype, k, n, nb, stride_dst, s);
        }
        return (int)CQ_ERR_DTYPE;
    });
}

namespace {
template <int DT, int PRO, int EPI>
int launch_fused1(const void *w, const ActSrc &src, void *dst, int64_t k, int64_t n, hipStream_t s, const Fuse &fz) {
    if (cq_act_layout(DT, k, 1).total + 64 > LDS_BUDGET) return CQ_ERR_RANGE;
    // the plane-merging prologue keeps its range (rows of one wave step of qmv_kernel) whichever kernel runs
    if (!pro_is_split(PRO) || k / Fmt<DT>::UE <= 64) {
        const int rc = launch_stream<DT, PRO, EPI>(w, (const float *)src.x, dst, CQ_F32, k, n, s, fz);
        if (rc != CQ_ERR_RANGE) return rc;
    }
    if (k / Fmt<DT>::UE <= 64) return launch_cfg<DT, 1, CQ_F32, true, PRO, EPI>(w, src, dst, CQ_F32, k, n, n, s, fz);
    if constexpr (pro_is_split(PRO)) {
        return CQ_ERR_RANGE;                                 // one span per wave: rows of one wave step only
    } else {
        if (k / UnitFmt<DT, 1, false>::type::UE <= 256) return launch_cfg<DT, 1, CQ_F32, false, PRO, EPI, true>(w, src, dst, CQ_F32, k, n, n, s, fz);
        return launch_cfg<DT, 1, CQ_F32, false, PRO, EPI>(w, src, dst, CQ_F32, k, n, n, s, fz);
    }
}
template <int PRO, int EPI>
int launch_fused_dt(int w_dtype, const void *w, const ActSrc &src, void *dst, int64_t k, int64_t n, hipStream_t s, const Fuse &fz) {
    switch (w_dtype) {
        case CQ_Q4_0: return launch_fused1<CQ_Q4_0, PRO, EPI>(w, src, dst, k, n, s, fz);
        case CQ_Q8_0: return launch_fused1<CQ_Q8_0, PRO, EPI>(w, src, dst, k, n, s, fz);
        case CQ_Q4K: return launch_fused1<CQ_Q4K, PRO, EPI>(w, src, dst, k, n, s, fz);
        case CQ_Q5K: return launch_fused1<CQ_Q5K, PRO, EPI>(w, src, dst, k, n, s, fz);
        case CQ_Q6K: return launch_fused1<CQ_Q6K, PRO, EPI>(w, src, dst, k, n, s, fz);
    }
    // Q4_1, Q5_0, Q5_1, Q2_K, Q3_K have the three fusions a decoder step cannot do without: the rms_norm
    // prologue, and the residual epilogue with and without the silu * up prologue.
    if constexpr ((PRO == PRO_NORM && EPI == EPI_NONE) || ((PRO == PRO_NONE || PRO == PRO_SILU) && EPI == EPI_RESID)) {
        switch (w_dtype) {
            case CQ_Q4_1: return launch_fused1<CQ_Q4_1, PRO, EPI>(w, src, dst, k, n, s, fz);
            case CQ_Q5_0: return launch_fused1<CQ_Q5_0, PRO, EPI>(w, src, dst, k, n, s, fz);
            case CQ_Q5_1: return launch_fused1<CQ_Q5_1, PRO, EPI>(w, src, dst, k, n, s, fz);
            case CQ_Q2K: return launch_fused1<CQ_Q2K, PRO, EPI>(w, src, dst, k, n, s, fz);
            case CQ_Q3K: return launch_fused1<CQ_Q3K, PRO, EPI>(w, src, dst, k, n, s, fz);
        }
    }
    return CQ_ERR_DTYPE;
}
}  // namespace

// dst[n] = W . quantize(rms_norm(x) * norm_weight), sum(x^2) given as 256 partial sums
int cq_matvec_norm_launch(int w_dtype, const void *w, const float *x, const float *partials, const float *norm_weight, float eps, float *dst,
                          int64_t k, int64_t n, hipStream_t s) {
    if (n == 0) return CQ_OK;
    ActSrc src{x, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{norm_weight, partials, eps, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0};
    return launch_fused_dt<PRO_NORM, EPI_NONE>(w_dtype, w, src, dst, k, n, s, fz);
}

// residual[n] = (residual + planes[0] + ...) + W . quantize(up ? silu(x) * up : x); partials_out[256] = partial sums of residual^2
int cq_matvec_residual_launch(int w_dtype, const void *w, const float *x, const float *up, float *residual, float *partials_out,
                              const float *planes, int64_t n_planes, int64_t k, int64_t n, hipStream_t s) {
    if (n == 0) return CQ_OK;
    if (n_planes < 0 || n_planes > MAXP) return CQ_ERR_RANGE;
    ActSrc src{x, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{up, nullptr, 0.0f, residual, partials_out, 0, 0, 0, nullptr, nullptr, 0, planes, (int)n_planes};
    if (n_planes > 0) {
        if (up) return launch_fused_dt<PRO_SILU, EPI_RESID_SPLIT>(w_dtype, w, src, nullptr, k, n, s, fz);
        return launch_fused_dt<PRO_NONE, EPI_RESID_SPLIT>(w_dtype, w, src, nullptr, k, n, s, fz);
    }
    if (up) return launch_fused_dt<PRO_SILU, EPI_RESID>(w_dtype, w, src, nullptr, k, n, s, fz);
    return launch_fused_dt<PRO_NONE, EPI_RESID>(w_dtype, w, src, nullptr, k, n, s, fz);
}

namespace {
template <int DT>
int launch_merge1(const void *w, void *dst, int64_t k, int64_t n, hipStream_t s, const Fuse &fz) {
    if (k / Fmt<DT>::UE > 64) return CQ_ERR_RANGE;          // one wave step per row, one span per wave
    ActSrc src{nullptr, ActView{nullptr, nullptr, nullptr}};
    {
        const int rc = fz.n_planes > 0 ? launch_stream<DT, PRO_MERGE, EPI_RESID_SPLIT>(w, nullptr, dst, CQ_F32, k, n, s, fz)
                                       : launch_stream<DT, PRO_MERGE, EPI_RESID>(w, nullptr, dst, CQ_F32, k, n, s, fz);
        if (rc != CQ_ERR_RANGE) return rc;
    }
    if (fz.n_planes > 0) return launch_cfg<DT, 1, CQ_F32, true, PRO_MERGE, EPI_RESID_SPLIT>(w, src, dst, CQ_F32, k, n, n, s, fz);
    return launch_cfg<DT, 1, CQ_F32, true, PRO_MERGE, EPI_RESID>(w, src, dst, CQ_F32, k, n, n, s, fz);
}
}  // namespace

// residual[n] += W . quantize(merge(attention partials)); partials_out[256] = partial sums of residual^2.
// CQ_ERR_RANGE when the row is longer than one wave step (k > 4096 for K-quants, > 2048 for Q4_0 / Q8_0),
// when splits > 16, or when head_dim is not a power of two.
int cq_matvec_residual_attn_launch(int w_dtype, const void *w, const float *attn_partials, int64_t splits, int64_t head_dim, float *residual,
                                   float *partials_out, const float *planes, int64_t n_planes, int64_t k, int64_t n, hipStream_t s) {
    if (n == 0) return CQ_OK;
    if (splits < 1 || splits > MAXS || head_dim < 4 || (head_dim & (head_dim - 1)) || k % head_dim) return CQ_ERR_RANGE;
    if (n_planes < 0 || n_planes > MAXP) return CQ_ERR_RANGE;
    int sh = 0;
    while ((1 << sh) < head_dim) sh++;
    Fuse fz{attn_partials, nullptr, 0.0f, residual, partials_out, (int)splits, sh, 0, nullptr, nullptr, 0, planes, (int)n_planes};
    switch (w_dtype) {
        case CQ_Q4_0: return launch_merge1<CQ_Q4_0>(w, nullptr, k, n, s, fz);
        case CQ_Q8_0: return launch_merge1<CQ_Q8_0>(w, nullptr, k, n, s, fz);
        case CQ_Q4K: return launch_merge1<CQ_Q4K>(w, nullptr, k, n, s, fz);
        case CQ_Q5K: return launch_merge1<CQ_Q5K>(w, nullptr, k, n, s, fz);
        case CQ_Q6K: return launch_merge1<CQ_Q6K>(w, nullptr, k, n, s, fz);
    }
    return CQ_ERR_DTYPE;
}

namespace {
template <int DT>
int launch_swiglu1(const void *w1, int64_t pair_off, const ActSrc &src, float *dst, int64_t k, int64_t ffn, hipStream_t s, Fuse fz) {
    if (k / Fmt<DT>::UE > 64) return CQ_ERR_RANGE;
    fz.pair_off = pair_off;
    {
        const int rc = launch_stream<DT, PRO_NORM, EPI_SWIGLU>(w1, (const float *)src.x, dst, CQ_F32, k, ffn, s, fz);
        if (rc != CQ_ERR_RANGE) return rc;
    }
    return launch_cfg<DT, 1, CQ_F32, true, PRO_NORM, EPI_SWIGLU>(w1, src, dst, CQ_F32, k, ffn, ffn, s, fz);
}

// The two-tensor launch with tensor A (and tensor B, when its format and shape allow) on the streaming body.
// CQ_ERR_RANGE: tensor A is not a shape of the streaming kernel.
template <int DTA, int DTB, int NW, int XS, int MAXB, int PRO>
int launch_pair_stream_xs(const void *wa, float *dsta, const void *wb, int64_t nb, float *dstb, const float *x, int64_t k, hipStream_t s,
                          const Fuse &fz, const StreamGeom &ga, bool sb, const StreamGeom &gsb) {
    constexpr int XL = pro_is_split(PRO) ? 64 : 0;
    // 256 workgroups in total, shared between the tensors in proportion to their bytes
    const double bytes_a = (double)ga.n * BlockInfo<DTA>::bytes / BlockInfo<DTA>::elems, bytes_b = (double)nb * BlockInfo<DTB>::bytes / BlockInfo<DTB>::elems;
    int64_t share_a = (int64_t)(256.0 * bytes_a / (bytes_a + bytes_b) + 0.5);
    if (share_a < 1) share_a = 1;
    if (share_a > 255) share_a = 255;
    const int64_t groups_a = ga.total_steps < share_a ? ga.total_steps : share_a;
    QmvGeom gb{};
    int64_t groups_b;
    size_t lds_b = 0;
    if (sb) {
        groups_b = gsb.total_steps < 256 - share_a ? gsb.total_steps : 256 - share_a;
    } else {
        int waves = NW;
        const int rc = make_geom<DTB, 1>(gb, groups_b, waves, k, nb, nb, CQ_F32, XL, lds_b, 256 - share_a);
        if (rc) return rc;
    }
    size_t lds_a = (size_t)NW * StreamFmt<DTA>::NLD * 1024;
    if constexpr (qs_streams(DTB)) {
        if (sb && (size_t)NW * StreamFmt<DTB>::NLD * 1024 > lds_a) lds_a = (size_t)NW * StreamFmt<DTB>::NLD * 1024;
    }
    const size_t lds_bytes = lds_a > lds_b ? lds_a : lds_b;
    if (lds_bytes + StreamAct<MAXB>::BYTES + 256 > (size_t)LDS_BUDGET) return CQ_ERR_RANGE;
    const bool single = k / 64 <= 64;
    // tensor B and its output travel as 32-bit distances from tensor A's; a launch they do not fit takes qmv2_kernel
    const int64_t wdist = (const uint8_t *)wb - (const uint8_t *)wa, ddist = dstb - dsta;
    if (wdist % 16 || wdist / 16 > 0x7fffffffLL || wdist / 16 < -0x7fffffffLL || ddist > 0x7fffffffLL || ddist < -0x7fffffffLL) return CQ_ERR_RANGE;
    if (groups_a > 255 || groups_b > 255 || groups_b < 1 || fz.n_planes > 15) return CQ_ERR_RANGE;
    if (!sb) {
        // qmv_body's geometry is rebuilt in the kernel from (nb, blocks_b): it must be what make_geom() returned
        const int64_t rpw = (nb + groups_b - 1) / groups_b;
        if (gb.rows_per_wg != rpw || (nb + rpw - 1) / rpw != groups_b) return CQ_ERR_RANGE;
    }
    Qs2Args a;
    a.wa = (const uint8_t *)wa; a.x = x; a.aux = fz.aux; a.extra = PRO == PRO_NORM ? fz.part_in : fz.planes; a.dsta = dsta;
    a.na = ga.n; a.nb = (int)nb;
    a.meta = (uint32_t)ga.bpr | ((uint32_t)groups_a << 8) | ((uint32_t)groups_b << 16) | ((uint32_t)fz.n_planes << 24);
    a.eps = fz.eps; a.wb_off16 = (int)(wdist / 16); a.dstb_off = (int)ddist;
    dim3 grid((unsigned)(groups_a + groups_b)), block(64 * NW);
    auto go = [&](auto kern) {
        if (lds_bytes > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (e != hipSuccess) return (int)e;
        }
        hipLaunchKernelGGL(kern, grid, block, lds_bytes, s, a.wa, a.x, a.aux, a.extra, a.na, a.nb, a.meta, a.wb_off16, a.eps, a.dstb_off, a.dsta);
        return (int)hipGetLastError();
    };
    // (the sixteen-wave launch exists for a tensor B that does not stream)
    if (sb && NW != QS_NW) return CQ_ERR_RANGE;
    if constexpr (qs_streams(DTB) && NW == QS_NW) {
        if (sb) return go(qms2_kernel<DTA, DTB, NW, XS, MAXB, true, PRO, true>);
    }
    if (single) return go(qms2_kernel<DTA, DTB, NW, XS, MAXB, true, PRO, false>);
    return go(qms2_kernel<DTA, DTB, NW, XS, MAXB, false, PRO, false>);
}

template <int DTA, int DTB, int PRO>
int launch_pair_stream(const void *wa, int64_t na, float *dsta, const void *wb, int64_t nb, float *dstb, const float *x, int64_t k, hipStream_t s,
                       const Fuse &fz) {
    StreamGeom ga;
    if (!stream_geom<DTA>(ga, k, na, CQ_F32) || ((uintptr_t)wa & 15)) return CQ_ERR_RANGE;
    const int bpr = ga.bpr;
    if (bpr > 16) return CQ_ERR_RANGE;            // longer rows: the two-tensor launch of qmv_kernel
    StreamGeom gsb = ga;
    bool sb = false;
    if constexpr (qs_streams(DTB)) sb = stream_geom<DTB>(gsb, k, nb, CQ_F32);
    if (pro_is_split(PRO) && !sb) {
        // qmv_body merges the planes with one activation span per wave: sixteen waves (and one span per wave here too)
        if (StreamFmt<DTA>::NLD * 16 * 1024 + StreamAct<16>::BYTES + 256 > LDS_BUDGET) return CQ_ERR_RANGE;
        return launch_pair_stream_xs<DTA, DTB, 16, 1, 16, PRO>(wa, dsta, wb, nb, dstb, x, k, s, fz, ga, sb, gsb);
    }
    if (bpr <= 8) return launch_pair_stream_xs<DTA, DTB, QS_NW, 1, 16, PRO>(wa, dsta, wb, nb, dstb, x, k, s, fz, ga, sb, gsb);
    return launch_pair_stream_xs<DTA, DTB, QS_NW, 2, 16, PRO>(wa, dsta, wb, nb, dstb, x, k, s, fz, ga, sb, gsb);
}

template <int DTA, int DTB, int PRO>
int launch_pair(const void *wa, int64_t na, float *dsta, const void *wb, int64_t nb, float *dstb, const ActSrc &src, int64_t k, hipStream_t s,
                const Fuse &fz_in) {
    constexpr int XL = pro_is_split(PRO) ? 64 : 0;
    if constexpr (qs_streams(DTA) || qs_streams(DTB)) {
        // rows the streaming kernel takes but its two-tensor launch does not (more than 4096 elements): two launches,
        // each on the kernel a single call would get
        StreamGeom gt;
        const bool sa = stream_geom<DTA>(gt, k, na, CQ_F32), sbb = stream_geom<DTB>(gt, k, nb, CQ_F32);
        if ((sa || sbb) && k / 256 > 16) {
            const int rc = launch_fused1<DTA, PRO, EPI_NONE>(wa, src, dsta, k, na, s, fz_in);
            return rc ? rc : launch_fused1<DTB, PRO, EPI_NONE>(wb, src, dstb, k, nb, s, fz_in);
        }
    }
    if constexpr (!qs_streams(DTA) && qs_streams(DTB)) {
        // only tensor B has a streaming body: the same launch with the tensors exchanged
        StreamGeom gt;
        if (stream_geom<DTB>(gt, k, nb, CQ_F32) && gt.bpr <= 16) return launch_pair<DTB, DTA, PRO>(wb, nb, dstb, wa, na, dsta, src, k, s, fz_in);
    }
    if constexpr (qs_streams(DTA)) {
        int rc = launch_pair_stream<DTA, DTB, PRO>(wa, na, dsta, wb, nb, dstb, (const float *)src.x, k, s, fz_in);
        if (rc != CQ_ERR_RANGE) return rc;
        // the two-tensor launch does not take this call (the tensors or their outputs lie further apart than its 32-bit
        // distances, or a geometry it has no kernel for): when a single call would stream, two launches, each on the
        // kernel a single call gets, so that the results do not depend on where the buffers happen to lie
        StreamGeom gt;
        if (stream_geom<DTA>(gt, k, na, CQ_F32) || stream_geom<DTB>(gt, k, nb, CQ_F32)) {
            rc = launch_fused1<DTA, PRO, EPI_NONE>(wa, src, dsta, k, na, s, fz_in);
            return rc ? rc : launch_fused1<DTB, PRO, EPI_NONE>(wb, src, dstb, k, nb, s, fz_in);
        }
    }
    QmvGeom ga, gb;
    int64_t groups_a, groups_b;
    size_t lds_a, lds_b;
    // one block size for both segments: that of the larger tensor
    int waves = 0;
    int rc = na >= nb ? make_geom<DTA, 1>(ga, groups_a, waves, k, na, na, CQ_F32, XL, lds_a) : make_geom<DTB, 1>(gb, groups_b, waves, k, nb, nb, CQ_F32, XL, lds_b);
    if (rc) return rc;
    if (pro_is_split(PRO)) {
        const int need = split_min_waves(k);                        // one span per wave
        if (need == 0) return CQ_ERR_RANGE;
        if (waves < need) waves = need;
    }
    // 256 workgroups in total (one per CU: a 16-wave workgroup fills a CU's registers, so a 257th would wait for a
    // whole workgroup to finish), shared between the tensors in proportion to their bytes
    const double bytes_a = (double)na * BlockInfo<DTA>::bytes / BlockInfo<DTA>::elems, bytes_b = (double)nb * BlockInfo<DTB>::bytes / BlockInfo<DTB>::elems;
    int64_t share_a = (int64_t)(256.0 * bytes_a / (bytes_a + bytes_b) + 0.5);
    if (share_a < 1) share_a = 1;
    if (share_a > 255) share_a = 255;
    if ((rc = make_geom<DTA, 1>(ga, groups_a, waves, k, na, na, CQ_F32, XL, lds_a, share_a))) return rc;
    if ((rc = make_geom<DTB, 1>(gb, groups_b, waves, k, nb, nb, CQ_F32, XL, lds_b, 256 - share_a))) return rc;
    const size_t lds_bytes = lds_a > lds_b ? lds_a : lds_b;
    const bool single = k / 64 <= 64;                     // every K-quant unit is 64 elements
    const Fuse &fz = fz_in;
    if (lds_bytes > 48 * 1024) {
        const void *kp = single ? (const void *)qmv2_kernel<DTA, DTB, true, PRO> : (const void *)qmv2_kernel<DTA, DTB, false, PRO>;
        hipError_t e = hipFuncSetAttribute(kp, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    dim3 grid((unsigned)(groups_a + groups_b)), block(64 * waves);
    if (single)
        hipLaunchKernelGGL((qmv2_kernel<DTA, DTB, true, PRO>), grid, block, lds_bytes, s, (const uint8_t *)wa, (const uint8_t *)wb, src,
                           (void *)dsta, (void *)dstb, ga, gb, fz, (int)groups_a);
    else
        hipLaunchKernelGGL((qmv2_kernel<DTA, DTB, false, PRO>), grid, block, lds_bytes, s, (const uint8_t *)wa, (const uint8_t *)wb, src,
                           (void *)dsta, (void *)dstb, ga, gb, fz, (int)groups_a);
    return (int)hipGetLastError();
}

template <int DTA, int PRO>
int launch_pair_b(int dtb, const void *wa, int64_t na, float *dsta, const void *wb, int64_t nb, float *dstb, const ActSrc &src, int64_t k,
                  hipStream_t s, const Fuse &fz) {
    switch (dtb) {
        case CQ_Q4K: return launch_pair<DTA, CQ_Q4K, PRO>(wa, na, dsta, wb, nb, dstb, src, k, s, fz);
        case CQ_Q5K: return launch_pair<DTA, CQ_Q5K, PRO>(wa, na, dsta, wb, nb, dstb, src, k, s, fz);
        case CQ_Q6K: return launch_pair<DTA, CQ_Q6K, PRO>(wa, na, dsta, wb, nb, dstb, src, k, s, fz);
    }
    return CQ_ERR_DTYPE;
}
template <int PRO>
int launch_pair_a(int dta, int dtb, const void *wa, int64_t na, float *dsta, const void *wb, int64_t nb, float *dstb, const ActSrc &src, int64_t k,
                  hipStream_t s, const Fuse &fz) {
    switch (dta) {
        case CQ_Q4K: return launch_pair_b<CQ_Q4K, PRO>(dtb, wa, na, dsta, wb, nb, dstb, src, k, s, fz);
        case CQ_Q5K: return launch_pair_b<CQ_Q5K, PRO>(dtb, wa, na, dsta, wb, nb, dstb, src, k, s, fz);
        case CQ_Q6K: return launch_pair_b<CQ_Q6K, PRO>(dtb, wa, na, dsta, wb, nb, dstb, src, k, s, fz);
    }
    return CQ_ERR_DTYPE;
}
}  // namespace

// h[ffn] = silu(W1 . xn) * (W3 . xn), xn = quantize(rms_norm(x) * norm_weight); W3 row r lies pair_off bytes behind W1 row r.
// CQ_ERR_RANGE when a row is longer than one wave step.
int cq_matvec_norm_swiglu_launch(int w_dtype, const void *w1, const void *w3, const float *x, const float *partials, const float *norm_weight,
                                 float eps, float *dst, int64_t k, int64_t ffn, hipStream_t s) {
    if (ffn == 0) return CQ_OK;
    ActSrc src{x, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{norm_weight, partials, eps, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0};
    const int64_t off = (const uint8_t *)w3 - (const uint8_t *)w1;
    switch (w_dtype) {
        case CQ_Q4_0: return launch_swiglu1<CQ_Q4_0>(w1, off, src, dst, k, ffn, s, fz);
        case CQ_Q8_0: return launch_swiglu1<CQ_Q8_0>(w1, off, src, dst, k, ffn, s, fz);
        case CQ_Q4K: return launch_swiglu1<CQ_Q4K>(w1, off, src, dst, k, ffn, s, fz);
        case CQ_Q5K: return launch_swiglu1<CQ_Q5K>(w1, off, src, dst, k, ffn, s, fz);
        case CQ_Q6K: return launch_swiglu1<CQ_Q6K>(w1, off, src, dst, k, ffn, s, fz);
    }
    return CQ_ERR_DTYPE;
}

// dst_a[na] = Wa . xn and dst_b[nb] = Wb . xn in one launch, xn = quantize(rms_norm(x) * norm_weight); both K-quants.
int cq_matvec_norm_pair_launch(int dta, const void *wa, int64_t na, float *dsta, int dtb, const void *wb, int64_t nb, float *dstb, const float *x,
                               const float *partials, const float *norm_weight, float eps, int64_t k, hipStream_t s) {
    if (!cq_is_kquant(dta) || !cq_is_kquant(dtb) || dta == CQ_Q8K || dtb == CQ_Q8K) return CQ_ERR_DTYPE;
    if (na == 0 || nb == 0) return CQ_ERR_SHAPE;
    if (cq_act_layout(dta, k, 1).total > LDS_BUDGET) return CQ_ERR_RANGE;
    ActSrc src{x, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{norm_weight, partials, eps, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0};
    return launch_pair_a<PRO_NORM>(dta, dtb, wa, na, dsta, wb, nb, dstb, src, k, s, fz);
}

// The same two launches for a row still split over K-slice planes: ((x + planes[0]) + planes[1]) + ... is
// normalized, with the sum of squares computed in the kernel.
int cq_matvec_norm_pair_merge_launch(int dta, const void *wa, int64_t na, float *dsta, int dtb, const void *wb, int64_t nb, float *dstb,
                                     const float *x, const float *planes, int64_t n_planes, const float *norm_weight, float eps, int64_t k,
                                     hipStream_t s) {
    if (!cq_is_kquant(dta) || !cq_is_kquant(dtb) || dta == CQ_Q8K || dtb == CQ_Q8K) return CQ_ERR_DTYPE;
    if (na == 0 || nb == 0) return CQ_ERR_SHAPE;
    if (n_planes < 1 || n_planes > MAXP) return CQ_ERR_RANGE;
    if (cq_act_layout(dta, k, 1).total + 64 > LDS_BUDGET) return CQ_ERR_RANGE;
    ActSrc src{x, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{norm_weight, nullptr, eps, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0, planes, (int)n_planes};
    return launch_pair_a<PRO_NORM_SPLIT>(dta, dtb, wa, na, dsta, wb, nb, dstb, src, k, s, fz);
}

int cq_matvec_norm_merge_launch(int w_dtype, const void *w, const float *x, const float *planes, int64_t n_planes, const float *norm_weight,
                                float eps, float *dst, int64_t k, int64_t n, hipStream_t s) {
    if (n == 0) return CQ_OK;
    if (n_planes < 1 || n_planes > MAXP) return CQ_ERR_RANGE;
    ActSrc src{x, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{norm_weight, nullptr, eps, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0, planes, (int)n_planes};
    return launch_fused_dt<PRO_NORM_SPLIT, EPI_NONE>(w_dtype, w, src, dst, k, n, s, fz);
}

// ---- a matvec split along K: plane s holds W[:, slice s] . quantize(x[slice s]) for every row ----
// Each workgroup quantizes only its slice of the activation row (the cost of quantizing a long row in every
// workgroup is what this removes); the planes are added in a fixed order by the consumers' PRO_NORM_SPLIT prologue
// and EPI_RESID_SPLIT epilogue.
namespace {
template <int DT, int PRO>
__global__ __launch_bounds__(1024) void qmv_ksplit_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, const float *__restrict__ up,
                                                          float *__restrict__ planes, QmvGeom g, int slice_bytes) {
    const int ks = blockIdx.y;
    ActSrc src{x + (int64_t)ks * g.k, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{PRO == PRO_SILU ? up + (int64_t)ks * g.k : nullptr, nullptr, 0.0f, nullptr, nullptr, 0, 0, 0, nullptr, nullptr, 0};
    qmv_body<DT, 1, CQ_F32, true, PRO, EPI_NONE, false>(w + (int64_t)ks * slice_bytes, src, planes + (int64_t)ks * g.n, g, fz, blockIdx.x, gridDim.x);
}

// The fewest equal slices (2 .. MAXP, whole blocks each) that one wave step per row covers; 0: none.  Few planes keep
// the consumers cheap: every workgroup of a consumer reads every plane.
template <int DT>
int64_t ksplit_planes(int64_t k) {
    constexpr int be = BlockInfo<DT>::elems;
    if (k <= 0 || k % be) return 0;
    const int64_t nblk = k / be;
    for (int64_t p = 2; p <= MAXP; p++)
        if (nblk % p == 0 && (k / p) / Fmt<DT>::UE <= 64) return p;
    return 0;
}

template <int DT>
int launch_ksplit(const void *w, const float *x, const float *up, float *planes, int64_t k, int64_t n, hipStream_t s) {
    const int64_t n_planes = ksplit_planes<DT>(k);
    if (n_planes == 0) return CQ_ERR_RANGE;
    const int64_t slice = k / n_planes;
    QmvGeom g;
    int64_t groups;
    int waves = 0;
    size_t lds_bytes;
    int rc = make_geom<DT, 1>(g, groups, waves, slice, n, n, CQ_F32, 0, lds_bytes, 256 / n_planes);
    if (rc) return rc;
    const int slice_bytes = g.row_bytes;
    const int64_t rb = (k / BlockInfo<DT>::elems) * BlockInfo<DT>::bytes;
    if (rb > 0x3fffffff) return CQ_ERR_RANGE;
    g.row_bytes = (int)rb;                                  // rows are still a whole row of W apart
    dim3 grid((unsigned)groups, (unsigned)n_planes), block(64 * waves);
    if (up)
        hipLaunchKernelGGL((qmv_ksplit_kernel<DT, PRO_SILU>), grid, block, lds_bytes, s, (const uint8_t *)w, x, up, planes, g, slice_bytes);
    else
        hipLaunchKernelGGL((qmv_ksplit_kernel<DT, PRO_NONE>), grid, block, lds_bytes, s, (const uint8_t *)w, x, up, planes, g, slice_bytes);
    return (int)hipGetLastError();
}
}  // namespace

// number of planes cq_matvec_ksplit_launch writes for this format and row length; 0: not available
int64_t cq_matvec_ksplit_planes(int w_dtype, int64_t k) {
    switch (w_dtype) {
        case CQ_Q4_0: return ksplit_planes<CQ_Q4_0>(k);
        case CQ_Q8_0: return ksplit_planes<CQ_Q8_0>(k);
        case CQ_Q4K: return ksplit_planes<CQ_Q4K>(k);
        case CQ_Q5K: return ksplit_planes<CQ_Q5K>(k);
        case CQ_Q6K: return ksplit_planes<CQ_Q6K>(k);
    }
    return 0;
}

// planes[s][n] = W[:, slice s] . quantize((up ? silu(x) * up : x)[slice s])
int cq_matvec_ksplit_launch(int w_dtype, const void *w, const float *x, const float *up, float *planes, int64_t k, int64_t n, hipStream_t s) {
    if (n == 0) return CQ_OK;
    switch (w_dtype) {
        case CQ_Q4_0: return launch_ksplit<CQ_Q4_0>(w, x, up, planes, k, n, s);
        case CQ_Q8_0: return launch_ksplit<CQ_Q8_0>(w, x, up, planes, k, n, s);
        case CQ_Q4K: return launch_ksplit<CQ_Q4K>(w, x, up, planes, k, n, s);
        case CQ_Q5K: return launch_ksplit<CQ_Q5K>(w, x, up, planes, k, n, s);
        case CQ_Q6K: return launch_ksplit<CQ_Q6K>(w, x, up, planes, k, n, s);
    }
    return CQ_ERR_DTYPE;
}

// ---- MoE with few pairs: block (tile, pair) is one fused matvec over the pair's expert ----
namespace {
// SWIGLU: w is the gate expert tensor, the up experts lie pair_off bytes behind it, and the pair's row is
// silu(gate . x) * (up . x) (rows of one wave step only).
template <int DT, bool SINGLE, bool SWIGLU = false>
__global__ __launch_bounds__(1024) void moe_pair_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ out, QmvGeom g,
                                                        PairSource ps, int64_t expert_bytes, int64_t pair_off) {
    const int p = blockIdx.y;
    int e, in_row, out_row;
    float scale;
    if (!pair_decode(ps, p, e, in_row, out_row, scale)) {       // uniform over the workgroup
        if (ps.mode == MOE_INDEXED) {                           // an out-of-range id: that output row is zero
            const int r0 = blockIdx.x * g.rows_per_wg, r1 = min(g.n, r0 + g.rows_per_wg);
            for (int r = r0 + (int)threadIdx.x; r < r1; r += (int)blockDim.x) out[(int64_t)p * g.n + r] = 0.0f;
        }
        return;
    }
    ActSrc src{x + (int64_t)in_row * g.k, ActView{nullptr, nullptr, nullptr}};
    Fuse fz{nullptr, nullptr, scale, nullptr, nullptr, 0, 0, pair_off, nullptr, nullptr, 0};
    qmv_body<DT, 1, CQ_F32, SINGLE, PRO_NONE, SWIGLU ? EPI_SWIGLU : EPI_SCALE, false>(w + (int64_t)e * expert_bytes, src,
                                                                                      out + (int64_t)out_row * g.n, g, fz, blockIdx.x, gridDim.x);
}

// Short expert rows (at most 32 units per row: k <= 2048 for K-quants, e.g. the 768- and 2048-element rows of a
// Qwen3-30B-A3B expert): one wave step takes 64 / SEG weight rows, SEG = 32 or 16 lanes each, instead of leaving half or
// more of the lanes idle.  Lane l works on unit l % SEG of row (l / SEG) of the step; the sums stay inside their
// 16-lane DPP rows (SEG = 16) or are folded pairwise with one row broadcast (SEG = 32) and lane SEG - 1 of each segment
// stores.  Otherwise the body of moe_pair_kernel for rows of one wave step: activation row quantized into LDS by the
// workgroup, weights of the next step in flight while this one is reduced.
template <int SEG> __device__ __forceinline__ float seg_sum_to_last(float v) {
#define CQ_DPP(ctrl, rmask, bc) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, rmask, 0xf, bc))
    v += CQ_DPP(0x111, 0xf, true);     // row_shr:1
    v += CQ_DPP(0x112, 0xf, true);     // row_shr:2
    v += CQ_DPP(0x114, 0xf, true);     // row_shr:4
    v += CQ_DPP(0x118, 0xf, true);     // row_shr:8   -> lane 15 of each 16-lane row holds the row sum
    if (SEG == 32) v += CQ_DPP(0x142, 0xa, false);    // row_bcast:15 into rows 1 and 3 -> lanes 31 and 63 hold the segment sums
#undef CQ_DPP
    return v;
}

template <int DT, int SEG, bool SWIGLU>
__global__ __launch_bounds__(1024) void moe_pair_short_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ out,
                                                              QmvGeom g, PairSource ps, int64_t expert_bytes, int64_t pair_off) {
    typedef Fmt<DT> F;
    constexpr int RPS = 64 / SEG;                      // weight rows per wave step
    const int p = blockIdx.y;
    int e, in_row, out_row;
    float scale;
    const int wg_row0 = blockIdx.x * g.rows_per_wg, wg_row1 = min(g.n, wg_row0 + g.rows_per_wg);
    if (!pair_decode(ps, p, e, in_row, out_row, scale)) {       // uniform over the workgroup
        if (ps.mode == MOE_INDEXED)                             // an out-of-range id: that output row is zero
            for (int r = wg_row0 + (int)threadIdx.x; r < wg_row1; r += (int)blockDim.x) out[(int64_t)p * g.n + r] = 0.0f;
        return;
    }
    extern __shared__ __align__(16) uint8_t lds[];
    int8_t *lqs = (int8_t *)lds;
    float *ld = (float *)(lds + g.lds_d_off);
    int16_t *lbs = (int16_t *)(lds + g.lds_bs_off);
    const int k = g.k, n = g.n;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = 1 << g.nw_shift;
    const int sl = lane & (SEG - 1), sub = lane / SEG;
    const bool valid = sl < g.units;
    const int u0 = min(sl, g.units - 1);
    const float *xr = x + (int64_t)in_row * k;
    float *orow = out + (int64_t)out_row * n;
    w += (int64_t)e * expert_bytes;

    // the activation load goes out first (vector loads complete in order), then the first weights
    const int total = k, spans = (k + 255) >> 8;
    const int xbase = wv * 256 + lane * 4;
    float xv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (xbase < total) cq_load4<CQ_F32>(xr, xbase, xv);
    const int step_rows = RPS << g.nw_shift;           // rows the workgroup covers per step
    int row = wg_row0 + wv * RPS + sub;                // this lane's row of the wave's current step
    const int base0 = wg_row0 + wv * RPS;
    const int my_steps = base0 < wg_row1 ? (wg_row1 - base0 + step_rows - 1) / step_rows : 0;
    const int64_t row_bytes = g.row_bytes;
    typename F::W wa, wb;
    F::load_w(wa, w + (int64_t)min(row, n - 1) * row_bytes, u0);

    if (wv < spans) {
        if (cq_is_kquant(DT)) cq_quantize_q8k_vals(xv, wv, lane, lqs, ld, lbs);
        else cq_quantize_q80_vals(xv, xbase < total, xbase, lane, lqs, ld);
    }
    for (int span = wv + nwaves; span < spans; span += nwaves) {
        if (cq_is_kquant(DT)) cq_quantize_q8k_span<CQ_F32>(xr, span, lane, lqs, ld, lbs);
        else cq_quantize_q80_span<CQ_F32>(xr, span, lane, total, lqs, ld);
    }
    __syncthreads();
    if (my_steps == 0) return;
    typename F::A areg;
    F::load_a(areg, act_row(lqs, ld, lbs, DT, 0, k), u0);

    if (SWIGLU) {
        // wa = gate row (in flight), wb = up row; the next gate row is requested before the up row is reduced
        for (int j = 0; j < my_steps; j++) {
            const uint8_t *rp = w + (int64_t)min(row, n - 1) * row_bytes;
            F::load_w(wb, rp + pair_off, u0);
            float gate = seg_sum_to_last<SEG>(valid ? F::dot(wa, areg, u0) : 0.0f);
            const int nrow = j + 1 < my_steps ? row + step_rows : row;
            F::load_w(wa, w + (int64_t)min(nrow, n - 1) * row_bytes, u0);
            float up = seg_sum_to_last<SEG>(valid ? F::dot(wb, areg, u0) : 0.0f);
            if (sl == SEG - 1 && row < wg_row1) orow[row] = gate / (1.0f + expf(-gate)) * up;
            row = nrow;
        }
        return;
    }
    for (int j = 0; j < my_steps; j += 2) {
        const int r1 = j + 1 < my_steps ? row + step_rows : row;
        F::load_w(wb, w + (int64_t)min(r1, n - 1) * row_bytes, u0);
        float v = seg_sum_to_last<SEG>(valid ? F::dot(wa, areg, u0) : 0.0f);
        if (sl == SEG - 1 && row < wg_row1) orow[row] = v * scale;
        if (j + 1 >= my_steps) break;
        const int r2 = j + 2 < my_steps ? r1 + step_rows : r1;
        F::load_w(wa, w + (int64_t)min(r2, n - 1) * row_bytes, u0);
        v = seg_sum_to_last<SEG>(valid ? F::dot(wb, areg, u0) : 0.0f);
        if (sl == SEG - 1 && r1 < wg_row1) orow[r1] = v * scale;
        row = r2;
    }
}

template <int DT, int SEG>
int launch_moe_pairs_short(const void *w, const float *x, float *out, const PairSource &ps, int64_t k, int64_t n, hipStream_t s, bool swiglu,
                           int64_t pair_off) {
    constexpr int RPS = 64 / SEG;
    QmvGeom g;
    int64_t groups;
    size_t lds_bytes;
    // the geometry of launch_moe_pairs in units of wave steps (RPS rows each)
    const int64_t n_steps = (n + RPS - 1) / RPS;
    int waves = 16;
    if ((int64_t)ps.n_pairs * n_steps < 256 * 16) {
        while (waves > 1 && n_steps < 256 * (int64_t)waves) waves >>= 1;
        // ... but at least one wave per 256-element span of the activation row (up to 8): a lone wave quantizing a
        // 2048-element row span by span takes longer than the rows it then streams
        const int64_t spans = (k + 255) / 256;
        while (waves < 8 && waves < spans) waves <<= 1;
    }
    const int64_t per_pair = ((swiglu ? 2048 : 1024) + ps.n_pairs - 1) / ps.n_pairs;
    int rc = make_geom<DT, 1>(g, groups, waves, k, n_steps, n, CQ_F32, 0, lds_bytes, per_pair < 256 ? per_pair : 256);
    if (rc) return rc;
    g.n = (int)n;
    g.rows_per_wg *= RPS;
    if (ps.n_pairs > 65535) return CQ_ERR_RANGE;
    const int64_t expert_bytes = n * (int64_t)g.row_bytes;
    dim3 grid((unsigned)groups, (unsigned)ps.n_pairs), block(64 * waves);
    if (swiglu)
        hipLaunchKernelGGL((moe_pair_short_kernel<DT, SEG, true>), grid, block, lds_bytes, s, (const uint8_t *)w, x, out, g, ps, expert_bytes, pair_off);
    else
        hipLaunchKernelGGL((moe_pair_short_kernel<DT, SEG, false>), grid, block, lds_bytes, s, (const uint8_t *)w, x, out, g, ps, expert_bytes, (int64_t)0);
    return (int)hipGetLastError();
}

template <int DT>
int launch_moe_pairs(const void *w, const float *x, float *out, const PairSource &ps, int64_t k, int64_t n, hipStream_t s, bool swiglu = false,
                     int64_t pair_off = 0) {
    if (cq_act_layout(DT, k, 1).total > LDS_BUDGET) return CQ_ERR_RANGE;
    if (swiglu && k / Fmt<DT>::UE > 64) return CQ_ERR_RANGE;         // the paired-row epilogue is for rows of one wave step
    // short rows: several weight rows per wave step
    if (k / Fmt<DT>::UE <= 16) return launch_moe_pairs_short<DT, 16>(w, x, out, ps, k, n, s, swiglu, pair_off);
    if (k / Fmt<DT>::UE <= 32) return launch_moe_pairs_short<DT, 32>(w, x, out, ps, k, n, s, swiglu, pair_off);
    QmvGeom g;
    int64_t groups;
    size_t lds_bytes;
    // wide workgroups once the pairs together hold enough rows: the activation row is quantized once per workgroup
    int waves = (int64_t)ps.n_pairs * n >= 256 * 16 ? 16 : 0;
    // about a thousand workgroups in total: with many pairs each workgroup takes more rows of its expert, so that
    // the activation prologue is paid once per many rows
    const int64_t per_pair = ((swiglu ? 2048 : 1024) + ps.n_pairs - 1) / ps.n_pairs;
    int rc = make_geom<DT, 1>(g, groups, waves, k, n, n, CQ_F32, 0, lds_bytes, per_pair < 256 ? per_pair : 256);
    if (rc) return rc;
    if (ps.n_pairs > 65535) return CQ_ERR_RANGE;
    const int64_t expert_bytes = n * (int64_t)g.row_bytes;
    const bool single = k / Fmt<DT>::UE <= 64;
    const void *kp = swiglu   ? (const void *)moe_pair_kernel<DT, true, true>
                     : single ? (const void *)moe_pair_kernel<DT, true>
                              : (const void *)moe_pair_kernel<DT, false>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(kp, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    dim3 grid((unsigned)groups, (unsigned)ps.n_pairs), block(64 * waves);
    if (swiglu)
        hipLaunchKernelGGL((moe_pair_kernel<DT, true, true>), grid, block, lds_bytes, s, (const uint8_t *)w, x, out, g, ps, expert_bytes, pair_off);
    else if (single)
        hipLaunchKernelGGL((moe_pair_kernel<DT, true>), grid, block, lds_bytes, s, (const uint8_t *)w, x, out, g, ps, expert_bytes, (int64_t)0);
    else
        hipLaunchKernelGGL((moe_pair_kernel<DT, false>), grid, block, lds_bytes, s, (const uint8_t *)w, x, out, g, ps, expert_bytes, (int64_t)0);
    return (int)hipGetLastError();
}
}  // namespace

int cq_moe_pairs_launch(int w_dtype, const void *w, const float *x, float *out, const PairSource &ps, int64_t k, int64_t n, hipStream_t s) {
    if (ps.n_pairs == 0 || n == 0) return CQ_OK;
    switch (w_dtype) {
        case CQ_Q4_0: return launch_moe_pairs<CQ_Q4_0>(w, x, out, ps, k, n, s);
        case CQ_Q8_0: return launch_moe_pairs<CQ_Q8_0>(w, x, out, ps, k, n, s);
        case CQ_Q4K: return launch_moe_pairs<CQ_Q4K>(w, x, out, ps, k, n, s);
        case CQ_Q5K: return launch_moe_pairs<CQ_Q5K>(w, x, out, ps, k, n, s);
        case CQ_Q6K: return launch_moe_pairs<CQ_Q6K>(w, x, out, ps, k, n, s);
        case CQ_Q2K: return launch_moe_pairs<CQ_Q2K>(w, x, out, ps, k, n, s);
        case CQ_Q3K: return launch_moe_pairs<CQ_Q3K>(w, x, out, ps, k, n, s);
    }
    return CQ_ERR_DTYPE;
}

// out[pair, :] = silu(W_gate[e] . x) * (W_up[e] . x) for at most CQ_MOE_DIRECT_MAX_PAIRS pairs; the two expert tensors have one
// shape and format.  CQ_ERR_RANGE when a row is longer than one wave step.
int cq_moe_pairs_swiglu_launch(int w_dtype, const void *w_gate, const void *w_up, const float *x, float *out, const PairSource &ps, int64_t k,
                               int64_t n, hipStream_t s) {
    if (ps.n_pairs == 0 || n == 0) return CQ_OK;
    const int64_t off = (const uint8_t *)w_up - (const uint8_t *)w_gate;
    switch (w_dtype) {
        case CQ_Q4_0: return launch_moe_pairs<CQ_Q4_0>(w_gate, x, out, ps, k, n, s, true, off);
        case CQ_Q8_0: return launch_moe_pairs<CQ_Q8_0>(w_gate, x, out, ps, k, n, s, true, off);
        case CQ_Q4K: return launch_moe_pairs<CQ_Q4K>(w_gate, x, out, ps, k, n, s, true, off);
        case CQ_Q5K: return launch_moe_pairs<CQ_Q5K>(w_gate, x, out, ps, k, n, s, true, off);
        case CQ_Q6K: return launch_moe_pairs<CQ_Q6K>(w_gate, x, out, ps, k, n, s, true, off);
        case CQ_Q2K: return launch_moe_pairs<CQ_Q2K>(w_gate, x, out, ps, k, n, s, true, off);
        case CQ_Q3K: return launch_moe_pairs<CQ_Q3K>(w_gate, x, out, ps, k, n, s, true, off);
    }
    return CQ_ERR_DTYPE;
}

// ---- MoE grouped by expert: block (tile, chunk) runs up to 8 pairs of one expert against one pass over its rows ----
namespace {
template <int DT, bool SINGLE>
__global__ __launch_bounds__(512) void moe_chunk_kernel(const uint8_t *__restrict__ w, ActView av, float *__restrict__ out, QmvGeom g, MoeChunks mc,
                                                         int64_t expert_bytes) {
    const int c = blockIdx.y;
    if (c >= mc.n_chunks[0]) return;                            // uniform over the workgroup
    const int first = mc.first[c];
    ActSrc src{nullptr, cq_act_view_rows(av, DT, g.k, first)};
    Fuse fz{nullptr, nullptr, 0.0f, nullptr, nullptr, 0, 0, 0, mc.pair_out + first, mc.pair_scale + first, mc.count[c]};
    qmv_body<DT, CQ_MOE_CHUNK, SRC_SCRATCH, SINGLE, PRO_NONE, EPI_MOE, false>(w + (int64_t)mc.expert[c] * expert_bytes, src, out, g, fz, blockIdx.x,
                                                                              gridDim.x);
}

template <int DT>
int launch_moe_chunks(const void *w, const void *scratch, int64_t rows_alloc, float *out, const MoeChunks &mc, int64_t k, int64_t n,
                      hipStream_t s) {
    if (cq_act_layout(DT, k, CQ_MOE_CHUNK).total > LDS_BUDGET) return CQ_ERR_RANGE;
    QmvGeom g;
    int64_t groups;
    size_t lds_bytes;
    int waves = 8;
    const int64_t per_chunk = (2048 + mc.max_chunks - 1) / mc.max_chunks;
    int rc = make_geom<DT, CQ_MOE_CHUNK>(g, groups, waves, k, n, n, CQ_F32, 0, lds_bytes, per_chunk < 256 ? per_chunk : 256);
    if (rc) return rc;
    if (mc.max_chunks > 65535) return CQ_ERR_RANGE;
    const int64_t expert_bytes = n * (int64_t)g.row_bytes;
    const bool single = k / Fmt<DT>::UE <= 64;
    const void *kp = single ? (const void *)moe_chunk_kernel<DT, true> : (const void *)moe_chunk_kernel<DT, false>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(kp, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    ActView av = cq_act_view(scratch, DT, k, rows_alloc);
    dim3 grid((unsigned)groups, (unsigned)mc.max_chunks), block(64 * waves);
    if (single)
        hipLaunchKernelGGL((moe_chunk_kernel<DT, true>), grid, block, lds_bytes, s, (const uint8_t *)w, av, out, g, mc, expert_bytes);
    else
        hipLaunchKernelGGL((moe_chunk_kernel<DT, false>), grid, block, lds_bytes, s, (const uint8_t *)w, av, out, g, mc, expert_bytes);
    return (int)hipGetLastError();
}
}  // namespace

int cq_moe_chunks_launch(int w_dtype, const void *w, const void *scratch, int64_t rows_alloc, float *out, const MoeChunks &mc, int64_t k,
                         int64_t n, hipStream_t s) {
    if (mc.max_chunks == 0 || n == 0) return CQ_OK;
    switch (w_dtype) {
        case CQ_Q4_0: return launch_moe_chunks<CQ_Q4_0>(w, scratch, rows_alloc, out, mc, k, n, s);
        case CQ_Q8_0: return launch_moe_chunks<CQ_Q8_0>(w, scratch, rows_alloc, out, mc, k, n, s);
        case CQ_Q4K: return launch_moe_chunks<CQ_Q4K>(w, scratch, rows_alloc, out, mc, k, n, s);
        case CQ_Q5K: return launch_moe_chunks<CQ_Q5K>(w, scratch, rows_alloc, out, mc, k, n, s);
        case CQ_Q6K: return launch_moe_chunks<CQ_Q6K>(w, scratch, rows_alloc, out, mc, k, n, s);
        case CQ_Q2K: return launch_moe_chunks<CQ_Q2K>(w, scratch, rows_alloc, out, mc, k, n, s);
        case CQ_Q3K: return launch_moe_chunks<CQ_Q3K>(w, scratch, rows_alloc, out, mc, k, n, s);
    }
    return CQ_ERR_DTYPE;
}
