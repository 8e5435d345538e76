// Shared device code of the fused decode matvecs: the fusion descriptors (prologues / epilogues around a single-row matvec)
// and the body of the streaming kernel (cq_stream.h), used by the matvec launches of cq_matvec.hip and by the cooperative
// decoder kernels of cq_layer.hip.
#pragma once
#include "cq_actquant.h"
#include "cq_device.h"
#include "cq_fmt.h"
#include "cq_launch.h"
#include "cq_stream.h"

// Per-wave timeline stamps for a private instrumented build (-DCL_STAMPS); nothing in a normal build.
#ifdef CL_STAMPS
#define CQ_STAMP(i) do { if ((threadIdx.x & 63) == 0) cq_stamp_lds[threadIdx.x >> 6][(i)] = (uint32_t)__builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define CQ_STAMP(i) do { } while (0)
#endif

namespace {

#ifdef CL_STAMPS
__shared__ uint32_t cq_stamp_lds[16][32];
#endif

constexpr int SRC_SCRATCH = -1;   // activations come pre-quantized (cq_quantize_act); otherwise SRC is the x dtype
constexpr int64_t LDS_BUDGET = 160 * 1024 - 1024;

struct ActSrc {
    const void *x;   // fused: [NB, k] activations
    ActView av;      // pre-quantized: section pointers of the scratch buffer (possibly row-offset)
};

// Decoder fusions around a single-row f32 matvec (none of them changes what the plain kernel does):
//   PRO_NORM  the activation row is rms_norm(x) * norm_weight; sum(x^2) arrives as CQ_NN_PARTIALS partial sums
//             written by the producer of x, so no workgroup-wide reduction is needed before quantizing
//   PRO_SILU  the activation row is silu(x) * up
//   PRO_MERGE the activation row is the attention output, merged on the fly from the per-split partials
//             { acc[hd], m, l, 0, 0 } the single-token attention kernel leaves (rows of one wave step only)
//   EPI_SWIGLU a logical row r is the pair (W[r], W[r] + pair_off bytes) = (feed_forward_w1, feed_forward_w3):
//             dst[r] = silu(W1[r] . x) * (W3[r] . x)   (rows of one wave step only)
//   EPI_SCALE the result is multiplied by a per-launch-block scalar (Fuse::eps) before it is stored (MoE top-k weight)
//   EPI_MOE   activation row b of the launch block belongs to output row row_map[b] and is scaled by row_scale[b];
//             rows b >= nvalid are padding and are not stored (8 router pairs of one expert per weight pass)
//   EPI_RESID the result is added to a residual row in place of being stored, and the workgroup leaves
//             its partial sum of residual^2 for the next PRO_NORM consumer
//   PRO_NORM_SPLIT like PRO_NORM, but the row is ((x + planes[0]) + planes[1]) + ... (the K-slice partial results of a
//             split matvec, added in this fixed order); sum(x^2) is computed here.  x itself is left as it is
//   EPI_RESID_SPLIT like EPI_RESID, with the same planes added to the residual row first (same order), so the row
//             leaves this kernel merged
enum { PRO_NONE = 0, PRO_NORM = 1, PRO_SILU = 2, PRO_MERGE = 3, PRO_NORM_SPLIT = 4 };
constexpr bool pro_is_split(int pro) { return pro == PRO_NORM_SPLIT; }
constexpr int MAXS = 16;     // attention splits a PRO_MERGE prologue can merge
constexpr int MAXP = 4;      // K-slice planes a PRO_NORM_SPLIT prologue / EPI_RESID_SPLIT epilogue can add
enum { EPI_NONE = 0, EPI_RESID = 1, EPI_SWIGLU = 2, EPI_SCALE = 3, EPI_MOE = 4, EPI_RESID_SPLIT = 5 };
constexpr bool epi_is_resid(int epi) { return epi == EPI_RESID || epi == EPI_RESID_SPLIT; }
constexpr int NPART = 256;   // == CQ_NN_PARTIALS
struct Fuse {
    const float *aux;        // PRO_NORM: norm weight [k];  PRO_SILU: up [k];  PRO_MERGE: partials [k/hd][splits][hd + 4]
    const float *part_in;    // PRO_NORM: [NPART]
    float eps;
    float *resid;            // EPI_RESID: [n], updated in place
    float *part_out;         // EPI_RESID: [NPART]
    int splits, hd_shift;    // PRO_MERGE
    int64_t pair_off;        // EPI_SWIGLU: byte distance from a row of w1 to the same row of w3
    const int *row_map;      // EPI_MOE
    const float *row_scale;
    int nvalid;
    const float *planes;     // PRO_NORM_SPLIT: [n_planes][k];  EPI_RESID_SPLIT: [n_planes][n]
    int n_planes;
};

// Launch geometry, computed once on the host so the kernel prologue is a handful of scalar loads
// instead of 64-bit divisions and multiplications in front of the first memory access.
struct QmvGeom {
    int k, n, rows_per_wg;
    int units, steps;          // units per row, wave steps per row
    int lds_d_off, lds_bs_off; // LDS sections (the scratch layout for NB rows)
    int nw_shift;              // log2(waves per workgroup)
    int row_bytes;             // bytes of one row of W
    int lds_red_off;           // EPI_RESID / PRO_NORM_SPLIT: 16 floats behind the activation sections
    int dst_dtype;
    int64_t stride_dst;
};

// the lane's four activation values of one 256-element span after the prologue op
template <int PRO>
__device__ __forceinline__ void pro_apply(float v[4], const float a[4], float m) {
    if (PRO == PRO_NORM) {
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = v[i] / m * a[i];                   // candle-nn/src/ops.rs:507-509
    } else if (PRO == PRO_SILU) {
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = v[i] / (1.0f + expf(-v[i])) * a[i];   // Silu::f32, then * up
    }
}

// PRO_MERGE: the lane's four consecutive elements [base, base + 4) of the attention output, from the partials
template <int MS> struct MergeRegs { float m[MS], l[MS]; f32x4 a[MS]; };
template <int MS>
__device__ __forceinline__ void merge_load(const Fuse &fz, int base, bool ok, MergeRegs<MS> &r) {
    const int hd = 1 << fz.hd_shift;
    const float *pp = fz.aux + (int64_t)(base >> fz.hd_shift) * fz.splits * (hd + 4);
    const int d = base & (hd - 1);
#pragma unroll
    for (int sI = 0; sI < MS; sI++) {
        r.m[sI] = -INFINITY; r.l[sI] = 0.0f; r.a[sI] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (ok && sI < fz.splits) {
            const float *rec = pp + sI * (hd + 4);
            r.a[sI] = *reinterpret_cast<const f32x4 *>(rec + d);
            const float2 t = *reinterpret_cast<const float2 *>(rec + hd);
            r.m[sI] = t.x; r.l[sI] = t.y;
        }
    }
}
template <int MS>
__device__ __forceinline__ void merge_reduce(const MergeRegs<MS> &r, bool ok, float v[4]) {
    // same operation order as the stand-alone merge kernel: identical bits
    float M = -INFINITY;
#pragma unroll
    for (int sI = 0; sI < MS; sI++) M = fmaxf(M, r.l[sI] > 0.0f ? r.m[sI] : -INFINITY);
    f32x4 num = {0.0f, 0.0f, 0.0f, 0.0f};
    float den = 0.0f;
#pragma unroll
    for (int sI = 0; sI < MS; sI++) {
        if (r.l[sI] > 0.0f) {
            const float wgt = __expf(r.m[sI] - M);
            num.x += wgt * r.a[sI].x; num.y += wgt * r.a[sI].y; num.z += wgt * r.a[sI].z; num.w += wgt * r.a[sI].w;
            den += wgt * r.l[sI];
        }
    }
    if (ok) { v[0] = num.x / den; v[1] = num.y / den; v[2] = num.z / den; v[3] = num.w / den; }
}

// A pointer rebuilt from integers (the fourteen-dword argument block) has no address space the compiler knows, and through
// a plain pointer every access is a flat instruction.  Flat loads cannot be waited for by count: the wait for an
// activation load becomes vmcnt(0), which also waits for every weight copy requested before it.  A round trip through
// the global address space that the optimizer cannot see through (the empty asm) tells the compiler where the memory is.
template <typename T> __device__ __forceinline__ T *qs_global(const void *p) {
    auto gp = (__attribute__((address_space(1))) T *)p;
    asm("" : "+s"(gp));
    return (T *)gp;
}


// ---------------------------------------------------------------------------------------------
// Streaming kernel (cq_stream.h): one lane per super-block, weights copied HBM -> LDS.  Q4_K / Q5_K, one f32 row,
// the same prologues and epilogues as qmv_body.  Workgroups of QS_NW waves; step s of the weight stream goes to wave
// (s / grid) % QS_NW of workgroup s % grid, so at any moment the whole chip reads one compact window of the tensor.
// ---------------------------------------------------------------------------------------------
constexpr int QS_NW = 8;
constexpr bool qs_streams(int dt) { return dt == CQ_Q4K || dt == CQ_Q5K || dt == CQ_Q6K || dt == CQ_Q4_0 || dt == CQ_Q8_0; }     // formats with a StreamFmt
constexpr bool qs_wide_aux(int dt) { return dt == CQ_Q6K || dt == CQ_Q4_0 || dt == CQ_Q8_0; }      // ... whose lanes keep the whole 64-byte span record
// the activation quantization a weight format asks for: Q8_K spans (with the 16-element sums for Q6_K) or Q8_0 blocks
template <int DT, int NS>
__device__ __forceinline__ void qs_quantize(const float (&v)[NS][4], int span0, int stride, int limit, int dump, int lane, uint8_t *act, int aux_off) {
    if constexpr (DT == CQ_Q4_0 || DT == CQ_Q8_0) {
#pragma unroll
        for (int j = 0; j < NS; j++) {
            const int span = span0 + j * stride;
            qs_quantize_span_q80(v[j], span < limit ? span : dump, lane, act, aux_off);
        }
    } else {
        qs_quantize_spans<DT == CQ_Q6K, NS>(v, span0, stride, limit, dump, lane, act, aux_off);
    }
}

// Use of the body as one phase of a cooperative multi-phase kernel (cq_layer.hip), where phases follow each other behind a
// barrier across the launch's workgroups instead of a kernel boundary:
//   CO_SLOTS  every wave's LDS slot is CO_SLOT bytes whatever the format, so that a wave may request the first step of the
//             next phase into its slot while other waves still work on the current one;
//   CO_PRE    the caller has requested the wave's first step already (qms_issue_first);
//   CO_SC1    results go out as device-scope stores: workgroups on other XCDs read them later in the same launch.
enum { CO_NONE = 0, CO_SLOTS = 1, CO_PRE = 2, CO_SC1 = 4 };
constexpr int CO_SLOT = 14 * 1024;

// the copies of step `step` of a weight stream into the calling wave's slot (absent steps: a descriptor of zero bytes)
template <int DT>
__device__ __forceinline__ void qms_issue_step(const uint8_t *wbase, uint8_t *slot, int step, int total_steps, int step_bytes, int64_t w_bytes, int lane) {
    typedef StreamFmt<DT> SF;
    const bool live = step < total_steps;
    const int64_t off = (int64_t)(live ? step : 0) * step_bytes;
    const int64_t left = w_bytes - off;
    const int bytes = live ? (int)(left < step_bytes ? left : step_bytes) : 0;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(wbase + off), 0, bytes, 0x00020000);
#pragma unroll
    for (int j = 0; j < SF::NLD; j++) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (cq_lds_void *)(slot + j * 1024), 16, lane * 16, j * 1024, 0, 0);
}
// what a CO_PRE phase expects to be on its way: the first step of wave `wv` of workgroup `block` (of `nblocks`)
template <int DT, int NW>
__device__ __forceinline__ void qms_issue_first(const uint8_t *w, uint8_t *slots, const StreamGeom &g, int block, int nblocks, int wv, int lane) {
    static_assert(StreamFmt<DT>::NLD * 1024 <= CO_SLOT, "a step of this format does not fit a cooperative slot");
    qms_issue_step<DT>(w, slots + wv * CO_SLOT, wv * nblocks + block, g.total_steps, g.step_bytes, g.w_bytes, lane);
}

template <int DT, int NW, int XS, int MAXB, int PRO, int EPI, int MSP = MAXS, int COOP = CO_NONE>
__device__ __forceinline__ void qms_body(const uint8_t *__restrict__ w, const float *__restrict__ x, void *__restrict__ dst, const StreamGeom &g,
                                         const Fuse &fz, const int block, const int nblocks) {
    typedef StreamFmt<DT> SF;
    typedef StreamAct<MAXB> SA;
    constexpr bool RESID = epi_is_resid(EPI);
    [[maybe_unused]] constexpr int SB = (COOP & CO_PRE) ? 8 : 0;            // (instrumented builds: where this phase's stamps go)
    constexpr bool PAIR = EPI == EPI_SWIGLU;               // two weight rows per output row: a step is two sub-steps, gate rows then up rows
    constexpr int SUBS = PAIR ? 2 : 1;
    // 16-byte-per-lane copies of the first step requested before the activation prologue; the rest follows it.
    // Requests beyond what the memory pipeline takes at once block the wave's instruction stream, and the prologue
    // queued behind them would wait for the weights instead of running under their latency.
    // (measured on the Q6_K 4096 x 14336 matvec, 14 copies per step and seven spans per wave: 4 copies first 14.8 us,
    // all 14 first 16.2 us, the rest spread behind the spans 15.2 us)
    constexpr int PRE = NW == 16 ? 2 : 4;
    constexpr int ME = EPI == EPI_RESID_SPLIT ? MAXP : 1;
    constexpr int SLOT = (COOP & (CO_SLOTS | CO_PRE)) ? CO_SLOT : SF::NLD * 1024;
    static_assert(SF::NLD * 1024 <= SLOT, "a step of this format does not fit a cooperative slot");
    static_assert(PRO != PRO_MERGE || XS <= 2, "the merge prologue holds its partials in registers");
    // two LDS variables on purpose: the compiler then knows that the LDS copies in flight (into `slots`) never touch
    // `act` and does not wait for them before the activation accesses
    extern __shared__ __align__(16) uint8_t slots[];
    __shared__ __align__(16) uint8_t act[SA::BYTES];
    __shared__ __align__(16) float red[32];                // [0, 16): sum(x^2) of the prologue, [16, 32): residual^2 of the epilogue
    static_assert(NW == 8 || NW == 16, "the fixed-order sums below read 8 or 16 slots");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int k = g.k, n = g.n, bpr = g.bpr;
    const int sstride = NW * nblocks;
    // sub-step t of wave wq: step wq * nblocks + block + (t / SUBS) * sstride, of the gate tensor (even t) or the up tensor
    // (odd t); copies [j0, j1) of it.  The loads are unconditional: a step that does not exist gets a descriptor of zero
    // bytes (its loads read nothing), so that the waits below stay counted waits.
    auto issue_for = [&](int wq, int t, int j0, int j1) {
        const int s0 = wq * nblocks + block;
        const int st = s0 + (PAIR ? t >> 1 : t) * sstride;
        const uint8_t *wbase = PAIR && (t & 1) ? w + fz.pair_off : w;
        const bool live = st < g.total_steps;
        const int64_t off = (int64_t)(live ? st : 0) * g.step_bytes;
        const int64_t left = g.w_bytes - off;
        const int bytes = live ? (int)(left < g.step_bytes ? left : g.step_bytes) : 0;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(wbase + off), 0, bytes, 0x00020000);
#pragma unroll
        for (int j = 0; j < SF::NLD; j++)
            if (j >= j0 && j < j1) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (cq_lds_void *)(slots + wq * SLOT + j * 1024), 16, lane * 16, j * 1024, 0, 0);
    };
    // 0. activation loads first (vector loads complete in order: what is asked for after the weights waits for them)
    f32x4 xt[XS], at[XS];
    float pp[NPART / 64] = {0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int MS = PRO == PRO_MERGE ? MSP : 1;         // splits the merge prologue holds (the launch picks the smallest that fits)
    MergeRegs<MS> mg[PRO == PRO_MERGE ? XS : 1];
    constexpr int MP = PRO == PRO_NORM_SPLIT ? MAXP : 1;
    f32x4 pl[PRO == PRO_NORM_SPLIT ? XS : 1][MP];
#pragma unroll
    for (int j = 0; j < XS; j++) {
        const int sc = min(wv + j * NW, bpr - 1);          // a wave without a span re-reads the last one (and dumps its result)
        const int base = sc * 256 + lane * 4;
        if (PRO == PRO_MERGE) {
            merge_load<MS>(fz, base, true, mg[PRO == PRO_MERGE ? j : 0]);
        } else {
            xt[j] = *(const f32x4 *)(x + base);
            if (PRO != PRO_NONE) at[j] = *(const f32x4 *)(fz.aux + base);
            if (PRO == PRO_NORM_SPLIT) {
#pragma unroll
                for (int sI = 0; sI < MP; sI++) pl[PRO == PRO_NORM_SPLIT ? j : 0][sI] = *(const f32x4 *)(fz.planes + (int64_t)min(sI, fz.n_planes - 1) * k + base);
            }
        }
    }
    if (PRO == PRO_NORM) {
#pragma unroll
        for (int i = 0; i < NPART / 64; i++) pp[i] = fz.part_in[lane + 64 * i];
    }
    asm volatile("" ::: "memory");

    CQ_STAMP(SB + 0);
    // 1. the wave's first step on its way into LDS
    uint8_t *slot = slots + wv * SLOT;
    const int step0 = wv * nblocks + block;
    const int my = step0 < g.total_steps ? (g.total_steps - step0 + sstride - 1) / sstride : 0;
    auto issue = [&](int t, int j0, int j1) { issue_for(wv, t, j0, j1); };
    if constexpr (!(COOP & CO_PRE)) issue(0, 0, PRE);
    asm volatile("" ::: "memory");
    // With a norm prologue nothing of it may be scheduled in front of these copies: left to itself the compiler places the
    // whole sum of squares (which waits for the partial sums) before them, and the weights start a memory trip late.
    // Without one the barrier gains nothing (measured: the same to slightly slower), so the compiler keeps its freedom there.
    if constexpr (PRO == PRO_NORM || PRO == PRO_NORM_SPLIT) __builtin_amdgcn_sched_barrier(0);

    // 2. activations -> LDS
    float pm = 1.0f;
    if (PRO == PRO_NORM) {
        const float sum2 = wave_sum((pp[0] + pp[1]) + (pp[2] + pp[3]));      // fixed order: the same bits in every wave and replay
        pm = sqrtf(sum2 / (float)k + fz.eps);
    }
    float xv[XS][4];
#pragma unroll
    for (int j = 0; j < XS; j++) {
        if (PRO == PRO_MERGE) {
            merge_reduce<MS>(mg[PRO == PRO_MERGE ? j : 0], true, xv[j]);
        } else {
            xv[j][0] = xt[j].x; xv[j][1] = xt[j].y; xv[j][2] = xt[j].z; xv[j][3] = xt[j].w;
        }
    }
    if (PRO == PRO_NORM_SPLIT) {
        // the merged row (absent planes count as zeros) and sum(x^2) over the whole row, in a fixed order
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < XS; j++) {
            const bool own = wv + j * NW < bpr;
#pragma unroll
            for (int sI = 0; sI < MP; sI++) {
                const f32x4 t = pl[PRO == PRO_NORM_SPLIT ? j : 0][sI];
                const bool on = sI < fz.n_planes;
                xv[j][0] += on ? t.x : 0.0f; xv[j][1] += on ? t.y : 0.0f; xv[j][2] += on ? t.z : 0.0f; xv[j][3] += on ? t.w : 0.0f;
            }
            const float s4 = (xv[j][0] * xv[j][0] + xv[j][1] * xv[j][1]) + (xv[j][2] * xv[j][2] + xv[j][3] * xv[j][3]);
            ss += own ? wave_sum(s4) : 0.0f;
        }
        if (lane == 0) red[wv] = ss;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        const f32x4 r0 = ((const f32x4 *)red)[0], r1 = ((const f32x4 *)red)[1];
        float sum2 = ((r0.x + r0.y) + (r0.z + r0.w)) + ((r1.x + r1.y) + (r1.z + r1.w));
        if (NW == 16) {
            const f32x4 r2 = ((const f32x4 *)red)[2], r3 = ((const f32x4 *)red)[3];
            sum2 += ((r2.x + r2.y) + (r2.z + r2.w)) + ((r3.x + r3.y) + (r3.z + r3.w));
        }
        pm = sqrtf(sum2 / (float)k + fz.eps);
    }
#pragma unroll
    for (int j = 0; j < XS; j++) {
        const float a4[4] = {at[j].x, at[j].y, at[j].z, at[j].w};
        if (PRO == PRO_NORM || PRO == PRO_SILU) pro_apply<PRO>(xv[j], a4, pm);
        if (PRO == PRO_NORM_SPLIT) pro_apply<PRO_NORM>(xv[j], a4, pm);
    }
    qs_quantize<DT, XS>(xv, wv, NW, bpr, MAXB, lane, act, SA::AUX_OFF);
    asm volatile("" ::: "memory");
    if constexpr (!(COOP & CO_PRE)) issue(0, PRE, SF::NLD);
    // The residual value of the wave's first row is asked for right behind its first step's copies (vector loads complete
    // in order: it is there when they are); every later one travels in front of the next step's copies.  Asked for when
    // its step begins, the last one of a wave would be waited for at the very end of the kernel, a memory trip long.
    float rv_next = 0.0f;
    if (RESID) rv_next = fz.resid[min(step0 * g.step_rows + (lane >> g.lp_shift), n - 1)];
    asm volatile("" ::: "memory");
    // a barrier without the fence of __syncthreads(): the fence would wait for the LDS copies in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    CQ_STAMP(SB + 1);
    // 3. the lane's place: row `rin` of the step, super-block `sb` of the row; its activations stay in registers
    const int lp = 1 << g.lp_shift;
    const int rin = lane >> g.lp_shift, sb = lane & (lp - 1);
    const bool valid_sb = sb < bpr;
    const int sbc = valid_sb ? sb : bpr - 1;
    u32x4 areg[16];
#pragma unroll
    for (int i = 0; i < 16; i++) areg[i] = *(const u32x4 *)(act + sbc * QS_ACT_STRIDE + 16 * i);
    const uint8_t *auxp = act + SA::AUX_OFF + sbc * QS_AUX_STRIDE;
    const u32x4 aux0 = *(const u32x4 *)auxp;
    QsAux aux1;
    aux1.s32 = *(const u32x4 *)(auxp + 16);
    if constexpr (qs_wide_aux(DT)) {
        aux1.bl16 = *(const u32x4 *)(auxp + 32);
        aux1.bh16 = *(const u32x4 *)(auxp + 48);
    }
    const float d8 = __uint_as_float(aux0.x);
    const int boff = (rin * bpr + sbc) * SF::BB;
    const bool last = sb == lp - 1;                     // this lane ends up with the row's sum
    float ssq = 0.0f;

    auto out1 = [&](int row, float v) {
        if constexpr (COOP & CO_SC1)
            __hip_atomic_store((float *)dst + row, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);       // f32 outputs only
        else
            store_out(dst, g.dst_dtype, row, v);
    };
    float gate = 0.0f;
    for (int t = 0; t < SUBS * my; t++) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // this wave's copies have landed
        if (t == 0) CQ_STAMP(SB + 2);
        const int step = step0 + (PAIR ? t >> 1 : t) * sstride;
        const int row = step * g.step_rows + rin;
        const bool store = last && row < n;
        // the residual value was asked for a step ahead; the planes to add to it travel in front of the next step's copies
        float rv = rv_next, pv[ME];
        if (EPI == EPI_RESID_SPLIT) {
            const int rc = min(row, n - 1);
#pragma unroll
            for (int sI = 0; sI < ME; sI++) pv[sI] = fz.planes[(int64_t)min(sI, fz.n_planes - 1) * n + rc];
        }
        typename SF::Blk b0;
        SF::read(b0, slot + boff);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // every lane has its block in registers: the slot is free
        if (RESID && t + 1 < my) rv_next = fz.resid[min(row + sstride * g.step_rows, n - 1)];
        issue(t + 1, 0, SF::NLD);
        asm volatile("" ::: "memory");
        float r = SF::dot(b0, areg, d8, aux1);
        r = qs_group_sum(valid_sb ? r : 0.0f, g.lp_shift);
        if (PAIR) {
            if (t & 1) {
                if (store) out1(row, gate / (1.0f + expf(-gate)) * r);      // Mlp::forward, quantized_llama.rs:56-63
            } else {
                gate = r;
            }
        } else if (RESID) {
            if (store) {
                if (EPI == EPI_RESID_SPLIT) {
#pragma unroll
                    for (int sI = 0; sI < ME; sI++) rv += sI < fz.n_planes ? pv[sI] : 0.0f;
                }
                const float sres = rv + r;                     // (x + residual), quantized_llama.rs:584,591
                fz.resid[row] = sres;
                ssq += sres * sres;
            }
        } else if (store) {
            out1(row, EPI == EPI_SCALE ? r * fz.eps : r);
        }
    }
    CQ_STAMP(SB + 3);
    if (RESID) {
        // the workgroup's partial of sum(residual^2), added in a fixed order; block 0 clears the unused slots
        ssq = wave_sum(ssq);
        if (lane == 0) red[16 + wv] = ssq;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (tid == 0) {
            const f32x4 r0 = ((const f32x4 *)red)[4], r1 = ((const f32x4 *)red)[5];
            float t = ((r0.x + r0.y) + (r0.z + r0.w)) + ((r1.x + r1.y) + (r1.z + r1.w));
            if (NW == 16) {
                const f32x4 r2 = ((const f32x4 *)red)[6], r3 = ((const f32x4 *)red)[7];
                t += ((r2.x + r2.y) + (r2.z + r2.w)) + ((r3.x + r3.y) + (r3.z + r3.w));
            }
            fz.part_out[block] = t;
        }
        if (block == 0)
            for (int i = nblocks + tid; i < NPART; i += NW * 64) fz.part_out[i] = 0.0f;
    }
}

// Does the streaming kernel take this (format, k, n)?  Rows of a power of two of super-blocks (up to 64) fill every
// lane; other row lengths put one row on a wave step and need at least three quarters of the lanes busy.
template <int DT>
bool stream_geom(StreamGeom &g, int64_t k, int64_t n, int dst_dtype) {
    if (!qs_streams(DT)) return false;
    if (k % 256 || k <= 0 || n < 64) return false;
    const int64_t bpr = k / 256;
    if (bpr > 64) return false;
    int sh = 0;
    while ((1 << sh) < bpr) sh++;
    if ((1 << sh) != bpr && 4 * bpr < 3 * (1 << sh)) return false;
    const int64_t bb = BlockInfo<DT>::bytes * (256 / BlockInfo<DT>::elems);       // bytes of 256 elements: a super-block, or eight blocks
    // every wave step must start on 16 bytes of the stream (Q6_K blocks are 210 bytes: steps of a multiple of 8 blocks)
    if (((64 >> sh) * bpr * bb) % 16) return false;
    // the copies move whole dwords and their range check is per dword: a tensor of 2 (mod 4) bytes (Q6_K, odd block count)
    // would lose the dword that holds its last two bytes, the f16 scale of the last block
    if ((n * bpr * bb) % 4) return false;
    g.k = (int)k; g.n = (int)n; g.bpr = (int)bpr; g.lp_shift = sh;
    g.step_rows = 64 >> sh;
    g.step_bytes = (int)(g.step_rows * bpr * bb);
    g.total_steps = (int)((n + g.step_rows - 1) / g.step_rows);
    g.dst_dtype = dst_dtype; g.stride_dst = n;
    g.w_bytes = n * bpr * bb;
    return n <= 0x7fffffff / 64;
}

}  // namespace
