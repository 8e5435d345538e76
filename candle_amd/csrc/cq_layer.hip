// Cooperative decode kernels: several dependent single-row matvecs of a decoder layer in ONE launch of 256 workgroups, the
// phases separated by a barrier across the launch (cq_coop.h) instead of a kernel boundary.  What that buys: while a
// workgroup waits for the others it has already asked for the first weight steps of the next phase, so the HBM keeps
// streaming across the hand-over, where a chain of launches leaves it idle for the launch gap, the argument fetch and the
// activation prologue of every kernel.  Each phase is the body of the streaming matvec kernel (cq_stream_body.h) with the
// same step -> (workgroup, wave) assignment as the stand-alone launch, so results are bit-identical to the chain of launches.
//
// (-DCL_STAMPS compiles per-wave s_memrealtime stamps into the kernel for a timeline of the launch; the library is built without.)
//
// candle runs these as separate tensor ops (candle-transformers/src/models/quantized_llama.rs:56-63, 191-266, 584-591).
#include "../../include/candle_hip_nn.h"
#include "../../include/candle_hip_quant.h"
#include "cq_coop.h"
#include "cq_stream_body.h"

namespace {

constexpr int CL_NW = QS_NW;                      // waves per workgroup, as in the stand-alone streaming launches
constexpr int CL_SLOTS_BYTES = CL_NW * CO_SLOT;   // dynamic LDS: one uniform slot per wave

template <int DT>
__device__ __forceinline__ StreamGeom cl_geom(int n, int bpr) {
    StreamGeom g;
    g.k = bpr * 256; g.n = n; g.bpr = bpr;
    g.lp_shift = bpr > 1 ? 32 - __builtin_clz(bpr - 1) : 0;
    g.step_rows = 64 >> g.lp_shift;
    g.step_bytes = g.step_rows * bpr * StreamFmt<DT>::BB;
    g.total_steps = (n + g.step_rows - 1) >> (6 - g.lp_shift);
    g.dst_dtype = CQ_F32; g.stride_dst = n;
    g.w_bytes = (int64_t)n * (bpr * StreamFmt<DT>::BB);
    return g;
}

// ---- the feed-forward half of a layer: h = silu(W1 xn) * (W3 xn), xn = rms_norm(x); x += W2 h ------------------------------
struct MlpArgs {
    const uint8_t *w1; int64_t pair_off; const uint8_t *w2;
    float *resid; float *part; const float *norm_w; float *h; uint32_t *sync;
    float eps; int hidden, ffn;
#ifdef CL_STAMPS
    uint32_t *stamps;
#endif
};

template <int DT13, int DT2, int XS1, int XS2, int MAXB2>
__global__ __launch_bounds__(CL_NW * 64) void mlp_coop_kernel(MlpArgs a) {
    extern __shared__ __align__(16) uint8_t slots[];
    __shared__ uint32_t co_cnt;
    const int tid = threadIdx.x, lane = tid & 63, block = blockIdx.x;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (tid == 0) co_cnt = 0;                     // (the phase below has a workgroup barrier before any wave arrives)
    Coop co;
    coop_init(co, a.sync, block);
    const StreamGeom g1 = cl_geom<DT13>(a.ffn, a.hidden / 256), g2 = cl_geom<DT2>(a.hidden, a.ffn / 256);
    {
        Fuse fz{a.norm_w, a.part, a.eps, nullptr, nullptr, 0, 0, a.pair_off, nullptr, nullptr, 0, nullptr, 0};
        qms_body<DT13, CL_NW, XS1, 16, PRO_NORM, EPI_SWIGLU, MAXS, CO_SLOTS | CO_SC1>(a.w1, a.resid, a.h, g1, fz, block, COOP_GRID);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // this wave's part of h is where every XCD reads it
    CQ_STAMP(5);
    coop_arrive(co, &co_cnt, CL_NW, lane);
    qms_issue_first<DT2, CL_NW>(a.w2, slots, g2, block, COOP_GRID, wv, lane);
    CQ_STAMP(6);
    coop_wait(co);
    CQ_STAMP(7);
    {
        Fuse fz{nullptr, nullptr, 0.0f, a.resid, a.part, 0, 0, 0, nullptr, nullptr, 0, nullptr, 0};
        qms_body<DT2, CL_NW, XS2, MAXB2, PRO_NONE, EPI_RESID, MAXS, CO_PRE>(a.w2, a.h, nullptr, g2, fz, block, COOP_GRID);
    }
#ifdef CL_STAMPS
    CQ_STAMP(12);
    __syncthreads();
    if (tid < CL_NW * 16) a.stamps[(block * CL_NW + tid / 16) * 16 + tid % 16] = cq_stamp_lds[tid / 16][tid % 16];
#endif
}

int coop_device_ok() {
    static int cached = -1;
    if (cached < 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached = cus >= COOP_GRID ? 1 : 0;
    }
    return cached;
}

template <int DT13, int DT2>
int launch_mlp(const MlpArgs &a, hipStream_t s) {
    StreamGeom gt;
    if (!stream_geom<DT13>(gt, a.hidden, a.ffn, CQ_F32) || gt.bpr > 16 || !stream_geom<DT2>(gt, a.ffn, a.hidden, CQ_F32)) return CQ_ERR_RANGE;
    if (((uintptr_t)a.w1 & 15) || ((uintptr_t)a.w2 & 15) || (a.pair_off & 15)) return CQ_ERR_RANGE;
    const int bpr1 = a.hidden / 256, bpr2 = a.ffn / 256;
    auto go = [&](auto kern) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, CL_SLOTS_BYTES);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, dim3(COOP_GRID), dim3(CL_NW * 64), CL_SLOTS_BYTES, s, a);
        return (int)hipGetLastError();
    };
    // activation spans per wave of each phase: as the stand-alone launches choose them (launch_stream)
    if (bpr1 <= 8) {
        if (bpr2 <= 8) return go(mlp_coop_kernel<DT13, DT2, 1, 1, 16>);
        if (bpr2 <= 16) return go(mlp_coop_kernel<DT13, DT2, 1, 2, 16>);
        if (bpr2 <= 32) return go(mlp_coop_kernel<DT13, DT2, 1, 4, 64>);
        return CQ_ERR_RANGE;
    }
    if (bpr2 <= 16) return go(mlp_coop_kernel<DT13, DT2, 2, 2, 16>);
    if (bpr2 <= 32) return go(mlp_coop_kernel<DT13, DT2, 2, 4, 64>);
    if (bpr2 <= 56) return go(mlp_coop_kernel<DT13, DT2, 2, 7, 64>);
    return go(mlp_coop_kernel<DT13, DT2, 2, 8, 64>);
}

}  // namespace

#ifdef CL_STAMPS
static uint32_t *cl_stamps_dev = nullptr;
extern "C" void cl_set_stamps(uint32_t *p) { cl_stamps_dev = p; }
#endif

extern "C" {

// bytes of one wave step of the streaming decode matvec over this weight (the unit in which its workgroups, and so the
// XCDs, take turns along the tensor); 0 when the (format, k, n) does not take the streaming kernel
int64_t cq_qmatmul_stream_step_bytes(int w_dtype, int64_t k, int64_t n) {
    StreamGeom g;
    bool okk = false;
    switch (w_dtype) {
        case CQ_Q4_0: okk = stream_geom<CQ_Q4_0>(g, k, n, CQ_F32); break;
        case CQ_Q8_0: okk = stream_geom<CQ_Q8_0>(g, k, n, CQ_F32); break;
        case CQ_Q4K: okk = stream_geom<CQ_Q4K>(g, k, n, CQ_F32); break;
        case CQ_Q5K: okk = stream_geom<CQ_Q5K>(g, k, n, CQ_F32); break;
        case CQ_Q6K: okk = stream_geom<CQ_Q6K>(g, k, n, CQ_F32); break;
        default: break;
    }
    return okk ? g.step_bytes : 0;
}

int64_t cq_nn_coop_sync_bytes(void) { return COOP_SYNC_BYTES; }

int cq_nn_decode_mlp(int w13_dtype, const void *w1_dev, const void *w3_dev, int w2_dtype, const void *w2_dev, float *residual_dev,
                     float *sumsq_partials_dev, const float *norm_weight_dev, float eps, float *h_dev, int64_t hidden, int64_t ffn, void *sync_dev,
                     void *stream) {
    if (hidden <= 0 || ffn <= 0 || hidden % 256 || ffn % 256) return CQ_ERR_SHAPE;
    if (!w1_dev || !w3_dev || !w2_dev || !residual_dev || !sumsq_partials_dev || !norm_weight_dev || !h_dev || !sync_dev) return CQ_ERR_NULL;
    if (((uintptr_t)residual_dev | (uintptr_t)h_dev | (uintptr_t)norm_weight_dev) & 15 || ((uintptr_t)sync_dev & 127)) return CQ_ERR_ALIGN;
    if (!coop_device_ok()) return CQ_ERR_RANGE;
    MlpArgs a{(const uint8_t *)w1_dev, (const uint8_t *)w3_dev - (const uint8_t *)w1_dev, (const uint8_t *)w2_dev, residual_dev, sumsq_partials_dev,
              norm_weight_dev, h_dev, (uint32_t *)sync_dev, eps, (int)hidden, (int)ffn};
#ifdef CL_STAMPS
    a.stamps = cl_stamps_dev;
#endif
    hipStream_t s = (hipStream_t)stream;
    if (w13_dtype == CQ_Q4K && w2_dtype == CQ_Q6K) return launch_mlp<CQ_Q4K, CQ_Q6K>(a, s);
    if (w13_dtype == CQ_Q4K && w2_dtype == CQ_Q4K) return launch_mlp<CQ_Q4K, CQ_Q4K>(a, s);
    return CQ_ERR_RANGE;
}

}  // extern "C"
