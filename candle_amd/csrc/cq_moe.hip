// Expert-grouped quantized matmul for gfx950: QTensor::indexed_moe_forward and
// candle_nn::moe::moe_gemm_gguf behind one kernel pair.
//
// Both entry points are lists of "pairs" (expert, activation row, output row, scale):
//   indexed_moe_forward (candle-core/src/quantized/cuda.rs:505-584, candle-kernels/src/quantized.cu:4670-4760)
//       pair p = b * topk + t : expert ids[p], activation row (input_dim1 == 1 ? b : p), output row p, scale 1
//   moe_gemm_gguf (candle-nn/src/moe.rs:169-337, candle-kernels/src/moe/moe_gguf.cu:55-132)
//       pair m : expert expert_ids[m], tok = sorted_token_ids[m],
//                activation row (topk_weights ? tok : tok / topk), output row tok, scale topk_weights[tok] or 1
//
// Step 1 quantizes the activation rows exactly as the CPU path does.  Step 2 (one workgroup)
// buckets the pairs by expert with a counting sort, so the input order does not matter (the
// reference sorts with an unstable sort, candle-core/src/sort.rs:282-297).  Step 3 streams every
// hit expert's rows once: workgroup (row tile, expert) keeps the decoded weight registers and loops
// over that expert's pairs — unlike the reference kernels, which re-read the expert's weights for
// every pair routed to it.  (Few pairs skip steps 1 and 2: a fused matvec per pair.  Hundreds of pairs take step 3 on the matrix
// cores: Q4_K experts with up to 64 pairs each as batched matvecs over their pairs, cq_matvec_batch.hip, the rest as tiles of
// expert-sorted rows through the prefill kernel of the format.)
#include <algorithm>
#include "cq_device.h"
#include "cq_fmt.h"
#include "cq_launch.h"

namespace {

struct MoeWorkspace {
    int64_t act_off, offsets_off, cursor_off, pin_off, pout_off, pscale_off, chunk_off, max_chunks, rows_alloc, extra_off, total;
};

inline MoeWorkspace moe_workspace(int w_dtype, int64_t num_experts, int64_t n_pairs, int64_t x_rows, int64_t k) {
    MoeWorkspace w;
    w.act_off = 0;
    // the chunked path quantizes the activation rows in expert-sorted pair order (plus one chunk of padding rows);
    // the older per-expert kernel quantizes the x rows as they are: room for the larger of the two
    w.rows_alloc = n_pairs + CQ_MOE_CHUNK;
    w.max_chunks = n_pairs / CQ_MOE_CHUNK + (num_experts < n_pairs ? num_experts : n_pairs) + 1;
    w.offsets_off = cq_act_layout(w_dtype, k, w.rows_alloc > x_rows ? w.rows_alloc : x_rows).total;
    // (experts run as batched matvecs keep their pairs' rows as operand tiles instead)
    if ((w_dtype == CQ_Q4K || w_dtype == CQ_Q5K) && k % 256 == 0) w.offsets_off = std::max<int64_t>(w.offsets_off, cq_align256(cq_moe_stream_operand_bytes(num_experts, n_pairs, k)));
    w.cursor_off = w.offsets_off + cq_align256((num_experts + 1) * 4);
    w.pin_off = w.cursor_off + cq_align256(num_experts * 4);
    w.pout_off = w.pin_off + cq_align256(n_pairs * 4);
    w.pscale_off = w.pout_off + cq_align256(n_pairs * 4);
    w.chunk_off = w.pscale_off + cq_align256(n_pairs * 4);
    w.extra_off = w.chunk_off + cq_align256((3 * w.max_chunks + 1) * 4);  // n_chunks | expert[] | first[] | count[]
    // further passes of the experts with more than 32 pairs, for the batched-matvec form: n | two counters | (expert, pass)[]
    w.total = w.extra_off + cq_align256((CQ_MOE_EXTRA_HEADER + 2 * (n_pairs / 32 + 1)) * 4);
    return w;
}

// offsets[e] .. offsets[e+1] is expert e's segment of pair_in / pair_out / pair_scale.
// LC: the per-expert counters live in LDS (up to GROUP_LDS_EXPERTS experts) instead of the global `cursor` array: the
// two passes of atomics are then LDS atomics, not trips of one workgroup to the L2.
constexpr int GROUP_LDS_EXPERTS = 4096;
template <bool LC>
__global__ __launch_bounds__(1024) void moe_group_kernel(PairSource ps, int *__restrict__ offsets, int *__restrict__ cursor,
                                                         int *__restrict__ pair_in, int *__restrict__ pair_out,
                                                         float *__restrict__ pair_scale, float *__restrict__ out, int n, int *__restrict__ chunks,
                                                         int max_chunks, int chunk, int *__restrict__ extra) {
    __shared__ int carry, n_chunks, n_extra;
    __shared__ int buf[1024];
    __shared__ int lcur[LC ? GROUP_LDS_EXPERTS : 1];
    int *cur = LC ? lcur : cursor;
    const int tid = threadIdx.x;
    const int E = ps.num_experts;
    for (int e = tid; e < E; e += 1024) cur[e] = 0;
    __syncthreads();
    // the first KEEP pairs of every thread stay in registers between the two sweeps (decoding a pair is two dependent loads)
    constexpr int KEEP = 4;
    int ke[KEEP], kin[KEEP], kout[KEEP];
    float ksc[KEEP];
    bool kok[KEEP];
#pragma unroll
    for (int i = 0; i < KEEP; i++) {
        const int p = tid + i * 1024;
        kok[i] = p < ps.n_pairs && pair_decode(ps, p, ke[i], kin[i], kout[i], ksc[i]);
        if (kok[i]) atomicAdd(&cur[ke[i]], 1);
    }
    for (int p = tid + KEEP * 1024; p < ps.n_pairs; p += 1024) {
        int e, in_row, out_row;
        float scale;
        if (pair_decode(ps, p, e, in_row, out_row, scale)) atomicAdd(&cur[e], 1);
    }
    if (tid == 0) { carry = 0; n_chunks = 0; n_extra = 0; }
    __syncthreads();
    // exclusive scan of the counts, 1024 experts per sweep (only as many doubling steps as the sweep is wide)
    for (int base = 0; base < E; base += 1024) {
        int e = base + tid;
        int c = e < E ? cur[e] : 0;
        const int width = min(1024, E - base);
        buf[tid] = c;
        __syncthreads();
        for (int o = 1; o < width; o <<= 1) {
            int v = tid >= o ? buf[tid - o] : 0;
            __syncthreads();
            buf[tid] += v;
            __syncthreads();
        }
        int start = carry + buf[tid] - c;
        if (e < E) {
            offsets[e] = start;
            cur[e] = start;
            // chunk table: expert e's segment in pieces of `chunk` pairs (any order: chunks are independent)
            // (the batched-matvec form takes 32 pairs of an expert per pass over its weights: every further pass is an item of a
            // list that the workgroups of that launch share out among themselves once their own pass is done)
            if (extra && c > 32) {
                const int np = (c + 31) / 32 - 1;
                const int eb = atomicAdd(&n_extra, np);
                for (int i = 0; i < np; i++) {
                    extra[CQ_MOE_EXTRA_HEADER + 2 * (eb + i)] = e;
                    extra[CQ_MOE_EXTRA_HEADER + 2 * (eb + i) + 1] = i + 1;
                }
            }
            const int cc = (c + chunk - 1) / chunk;
            if (cc > 0) {
                const int cb = atomicAdd(&n_chunks, cc);
                for (int i = 0; i < cc; i++) {
                    chunks[1 + cb + i] = e;
                    chunks[1 + max_chunks + cb + i] = start + i * chunk;
                    chunks[1 + 2 * max_chunks + cb + i] = min(chunk, c - i * chunk);
                }
            }
        }
        __syncthreads();
        if (tid == width - 1) carry += buf[tid];              // the inclusive sum of the sweep
        __syncthreads();
    }
    if (tid == 0) {
        offsets[E] = carry;
        chunks[0] = n_chunks;
        if (extra) { extra[0] = n_extra; extra[1] = 0; extra[2] = 0; }         // the list's length, and the two launches' counters
    }
    // positions behind the last valid pair are never part of a chunk, but the gathering quantizer walks all n_pairs
    // rows: give them a valid source row
    for (int p = carry + tid; p < ps.n_pairs; p += 1024) pair_in[p] = 0;
    auto place = [&](int p, bool ok, int e, int in_row, int out_row, float scale) {
        if (ok) {
            int pos = atomicAdd(&cur[e], 1);
            pair_in[pos] = in_row;
            pair_out[pos] = out_row;
            pair_scale[pos] = scale;
        } else if (ps.mode == MOE_INDEXED) {
            for (int c = 0; c < n; c++) out[(int64_t)p * n + c] = 0.0f;   // id out of range: defined output
        }
    };
#pragma unroll
    for (int i = 0; i < KEEP; i++)
        if (tid + i * 1024 < ps.n_pairs) place(tid + i * 1024, kok[i], ke[i], kin[i], kout[i], ksc[i]);
    for (int p = tid + KEEP * 1024; p < ps.n_pairs; p += 1024) {
        int e, in_row, out_row;
        float scale;
        const bool ok = pair_decode(ps, p, e, in_row, out_row, scale);
        place(p, ok, e, in_row, out_row, scale);
    }
}

// Workgroup (blockIdx.x = row tile, blockIdx.y = expert); 4 waves x R rows.  Pairs of the expert are
// taken PB at a time with the decoded weight registers held across them.
template <int DT, int R, int PB>
__global__ __launch_bounds__(256) void moe_matvec_kernel(const uint8_t *__restrict__ w, ActView av, float *__restrict__ out,
                                                         const int *__restrict__ offsets, const int *__restrict__ pair_in,
                                                         const int *__restrict__ pair_out, const float *__restrict__ pair_scale,
                                                         int k, int n) {
    typedef Fmt<DT> F;
    const int e = blockIdx.y;
    const int seg0 = offsets[e], seg1 = offsets[e + 1];
    if (seg0 == seg1) return;
    const int lane = threadIdx.x & 63;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * R;
    if (row0 >= n) return;
    const int nblk = k / BlockInfo<DT>::elems;
    const int units = nblk * F::UPB;
    const int64_t row_bytes = (int64_t)nblk * BlockInfo<DT>::bytes;
    const uint8_t *we = w + (int64_t)e * n * row_bytes;

    for (int s0 = seg0; s0 < seg1; s0 += PB) {
        int arow[PB];
#pragma unroll
        for (int b = 0; b < PB; b++) arow[b] = pair_in[s0 + b < seg1 ? s0 + b : seg1 - 1];
        float acc[R][PB];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int b = 0; b < PB; b++) acc[r][b] = 0.0f;

        ActRow arow_p[PB];
#pragma unroll
        for (int b = 0; b < PB; b++) arow_p[b] = act_row(av.qs, av.d, av.bsums, DT, arow[b], k);
        for (int u = lane; u < units; u += CQ_WAVE) {
            typename F::W wr[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                int64_t row = row0 + r < n ? row0 + r : n - 1;
                F::load_w(wr[r], we + row * row_bytes, u);
            }
            typename F::A ar[PB];
#pragma unroll
            for (int b = 0; b < PB; b++) F::load_a(ar[b], arow_p[b], u);
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int b = 0; b < PB; b++) acc[r][b] += F::dot(wr[r], ar[b], u);
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int b = 0; b < PB; b++) {
                float v = wave_sum(acc[r][b]);
                if (lane == 0 && row0 + r < n && s0 + b < seg1)
                    out[(int64_t)pair_out[s0 + b] * n + row0 + r] = v * pair_scale[s0 + b];
            }
    }
}

template <int DT>
int launch_moe_matvec(const MoeArgs &a, const ActView &av, const int *offsets, const int *pin, const int *pout, const float *pscale,
                      hipStream_t s) {
    constexpr int R = 2, PB = 4;
    int64_t tiles = (a.n + 4 * R - 1) / (4 * R);
    if (tiles > 0x7fffffffLL || a.num_experts > 65535) return CQ_ERR_RANGE;
    hipLaunchKernelGGL((moe_matvec_kernel<DT, R, PB>), dim3((unsigned)tiles, (unsigned)a.num_experts), dim3(256), 0, s,
                       (const uint8_t *)a.w, av, a.out, offsets, pin, pout, pscale, (int)a.k, (int)a.n);
    return (int)hipGetLastError();
}

}  // namespace

int64_t cq_moe_workspace_bytes_impl(int w_dtype, int64_t num_experts, int64_t n_pairs, int64_t x_rows, int64_t k) {
    return moe_workspace(w_dtype, num_experts, n_pairs, x_rows, k).total;
}

// Does a call with this many pairs group them by expert and run the matrix-core kernel of the format over expert tiles?
static bool moe_takes_mfma(int w_dtype, const void *w, const void *w_b, int64_t n_pairs, int64_t k) {
    // (the matrix-core kernel of the 32-element formats copies weight rows in 8-byte pieces: experts at another alignment take
    // the matvec passes)
    const bool q0_ok = (w_dtype == CQ_Q4_0 || w_dtype == CQ_Q8_0) && ((uintptr_t)w & 7) == 0 && (!w_b || ((uintptr_t)w_b & 7) == 0);
    return k % 256 == 0 && (cq_is_kquant(w_dtype) || q0_ok) && cq_has_mfma(w_dtype) && n_pairs >= CQ_MOE_MFMA_MIN_PAIRS;
}
static int moe_tile_rows(int64_t n_pairs, int64_t num_experts) { return n_pairs < 40 * num_experts ? CQ_MOE_TILE_SMALL : CQ_MOE_TILE_LARGE; }

int cq_moe_down_after_pair_launch(int w_dtype, const void *w_down, const float *gate, const float *up, const float *topk_weights, float *out,
                                  int64_t num_experts, int64_t topk, int64_t n_pairs, int64_t n, int64_t k, int64_t k_pair, void *workspace,
                                  hipStream_t s) {
    if (n_pairs > 0x7fffffffLL || topk <= 0 || n_pairs % topk) return CQ_ERR_RANGE;
    // what the gate / up call did with these pairs, and what this one needs
    // (K-quants only: whether Q4_0 / Q8_0 experts were grouped for the matrix cores also depended on that call's weight addresses)
    if (!cq_is_kquant(w_dtype)) return CQ_ERR_RANGE;
    if (cq_moe_direct(w_dtype, num_experts, n_pairs, k_pair) || !moe_takes_mfma(w_dtype, nullptr, nullptr, n_pairs, k_pair)) return CQ_ERR_RANGE;
    if (!moe_takes_mfma(w_dtype, w_down, nullptr, n_pairs, k)) return CQ_ERR_RANGE;
    const MoeWorkspace ws = moe_workspace(w_dtype, num_experts, n_pairs, n_pairs / topk, k_pair);
    // the pair call ran its experts as batched matvecs (chunks of 16 pairs): this one must be able to as well
    // (n of the pair call = this call's k; its expert tensors were 16-byte aligned or it returned CQ_ERR_ALIGN)
    if (cq_moe_stream_shape(w_dtype, num_experts, n_pairs, k_pair, k)) {
        if (!cq_moe_stream_takes(w_dtype, w_down, nullptr, num_experts, n_pairs, k, n)) return CQ_ERR_RANGE;
        if (cq_align256(cq_moe_stream_operand_bytes(num_experts, n_pairs, k)) > ws.offsets_off) return CQ_ERR_RANGE;
        uint8_t *b = (uint8_t *)workspace;
        const int *offsets = (const int *)(b + ws.offsets_off);
        const int *pout = (const int *)(b + ws.pout_off);
        float *pscale = (float *)(b + ws.pscale_off);
        const int *chunks = (const int *)(b + ws.chunk_off);
        int rc = cq_moe_stream_quantize_launch(gate, up, pout, topk_weights, pscale, chunks, ws.max_chunks, num_experts, n_pairs, offsets, b + ws.act_off, k, s);
        if (rc) return rc;
        return cq_moe_stream_launch(w_dtype, w_down, nullptr, out, nullptr, b + ws.act_off, offsets, pout, pscale, (int *)(b + ws.extra_off), 1,
                                    num_experts, k, n, s);
    }
    // the rows of this call are quantized into the front of the workspace: they must end before that call's tables begin
    if (cq_act_layout(w_dtype, k, ws.rows_alloc).total > ws.offsets_off) return CQ_ERR_RANGE;
    uint8_t *b = (uint8_t *)workspace;
    const int *pout = (const int *)(b + ws.pout_off);
    float *pscale = (float *)(b + ws.pscale_off);
    const int *chunks = (const int *)(b + ws.chunk_off);
    // pair i of the expert-sorted list reads row pair_out[i] (one row per pair here) and is scaled by that pair's routing weight
    const int *n_valid = (const int *)(b + ws.offsets_off) + num_experts;          // the end of the last expert's segment
    int rc = cq_quantize_act_swiglu_gather_launch(w_dtype, gate, up, pout, n_valid, topk_weights, pscale, b + ws.act_off, k, n_pairs, ws.rows_alloc, s);
    if (rc) return rc;
    MoeChunks mc{chunks, chunks + 1, chunks + 1 + ws.max_chunks, chunks + 1 + 2 * ws.max_chunks, pout, pscale, (int)ws.max_chunks};
    return cq_matmul_moe_launch(w_dtype, w_down, b + ws.act_off, ws.rows_alloc, out, mc, k, n, moe_tile_rows(n_pairs, num_experts), s);
}

int cq_moe_launch(const MoeArgs &a, void *workspace, hipStream_t s) {
    if (a.n_pairs > 0x7fffffffLL || a.x_rows > 0x7fffffffLL) return CQ_ERR_RANGE;
    const bool mfma = moe_takes_mfma(a.w_dtype, a.w, a.w_b, a.n_pairs, a.k);
    const bool stream_shape = mfma && !cq_moe_direct(a.w_dtype, a.num_experts, a.n_pairs, a.k) && cq_moe_stream_shape(a.w_dtype, a.num_experts, a.n_pairs, a.k, a.n);
    const bool stream = stream_shape && cq_moe_stream_takes(a.w_dtype, a.w, a.w_b, a.num_experts, a.n_pairs, a.k, a.n);
    // (a later cq_moe_down_after_pair_launch tells from the shape alone how this call chunked its pairs)
    if (a.w_b && stream_shape && !stream) return CQ_ERR_ALIGN;
    if (a.w_b && !mfma) {
        // only the MFMA path shares its grouping pass and quantized activations between two weight tensors
        MoeArgs one = a;
        one.w_b = nullptr; one.out_b = nullptr;
        int rc = cq_moe_launch(one, workspace, s);
        if (rc) return rc;
        one.w = a.w_b; one.out = a.out_b;
        return cq_moe_launch(one, workspace, s);
    }
    PairSource ps;
    ps.mode = a.mode; ps.ids_u32 = a.ids_u32; ps.sorted_token_ids = a.sorted_token_ids; ps.expert_ids = a.expert_ids;
    ps.topk_weights = a.topk_weights; ps.topk = (int)a.topk; ps.input_dim1 = (int)a.input_dim1;
    ps.n_pairs = (int)a.n_pairs; ps.num_experts = (int)a.num_experts; ps.x_rows = (int)a.x_rows;
    // Few pairs (decode): every pair is its own fused matvec (activation quantization in the kernel, no scratch,
    // no grouping pass); an expert hit by two pairs is simply read twice, the second time from cache.
    if (cq_moe_direct(a.w_dtype, a.num_experts, a.n_pairs, a.k)) {
        int rc = cq_moe_pairs_launch(a.w_dtype, a.w, a.x, a.out, ps, a.k, a.n, s);
        if (rc != CQ_ERR_RANGE) return rc;
    }
    MoeWorkspace ws = moe_workspace(a.w_dtype, a.num_experts, a.n_pairs, a.x_rows, a.k);
    uint8_t *b = (uint8_t *)workspace;
    int rc;
    int *offsets = (int *)(b + ws.offsets_off), *cursor = (int *)(b + ws.cursor_off);
    int *pin = (int *)(b + ws.pin_off), *pout = (int *)(b + ws.pout_off);
    float *pscale = (float *)(b + ws.pscale_off);
    int *chunks = (int *)(b + ws.chunk_off);
    int *extra = (int *)(b + ws.extra_off);
    // Hundreds of pairs per call: the expert-sorted rows go through the MFMA prefill kernel of the format in tiles of up to
    // 128 rows of one expert (integer-exact like the dense paths).  Otherwise 8 pairs per matvec pass.
    const int tile_rows = moe_tile_rows(a.n_pairs, a.num_experts);
    if (a.num_experts <= GROUP_LDS_EXPERTS)
        hipLaunchKernelGGL(moe_group_kernel<true>, dim3(1), dim3(1024), 0, s, ps, offsets, cursor, pin, pout, pscale, a.out, (int)a.n, chunks,
                           (int)ws.max_chunks, stream ? CQ_MOE_STREAM_CHUNK : mfma ? tile_rows : CQ_MOE_CHUNK, stream ? extra : nullptr);
    else
        hipLaunchKernelGGL(moe_group_kernel<false>, dim3(1), dim3(1024), 0, s, ps, offsets, cursor, pin, pout, pscale, a.out, (int)a.n, chunks,
                           (int)ws.max_chunks, stream ? CQ_MOE_STREAM_CHUNK : mfma ? tile_rows : CQ_MOE_CHUNK, stream ? extra : nullptr);
    if ((rc = (int)hipGetLastError())) return rc;
    if (stream) {
        // every expert a batched matvec over its own pairs: the weights of an expert are streamed once per 32 pairs
        if (cq_align256(cq_moe_stream_operand_bytes(a.num_experts, a.n_pairs, a.k)) > ws.offsets_off) return CQ_ERR_RANGE;      // (the workspace layout above reserves it)
        if ((rc = cq_moe_stream_quantize_launch(a.x, nullptr, pin, nullptr, nullptr, chunks, ws.max_chunks, a.num_experts, a.n_pairs, offsets, b + ws.act_off, a.k, s))) return rc;
        return cq_moe_stream_launch(a.w_dtype, a.w, a.w_b, a.out, a.out_b, b + ws.act_off, offsets, pout, pscale, extra, 0, a.num_experts, a.k, a.n, s);
    }
    if (mfma) {
        if ((rc = cq_quantize_act_gather_launch(a.w_dtype, a.x, pin, b + ws.act_off, a.k, a.n_pairs, ws.rows_alloc, s))) return rc;
        MoeChunks mc{chunks, chunks + 1, chunks + 1 + ws.max_chunks, chunks + 1 + 2 * ws.max_chunks, pout, pscale, (int)ws.max_chunks};
        rc = cq_matmul_moe_launch(a.w_dtype, a.w, b + ws.act_off, ws.rows_alloc, a.out, mc, a.k, a.n, tile_rows, s);
        if (!rc && a.w_b) rc = cq_matmul_moe_launch(a.w_dtype, a.w_b, b + ws.act_off, ws.rows_alloc, a.out_b, mc, a.k, a.n, tile_rows, s);
        return rc;
    }
    if (a.k % 256 == 0) {
        // Many pairs: activation rows quantized in expert-sorted order, then CQ_MOE_CHUNK pairs of an expert per pass
        // over its rows (the matvec body with 8 activation rows in LDS).
        if ((rc = cq_quantize_act_gather_launch(a.w_dtype, a.x, pin, b + ws.act_off, a.k, a.n_pairs, ws.rows_alloc, s))) return rc;
        MoeChunks mc{chunks, chunks + 1, chunks + 1 + ws.max_chunks, chunks + 1 + 2 * ws.max_chunks, pout, pscale, (int)ws.max_chunks};
        rc = cq_moe_chunks_launch(a.w_dtype, a.w, b + ws.act_off, ws.rows_alloc, a.out, mc, a.k, a.n, s);
        if (rc != CQ_ERR_RANGE) return rc;
    }
    if ((rc = cq_quantize_act_launch(a.w_dtype, a.x, CQ_F32, b + ws.act_off, a.k, a.x_rows, s))) return rc;
    ActView av = cq_act_view(b + ws.act_off, a.w_dtype, a.k, a.x_rows);
    switch (a.w_dtype) {
        case CQ_Q4_0: return launch_moe_matvec<CQ_Q4_0>(a, av, offsets, pin, pout, pscale, s);
        case CQ_Q8_0: return launch_moe_matvec<CQ_Q8_0>(a, av, offsets, pin, pout, pscale, s);
        case CQ_Q4K: return launch_moe_matvec<CQ_Q4K>(a, av, offsets, pin, pout, pscale, s);
        case CQ_Q5K: return launch_moe_matvec<CQ_Q5K>(a, av, offsets, pin, pout, pscale, s);
        case CQ_Q6K: return launch_moe_matvec<CQ_Q6K>(a, av, offsets, pin, pout, pscale, s);
        case CQ_Q2K: return launch_moe_matvec<CQ_Q2K>(a, av, offsets, pin, pout, pscale, s);
        case CQ_Q3K: return launch_moe_matvec<CQ_Q3K>(a, av, offsets, pin, pout, pscale, s);
    }
    return CQ_ERR_DTYPE;
}
