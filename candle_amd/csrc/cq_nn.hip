// Decoder glue around the quantized matmuls of candle's quantized llama
// (candle-transformers/src/models/quantized_llama.rs:191-266, 568-596): embedding lookup, residual add +
// RMS norm, interleaved rotary embedding + KV-cache append, causal GQA attention over the cache,
// silu(gate) * up, and greedy argmax; and the routing glue of the fused MoE layer (candle-transformers/src/fused_moe.rs:
// 222-301): router + softmax + top-k, the sort of the pairs by expert, the sum over top-k.  All f32, like the reference's CPU path.  Token ids and the
// decode position can be read from device memory so that a whole decode step (including "pick the next
// token, advance the position") can be captured in a HIP graph and replayed without host round trips.
#include "cq_device.h"
#include "../../include/candle_hip_nn.h"

namespace {

__device__ __forceinline__ float block_sum_256(float v, float *red) {     // red: >= 4 floats of LDS
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// ---- embedding: out[r, :] = table[ids[r], :] (candle_nn::Embedding, index_select) ---------------
__global__ __launch_bounds__(256) void embedding_kernel(const float *__restrict__ table, const int32_t *__restrict__ ids, float *__restrict__ out,
                                                        int dim, int64_t vocab, float *__restrict__ partials) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const int64_t id = ids[r];
    const bool ok = id >= 0 && id < vocab;
    const float4 *src = reinterpret_cast<const float4 *>(table + (ok ? id : 0) * dim);
    float4 *dst = reinterpret_cast<float4 *>(out + (int64_t)r * dim);
    float acc = 0.0f;
    for (int i = threadIdx.x; i < dim / 4; i += 256) {
        const float4 v = ok ? src[i] : float4{0.f, 0.f, 0.f, 0.f};
        dst[i] = v;
        acc += v.x * v.x;
        acc += v.y * v.y;
        acc += v.z * v.z;
        acc += v.w * v.w;
    }
    if (partials) {                       // uniform branch
        const float t = block_sum_256(acc, red);
        partials[threadIdx.x] = threadIdx.x == 0 ? t : 0.0f;      // 256 threads == CQ_NN_PARTIALS slots
    }
}

// ---- s = x (+ delta); sum_out = s; out = s / sqrt(mean(s^2) + eps) * w  (candle-nn/src/ops.rs:499-510) ----
__global__ __launch_bounds__(256) void rms_norm_kernel(const float *x, const float *__restrict__ delta, const float *__restrict__ w, float *sum_out,
                                                       float *__restrict__ out, int dim, float eps) {
    __shared__ float red[4];
    const int64_t base = (int64_t)blockIdx.x * dim;
    const float4 *x4 = reinterpret_cast<const float4 *>(x + base);
    const float4 *d4 = delta ? reinterpret_cast<const float4 *>(delta + base) : nullptr;
    float4 *s4 = sum_out ? reinterpret_cast<float4 *>(sum_out + base) : nullptr;
    const float4 *w4 = reinterpret_cast<const float4 *>(w);
    float4 *o4 = reinterpret_cast<float4 *>(out + base);
    const int n4 = dim >> 2;
    // up to 4 float4 per thread stay in registers (dim <= 4096); longer rows are re-read
    float4 keep[4];
    float acc = 0.0f;
    auto fetch = [&](int i) {
        float4 v = x4[i];
        if (d4) {
            float4 d = d4[i];
            v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        return v;
    };
    auto square = [&](const float4 &v) {
        acc += v.x * v.x;
        acc += v.y * v.y;
        acc += v.z * v.z;
        acc += v.w * v.w;
    };
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int i = threadIdx.x + 256 * c;
        if (i < n4) {
            keep[c] = fetch(i);
            if (s4) s4[i] = keep[c];
            square(keep[c]);
        }
    }
    for (int i = threadIdx.x + 1024; i < n4; i += 256) {
        const float4 v = fetch(i);
        if (s4) s4[i] = v;
        square(v);
    }
    const float sum2 = block_sum_256(acc, red);
    const float m = sqrtf(sum2 / (float)dim + eps);
    auto emit = [&](int i, const float4 &v) {
        const float4 a = w4[i];
        o4[i] = float4{v.x / m * a.x, v.y / m * a.y, v.z / m * a.z, v.w / m * a.w};
    };
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int i = threadIdx.x + 256 * c;
        if (i < n4) emit(i, keep[c]);
    }
    // x may alias sum_out: each thread re-reads only elements it wrote itself
    for (int i = threadIdx.x + 1024; i < n4; i += 256) emit(i, s4 ? s4[i] : fetch(i));
}

// ---- rope_i on q (in place) and k (into the cache), v copied into the cache -------------------------
// candle-nn/src/rotary_emb.rs:52-70: dst[2i] = x[2i] cos - x[2i+1] sin ; dst[2i+1] = x[2i] sin + x[2i+1] cos,
// cos/sin rows indexed by the absolute position (quantized_llama.rs:174-189).
// caches: [n_kv_head][ctx][head_dim]
__global__ __launch_bounds__(256) void rope_kv_kernel(float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
                                                      float *__restrict__ k_cache, float *__restrict__ v_cache, const float *__restrict__ cos_t,
                                                      const float *__restrict__ sin_t, const int32_t *__restrict__ pos_dev, int pos0, int n_head,
                                                      int n_kv_head, int hd, int ctx, int64_t q_stride, int64_t k_stride, int64_t v_stride) {
    const int r = blockIdx.x;
    const int p = pos0 + (pos_dev ? pos_dev[0] : 0) + r;
    if (p >= ctx) return;
    const int half = hd >> 1;
    const float *cs = cos_t + (int64_t)p * half, *sn = sin_t + (int64_t)p * half;
    float *qr = q + r * q_stride;
    const float *kr = k + r * k_stride, *vr = v + r * v_stride;
    for (int i = threadIdx.x; i < n_head * half; i += 256) {
        const int h = i / half, j = i - h * half;
        float2 x = *reinterpret_cast<float2 *>(qr + h * hd + 2 * j);
        const float c = cs[j], s = sn[j];
        *reinterpret_cast<float2 *>(qr + h * hd + 2 * j) = float2{x.x * c - x.y * s, x.x * s + x.y * c};
    }
    for (int i = threadIdx.x; i < n_kv_head * half; i += 256) {
        const int h = i / half, j = i - h * half;
        float2 x = *reinterpret_cast<const float2 *>(kr + h * hd + 2 * j);
        const float c = cs[j], s = sn[j];
        *reinterpret_cast<float2 *>(k_cache + ((int64_t)h * ctx + p) * hd + 2 * j) = float2{x.x * c - x.y * s, x.x * s + x.y * c};
        *reinterpret_cast<float2 *>(v_cache + ((int64_t)h * ctx + p) * hd + 2 * j) = *reinterpret_cast<const float2 *>(vr + h * hd + 2 * j);
    }
}

// ---- causal attention of `rows` new queries over the cache -------------------------------------------
// Query row r sits at absolute position p = pos + r and attends keys [0, p] (quantized_llama.rs:246-261:
// q k^T / sqrt(d), causal mask, softmax_last_dim, . v, with repeat_kv for grouped heads).
// One workgroup = one kv head x one query row x one split of 128 keys; the G = n_head / n_kv_head query
// heads that share the kv head are processed together so K and V are read once.
//   phase 1: 16 lanes share one key (each holds HD/16 consecutive dims of it and of the G queries), a wave
//            covers 4 keys per step, the workgroup 16; all K loads of the split are issued before any use;
//            16-lane DPP sums give the scores
//   phase 2: per query head: max, exp, sum over the split
//   phase 3: lanes own output dims, each wave takes 8 keys per step (loads first, then FMAs), p[j] broadcast
//            from LDS; waves summed via LDS
// With one split the normalized result is written directly; otherwise (m, l, unnormalized acc) partials
// go to the workspace and attn_combine_kernel merges them.
constexpr int ATT_SPLIT = 128;
constexpr int CQ_ATTN_MFMA_MIN = 64;         // query rows from which attn_mfma_kernel is used (head_dim 128)
constexpr int CQ_ATTN_ROWS_MIN = 16;        // query rows from which a workgroup takes several rows (attn_rows_kernel)

__device__ __forceinline__ float row16_sum(float v) {      // sum over each aligned group of 16 lanes, in every lane
#define CQ_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))
    CQ_ADD(CQ_DPP_QUAD_XOR1);
    CQ_ADD(CQ_DPP_QUAD_XOR2);
    CQ_ADD(CQ_DPP_ROW_HALF_MIRROR);
    CQ_ADD(0x140);                                          // row_mirror
#undef CQ_ADD
    return v;
}

template <int HD, int G>
__global__ __launch_bounds__(256) void attn_kernel(const float *__restrict__ q, int64_t q_stride, const float *__restrict__ k_cache,
                                                   const float *__restrict__ v_cache, float *__restrict__ out, float *__restrict__ part,
                                                   const int32_t *__restrict__ pos_dev, int pos0, int n_head, int ctx, float scale, int splits) {
    constexpr int DPL = HD / 64;                  // output dims per lane (phase 3)
    constexpr int EPL = HD / 16;                  // dims per lane (phase 1): 16 lanes per key
    constexpr int IT = ATT_SPLIT / 16;            // phase-1 steps: 16 keys per workgroup step
    __shared__ float sc[G * ATT_SPLIT];
    __shared__ float red[4 * G * HD];
    __shared__ float ml[2 * G];
    const int kvh = blockIdx.x, r = blockIdx.y, sp = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int kv_len = min(pos0 + (pos_dev ? pos_dev[0] : 0) + r + 1, ctx);
    const int j0 = sp * ATT_SPLIT;
    const int cnt = min(kv_len - j0, ATT_SPLIT);      // keys in this split (may be <= 0)
    if (cnt <= 0 && splits > 1) {
        // a split entirely behind this row's position (the grid is sized for the last row): an empty partial, which the
        // combine kernel skips, and nothing else — with a causal prompt that is three splits in eight
        if (tid < G) {
            float *pp = part + (((int64_t)r * n_head + kvh * G + tid) * splits + sp) * (HD + 2);
            pp[0] = -INFINITY;
            pp[1] = 0.0f;
        }
        return;
    }
    const float *kb = k_cache + (int64_t)kvh * ctx * HD, *vb = v_cache + (int64_t)kvh * ctx * HD;
    const int last = max(cnt - 1, 0);                 // loads of masked keys are redirected to a valid row

    // ---- phase 1 ----
    {
        const int sub = lane & 15, kq = lane >> 4;
        f32x4 kd[IT][EPL / 4];
#pragma unroll
        for (int it = 0; it < IT; it++) {
            const int key = min(it * 16 + wv * 4 + kq, last);
            const f32x4 *kr = reinterpret_cast<const f32x4 *>(kb + (int64_t)(j0 + key) * HD + EPL * sub);
#pragma unroll
            for (int c = 0; c < EPL / 4; c++) kd[it][c] = kr[c];
        }
        f32x4 qf[G][EPL / 4];
#pragma unroll
        for (int g = 0; g < G; g++) {
            const f32x4 *qr = reinterpret_cast<const f32x4 *>(q + r * q_stride + (int64_t)(kvh * G + g) * HD + EPL * sub);
#pragma unroll
            for (int c = 0; c < EPL / 4; c++) qf[g][c] = qr[c];
        }
#pragma unroll
        for (int it = 0; it < IT; it++) {
            const int key = it * 16 + wv * 4 + kq;
#pragma unroll
            for (int g = 0; g < G; g++) {
                float a = 0.0f;
#pragma unroll
                for (int c = 0; c < EPL / 4; c++) {
                    a += qf[g][c].x * kd[it][c].x;
                    a += qf[g][c].y * kd[it][c].y;
                    a += qf[g][c].z * kd[it][c].z;
                    a += qf[g][c].w * kd[it][c].w;
                }
                a = row16_sum(a);
                if (sub == 0) sc[g * ATT_SPLIT + key] = key < cnt ? a * scale : -INFINITY;
            }
        }
    }
    __syncthreads();

    // ---- phase 2: wave w reduces heads g = w, w + 4, ... ----
    for (int g = wv; g < G; g += 4) {
        float s[ATT_SPLIT / 64], m = -INFINITY;
#pragma unroll
        for (int i = 0; i < ATT_SPLIT / 64; i++) {
            s[i] = sc[g * ATT_SPLIT + lane + 64 * i];
            m = fmaxf(m, s[i]);
        }
        m = wave_max(m);
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < ATT_SPLIT / 64; i++) {
            const float p = (cnt > 0 && s[i] > -INFINITY) ? __expf(s[i] - m) : 0.0f;
            sc[g * ATT_SPLIT + lane + 64 * i] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) { ml[2 * g] = m; ml[2 * g + 1] = l; }
    }
    __syncthreads();

    // ---- phase 3 ----
    float o[G][DPL];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < DPL; e++) o[g][e] = 0.0f;
    for (int jb = 0; jb < cnt; jb += 32) {
        float vv[8][DPL];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int j = min(jb + wv + 4 * u, last);
            if (DPL == 2) {
                const float2 t = *reinterpret_cast<const float2 *>(vb + (int64_t)(j0 + j) * HD + 2 * lane);
                vv[u][0] = t.x; vv[u][DPL - 1] = t.y;
            } else {
#pragma unroll
                for (int e = 0; e < DPL; e++) vv[u][e] = vb[(int64_t)(j0 + j) * HD + DPL * lane + e];
            }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int j = jb + wv + 4 * u;                // < ATT_SPLIT; entries at or beyond cnt hold p = 0
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float p = sc[g * ATT_SPLIT + j];
#pragma unroll
                for (int e = 0; e < DPL; e++) o[g][e] += p * vv[u][e];
            }
        }
    }
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < DPL; e++) red[(wv * G + g) * HD + DPL * lane + e] = o[g][e];
    __syncthreads();
    for (int i = tid; i < G * HD; i += 256) {
        const int g = i / HD, d = i - g * HD;
        const float a = red[(0 * G + g) * HD + d] + red[(1 * G + g) * HD + d] + red[(2 * G + g) * HD + d] + red[(3 * G + g) * HD + d];
        const int head = kvh * G + g;
        if (splits == 1) {
            out[((int64_t)r * n_head + head) * HD + d] = a / ml[2 * g + 1];
        } else {
            float *pp = part + (((int64_t)r * n_head + head) * splits + sp) * (HD + 2);
            pp[2 + d] = a;
            if (d == 0) { pp[0] = ml[2 * g]; pp[1] = ml[2 * g + 1]; }
        }
    }
}

// The same attention for R consecutive query rows per workgroup (prompts and wide batches): the K and V rows of a split
// are loaded once for the R * G (row, head) pairs that use them instead of once per row, which is what bounds the
// one-row kernel on a long prompt (every workgroup pulls 2 * ATT_SPLIT * HD floats through the L2).  Per (row, head) the
// arithmetic and its order are those of attn_kernel; each row keeps its own causal length.
template <int HD, int G, int R>
__global__ __launch_bounds__(256) void attn_rows_kernel(const float *__restrict__ q, int64_t q_stride, const float *__restrict__ k_cache,
                                                        const float *__restrict__ v_cache, float *__restrict__ out, float *__restrict__ part,
                                                        const int32_t *__restrict__ pos_dev, int pos0, int rows, int n_head, int ctx,
                                                        float scale, int splits) {
    constexpr int VH = G * R;                     // (row, head) pairs of the workgroup, vh = rr * G + g
    static_assert(VH % 4 == 0 && VH <= 16, "pairs per workgroup");
    constexpr int DPL = HD / 64, EPL = HD / 16, IT = ATT_SPLIT / 16;
    __shared__ __attribute__((aligned(16))) float sc[ATT_SPLIT * VH];       // [key][vh]
    __shared__ float red[4 * VH * HD];
    __shared__ float ml[2 * VH];
    const int kvh = blockIdx.x, r0 = blockIdx.y * R, sp = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int nr = min(R, rows - r0);                 // valid rows of this workgroup (>= 1)
    const int base_len = pos0 + (pos_dev ? pos_dev[0] : 0) + r0 + 1;
    const int j0 = sp * ATT_SPLIT;
    const int cnt_max = min(min(base_len + nr - 1, ctx) - j0, ATT_SPLIT);   // keys of the last valid row
    if (cnt_max <= 0 && splits > 1) {
        if (tid < VH && tid / G < nr) {
            float *pp = part + (((int64_t)(r0 + tid / G) * n_head + kvh * G + tid % G) * splits + sp) * (HD + 2);
            pp[0] = -INFINITY;
            pp[1] = 0.0f;
        }
        return;
    }
    const float *kb = k_cache + (int64_t)kvh * ctx * HD, *vb = v_cache + (int64_t)kvh * ctx * HD;
    const int last = max(cnt_max - 1, 0);

    // ---- phase 1: scores of 16 keys per step, the K rows held in registers across the R rows ----
    {
        const int sub = lane & 15, kq = lane >> 4;
        f32x4 kd[IT][EPL / 4];
#pragma unroll
        for (int it = 0; it < IT; it++) {
            const int key = min(it * 16 + wv * 4 + kq, last);
            const f32x4 *kr = reinterpret_cast<const f32x4 *>(kb + (int64_t)(j0 + key) * HD + EPL * sub);
#pragma unroll
            for (int c = 0; c < EPL / 4; c++) kd[it][c] = kr[c];
        }
#pragma unroll
        for (int rr = 0; rr < R; rr++) {
            const int row = r0 + min(rr, nr - 1);
            const int cnt = min(min(base_len + rr, ctx) - j0, ATT_SPLIT);
            f32x4 qf[G][EPL / 4];
#pragma unroll
            for (int g = 0; g < G; g++) {
                const f32x4 *qr = reinterpret_cast<const f32x4 *>(q + row * q_stride + (int64_t)(kvh * G + g) * HD + EPL * sub);
#pragma unroll
                for (int c = 0; c < EPL / 4; c++) qf[g][c] = qr[c];
            }
#pragma unroll
            for (int it = 0; it < IT; it++) {
                const int key = it * 16 + wv * 4 + kq;
#pragma unroll
                for (int g = 0; g < G; g++) {
                    float a = 0.0f;
#pragma unroll
                    for (int c = 0; c < EPL / 4; c++) {
                        a += qf[g][c].x * kd[it][c].x;
                        a += qf[g][c].y * kd[it][c].y;
                        a += qf[g][c].z * kd[it][c].z;
                        a += qf[g][c].w * kd[it][c].w;
                    }
                    a = row16_sum(a);
                    if (sub == 0) sc[key * VH + rr * G + g] = key < cnt ? a * scale : -INFINITY;
                }
            }
        }
    }
    __syncthreads();

    // ---- phase 2: wave w reduces pairs vh = w, w + 4, ... ----
    for (int vh = wv; vh < VH; vh += 4) {
        float s[ATT_SPLIT / 64], m = -INFINITY;
#pragma unroll
        for (int i = 0; i < ATT_SPLIT / 64; i++) {
            s[i] = sc[(lane + 64 * i) * VH + vh];
            m = fmaxf(m, s[i]);
        }
        m = wave_max(m);
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < ATT_SPLIT / 64; i++) {
            const float p = s[i] > -INFINITY ? __expf(s[i] - m) : 0.0f;
            sc[(lane + 64 * i) * VH + vh] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) { ml[2 * vh] = m; ml[2 * vh + 1] = l; }
    }
    __syncthreads();

    // ---- phase 3: wave w accumulates the values of keys w, w + 4, ... for every pair ----
    float o[VH][DPL];
#pragma unroll
    for (int v = 0; v < VH; v++)
#pragma unroll
        for (int e = 0; e < DPL; e++) o[v][e] = 0.0f;
    for (int jb = 0; jb < cnt_max; jb += 32) {
        float vv[8][DPL];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int j = min(jb + wv + 4 * u, last);
            if (DPL == 2) {
                const float2 t = *reinterpret_cast<const float2 *>(vb + (int64_t)(j0 + j) * HD + 2 * lane);
                vv[u][0] = t.x; vv[u][DPL - 1] = t.y;
            } else {
#pragma unroll
                for (int e = 0; e < DPL; e++) vv[u][e] = vb[(int64_t)(j0 + j) * HD + DPL * lane + e];
            }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int j = jb + wv + 4 * u;                // < ATT_SPLIT; masked entries hold p = 0
#pragma unroll
            for (int v4 = 0; v4 < VH / 4; v4++) {
                const f32x4 p = *reinterpret_cast<const f32x4 *>(&sc[j * VH + 4 * v4]);
#pragma unroll
                for (int e = 0; e < DPL; e++) {
                    o[4 * v4 + 0][e] += p.x * vv[u][e];
                    o[4 * v4 + 1][e] += p.y * vv[u][e];
                    o[4 * v4 + 2][e] += p.z * vv[u][e];
                    o[4 * v4 + 3][e] += p.w * vv[u][e];
                }
            }
        }
    }
#pragma unroll
    for (int v = 0; v < VH; v++)
#pragma unroll
        for (int e = 0; e < DPL; e++) red[(wv * VH + v) * HD + DPL * lane + e] = o[v][e];
    __syncthreads();
    for (int i = tid; i < VH * HD; i += 256) {
        const int vh = i / HD, d = i - vh * HD;
        const int rr = vh / G, g = vh - rr * G;
        if (rr >= nr) continue;
        const float a = red[(0 * VH + vh) * HD + d] + red[(1 * VH + vh) * HD + d] + red[(2 * VH + vh) * HD + d] + red[(3 * VH + vh) * HD + d];
        const int head = kvh * G + g;
        if (splits == 1) {
            out[((int64_t)(r0 + rr) * n_head + head) * HD + d] = a / ml[2 * vh + 1];
        } else {
            float *pp = part + (((int64_t)(r0 + rr) * n_head + head) * splits + sp) * (HD + 2);
            pp[2 + d] = a;
            if (d == 0) { pp[0] = ml[2 * vh]; pp[1] = ml[2 * vh + 1]; }
        }
    }
}

// The prompt's attention on the f32 matrix cores (head_dim 128): a workgroup takes the 32 (row, head) pairs of 32 / G
// consecutive query rows and walks over the keys in splits of 128, keeping a running maximum, sum and output per pair
// (no partial results in memory, no combine pass).  Per split: wave w forms the 32 x 32 score tile of its 32 keys with 64
// v_mfma_f32_32x32x2f32 steps over the head dimension (A = q, B = k, one float4 per lane and eight dims); the tiles meet
// in LDS (key-major, row stride 33 floats so that neither the tile's column-wise writes nor the row-wise reads collide),
// the softmax over the split runs as in attn_kernel, wave w forms output columns [32 w, 32 w + 32) of the split with 64
// steps over the keys (A = p from LDS, B = v), and the split is merged into the running state:
//   M' = max(M, m), out = out e^{M - M'} + out_split e^{m - M'}, L likewise.   f32 throughout.
typedef float mf32x16 __attribute__((ext_vector_type(16)));
constexpr int ATT_SCP = 33;                       // floats per key in the score tile

template <int G>
__global__ __launch_bounds__(256) void attn_mfma_kernel(const float *__restrict__ q, int64_t q_stride, const float *__restrict__ k_cache,
                                                        const float *__restrict__ v_cache, float *__restrict__ out,
                                                        const int32_t *__restrict__ pos_dev, int pos0, int rows, int n_head, int ctx,
                                                        float scale) {
    constexpr int HD = 128, VH = 32, R = VH / G;     // pair vh = rr * G + g
    static_assert(ATT_SPLIT == 128, "one 32-key tile per wave");
    __shared__ float sc[ATT_SPLIT * ATT_SCP];
    __shared__ float ml[2 * VH];                      // (m, l) of the current split
    __shared__ float run[2 * VH];                     // running (M, L)
    __shared__ float fac[2 * VH];                     // e^{M - M'}, e^{m - M'}
    const int kvh = blockIdx.x, r0 = blockIdx.y * R;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int x = lane & 31, kk = lane >> 5;          // operand row / column of this lane, and which of a step's two k
    const int nr = min(R, rows - r0);                 // valid rows of this workgroup (>= 1)
    const int base_len = pos0 + (pos_dev ? pos_dev[0] : 0) + r0 + 1;
    const int len_last = min(base_len + nr - 1, ctx);                       // keys of the last valid row (>= 1)
    const int n_sp = (len_last + ATT_SPLIT - 1) / ATT_SPLIT;
    const float *kb = k_cache + (int64_t)kvh * ctx * HD, *vb = v_cache + (int64_t)kvh * ctx * HD;
    if (tid < VH) { run[2 * tid] = -INFINITY; run[2 * tid + 1] = 0.0f; }

    // q of pair x: dims 8 c + 4 kk + i go to MFMA step 4 c + i
    f32x4 qd[HD / 8];
    {
        const float *qr = q + (int64_t)(r0 + min(x / G, nr - 1)) * q_stride + (int64_t)(kvh * G + x % G) * HD + 4 * kk;
#pragma unroll
        for (int c = 0; c < HD / 8; c++) qd[c] = *reinterpret_cast<const f32x4 *>(qr + 8 * c);
    }
    mf32x16 o;
#pragma unroll
    for (int e = 0; e < 16; e++) o[e] = 0.0f;

    for (int sp = 0; sp < n_sp; sp++) {
        const int j0 = sp * ATT_SPLIT;
        const int cnt_max = min(len_last - j0, ATT_SPLIT);                  // >= 1
        const int last = cnt_max - 1;                 // loads of masked keys are redirected to a valid row
        // ---- scores of keys [32 wv, 32 wv + 32) ----
        {
            f32x4 kd[HD / 8];
            const float *kr = kb + (int64_t)(j0 + min(32 * wv + x, last)) * HD + 4 * kk;
#pragma unroll
            for (int c = 0; c < HD / 8; c++) kd[c] = *reinterpret_cast<const f32x4 *>(kr + 8 * c);
            mf32x16 s;
#pragma unroll
            for (int e = 0; e < 16; e++) s[e] = 0.0f;
#pragma unroll
            for (int c = 0; c < HD / 8; c++) {
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(qd[c].x, kd[c].x, s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(qd[c].y, kd[c].y, s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(qd[c].z, kd[c].z, s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(qd[c].w, kd[c].w, s, 0, 0, 0);
            }
            // tile layout: column (key) = x, row (pair) = 8 (e / 4) + 4 kk + e % 4
            const int key = 32 * wv + x;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int vh = 8 * (e >> 2) + 4 * kk + (e & 3);
                const int cnt = min(base_len + vh / G, ctx) - j0;            // keys of this pair's row in the split (may be <= 0)
                sc[key * ATT_SCP + vh] = key < cnt ? s[e] * scale : -INFINITY;
            }
        }
        __syncthreads();

        // ---- softmax over the split: wave w reduces pairs vh = w, w + 4, ... ----
        for (int vh = wv; vh < VH; vh += 4) {
            float s[ATT_SPLIT / 64], m = -INFINITY;
#pragma unroll
            for (int i = 0; i < ATT_SPLIT / 64; i++) {
                s[i] = sc[(lane + 64 * i) * ATT_SCP + vh];
                m = fmaxf(m, s[i]);
            }
            m = wave_max(m);
            float l = 0.0f;
#pragma unroll
            for (int i = 0; i < ATT_SPLIT / 64; i++) {
                const float p = s[i] > -INFINITY ? __expf(s[i] - m) : 0.0f;
                sc[(lane + 64 * i) * ATT_SCP + vh] = p;
                l += p;
            }
            l = wave_sum(l);
            if (lane == 0) { ml[2 * vh] = m; ml[2 * vh + 1] = l; }
        }
        __syncthreads();
        if (tid < VH) {
            const float m = ml[2 * tid], l = ml[2 * tid + 1], M = run[2 * tid], L = run[2 * tid + 1];
            const float Mn = fmaxf(M, m);
            const float fa = L > 0.0f ? __expf(M - Mn) : 0.0f, fb = l > 0.0f ? __expf(m - Mn) : 0.0f;
            run[2 * tid] = Mn;
            run[2 * tid + 1] = L * fa + l * fb;
            fac[2 * tid] = fa;
            fac[2 * tid + 1] = fb;
        }

        // ---- output columns [32 wv, 32 wv + 32) of the split: step t takes keys 2 t + kk (masked keys hold p = 0) ----
        mf32x16 os;
#pragma unroll
        for (int e = 0; e < 16; e++) os[e] = 0.0f;
        const int nsteps = (cnt_max + 1) >> 1;                       // uniform over the workgroup
        for (int t0 = 0; t0 < nsteps; t0 += 16) {
            float vv[16], pv[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const int key = 2 * (t0 + u) + kk;                     // < ATT_SPLIT; clamped for the loads, p = 0 beyond cnt
                vv[u] = vb[(int64_t)(j0 + min(key, last)) * HD + 32 * wv + x];
                pv[u] = sc[key * ATT_SCP + x];
            }
#pragma unroll
            for (int u = 0; u < 16; u++) os = __builtin_amdgcn_mfma_f32_32x32x2f32(pv[u], vv[u], os, 0, 0, 0);
        }
        __syncthreads();                              // fac is written, and every wave is done with sc
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int vh = 8 * (e >> 2) + 4 * kk + (e & 3);
            o[e] = o[e] * fac[2 * vh] + os[e] * fac[2 * vh + 1];
        }
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const int vh = 8 * (e >> 2) + 4 * kk + (e & 3);
        const int rr = vh / G, g = vh - rr * G;
        if (rr >= nr) continue;
        out[((int64_t)(r0 + rr) * n_head + kvh * G + g) * HD + 32 * wv + x] = o[e] / run[2 * vh + 1];
    }
}

// merge the splits of one (row, head): out = sum_s e^{m_s - M} acc_s / sum_s e^{m_s - M} l_s
template <int HD>
__global__ __launch_bounds__(HD) void attn_combine_kernel(const float *__restrict__ part, float *__restrict__ out, int splits) {
    const int64_t rh = blockIdx.x;
    const float *pp = part + rh * splits * (HD + 2);
    float M = -INFINITY;
    for (int s = 0; s < splits; s++) M = fmaxf(M, pp[s * (HD + 2) + 1] > 0.0f ? pp[s * (HD + 2)] : -INFINITY);
    float num = 0.0f, den = 0.0f;
    for (int s = 0; s < splits; s++) {
        const float l = pp[s * (HD + 2) + 1];
        if (l > 0.0f) {
            const float w = __expf(pp[s * (HD + 2)] - M);
            num += w * pp[s * (HD + 2) + 2 + threadIdx.x];
            den += w * l;
        }
    }
    out[rh * HD + threadIdx.x] = num / den;
}

// ---- one decode step of attention (one new token) ------------------------------------------------------
// rope_i on q and on the new k, append of the new k / v to the cache, attention over keys [0, p].  Same
// arithmetic as rope_kv_kernel + attn_kernel; what changes is where it runs:
//   * q is rotated in registers; the workgroup whose split contains position p takes the new key and value
//     from the projection outputs instead of the cache, rotates the key, uses both, and writes them to the cache;
//   * a workgroup is 16 waves over one split of 128 keys, so a wave scores 8 keys and accumulates 8 values, and
//     every K and V row is requested before anything is consumed (one memory round trip);
//   * the result is left as per-split partials { acc[HD], m, l, 0, 0 } (stride HD + 4 floats, 16-byte aligned
//     rows); the last workgroup of each kv head, or the prologue of the attention_wo matvec, merges them.
constexpr int ATTD_MAX_SPLITS = 32;           // 4096 keys in splits of 128 (MAX_SEQ_LEN, quantized_llama.rs:27)
constexpr int ATTD_FINE_SPLITS = 32;          // up to this many splits they are 64 keys long
constexpr int ATTD_COUNTER_BYTES = CQ_NN_ATTD_HEADER_BYTES;      // arrival counters of the in-kernel merge, one int per kv head, in front of the partials
// Keys per split: 64 (workgroups of 8 waves) while that gives at most ATTD_FINE_SPLITS splits, else 128 (16 waves).  The
// vector memory pipeline of a CU takes one instruction of a wave per 16 cycles whatever it loads, and a split asks for
// about 28 of them per wave: with 128-key splits of 16 waves the 48 workgroups of a 768-key step spent 3 us getting
// their loads accepted; twice the workgroups of half the size halve that.
__host__ __device__ inline int64_t attd_split_keys(int64_t max_kv_len) { return (max_kv_len + 63) / 64 <= ATTD_FINE_SPLITS ? 64 : 128; }
__host__ __device__ inline int64_t attd_splits(int64_t max_kv_len) { const int64_t sk = attd_split_keys(max_kv_len); return (max_kv_len + sk - 1) / sk; }

// The merge of a kv head's splits by the workgroup that arrived last: out = sum_s e^{m_s - M} acc_s / sum_s e^{m_s - M} l_s,
// split by split, in order (the arithmetic of attn_combine_kernel and of the merge prologue of the attention_wo matvec).
// MS: the number of splits the registers hold (16 or 32).
template <int HD, int G, int NW, int MS>
__device__ __forceinline__ void attd_merge(const float *__restrict__ part, float *__restrict__ out, int kvh, int stride, int splits, int tid) {
    const int lane = tid & 63;
    auto ld = [](const float *q) { return __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    for (int i = tid; i < G * HD; i += 64 * NW) {
        const int g = i / HD, d = i - g * HD;                 // g is the same in all lanes of a wave
        const float *pp = part + (int64_t)(kvh * G + g) * stride * (HD + 4);           // `stride` records per head, the first `splits` in use
        // Every load first (these bypass the caches: one after the other they would be a trip to memory each), and as few
        // load instructions as possible, they are what the last workgroup's time goes into: one instruction fetches
        // the (m, l) of all splits of the head (lane s: m of split s, lane MS + s: l), one per existing split the
        // accumulators.  A split that does not exist re-reads the last one and is left out of the sums.
        const float mlv = ld(pp + min(lane & (MS - 1), splits - 1) * (HD + 4) + HD + ((lane / MS) & 1));
        float av[MS];
#pragma unroll
        for (int sI = 0; sI < MS; sI++) av[sI] = sI < splits ? ld(pp + sI * (HD + 4) + d) : 0.0f;
        float mv[MS], lv[MS];
#pragma unroll
        for (int sI = 0; sI < MS; sI++) {
            mv[sI] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mlv), sI));
            lv[sI] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mlv), MS + sI));
        }
        float M = -INFINITY;
#pragma unroll
        for (int sI = 0; sI < MS; sI++)
            if (sI < splits) M = fmaxf(M, lv[sI] > 0.0f ? mv[sI] : -INFINITY);
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int sI = 0; sI < MS; sI++) {
            if (sI < splits && lv[sI] > 0.0f) {
                const float wgt = __expf(mv[sI] - M);
                num += wgt * av[sI];
                den += wgt * lv[sI];
            }
        }
        out[(int64_t)(kvh * G + g) * HD + d] = num / den;
    }
}

// The read-only work of the single-token attention launch: workgroup `rank` of `count` read-only workgroups per grid column
// pulls its share of the weights the following kernels will stream (attention_wo, feed_forward_w1 / w3) towards the caches
// while this latency-bound kernel leaves the HBM idle.  Nothing is computed from the data; the store never executes for real weights.
template <int NW>
__device__ __forceinline__ void attd_prefetch(const u32x4 *__restrict__ pf, int64_t pf_chunks, int pf_piece16, uint32_t *__restrict__ pf_sink, int rank,
                                              int count) {
    uint32_t acc = 0;
    if (pf_piece16 > 0) {
        // Piece p of the range (pf_piece16 chunks: one wave step of the matvec that will stream it) is read later by a workgroup
        // on XCD p % 8; workgroups are dealt to the XCDs round-robin by their linear index, so this one reads pieces of its own
        // XCD only and they land in the L2 that the consumer will look in (grids of 8 columns).
        const int lin = (int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x;
        const int xcd = lin & 7;
        const int64_t npieces = pf_chunks / pf_piece16;
        const int64_t mine = (npieces - xcd + 7) / 8;                       // pieces of this XCD
        const int64_t vtotal = mine * pf_piece16, T = (int64_t)count * (64 * NW);
        for (int64_t v = (int64_t)rank * (64 * NW) + threadIdx.x; v < vtotal; v += 2 * T) {
            const int64_t v2 = v + T;
            const int64_t q = v / pf_piece16, o = v - q * pf_piece16;
            const u32x4 a = pf[(xcd + 8 * q) * pf_piece16 + o];
            u32x4 b = {0, 0, 0, 0};
            if (v2 < vtotal) {
                const int64_t q2 = v2 / pf_piece16, o2 = v2 - q2 * pf_piece16;
                b = pf[(xcd + 8 * q2) * pf_piece16 + o2];
            }
            acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w;
        }
        if (acc == 0x9e3779b9u && pf_sink) pf_sink[0] = acc;
        return;
    }
    const int64_t nthreads = (int64_t)gridDim.x * count * (64 * NW);
    int64_t i = ((int64_t)rank * gridDim.x + blockIdx.x) * (64 * NW) + threadIdx.x;
    for (; i + 3 * nthreads < pf_chunks; i += 4 * nthreads) {
        const u32x4 a = pf[i], b = pf[i + nthreads], c = pf[i + 2 * nthreads], d = pf[i + 3 * nthreads];
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < pf_chunks; i += nthreads) {
        const u32x4 a = pf[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u && pf_sink) pf_sink[0] = acc;
}

// Splits that hold keys at this position: with the merge inside the kernel (out != NULL) only those take part -- a launch laid
// out for a long context costs what the keys that exist cost -- and the workgroups of the others leave at once.
template <int SPLIT>
__device__ __forceinline__ int attd_active(int splits, int kv_len, bool merged) {
    return merged ? min(splits, (kv_len + SPLIT - 1) / SPLIT) : splits;
}

template <int HD, int G, int NW, int SPLIT>
__global__ __launch_bounds__(64 * NW) void attn_decode_kernel(const int32_t *__restrict__ pos_dev, const float *__restrict__ q, float *k_cache,
                                                                      const float *__restrict__ cos_t, const float *__restrict__ sin_t, int pos0,
                                                                      int splits, int ctx, float scale, float *v_cache,
                                                                      const float *__restrict__ k_new, const float *__restrict__ v_new,
                                                                      float *__restrict__ part, const u32x4 *__restrict__ pf,
                                                                      int64_t pf_chunks, uint32_t *__restrict__ pf_sink, float *__restrict__ out,
                                                                      int *__restrict__ counters, int pf_piece16) {
    // (parameter order: the fourteen dwords that sit in SGPRs when the wave starts are all that the key and query loads
    // need, so that those go out without waiting for a scalar load: neither for further arguments nor for the position)
    if ((int)blockIdx.y >= splits) {
        // workgroups beyond the attention splits only read (they do not wait for the position: their share is fixed by the grid)
        if (pf_chunks > 0) attd_prefetch<NW>(pf, pf_chunks, pf_piece16, pf_sink, (int)blockIdx.y - splits, (int)gridDim.y - splits);
        return;
    }
    constexpr int DPL = HD / 64, EPL = HD / 16, IT = SPLIT / (4 * NW), VU = SPLIT / NW, QR = (G + 3) / 4;
    __shared__ __align__(16) float sc[SPLIT * G];          // [key][query head]
    __shared__ __align__(16) float red[NW * G * HD];
    __shared__ float ml[2 * G];
    const int kvh = blockIdx.x, sp = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int p_raw = pos_dev ? pos_dev[0] : 0;             // on its way while the loads below go out
    const int j0 = sp * SPLIT;
    float *kb = k_cache + (int64_t)kvh * ctx * HD, *vb = v_cache + (int64_t)kvh * ctx * HD;
    const int sub = lane & 15, kq = lane >> 4;

    // ---- every load of the kernel, issued before any use ----
    // What scoring needs goes first, and of that first what does not depend on the position: the split's key rows as they
    // lie in the cache (rows beyond the position are read and masked later; the row of the position itself is replaced by
    // the new key below) and the query heads.  A lane fetches its 16-dimension slice of one query head only (head kq of
    // every four); the wave exchanges the rotated slices through LDS, a quarter of the load instructions of every lane
    // fetching every head.
    f32x4 kd[IT][EPL / 4];
#pragma unroll
    for (int it = 0; it < IT; it++) {
        const int row = min(j0 + (it * NW + wv) * 4 + kq, ctx - 1);
        const float *src = kb + (int64_t)row * HD + EPL * sub;
#pragma unroll
        for (int c = 0; c < EPL / 4; c++) kd[it][c] = reinterpret_cast<const f32x4 *>(src)[c];
    }
    f32x4 qv[QR][EPL / 4];
#pragma unroll
    for (int r = 0; r < QR; r++) {
        const int g = min(4 * r + kq, G - 1);
        const f32x4 *qr = reinterpret_cast<const f32x4 *>(q + (int64_t)(kvh * G + g) * HD + EPL * sub);
#pragma unroll
        for (int c = 0; c < EPL / 4; c++) qv[r][c] = qr[c];
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // the arguments that did not arrive in registers, asked for here in one go (and waited for together with the position)
    asm volatile("" ::"s"(v_cache), "s"(k_new), "s"(v_new), "s"(part));
    const int p = min(pos0 + p_raw, ctx - 1);
    const int kv_len = p + 1;
    const int active = attd_active<SPLIT>(splits, kv_len, out != nullptr);
    if (sp >= active) return;                     // uniform over the workgroup: no key of this split exists yet
    const int cnt = min(kv_len - j0, SPLIT);
    const int last = max(cnt - 1, 0);
    const bool has_p = p >= j0 && p < j0 + SPLIT;           // this split holds the new token (the same in every wave)
    // cos / sin of position p for this lane's EPL/2 pairs
    float cs[EPL / 2], sn[EPL / 2];
    if constexpr (EPL / 2 == 4) {
        const f32x4 c4 = *reinterpret_cast<const f32x4 *>(cos_t + (int64_t)p * (HD / 2) + 4 * sub);
        const f32x4 s4 = *reinterpret_cast<const f32x4 *>(sin_t + (int64_t)p * (HD / 2) + 4 * sub);
        cs[0] = c4.x; cs[1] = c4.y; cs[2] = c4.z; cs[3] = c4.w;
        sn[0] = s4.x; sn[1] = s4.y; sn[2] = s4.z; sn[3] = s4.w;
    } else {
#pragma unroll
        for (int c = 0; c < EPL / 2; c++) {
            cs[c] = cos_t[(int64_t)p * (HD / 2) + (EPL / 2) * sub + c];
            sn[c] = sin_t[(int64_t)p * (HD / 2) + (EPL / 2) * sub + c];
        }
    }
    f32x4 kn[EPL / 4];
#pragma unroll
    for (int c = 0; c < EPL / 4; c++) kn[c] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (has_p) {
#pragma unroll
        for (int c = 0; c < EPL / 4; c++) kn[c] = reinterpret_cast<const f32x4 *>(k_new + kvh * HD + EPL * sub)[c];
    }
    asm volatile("" ::: "memory");
    // the values last: they are used after the softmax
    float vv[VU][DPL];
#pragma unroll
    for (int u = 0; u < VU; u++) {
        const int j = min(wv + NW * u, last);
        const float *src = (j0 + j == p) ? v_new + kvh * HD + DPL * lane : vb + (int64_t)(j0 + j) * HD + DPL * lane;
        if (DPL == 2) {
            const float2 t = *reinterpret_cast<const float2 *>(src);
            vv[u][0] = t.x; vv[u][DPL - 1] = t.y;
        } else {
#pragma unroll
            for (int e = 0; e < DPL; e++) vv[u][e] = src[e];
        }
    }
    // nothing that waits for data may be scheduled between the loads above: every one is requested before the first wait
    __builtin_amdgcn_sched_barrier(0);
    auto rope4 = [&](f32x4 &v, int c) {       // two interleaved pairs (rotary_emb.rs:52-70)
        const float a = v.x * cs[2 * c] - v.y * sn[2 * c], b = v.x * sn[2 * c] + v.y * cs[2 * c];
        const float e = v.z * cs[2 * c + 1] - v.w * sn[2 * c + 1], f = v.z * sn[2 * c + 1] + v.w * cs[2 * c + 1];
        v = f32x4{a, b, e, f};
    };
    // the lane's query slice rotated, then every head's slice back from the wave's own part of `red` (free until phase 3)
    f32x4 qf[G][EPL / 4];
    {
        float *qx = red + wv * G * HD + EPL * sub;
#pragma unroll
        for (int r = 0; r < QR; r++) {
            const int g = min(4 * r + kq, G - 1);         // G not a multiple of four: several lanes write the same head, the same values
#pragma unroll
            for (int c = 0; c < EPL / 4; c++) {
                rope4(qv[r][c], c);
                reinterpret_cast<f32x4 *>(qx + g * HD)[c] = qv[r][c];
            }
        }
        // the wave reads what its own lanes wrote: LDS operations of a wave complete in order, the fences keep the compiler
        // from moving the reads up
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int c = 0; c < EPL / 4; c++) qf[g][c] = reinterpret_cast<const f32x4 *>(qx + g * HD)[c];
    }

    // ---- phase 1: scores; the lanes holding the new key take it from the projection, rotate it and append it to the cache ----
#pragma unroll
    for (int it = 0; it < IT; it++) {
        const int key = (it * NW + wv) * 4 + kq;
        if (j0 + key == p) {
#pragma unroll
            for (int c = 0; c < EPL / 4; c++) {
                kd[it][c] = kn[c];
                rope4(kd[it][c], c);
                reinterpret_cast<f32x4 *>(kb + (int64_t)p * HD + EPL * sub)[c] = kd[it][c];
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            float a = 0.0f;
#pragma unroll
            for (int c = 0; c < EPL / 4; c++) {
                a += qf[g][c].x * kd[it][c].x;
                a += qf[g][c].y * kd[it][c].y;
                a += qf[g][c].z * kd[it][c].z;
                a += qf[g][c].w * kd[it][c].w;
            }
            a = row16_sum(a);
            if (sub == 0) sc[key * G + g] = key < cnt ? a * scale : -INFINITY;
        }
    }
    __syncthreads();

    // ---- phase 2: wave g handles query head g ----
    if (wv < G) {
        const int g = wv;
        float s[SPLIT / 64], m = -INFINITY;
#pragma unroll
        for (int i = 0; i < SPLIT / 64; i++) {
            s[i] = sc[(lane + 64 * i) * G + g];
            m = fmaxf(m, s[i]);
        }
        m = wave_max(m);
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < SPLIT / 64; i++) {
            const float pr = (cnt > 0 && s[i] > -INFINITY) ? __expf(s[i] - m) : 0.0f;
            sc[(lane + 64 * i) * G + g] = pr;
            l += pr;
        }
        l = wave_sum(l);
        if (lane == 0) { ml[2 * g] = m; ml[2 * g + 1] = l; }
    }
    __syncthreads();

    // ---- phase 3: p . v from registers; the wave holding the new value appends it ----
    // every probability of the wave's keys read first (one LDS round trip), and no branch around the sums: the value of a
    // key at or beyond cnt is replaced by zero (its probability is zero too, but what lies in the cache there need not be finite)
    float pr[VU][G];
#pragma unroll
    for (int u = 0; u < VU; u++)
#pragma unroll
        for (int g = 0; g < G; g++) pr[u][g] = sc[(wv + NW * u) * G + g];
    float o[G][DPL];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < DPL; e++) o[g][e] = 0.0f;
#pragma unroll
    for (int u = 0; u < VU; u++) {
        const int j = wv + NW * u;                    // < SPLIT
        if (j0 + j == p) {
#pragma unroll
            for (int e = 0; e < DPL; e++) vb[(int64_t)p * HD + DPL * lane + e] = vv[u][e];
        }
        const bool live = j < cnt;                    // wave-uniform
#pragma unroll
        for (int e = 0; e < DPL; e++) {
            const float v = live ? vv[u][e] : 0.0f;
#pragma unroll
            for (int g = 0; g < G; g++) o[g][e] += (live ? pr[u][g] : 0.0f) * v;
        }
    }
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < DPL; e++) red[(wv * G + g) * HD + DPL * lane + e] = o[g][e];
    __syncthreads();
    for (int i = tid; i < G * HD; i += 64 * NW) {
        const int g = i / HD, d = i - g * HD;
        float a = 0.0f;
#pragma unroll
        for (int w2 = 0; w2 < NW; w2++) a += red[(w2 * G + g) * HD + d];
        float *pp = part + ((int64_t)(kvh * G + g) * splits + sp) * (HD + 4);
        // device-scope stores (written through to where every CU of the GPU reads them): the in-kernel merge below reads
        // partials of workgroups on other XCDs, whose L2 caches are not coherent with this one's
        __hip_atomic_store(pp + d, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d < 4) __hip_atomic_store(pp + HD + d, d == 0 ? ml[2 * g] : d == 1 ? ml[2 * g + 1] : 0.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (out == nullptr) return;
    // The merge of the splits, once: the workgroup of this kv head that finishes last does it (no second launch, and no
    // consumer has to pull every partial through its own CU).  Arrival is counted after a device-wide release of the
    // partials; the last workgroup acquires, merges (split by split, in order, like the prologue of the attention_wo matvec), and leaves the counter zero.
    // No fence: a device-scope release would write back every dirty line of this XCD's L2 (measured: 24 us per launch).
    // The partials went out as device-scope stores; once they are acknowledged (vmcnt = 0) the arrival may be counted,
    // and the last workgroup reads them with device-scope loads.
    __shared__ int s_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) s_last = __hip_atomic_fetch_add(&counters[kvh], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == active - 1;
    __syncthreads();
    if (!s_last) return;
    static_assert(HD % 64 == 0 && ATTD_MAX_SPLITS <= 32, "a wave stays inside one query head; the lanes of a wave fetch the (m, l) pairs");
    if (active <= 16)
        attd_merge<HD, G, NW, 16>(part, out, kvh, splits, active, tid);
    else
        attd_merge<HD, G, NW, ATTD_MAX_SPLITS>(part, out, kvh, splits, active, tid);
    if (tid == 0) __hip_atomic_store(&counters[kvh], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- out = silu(gate) * up, silu(v) = v / (1 + exp(-v))  (candle-core/src/op.rs Silu; quantized_llama.rs:56-63) ----
__global__ __launch_bounds__(256) void silu_mul_kernel(const float *__restrict__ gate, const float *__restrict__ up, float *__restrict__ out, int dim,
                                                       int64_t gate_stride, int64_t up_stride) {
    const int r = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= dim / 4) return;
    const float4 g = reinterpret_cast<const float4 *>(gate + r * gate_stride)[i];
    const float4 u = reinterpret_cast<const float4 *>(up + r * up_stride)[i];
    float4 o;
    o.x = g.x / (1.0f + expf(-g.x)) * u.x;
    o.y = g.y / (1.0f + expf(-g.y)) * u.y;
    o.z = g.z / (1.0f + expf(-g.z)) * u.z;
    o.w = g.w / (1.0f + expf(-g.w)) * u.w;
    reinterpret_cast<float4 *>(out + (int64_t)r * dim)[i] = o;
}

// ---- greedy sampling: index of the largest logit, lowest index on ties (Sampling::ArgMax) ----
// One workgroup.  Optionally appends the token to history[*pos_dev + 1 ...] semantics are the caller's:
// token_out[0] = idx; if history: history[hist_index] = idx where hist_index = *counter; if counter: *counter += 1.
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ logits, int n, int32_t *__restrict__ token_out,
                                                      int32_t *__restrict__ history, int32_t *__restrict__ counter, int32_t *__restrict__ pos_dev) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += 1024) {
        const float v = logits[i];
        if (v > best || idx == 0x7fffffff) { best = v; idx = i; }      // ascending i per thread: strict > keeps the first
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(idx, o, 64);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = best; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++)
            if (bv[w] > best || (bv[w] == best && bi[w] < idx)) { best = bv[w]; idx = bi[w]; }
        token_out[0] = idx;
        if (history && counter) history[counter[0]] = idx;
        if (counter) counter[0] += 1;
        if (pos_dev) pos_dev[0] += 1;
    }
}

// Two-stage variant for long logit rows: up to 128 workgroups each leave (value, index) of their contiguous chunk,
// one small workgroup finishes.  Ties still resolve to the lowest index: chunks are contiguous and ordered.
constexpr int ARGMAX_PARTS = 128;
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float *__restrict__ logits, int n, int chunk, float *__restrict__ pv,
                                                             int *__restrict__ pi) {
    __shared__ float bv[4];
    __shared__ int bi[4];
    const int lo = blockIdx.x * chunk, hi = min(n, lo + chunk);
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
        const float v = logits[i];
        if (v > best || idx == 0x7fffffff) { best = v; idx = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(idx, o, 64);
        if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) { best = ov; idx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = best; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++)
            if (bi[w] != 0x7fffffff && (idx == 0x7fffffff || bv[w] > best || (bv[w] == best && bi[w] < idx))) { best = bv[w]; idx = bi[w]; }
        pv[blockIdx.x] = best;
        pi[blockIdx.x] = idx;
    }
}
__global__ __launch_bounds__(64) void argmax_final_kernel(const float *__restrict__ pv, const int *__restrict__ pi, int parts,
                                                          int32_t *__restrict__ token_out, int32_t *__restrict__ history,
                                                          int32_t *__restrict__ counter, int32_t *__restrict__ pos_dev) {
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < parts; i += 64) {
        const float v = pv[i];
        const int j = pi[i];
        if (j != 0x7fffffff && (idx == 0x7fffffff || v > best || (v == best && j < idx))) { best = v; idx = j; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(idx, o, 64);
        if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) { best = ov; idx = oi; }
    }
    if (threadIdx.x == 0) {
        token_out[0] = idx;
        if (history && counter) history[counter[0]] = idx;
        if (counter) counter[0] += 1;
        if (pos_dev) pos_dev[0] += 1;
    }
}

// The same last stage followed by the embedding lookup of the chosen token (embedding_kernel for one row, with its partial
// sums of squares): the next decode step finds its input row in place and starts with its first matvec.
__global__ __launch_bounds__(256) void argmax_final_embed_kernel(const float *__restrict__ pv, const int *__restrict__ pi, int parts,
                                                                 int32_t *__restrict__ token_out, int32_t *__restrict__ history,
                                                                 int32_t *__restrict__ counter, int32_t *__restrict__ pos_dev,
                                                                 const float *__restrict__ table, float *__restrict__ out, int dim, int64_t vocab,
                                                                 float *__restrict__ partials) {
    __shared__ float red[4];
    __shared__ int s_tok;
    if (threadIdx.x < 64) {
        float best = -INFINITY;
        int idx = 0x7fffffff;
        for (int i = threadIdx.x; i < parts; i += 64) {
            const float v = pv[i];
            const int j = pi[i];
            if (j != 0x7fffffff && (idx == 0x7fffffff || v > best || (v == best && j < idx))) { best = v; idx = j; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(idx, o, 64);
            if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) { best = ov; idx = oi; }
        }
        if (threadIdx.x == 0) {
            s_tok = idx;
            token_out[0] = idx;
            if (history && counter) history[counter[0]] = idx;
            if (counter) counter[0] += 1;
            if (pos_dev) pos_dev[0] += 1;
        }
    }
    __syncthreads();
    const int64_t id = s_tok;
    const bool ok = id >= 0 && id < vocab;
    const float4 *src = reinterpret_cast<const float4 *>(table + (ok ? id : 0) * dim);
    float4 *dst = reinterpret_cast<float4 *>(out);
    float acc = 0.0f;
    for (int i = threadIdx.x; i < dim / 4; i += 256) {
        const float4 v = ok ? src[i] : float4{0.f, 0.f, 0.f, 0.f};
        dst[i] = v;
        acc += v.x * v.x;
        acc += v.y * v.y;
        acc += v.z * v.z;
        acc += v.w * v.w;
    }
    if (partials) {                       // uniform branch
        const float t = block_sum_256(acc, red);
        partials[threadIdx.x] = threadIdx.x == 0 ? t : 0.0f;      // 256 threads == CQ_NN_PARTIALS slots
    }
}

// ---- MoE routing around the grouped expert matmuls (FusedMoeGGUF::forward, candle-transformers/src/fused_moe.rs:222-301) ----
constexpr int ROUTE_MAX_EXPERTS = 1024, ROUTE_MAX_TOPK = 64;

// router_logits = x . router_w^T (a bias-free f32 Linear, :233): a wave takes R experts of one token and walks the rows C
// column chunks of 256 at a time, every load of a trip issued before the first use (the router matrix of 128 x 2048 is
// 1 MB: walked chunk by chunk with a wait per chunk it took eight dependent memory trips, 5.2 us for one token).
// <1, 8>: few tokens, one row per wave, a 2048-element row is one trip; <4, 2>: many tokens, the token's row is loaded once
// per four experts.  Per lane the products are added in the same order in both, so the logits do not depend on the variant.
// T: tokens per wave (blockIdx.y is a group of T tokens): with hundreds of tokens the router rows a wave has loaded serve T
// tokens instead of one (one token per wave re-reads the 1 MB router matrix once per token: 14 us for 256 tokens).
template <int R, int C, int T = 1>
__global__ __launch_bounds__(256) void moe_logits_kernel(const float *__restrict__ x, const float *__restrict__ router_w, float *__restrict__ logits,
                                                         int hidden, int n_experts, int tokens) {
    const int t0 = blockIdx.y * T, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int e0 = (blockIdx.x * 4 + wv) * R;
    if (e0 >= n_experts) return;
    const float *xr[T];
#pragma unroll
    for (int j = 0; j < T; j++) xr[j] = x + (int64_t)min(t0 + j, tokens - 1) * hidden;
    const float *w[R];
#pragma unroll
    for (int i = 0; i < R; i++) w[i] = router_w + (int64_t)min(e0 + i, n_experts - 1) * hidden;
    float acc[T][R];
#pragma unroll
    for (int j = 0; j < T; j++)
#pragma unroll
        for (int i = 0; i < R; i++) acc[j][i] = 0.0f;
    for (int k0 = lane * 4; k0 < hidden; k0 += 256 * C) {
        f32x4 a[T][C], b[R][C];
#pragma unroll
        for (int c = 0; c < C; c++) {
            const int kc = min(k0 + 256 * c, hidden - 4);          // past the end: re-read the last vector, not used below
#pragma unroll
            for (int j = 0; j < T; j++) a[j][c] = *reinterpret_cast<const f32x4 *>(xr[j] + kc);
#pragma unroll
            for (int i = 0; i < R; i++) b[i][c] = *reinterpret_cast<const f32x4 *>(w[i] + kc);
        }
#pragma unroll
        for (int c = 0; c < C; c++) {
            if (k0 + 256 * c < hidden) {
#pragma unroll
                for (int j = 0; j < T; j++)
#pragma unroll
                    for (int i = 0; i < R; i++) {
                        acc[j][i] = fmaf(a[j][c].x, b[i][c].x, acc[j][i]);
                        acc[j][i] = fmaf(a[j][c].y, b[i][c].y, acc[j][i]);
                        acc[j][i] = fmaf(a[j][c].z, b[i][c].z, acc[j][i]);
                        acc[j][i] = fmaf(a[j][c].w, b[i][c].w, acc[j][i]);
                    }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < T; j++)
#pragma unroll
        for (int i = 0; i < R; i++) {
            const float v = wave_sum(acc[j][i]);
            if (lane == 0 && e0 + i < n_experts && t0 + j < tokens) logits[(int64_t)(t0 + j) * n_experts + e0 + i] = v;
        }
}

// One workgroup per token: softmax over the experts (:235-236), the topk largest probabilities in descending order
// (:238-243; equal values: lower expert first, as the stable descending arg_sort of candle-core/src/sort.rs:48-53
// leaves them) and the optional renormalisation (:245-247).
__global__ __launch_bounds__(256) void moe_topk_kernel(const float *__restrict__ logits, uint32_t *__restrict__ topk_ids,
                                                       float *__restrict__ topk_weights, int n_experts, int topk, int renorm) {
    __shared__ float prob[ROUTE_MAX_EXPERTS];
    __shared__ float sel[ROUTE_MAX_TOPK];
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    for (int e = tid; e < n_experts; e += 256) prob[e] = logits[(int64_t)t * n_experts + e];
    __syncthreads();
    // softmax_last_dim (candle-nn/src/ops.rs): max, exp(x - max), sum, divide
    float m = -INFINITY;
    for (int e = tid; e < n_experts; e += 256) m = fmaxf(m, prob[e]);
    m = wave_max(m);
    if (lane == 0) red[wv] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float part = 0.0f;
    for (int e = tid; e < n_experts; e += 256) {
        const float ex = expf(prob[e] - m);
        prob[e] = ex;
        part += ex;
    }
    const float total = block_sum_256(part, red);
    for (int e = tid; e < n_experts; e += 256) prob[e] = prob[e] / total;
    __syncthreads();
    if (wv != 0) return;
    // one wave picks the topk: every round the largest remaining probability, the lowest expert among equals
    volatile float *vp = prob;
    for (int j = 0; j < topk; j++) {
        // the largest remaining value (selected entries hold -2, NaNs never compare greater), then the lowest expert holding it
        float bv = -1.0f;
        for (int e = lane; e < n_experts; e += 64) bv = fmaxf(bv, vp[e]);
        bv = wave_max(bv);
        int bi = 0x7fffffff;
        if (bv > -1.0f) {
            for (int e0 = 0; e0 < n_experts; e0 += 64) {
                const unsigned long long hit = __ballot(e0 + lane < n_experts && vp[min(e0 + lane, n_experts - 1)] == bv);
                if (hit) { bi = e0 + __builtin_ctzll(hit); break; }
            }
        }
        if (lane == 0) {
            topk_ids[(int64_t)t * topk + j] = (uint32_t)bi;       // no finite probability left (NaN logits): an id no expert has
            sel[j] = bv;
            if (bi < n_experts) vp[bi] = -2.0f;
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (lane == 0) {
        float sum = 0.0f;
        for (int j = 0; j < topk; j++) sum += sel[j];
        for (int j = 0; j < topk; j++) topk_weights[(int64_t)t * topk + j] = renorm ? sel[j] / sum : sel[j];
    }
}

// The same routing for up to 256 experts with the row in the registers of one wave (expert e = lane + 64 i): no LDS
// round trips between the topk rounds and no barrier.  Sums are formed in the order of moe_topk_kernel (64 experts per
// wave sum, the four sums added in order; the selected probabilities added in slot order), so the two kernels return
// the same bits.
__global__ __launch_bounds__(64) void moe_topk_wave_kernel(const float *__restrict__ logits, uint32_t *__restrict__ topk_ids,
                                                           float *__restrict__ topk_weights, int n_experts, int topk, int renorm) {
    const int t = blockIdx.x, lane = threadIdx.x;
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; i++) p[i] = lane + 64 * i < n_experts ? logits[(int64_t)t * n_experts + lane + 64 * i] : -INFINITY;
    const float m = wave_max(fmaxf(fmaxf(p[0], p[1]), fmaxf(p[2], p[3])));
    float s4[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const bool live = lane + 64 * i < n_experts;
        p[i] = live ? expf(p[i] - m) : 0.0f;
        s4[i] = wave_sum(p[i]);
    }
    const float total = s4[0] + s4[1] + s4[2] + s4[3];
#pragma unroll
    for (int i = 0; i < 4; i++) p[i] = lane + 64 * i < n_experts ? p[i] / total : -2.0f;     // -2: not selectable
    float mysel = 0.0f;                                   // lane j keeps the probability of slot j
    for (int j = 0; j < topk; j++) {
        const float bv = wave_max(fmaxf(fmaxf(fmaxf(p[0], p[1]), fmaxf(p[2], p[3])), -1.0f));
        int bi = 0x7fffffff;
        if (bv > -1.0f) {                                 // uniform
            int cand = 0x7fffffff;
#pragma unroll
            for (int i = 3; i >= 0; i--)
                if (p[i] == bv) cand = lane + 64 * i;     // the lowest expert among equals
            bi = wave_min_int(cand);
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (lane + 64 * i == bi) p[i] = -2.0f;
        if (lane == 0) topk_ids[(int64_t)t * topk + j] = (uint32_t)bi;   // no finite probability left (NaN logits): an id no expert has
        if (lane == j) mysel = bv;
    }
    float sum = 0.0f;
    for (int j = 0; j < topk; j++) sum += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mysel), j));
    if (lane < topk) topk_weights[(int64_t)t * topk + lane] = renorm ? mysel / sum : mysel;
}

// (expert_ids, sorted_token_ids) = topk_ids.flatten().sort_last_dim(ascending) (fused_moe.rs:249-260) as a counting
// sort in one workgroup.  candle's sort is unstable (candle-core/src/sort.rs:282-297), so the order of the pairs
// inside an expert's segment is unspecified there too; here it depends on the order the LDS atomics are served in.
// Ids outside [0, n_experts) are larger than every valid id and end up behind them, unchanged.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const uint32_t *__restrict__ ids, int32_t *__restrict__ expert_ids,
                                                        int32_t *__restrict__ sorted_token_ids, int n_pairs, int n_experts) {
    extern __shared__ int cnt[];                 // [n_experts + 1] counts, then [n_experts + 1] running offsets
    int *off = cnt + n_experts + 1;
    const int tid = threadIdx.x;
    for (int e = tid; e <= n_experts; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += 1024) atomicAdd(&cnt[min(ids[p], (uint32_t)n_experts)], 1);
    __syncthreads();
    for (int e = tid; e <= n_experts; e += 1024) {
        int before = 0;
        for (int j = 0; j < e; j++) before += cnt[j];
        off[e] = before;
    }
    __syncthreads();
    for (int p = tid; p < n_pairs; p += 1024) {
        const uint32_t id = ids[p];
        const int pos = atomicAdd(&off[min(id, (uint32_t)n_experts)], 1);
        expert_ids[pos] = (int32_t)id;
        sorted_token_ids[pos] = p;
    }
}

// ys.reshape((tokens, topk, dim)).sum(-2) (fused_moe.rs:296): the topk rows of a token added in slot order
__global__ __launch_bounds__(256) void moe_sum_kernel(const float *__restrict__ y, float *__restrict__ out, int topk, int dim) {
    const int t = blockIdx.y;
    const int c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= dim) return;
    const float *src = y + (int64_t)t * topk * dim + c;
    f32x4 acc = *reinterpret_cast<const f32x4 *>(src);
    for (int j = 1; j < topk; j++) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(src + (int64_t)j * dim);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    *reinterpret_cast<f32x4 *>(out + (int64_t)t * dim + c) = acc;
}

inline bool misaligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

template <int HD>
int launch_attn(int G, dim3 grid, hipStream_t s, const float *q, int64_t q_stride, const float *kc, const float *vc, float *out, float *part,
                const int32_t *pos_dev, int pos0, int n_head, int ctx, float scale, int splits) {
#define CQ_ATT(GG)                                                                                                                   \
    case GG:                                                                                                                         \
        hipLaunchKernelGGL((attn_kernel<HD, GG>), grid, dim3(256), 0, s, q, q_stride, kc, vc, out, part, pos_dev, pos0, n_head, ctx, \
                           scale, splits);                                                                                           \
        break;
    switch (G) {
        CQ_ATT(1) CQ_ATT(2) CQ_ATT(4) CQ_ATT(8)
        default: return CQ_ERR_RANGE;
    }
#undef CQ_ATT
    return (int)hipGetLastError();
}

int launch_attn_mfma(int G, dim3 grid, hipStream_t s, const float *q, int64_t q_stride, const float *kc, const float *vc, float *out,
                     const int32_t *pos_dev, int pos0, int rows, int n_head, int ctx, float scale) {
#define CQ_ATT(GG)                                                                                                                \
    case GG:                                                                                                                      \
        hipLaunchKernelGGL((attn_mfma_kernel<GG>), grid, dim3(256), 0, s, q, q_stride, kc, vc, out, pos_dev, pos0, rows, n_head,  \
                           ctx, scale);                                                                                           \
        break;
    switch (G) {
        CQ_ATT(1) CQ_ATT(2) CQ_ATT(4) CQ_ATT(8)
        default: return CQ_ERR_RANGE;
    }
#undef CQ_ATT
    return (int)hipGetLastError();
}

// rows per workgroup of attn_rows_kernel for a grouping of G query heads per kv head (G * R <= 16 pairs)
inline int attn_rows_per_group(int G) { return G == 8 ? 2 : 4; }

template <int HD>
int launch_attn_rows(int G, dim3 grid, hipStream_t s, const float *q, int64_t q_stride, const float *kc, const float *vc, float *out,
                     float *part, const int32_t *pos_dev, int pos0, int rows, int n_head, int ctx, float scale, int splits) {
#define CQ_ATT(GG, RR)                                                                                                              \
    case GG:                                                                                                                        \
        hipLaunchKernelGGL((attn_rows_kernel<HD, GG, RR>), grid, dim3(256), 0, s, q, q_stride, kc, vc, out, part, pos_dev, pos0,    \
                           rows, n_head, ctx, scale, splits);                                                                       \
        break;
    switch (G) {
        CQ_ATT(1, 4) CQ_ATT(2, 4) CQ_ATT(4, 4) CQ_ATT(8, 2)
        default: return CQ_ERR_RANGE;
    }
#undef CQ_ATT
    return (int)hipGetLastError();
}

}  // namespace

extern "C" {

int cq_nn_embedding(const float *table_dev, const int32_t *ids_dev, float *out_dev, int64_t rows, int64_t dim, int64_t vocab,
                    float *sumsq_partials_dev, void *stream) {
    if (rows < 0 || dim <= 0 || vocab <= 0 || dim % 4) return CQ_ERR_SHAPE;
    if (sumsq_partials_dev && rows != 1) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    if (!table_dev || !ids_dev || !out_dev) return CQ_ERR_NULL;
    if (misaligned(table_dev, 16) || misaligned(out_dev, 16)) return CQ_ERR_ALIGN;
    if (rows > 0x7fffffffLL || dim > 0x7fffffffLL) return CQ_ERR_RANGE;
    hipLaunchKernelGGL(embedding_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, table_dev, ids_dev, out_dev, (int)dim, vocab,
                       sumsq_partials_dev);
    return (int)hipGetLastError();
}

int cq_nn_rms_norm(const float *x_dev, const float *delta_dev, const float *weight_dev, float *sum_out_dev, float *out_dev, int64_t rows,
                   int64_t dim, float eps, void *stream) {
    if (rows < 0 || dim <= 0 || dim % 4) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    if (!x_dev || !weight_dev || !out_dev) return CQ_ERR_NULL;
    if (misaligned(x_dev, 16) || misaligned(delta_dev, 16) || misaligned(weight_dev, 16) || misaligned(sum_out_dev, 16) || misaligned(out_dev, 16))
        return CQ_ERR_ALIGN;
    if (rows > 0x7fffffffLL || dim > (1 << 24)) return CQ_ERR_RANGE;
    hipLaunchKernelGGL(rms_norm_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, x_dev, delta_dev, weight_dev, sum_out_dev, out_dev,
                       (int)dim, eps);
    return (int)hipGetLastError();
}

int cq_nn_rope_i_kv(float *q_dev, const float *k_dev, const float *v_dev, float *k_cache_dev, float *v_cache_dev, const float *cos_dev,
                    const float *sin_dev, const int32_t *pos_dev, int64_t pos, int64_t rows, int64_t n_head, int64_t n_kv_head, int64_t head_dim,
                    int64_t ctx, int64_t q_stride, int64_t k_stride, int64_t v_stride, void *stream) {
    if (rows < 0 || n_head <= 0 || n_kv_head <= 0 || head_dim <= 0 || head_dim % 2 || ctx <= 0 || pos < 0) return CQ_ERR_SHAPE;
    if (q_stride < n_head * head_dim || k_stride < n_kv_head * head_dim || v_stride < n_kv_head * head_dim) return CQ_ERR_SHAPE;
    if (q_stride % 2 || k_stride % 2 || v_stride % 2) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    if (!q_dev || !k_dev || !v_dev || !k_cache_dev || !v_cache_dev || !cos_dev || !sin_dev) return CQ_ERR_NULL;
    if (misaligned(q_dev, 8) || misaligned(k_dev, 8) || misaligned(v_dev, 8) || misaligned(k_cache_dev, 8) || misaligned(v_cache_dev, 8))
        return CQ_ERR_ALIGN;
    if (!pos_dev && pos + rows > ctx) return CQ_ERR_RANGE;
    if (rows > 0x7fffffffLL || ctx > 0x7fffffffLL) return CQ_ERR_RANGE;
    hipLaunchKernelGGL(rope_kv_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, q_dev, k_dev, v_dev, k_cache_dev, v_cache_dev,
                       cos_dev, sin_dev, pos_dev, (int)pos, (int)n_head, (int)n_kv_head, (int)head_dim, (int)ctx, q_stride, k_stride, v_stride);
    return (int)hipGetLastError();
}

static int64_t attn_splits(int64_t max_kv_len) { return (max_kv_len + ATT_SPLIT - 1) / ATT_SPLIT; }

int64_t cq_nn_attention_workspace_bytes(int64_t rows, int64_t n_head, int64_t head_dim, int64_t max_kv_len) {
    if (rows < 0 || n_head <= 0 || head_dim <= 0 || max_kv_len <= 0) return -1;
    const int64_t splits = attn_splits(max_kv_len);
    return splits <= 1 ? 0 : rows * n_head * splits * (head_dim + 2) * 4;
}

int cq_nn_attention(const float *q_dev, int64_t q_stride, const float *k_cache_dev, const float *v_cache_dev, float *out_dev,
                    const int32_t *pos_dev, int64_t pos, int64_t rows, int64_t n_head, int64_t n_kv_head, int64_t head_dim, int64_t ctx,
                    int64_t max_kv_len, float scale, void *workspace_dev, int64_t workspace_bytes, void *stream) {
    if (rows < 0 || n_head <= 0 || n_kv_head <= 0 || n_head % n_kv_head || ctx <= 0 || pos < 0 || max_kv_len <= 0 || max_kv_len > ctx)
        return CQ_ERR_SHAPE;
    if (q_stride < n_head * head_dim) return CQ_ERR_SHAPE;
    if (head_dim != 64 && head_dim != 128) return CQ_ERR_RANGE;
    if (rows == 0) return CQ_OK;
    if (!q_dev || !k_cache_dev || !v_cache_dev || !out_dev) return CQ_ERR_NULL;
    if (misaligned(k_cache_dev, 16) || misaligned(v_cache_dev, 16)) return CQ_ERR_ALIGN;
    if (!pos_dev && pos + rows > max_kv_len) return CQ_ERR_RANGE;
    const int64_t splits = attn_splits(max_kv_len);
    const int64_t need = cq_nn_attention_workspace_bytes(rows, n_head, head_dim, max_kv_len);
    if (need > 0 && (!workspace_dev || workspace_bytes < need)) return CQ_ERR_WORKSPACE;
    if (rows > 65535 || splits > 65535 || ctx > 0x7fffffffLL) return CQ_ERR_RANGE;
    const int G = (int)(n_head / n_kv_head);
    dim3 grid((unsigned)n_kv_head, (unsigned)rows, (unsigned)splits);
    hipStream_t s = (hipStream_t)stream;
    int rc;
    if (rows >= CQ_ATTN_MFMA_MIN && head_dim == 128 && (G == 1 || G == 2 || G == 4 || G == 8)) {
        // prompts: 32 (row, head) pairs per workgroup on the f32 matrix cores, all splits in one pass (nothing to combine)
        const int R = 32 / G;
        return launch_attn_mfma(G, dim3((unsigned)n_kv_head, (unsigned)((rows + R - 1) / R)), s, q_dev, q_stride, k_cache_dev, v_cache_dev,
                                out_dev, pos_dev, (int)pos, (int)rows, (int)n_head, (int)ctx, scale);
    } else if (rows >= CQ_ATTN_ROWS_MIN && (G == 1 || G == 2 || G == 4 || G == 8)) {
        // prompts and wide batches: several query rows share each load of the keys and values
        const int R = attn_rows_per_group(G);
        grid.y = (unsigned)((rows + R - 1) / R);
        rc = head_dim == 128 ? launch_attn_rows<128>(G, grid, s, q_dev, q_stride, k_cache_dev, v_cache_dev, out_dev, (float *)workspace_dev,
                                                     pos_dev, (int)pos, (int)rows, (int)n_head, (int)ctx, scale, (int)splits)
                             : launch_attn_rows<64>(G, grid, s, q_dev, q_stride, k_cache_dev, v_cache_dev, out_dev, (float *)workspace_dev,
                                                    pos_dev, (int)pos, (int)rows, (int)n_head, (int)ctx, scale, (int)splits);
    } else {
        rc = head_dim == 128 ? launch_attn<128>(G, grid, s, q_dev, q_stride, k_cache_dev, v_cache_dev, out_dev, (float *)workspace_dev, pos_dev,
                                                (int)pos, (int)n_head, (int)ctx, scale, (int)splits)
                             : launch_attn<64>(G, grid, s, q_dev, q_stride, k_cache_dev, v_cache_dev, out_dev, (float *)workspace_dev, pos_dev,
                                               (int)pos, (int)n_head, (int)ctx, scale, (int)splits);
    }
    if (rc) return rc;
    if (splits > 1) {
        if (head_dim == 128)
            hipLaunchKernelGGL((attn_combine_kernel<128>), dim3((unsigned)(rows * n_head)), dim3(128), 0, s, (const float *)workspace_dev, out_dev,
                               (int)splits);
        else
            hipLaunchKernelGGL((attn_combine_kernel<64>), dim3((unsigned)(rows * n_head)), dim3(64), 0, s, (const float *)workspace_dev, out_dev,
                               (int)splits);
        return (int)hipGetLastError();
    }
    return CQ_OK;
}

int64_t cq_nn_attention_decode_workspace_bytes(int64_t n_head, int64_t head_dim, int64_t max_kv_len) {
    if (n_head <= 0 || head_dim <= 0 || max_kv_len <= 0) return -1;
    return ATTD_COUNTER_BYTES + n_head * attd_splits(max_kv_len) * (head_dim + 4) * 4;
}

int64_t cq_nn_attention_decode_splits(int64_t max_kv_len) {
    if (max_kv_len <= 0) return -1;
    const int64_t s = attd_splits(max_kv_len);
    return s <= ATTD_MAX_SPLITS ? s : -1;
}

int cq_nn_attention_decode(const float *q_dev, const float *k_new_dev, const float *v_new_dev, float *k_cache_dev, float *v_cache_dev,
                           const float *cos_dev, const float *sin_dev, float *out_dev, const int32_t *pos_dev, int64_t pos, int64_t n_head,
                           int64_t n_kv_head, int64_t head_dim, int64_t ctx, int64_t max_kv_len, float scale, void *partials_dev,
                           int64_t partials_bytes, const void *prefetch_dev, int64_t prefetch_bytes, int64_t prefetch_piece_bytes, void *stream) {
    if (n_head <= 0 || n_kv_head <= 0 || n_head % n_kv_head || ctx <= 0 || pos < 0 || max_kv_len <= 0 || max_kv_len > ctx) return CQ_ERR_SHAPE;
    if (prefetch_bytes < 0 || (prefetch_bytes > 0 && (!prefetch_dev || misaligned(prefetch_dev, 16)))) return CQ_ERR_ALIGN;
    if (prefetch_piece_bytes < 0 || prefetch_piece_bytes % 16 || prefetch_piece_bytes > 0x7fffffffLL) return CQ_ERR_ALIGN;
    if (head_dim != 64 && head_dim != 128) return CQ_ERR_RANGE;
    if (!q_dev || !k_new_dev || !v_new_dev || !k_cache_dev || !v_cache_dev || !cos_dev || !sin_dev || !partials_dev) return CQ_ERR_NULL;
    if (misaligned(q_dev, 16) || misaligned(k_new_dev, 16) || misaligned(v_new_dev, 16) || misaligned(k_cache_dev, 16) ||
        misaligned(v_cache_dev, 16) || misaligned(partials_dev, 16))
        return CQ_ERR_ALIGN;
    if (!pos_dev && pos + 1 > max_kv_len) return CQ_ERR_RANGE;
    if (partials_bytes < cq_nn_attention_decode_workspace_bytes(n_head, head_dim, max_kv_len)) return CQ_ERR_WORKSPACE;
    const int64_t splits = attd_splits(max_kv_len);
    if (splits > ATTD_MAX_SPLITS || ctx > 0x7fffffffLL || n_kv_head > ATTD_COUNTER_BYTES / 4) return CQ_ERR_RANGE;
    const bool fine = attd_split_keys(max_kv_len) == 64;
    // the counters lie in front of the records: their place does not move with max_kv_len, so one buffer serves every length
    int *counters = (int *)partials_dev;
    const int G = (int)(n_head / n_kv_head);
    float *part = (float *)((uint8_t *)partials_dev + ATTD_COUNTER_BYTES);
    // read-only workgroups for the prefetch range: enough, with the attention ones, for one per CU
    const int64_t pf_chunks = prefetch_bytes / 16;
    int64_t pf_rows = 0;
    if (pf_chunks > 0) {
        pf_rows = (256 - n_kv_head * splits + n_kv_head - 1) / n_kv_head;
        // ... and at least 160 of them (the splits beyond the position leave at once and make room): fewer would still be
        // reading when the attention itself has finished
        if (pf_rows < (160 + n_kv_head - 1) / n_kv_head) pf_rows = (160 + n_kv_head - 1) / n_kv_head;
    }
    dim3 grid((unsigned)n_kv_head, (unsigned)(splits + pf_rows));
    hipStream_t s = (hipStream_t)stream;
    // pieces go to the XCD of their consumer only where the grid's columns are the XCDs (workgroups are dealt to the 8 XCDs
    // round-robin by linear index); other head counts read the range linearly
    const int pf_piece16 = n_kv_head == 8 ? (int)(prefetch_piece_bytes / 16) : 0;
#define CQ_ATTD(HH, GG)                                                                                                                   \
    if (fine)                                                                                                                             \
        hipLaunchKernelGGL((attn_decode_kernel<HH, GG, 8, 64>), grid, dim3(64 * 8), 0, s, pos_dev, q_dev, k_cache_dev, cos_dev, sin_dev, (int)pos, \
                           (int)splits, (int)ctx, scale, v_cache_dev, k_new_dev, v_new_dev, part, (const u32x4 *)prefetch_dev, pf_chunks,   \
                           (uint32_t *)nullptr, out_dev, counters, pf_piece16);                                                           \
    else                                                                                                                                  \
        hipLaunchKernelGGL((attn_decode_kernel<HH, GG, 16, 128>), grid, dim3(64 * 16), 0, s, pos_dev, q_dev, k_cache_dev, cos_dev, sin_dev,       \
                           (int)pos, (int)splits, (int)ctx, scale, v_cache_dev, k_new_dev, v_new_dev, part, (const u32x4 *)prefetch_dev,     \
                           pf_chunks, (uint32_t *)nullptr, out_dev, counters, pf_piece16)
    if (head_dim == 128) {
        switch (G) {
            case 1: CQ_ATTD(128, 1); break;
            case 2: CQ_ATTD(128, 2); break;
            case 4: CQ_ATTD(128, 4); break;
            case 8: CQ_ATTD(128, 8); break;
            default: return CQ_ERR_RANGE;
        }
    } else {
        switch (G) {
            case 1: CQ_ATTD(64, 1); break;
            case 2: CQ_ATTD(64, 2); break;
            case 4: CQ_ATTD(64, 4); break;
            case 8: CQ_ATTD(64, 8); break;
            default: return CQ_ERR_RANGE;
        }
    }
#undef CQ_ATTD
    return (int)hipGetLastError();
}

int cq_nn_silu_mul(const float *gate_dev, const float *up_dev, float *out_dev, int64_t rows, int64_t dim, int64_t gate_stride, int64_t up_stride,
                   void *stream) {
    if (rows < 0 || dim <= 0 || dim % 4 || gate_stride < dim || up_stride < dim || gate_stride % 4 || up_stride % 4) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    if (!gate_dev || !up_dev || !out_dev) return CQ_ERR_NULL;
    if (misaligned(gate_dev, 16) || misaligned(up_dev, 16) || misaligned(out_dev, 16)) return CQ_ERR_ALIGN;
    if (rows > 65535 || dim > 0x7fffffffLL) return CQ_ERR_RANGE;
    dim3 grid((unsigned)((dim / 4 + 255) / 256), (unsigned)rows);
    hipLaunchKernelGGL(silu_mul_kernel, grid, dim3(256), 0, (hipStream_t)stream, gate_dev, up_dev, out_dev, (int)dim, gate_stride, up_stride);
    return (int)hipGetLastError();
}

int cq_nn_argmax(const float *logits_dev, int64_t n, int32_t *token_out_dev, int32_t *history_dev, int32_t *counter_dev, int32_t *pos_dev,
                 void *workspace_dev, void *stream) {
    if (n <= 0) return CQ_ERR_SHAPE;
    if (!logits_dev || !token_out_dev) return CQ_ERR_NULL;
    if (n > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (workspace_dev && misaligned(workspace_dev, 4)) return CQ_ERR_ALIGN;
    if (workspace_dev && n >= 8192) {
        const int chunk = (int)((n + ARGMAX_PARTS - 1) / ARGMAX_PARTS);
        const int parts = (int)((n + chunk - 1) / chunk);
        float *pv = (float *)workspace_dev;
        int *pi = (int *)workspace_dev + ARGMAX_PARTS;
        hipLaunchKernelGGL(argmax_partial_kernel, dim3(parts), dim3(256), 0, (hipStream_t)stream, logits_dev, (int)n, chunk, pv, pi);
        hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (const float *)pv, (const int *)pi, parts,
                           token_out_dev, history_dev, counter_dev, pos_dev);
        return (int)hipGetLastError();
    }
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, logits_dev, (int)n, token_out_dev, history_dev, counter_dev,
                       pos_dev);
    return (int)hipGetLastError();
}

int cq_nn_argmax_embed(const float *logits_dev, int64_t n, int32_t *token_out_dev, int32_t *history_dev, int32_t *counter_dev, int32_t *pos_dev,
                       void *workspace_dev, const float *table_dev, float *out_dev, int64_t dim, int64_t vocab, float *sumsq_partials_dev,
                       void *stream) {
    if (n <= 0 || dim <= 0 || dim % 4 || vocab <= 0) return CQ_ERR_SHAPE;
    if (!logits_dev || !token_out_dev || !workspace_dev || !table_dev || !out_dev) return CQ_ERR_NULL;
    if (n > 0x7fffffffLL || dim > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (misaligned(workspace_dev, 4) || misaligned(table_dev, 16) || misaligned(out_dev, 16)) return CQ_ERR_ALIGN;
    const int chunk = (int)((n + ARGMAX_PARTS - 1) / ARGMAX_PARTS);
    const int parts = (int)((n + chunk - 1) / chunk);
    float *pv = (float *)workspace_dev;
    int *pi = (int *)workspace_dev + ARGMAX_PARTS;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(parts), dim3(256), 0, (hipStream_t)stream, logits_dev, (int)n, chunk, pv, pi);
    hipLaunchKernelGGL(argmax_final_embed_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, (const float *)pv, (const int *)pi, parts, token_out_dev,
                       history_dev, counter_dev, pos_dev, table_dev, out_dev, (int)dim, vocab, sumsq_partials_dev);
    return (int)hipGetLastError();
}

int cq_nn_moe_route(const float *x_dev, const float *router_w_dev, uint32_t *topk_ids_dev, float *topk_weights_dev, float *logits_dev,
                    int64_t tokens, int64_t hidden, int64_t num_experts, int64_t topk, int norm_topk_prob, void *stream) {
    if (tokens < 0 || hidden <= 0 || hidden % 4 || num_experts <= 0 || topk <= 0 || topk > num_experts) return CQ_ERR_SHAPE;
    if (num_experts > ROUTE_MAX_EXPERTS || topk > ROUTE_MAX_TOPK || tokens > 65535 || hidden > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (tokens == 0) return CQ_OK;
    if (!x_dev || !router_w_dev || !topk_ids_dev || !topk_weights_dev || !logits_dev) return CQ_ERR_NULL;
    if (misaligned(x_dev, 16) || misaligned(router_w_dev, 16) || misaligned(topk_ids_dev, 4) || misaligned(topk_weights_dev, 4) ||
        misaligned(logits_dev, 4))
        return CQ_ERR_ALIGN;
    if (tokens * num_experts <= 4096)
        hipLaunchKernelGGL((moe_logits_kernel<1, 8>), dim3((unsigned)((num_experts + 3) / 4), (unsigned)tokens), dim3(256), 0, (hipStream_t)stream, x_dev,
                           router_w_dev, logits_dev, (int)hidden, (int)num_experts, (int)tokens);
    else if (tokens * num_experts <= 16384)
        hipLaunchKernelGGL((moe_logits_kernel<4, 2>), dim3((unsigned)((num_experts + 15) / 16), (unsigned)tokens), dim3(256), 0, (hipStream_t)stream, x_dev,
                           router_w_dev, logits_dev, (int)hidden, (int)num_experts, (int)tokens);
    else
        hipLaunchKernelGGL((moe_logits_kernel<4, 2, 2>), dim3((unsigned)((num_experts + 15) / 16), (unsigned)((tokens + 1) / 2)), dim3(256), 0,
                           (hipStream_t)stream, x_dev, router_w_dev, logits_dev, (int)hidden, (int)num_experts, (int)tokens);
    if (num_experts <= 256)
        hipLaunchKernelGGL(moe_topk_wave_kernel, dim3((unsigned)tokens), dim3(64), 0, (hipStream_t)stream, (const float *)logits_dev, topk_ids_dev,
                           topk_weights_dev, (int)num_experts, (int)topk, norm_topk_prob);
    else
        hipLaunchKernelGGL(moe_topk_kernel, dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, (const float *)logits_dev, topk_ids_dev,
                           topk_weights_dev, (int)num_experts, (int)topk, norm_topk_prob);
    return (int)hipGetLastError();
}

int cq_nn_moe_sort(const uint32_t *topk_ids_dev, int32_t *expert_ids_dev, int32_t *sorted_token_ids_dev, int64_t n_pairs, int64_t num_experts,
                   void *stream) {
    if (n_pairs < 0 || num_experts <= 0) return CQ_ERR_SHAPE;
    if (num_experts > 8191 || n_pairs > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (n_pairs == 0) return CQ_OK;
    if (!topk_ids_dev || !expert_ids_dev || !sorted_token_ids_dev) return CQ_ERR_NULL;
    if (misaligned(topk_ids_dev, 4) || misaligned(expert_ids_dev, 4) || misaligned(sorted_token_ids_dev, 4)) return CQ_ERR_ALIGN;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 2 * (num_experts + 1) * sizeof(int), (hipStream_t)stream, topk_ids_dev, expert_ids_dev,
                       sorted_token_ids_dev, (int)n_pairs, (int)num_experts);
    return (int)hipGetLastError();
}

int cq_nn_moe_sum(const float *y_dev, float *out_dev, int64_t tokens, int64_t topk, int64_t dim, void *stream) {
    if (tokens < 0 || topk <= 0 || dim <= 0 || dim % 4) return CQ_ERR_SHAPE;
    if (tokens > 65535 || topk > 0x7fffffffLL || dim > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (tokens == 0) return CQ_OK;
    if (!y_dev || !out_dev) return CQ_ERR_NULL;
    if (misaligned(y_dev, 16) || misaligned(out_dev, 16)) return CQ_ERR_ALIGN;
    hipLaunchKernelGGL(moe_sum_kernel, dim3((unsigned)((dim / 4 + 255) / 256), (unsigned)tokens), dim3(256), 0, (hipStream_t)stream, y_dev, out_dev,
                       (int)topk, (int)dim);
    return (int)hipGetLastError();
}

}  // extern "C"
