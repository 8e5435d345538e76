// Internal launcher interface between the extern "C" layer (cq_api.hip) and the kernel files.
// Every launcher enqueues on `s`, never synchronizes, and returns 0 or a hipError_t / CQ_ERR_* code.
#pragma once
#include "cq_device.h"

int cq_dequantize_launch(int dtype, const void *blocks, void *out, int64_t elems, int out_dtype, hipStream_t s);
int cq_quantize_launch(int dtype, const float *x, void *blocks, int64_t elems, hipStream_t s);
int cq_quantize_act_launch(int w_dtype, const void *x, int x_dtype, void *scratch, int64_t k, int64_t rows, hipStream_t s);
int cq_quantize_act_swiglu_launch(int w_dtype, const float *gate, const float *up, int64_t gate_stride, int64_t up_stride, void *scratch, int64_t k,
                                  int64_t rows, hipStream_t s);
int cq_matvec_launch(int w_dtype, const void *w, const void *scratch, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows,
                     int64_t stride_dst, hipStream_t s);
// same, over an already resolved (possibly row-offset) view of the activation scratch
int cq_matvec_launch_av(int w_dtype, const void *w, const ActView &av, void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows,
                        int64_t stride_dst, hipStream_t s);
// 3 .. 16 rows on the int8 matrix cores (quantized into `workspace` by a kernel of its own), the weights read once (cq_matvec_batch.hip); CQ_ERR_RANGE: not a call it takes
bool cq_matvec_batch_takes(int w_dtype, const void *w, int64_t k, int64_t n, int64_t rows);
int64_t cq_matvec_batch_workspace(int w_dtype, int64_t k, int64_t rows);
int cq_matvec_batch_launch(int w_dtype, const void *w, const void *x, int x_dtype, void *workspace, void *dst, int dst_dtype, int64_t k, int64_t n,
                           int64_t rows, int64_t stride_dst, hipStream_t s);
// the same over rows silu(gate[r]) * up[r] (f32, row strides in floats)
// 17 .. 64 f32 rows of Q4_K with rows of up to 16 super-blocks: the rows in sets of 16, two sets per pass over the weights
bool cq_matvec_batch_mid_takes(int w_dtype, const void *w, const void *x, int x_dtype, int dst_dtype, int64_t k, int64_t n, int64_t rows);
int64_t cq_matvec_batch_mid_workspace(int w_dtype, int64_t k, int64_t rows);
int cq_matvec_batch_mid_launch(int w_dtype, const void *w, const float *x, const float *up, int64_t x_stride, int64_t up_stride, void *workspace, float *dst,
                               int64_t k, int64_t n, int64_t rows, hipStream_t s);      // up != nullptr: rows silu(x[r]) * up[r]
int cq_matvec_batch_swiglu_launch(int w_dtype, const void *w, const float *gate, const float *up, int64_t gate_stride, int64_t up_stride, void *workspace,
                                  void *dst, int dst_dtype, int64_t k, int64_t n, int64_t rows, int64_t stride_dst, hipStream_t s);
// QMatMul::forward for <= CQ_MATVEC_MAX_ROWS rows with the activation quantization fused into the matvec kernel
int cq_matvec_fused_launch(int w_dtype, const void *w, const void *x, int x_dtype, void *dst, int dst_dtype, int64_t k, int64_t n,
                           int64_t rows, int64_t stride_dst, hipStream_t s);
// single-row decoder fusions (see the Fuse struct in cq_matvec.hip); partial-sum buffers hold 256 floats
int cq_matvec_norm_launch(int w_dtype, const void *w, const float *x, const float *partials, const float *norm_weight, float eps, float *dst,
                          int64_t k, int64_t n, hipStream_t s);
// planes / n_planes (optional, at most 4): K-slice planes of a split matvec still to be added to the residual row
int cq_matvec_residual_launch(int w_dtype, const void *w, const float *x, const float *up, float *residual, float *partials_out,
                              const float *planes, int64_t n_planes, int64_t k, int64_t n, hipStream_t s);
int cq_matvec_residual_attn_launch(int w_dtype, const void *w, const float *attn_partials, int64_t splits, int64_t head_dim, float *residual,
                                   float *partials_out, const float *planes, int64_t n_planes, int64_t k, int64_t n, hipStream_t s);
int cq_matvec_norm_swiglu_launch(int w_dtype, const void *w1, const void *w3, const float *x, const float *partials, const float *norm_weight,
                                 float eps, float *dst, int64_t k, int64_t ffn, hipStream_t s);
int cq_matvec_norm_pair_launch(int dta, const void *wa, int64_t na, float *dsta, int dtb, const void *wb, int64_t nb, float *dstb, const float *x,
                               const float *partials, const float *norm_weight, float eps, int64_t k, hipStream_t s);
// a long-row matvec split along K into planes, and the PRO_NORM consumers that add the planes back (see cq_matvec.hip)
int64_t cq_matvec_ksplit_planes(int w_dtype, int64_t k);
int cq_matvec_ksplit_launch(int w_dtype, const void *w, const float *x, const float *up, float *planes, int64_t k, int64_t n, hipStream_t s);
int cq_matvec_norm_merge_launch(int w_dtype, const void *w, const float *x, const float *planes, int64_t n_planes, const float *norm_weight,
                                float eps, float *dst, int64_t k, int64_t n, hipStream_t s);
int cq_matvec_norm_pair_merge_launch(int dta, const void *wa, int64_t na, float *dsta, int dtb, const void *wb, int64_t nb, float *dstb,
                                     const float *x, const float *planes, int64_t n_planes, const float *norm_weight, float eps, int64_t k,
                                     hipStream_t s);
// split_ws: optional workspace of cq_qmm_splits(k, n, rows) * rows * n floats for split-K partial planes (NULL: no split)
int cq_matmul_launch(int w_dtype, const void *w, const void *scratch, float *dst, int64_t k, int64_t n, int64_t rows,
                     int64_t stride_dst, hipStream_t s, float *split_ws = nullptr);
int cq_qmm_splits(int64_t k, int64_t n, int64_t rows);
bool cq_use_mfma(int w_dtype, int64_t rows, int64_t k);
int cq_embedding_launch(int dtype, const void *blocks, const uint32_t *ids, float *out, int64_t n_ids, int64_t rows, int64_t hidden, hipStream_t s);
int cq_convert_f32_launch(const float *src, void *dst, int dst_dtype, int64_t count, hipStream_t s);

// ---- MoE: both public entry points reduce to "pairs" (expert, activation row, output row, scale) ----
enum { MOE_INDEXED = 0, MOE_SORTED = 1 };
struct MoeArgs {
    int w_dtype;
    const void *w;           // [num_experts, n, k] blocks
    const float *x;          // [x_rows, k]
    float *out;              // [n_pairs, n]
    int64_t num_experts, n, k, n_pairs, x_rows;
    int mode;
    // MOE_INDEXED (QTensor::indexed_moe_forward): pair p = b * topk + t
    const uint32_t *ids_u32;
    int64_t topk, input_dim1;
    // MOE_SORTED (candle_nn::moe::moe_gemm_gguf): pair m of the router-sorted list
    const int32_t *sorted_token_ids, *expert_ids;
    const float *topk_weights;
    int prefill;
    // optional second grouped matmul over the same x and pairs (gate and up of an expert MLP): out_b = x W_b^T
    const void *w_b = nullptr;
    float *out_b = nullptr;
};
int64_t cq_moe_workspace_bytes_impl(int w_dtype, int64_t num_experts, int64_t n_pairs, int64_t x_rows, int64_t k);
int cq_moe_launch(const MoeArgs &a, void *workspace, hipStream_t s);
// The down projection of an expert MLP right after a grouped gate / up call (cq_moe_launch with w_b, more pairs than the per-pair
// kernels take) on the same workspace and pair list: out[pair] = topk_weights[pair] * W_down[e] . quantize(silu(gate[pair]) * up[pair]),
// with the grouping that call left in the workspace.  CQ_ERR_RANGE when that call did not group on the matrix-core path or the
// quantized rows of this one do not fit in front of its tables.
int cq_moe_down_after_pair_launch(int w_dtype, const void *w_down, const float *gate, const float *up, const float *topk_weights, float *out,
                                  int64_t num_experts, int64_t topk, int64_t n_pairs, int64_t n, int64_t k, int64_t k_pair, void *workspace,
                                  hipStream_t s);

// One (expert, activation row, output row, scale) pair of either MoE entry point.
struct PairSource {
    int mode;
    const uint32_t *ids_u32;
    const int32_t *sorted_token_ids, *expert_ids;
    const float *topk_weights;
    int topk, input_dim1;
    int n_pairs, num_experts, x_rows;
};

__device__ __forceinline__ bool pair_decode(const PairSource &ps, int p, int &e, int &in_row, int &out_row, float &scale) {
    if (ps.mode == MOE_INDEXED) {
        uint32_t id = ps.ids_u32[p];
        e = (int)id;
        in_row = ps.input_dim1 == 1 ? p / ps.topk : p;
        out_row = p;
        scale = 1.0f;
        return id < (uint32_t)ps.num_experts;
    }
    e = ps.expert_ids[p];
    int tok = ps.sorted_token_ids[p];
    out_row = tok;
    if (ps.topk_weights) {
        in_row = tok;
        // a token id outside the table would read past topk_weights; such pairs are dropped below
        scale = (tok >= 0 && tok < ps.n_pairs) ? ps.topk_weights[tok] : 0.0f;
    } else {
        in_row = tok / ps.topk;
        scale = 1.0f;
    }
    return e >= 0 && e < ps.num_experts && tok >= 0 && tok < ps.n_pairs && in_row < ps.x_rows;
}

// One workgroup: histogram of experts, exclusive scan, scatter of the pair descriptors.

// Pairs up to which cq_moe_launch runs every pair as its own fused matvec instead of grouping by expert: 256 for every
// shape; up to 512 when the rows are short enough for the several-rows-per-wave-step kernel (at most 32 units) and an expert
// is hit by three pairs at most on average.  Measured on 128 experts of 768 x 2048 / 2048 x 768, top-8: 256 pairs 99 us per
// layer of three matmuls, about 3 us per further 8 pairs; the grouped MFMA path 154-163 us for 264-512 pairs.
#define CQ_MOE_DIRECT_MAX_PAIRS 256
inline bool cq_moe_direct(int w_dtype, int64_t num_experts, int64_t n_pairs, int64_t k) {
    if (n_pairs <= CQ_MOE_DIRECT_MAX_PAIRS) return true;
    const int64_t unit = cq_is_kquant(w_dtype) ? 64 : 32;
    return k / unit <= 32 && n_pairs <= 512 && n_pairs <= 3 * num_experts;
}
// CQ_ERR_RANGE when the shape is not served by the fused kernel (the caller then takes the grouped path).
int cq_moe_pairs_launch(int w_dtype, const void *w, const float *x, float *out, const PairSource &ps, int64_t k, int64_t n, hipStream_t s);
int cq_moe_pairs_swiglu_launch(int w_dtype, const void *w_gate, const void *w_up, const float *x, float *out, const PairSource &ps, int64_t k,
                               int64_t n, hipStream_t s);

int cq_quantize_act_gather_launch(int w_dtype, const float *x, const int *row_map, void *scratch, int64_t k, int64_t rows, int64_t rows_alloc,
                                  hipStream_t s);
int cq_quantize_act_swiglu_gather_launch(int w_dtype, const float *gate, const float *up, const int *row_map, const int *n_valid, const float *scale_in,
                                         float *scale_out, void *scratch, int64_t k, int64_t rows, int64_t rows_alloc, hipStream_t s);
// Expert-grouped MoE, 8 pairs per weight pass.  Chunk c (c < *n_chunks) covers sorted pairs [first[c], first[c] + count[c]) of expert[c];
// the activation scratch holds the quantized rows in sorted-pair order (layout of rows_alloc rows).
#define CQ_MOE_CHUNK 8
struct MoeChunks {
    const int *n_chunks, *expert, *first, *count;
    const int *pair_out;
    const float *pair_scale;
    int max_chunks;
};
int cq_moe_chunks_launch(int w_dtype, const void *w, const void *scratch, int64_t rows_alloc, float *out, const MoeChunks &mc, int64_t k,
                         int64_t n, hipStream_t s);

// Q4_K experts hit by a few dozen pairs each as batched matvecs (cq_matvec_batch.hip): the expert-sorted pairs of an expert are the
// batch rows, in sets of 16 whose quantized rows sit in operand tiles.
bool cq_moe_stream_shape(int w_dtype, int64_t num_experts, int64_t n_pairs, int64_t k, int64_t n);      // ... by shape alone
bool cq_moe_stream_takes(int w_dtype, const void *w, const void *w_b, int64_t num_experts, int64_t n_pairs, int64_t k, int64_t n);
int64_t cq_moe_stream_operand_bytes(int64_t num_experts, int64_t n_pairs, int64_t k);
#define CQ_MOE_STREAM_CHUNK 16
int cq_moe_stream_quantize_launch(const float *x, const float *up, const int *row_map, const float *scale_in, float *scale_out, const int *chunks,
                                  int64_t max_chunks, int64_t num_experts, int64_t n_pairs, const int *offsets, void *op, int64_t k, hipStream_t s);
// extra: n | counter of launch 0 | counter of launch 1 | (expert, pass)[n]: the passes beyond the first of the experts with more than
// 32 pairs, written (counters zero) by the grouping pass; launch_slot: which counter this launch counts with
#define CQ_MOE_EXTRA_HEADER 3
int cq_moe_stream_launch(int w_dtype, const void *w_a, const void *w_b, float *out_a, float *out_b, const void *op, const int *offsets, const int *pair_out,
                         const float *pair_scale, int *extra, int launch_slot, int64_t num_experts, int64_t k, int64_t n, hipStream_t s);

// Pairs from which a K-quant MoE call goes through the MFMA kernel (tiles of expert-sorted rows): everything the
// per-pair kernels do not take.  Measured on 128 experts of 768 x 2048: 264-1016 pairs take 211-229 us per layer on
// 32-row tiles against 427-644 us on the 8-pairs-per-pass matvec.
#define CQ_MOE_MFMA_MIN_PAIRS 257
// rows of one MFMA tile of an expert: the small tile while experts average fewer than 40 rows (two small tiles cost
// more than one large one)
#define CQ_MOE_TILE_SMALL 32
#define CQ_MOE_TILE_LARGE 128
int cq_matmul_moe_launch(int w_dtype, const void *w, const void *scratch, int64_t rows_alloc, float *out, const MoeChunks &mc, int64_t k, int64_t n,
                         int tile_rows, hipStream_t s);
