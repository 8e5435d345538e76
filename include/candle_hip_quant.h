/*
 * candle_hip_quant.h — C ABI of the MI355X (gfx950) GGUF quantized-matmul library.
 *
 * This is the boundary a `hip` backend of candle-core binds through FFI, in the same way
 * candle-core binds candle-kernels' statically linked launchers
 * (candle-kernels/src/ffi.rs:4-631, called from candle-core/src/quantized/fast_mmvq.rs:227-248 and
 * candle-nn/src/moe.rs:279-317).  Conventions:
 *
 *   - plain pointers and sizes only; every pointer named *_dev is a device pointer;
 *   - the caller owns every buffer; the library never allocates, frees or synchronizes;
 *     scratch/workspace sizes come from the matching *_bytes() query;
 *   - everything is enqueued on the caller's stream (`stream` is a hipStream_t passed as void*,
 *     NULL = the default stream), so calls can be captured into a HIP graph;
 *   - every entry point returns a status: 0 = ok, negative = argument error (CQ_ERR_*),
 *     positive = the hipError_t reported by the launch;
 *   - weights are GGUF blocks exactly as stored on disk, rows contiguous, `n` rows of `k/blk` blocks
 *     (candle-core/src/quantized/k_quants.rs:77-190); kernels read only [ptr, ptr + size) and never
 *     rely on the 512-element tail padding the CUDA backend adds
 *     (candle-core/src/quantized/cuda.rs:624-637,989-1008);
 *   - activation quantization follows candle's CPU path bit for bit (Q8_K blocks for K-quants,
 *     Q8_0 blocks for Q4_0/Q5_0/Q8_0, Q8_1 blocks for Q4_1/Q5_1: k_quants.rs:2320-2358, 658-687, 770-799), so
 *     results match QMatMul::forward on the CPU up to f32 summation order;
 *   - weight formats of the matmul-family entry points (cq_quantize_act, cq_matvec, cq_matmul, cq_qmatmul_forward): Q4_0, Q4_1,
 *     Q5_0, Q5_1, Q8_0, Q2K, Q3K, Q4K, Q5K, Q6K, each with a matvec kernel (up to eight activation rows) and a matrix-core
 *     kernel; the MoE entry points take Q4_0, Q8_0, Q2K, Q3K, Q4K, Q5K, Q6K.
 */
#ifndef CANDLE_HIP_QUANT_H
#define CANDLE_HIP_QUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF type codes: GgmlDType::{from_u32,to_u32}, candle-core/src/quantized/mod.rs:300-342 */
enum cq_dtype {
    CQ_F32 = 0, CQ_F16 = 1, CQ_Q4_0 = 2, CQ_Q4_1 = 3, CQ_Q5_0 = 6, CQ_Q5_1 = 7, CQ_Q8_0 = 8,
    CQ_Q8_1 = 9, CQ_Q2K = 10, CQ_Q3K = 11, CQ_Q4K = 12, CQ_Q5K = 13, CQ_Q6K = 14, CQ_Q8K = 15,
    CQ_BF16 = 30
};

enum cq_status {
    CQ_OK = 0,
    CQ_ERR_DTYPE = -1,      /* dtype not supported by this entry point */
    CQ_ERR_SHAPE = -2,      /* k not a multiple of the block size, negative sizes, ... */
    CQ_ERR_ALIGN = -3,      /* a pointer does not meet the stated alignment */
    CQ_ERR_NULL = -4,       /* a required pointer is NULL */
    CQ_ERR_WORKSPACE = -5,  /* workspace smaller than the *_bytes() query asks for */
    CQ_ERR_RANGE = -6       /* a size exceeds what the entry point supports */
};

/* Human-readable text for a status returned by any entry point. */
const char *cq_status_string(int status);

/* GgmlDType::block_size / type_size (mod.rs:386-421). 0 for an unknown dtype. */
int64_t cq_block_size(int dtype);
int64_t cq_type_size(int dtype);
/* Bytes of `elem_count` elements stored as `dtype` blocks (QCudaStorage::storage_size_in_bytes,
 * cuda.rs:880-882, without the tail padding). -1 if elem_count is not a multiple of the block size. */
int64_t cq_storage_bytes(int dtype, int64_t elem_count);

/* ---------------------------------------------------------------------------------------------
 * QTensor::dequantize / dequantize_f16 (mod.rs:689-710; CUDA: cuda.rs:105-223,
 * candle-kernels/src/quantized.cu:780-1156).  Bit-exact with GgmlType::to_float on the CPU; the
 * f16 result equals the f32 result rounded to nearest even.
 *   dtype: every block format of GgmlDType — Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2K, Q3K, Q4K, Q5K, Q6K, Q8K.
 *   out_dtype: CQ_F32 or CQ_F16.
 *   blocks_dev: 2-byte aligned.  out_dev: 16-byte aligned.
 * ------------------------------------------------------------------------------------------- */
int cq_dequantize(int dtype, const void *blocks_dev, void *out_dev, int64_t elem_count, int out_dtype, void *stream);

/* ---------------------------------------------------------------------------------------------
 * QTensor::embedding (mod.rs:712-748, CPU kernel :449-473): out [n_ids, hidden] f32, row r = row ids[r] of the
 * [rows, hidden] block matrix, dequantized (bit-exact with dequantize + index_select).  Every block format of
 * cq_dequantize; hidden a multiple of the block size.  An id >= rows gives a row of zeros where the CPU path returns
 * an error (a launch cannot); callers that need the error check the ids first.
 *   blocks_dev: 2-byte aligned.  ids_dev: u32.  out_dev: 16-byte aligned.
 * ------------------------------------------------------------------------------------------- */
int cq_embedding(int dtype, const void *blocks_dev, const uint32_t *ids_dev, float *out_dev, int64_t n_ids, int64_t rows, int64_t hidden,
                 void *stream);

/* ---------------------------------------------------------------------------------------------
 * QTensor::quantize on a device tensor (mod.rs:543-562).  The CUDA backend copies to the host,
 * runs GgmlType::from_float and copies back (cuda.rs:704-725); here the same arithmetic runs on the
 * GPU, one thread per block, and produces the same bytes as the CPU from_float.
 *   dtype: every block format of cq_dequantize.   x_dev: f32, 4-byte aligned.  blocks_dev: 2-byte aligned.
 * ------------------------------------------------------------------------------------------- */
int cq_quantize(int dtype, const float *x_dev, void *blocks_dev, int64_t elem_count, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Activation quantization, the first half of k_quants::matmul (k_quants.rs:2419-2428): each of
 * `rows` activation rows of length k is quantized to the weight type's VecDotType — Q8_K for
 * Q2K/Q3K/Q4K/Q5K/Q6K/Q8K, Q8_0 for Q4_0/Q5_0/Q8_0 and for Q4_1/Q5_1 (whose Q8_1 blocks have the qs and d of Q8_0;
 * their field s = f16(f16(sum) * d) is formed from the {d, sum} pair where it is used) — with the same results as
 * the CPU from_float.  Replaces the
 * q8_1 quantize launch of the CUDA backend (cuda.rs:48-103, fast_mmvq.rs:296-303).
 *
 * Scratch layout (device-private, 256-byte aligned sections, in this order):
 *   K-quants : int8 qs[rows][k] | float d[rows][k/256] | int16 bsums[rows][k/16]
 *   32-element formats: int8 qs[rows][k] | struct { float d (f16-rounded); int32 sum; } ds[rows][k/32]
 *   x_dtype: CQ_F32, CQ_F16 or CQ_BF16.  x_dev: 16-byte aligned, rows contiguous.  scratch_dev: 256-byte aligned.
 * ------------------------------------------------------------------------------------------- */
int64_t cq_act_scratch_bytes(int w_dtype, int64_t k, int64_t rows);
int cq_quantize_act(int w_dtype, const void *x_dev, int x_dtype, void *scratch_dev, int64_t k, int64_t rows, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Decode matvec over pre-quantized activations:  dst[r, j] = sum_k W[j, k] * x^[r, k]
 * for r < rows <= CQ_MATVEC_MAX_ROWS.  Counterpart of launch_mmvq_gguf_<t>_<dst>_plain
 * (candle-kernels/src/ffi.rs:58-631, mmvq_gguf.cu:915-1008).
 *   w_dev: n rows of k/blk blocks; 16-byte aligned for Q4K/Q5K, 2-byte aligned otherwise.
 *   act_scratch_dev: written by cq_quantize_act with the same (w_dtype, k, rows).
 *   dst_dev: f32 / f16 / bf16 (dst_dtype), row stride `stride_dst` elements (>= n).
 * ------------------------------------------------------------------------------------------- */
#define CQ_MATVEC_MAX_ROWS 8
int cq_matvec(int w_dtype, const void *w_dev, const void *act_scratch_dev, void *dst_dev, int dst_dtype,
              int64_t k, int64_t n, int64_t rows, int64_t stride_dst, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Prefill matmul over pre-quantized activations (any rows >= 1): more than CQ_MATVEC_MAX_ROWS rows (Q4K: from 6 rows) with k a
 * multiple of 256 run on the matrix cores, every format integer-exact: Q4K, Q4_0, Q8_0, Q4_1, Q5_0, Q5_1 on the int8 cores (the
 * 32-element formats as one int8 MFMA per block, whose int32 result is the block sum the CPU forms; their weights must be 8-byte
 * aligned), Q2K, Q3K, Q5K, Q6K on the f16 cores with operands that are exact small integers.  Other shapes take 8 rows per
 * matvec pass.
 * Counterpart of launch_mmq_gguf_<t> (candle-core/src/quantized/fast_mmq.rs:71-111, candle-kernels/src/mmq_gguf/).
 * Same buffers as cq_matvec; dst is f32.
 * ------------------------------------------------------------------------------------------- */
int cq_matmul(int w_dtype, const void *w_dev, const void *act_scratch_dev, float *dst_dev,
              int64_t k, int64_t n, int64_t rows, int64_t stride_dst, void *stream);

/* ---------------------------------------------------------------------------------------------
 * QCudaStorage::fwd (cuda.rs:846-878), the body of CustomOp1::cuda_fwd for QTensor
 * (mod.rs:1007-1017): quantize the m activation rows, then matvec (m <= CQ_MATVEC_MAX_ROWS; for m <= 2 the
 * quantization happens inside the matvec kernel; Q4K / Q5K with 3 <= m <= 16, k a multiple of 256 up to 16384 (Q5K: 14336) and 16-byte
 * aligned weights: one pass over the weights on the int8 matrix cores with the rows as register operands, up to 8 f32 rows of
 * up to 6144 elements quantized inside that kernel; Q4K / Q5K with 17 <= m <= 64 f32 rows of up to 4096 elements to an f32 dst: the
 * same with the rows in sets of 16, one pass over the weights per 32 rows) or MFMA matmul
 * (split over k with an ordered reduction when the grid would be small).  x is [m, k] contiguous (f32 / f16 / bf16), dst is [m, n] contiguous in dst_dtype
 * (CUDA keeps the input dtype: fast_mmvq.rs:161-323).  workspace_dev: 256-byte aligned,
 * at least cq_qmatmul_workspace_bytes(w_dtype, m, k, n) bytes.
 * ------------------------------------------------------------------------------------------- */
int64_t cq_qmatmul_workspace_bytes(int w_dtype, int64_t m, int64_t k, int64_t n);
/* Bytes of one wave step of the single-row decode kernel over a [n, k] weight of this format, or 0 when the shape does not take
 * the streaming kernel.  Workgroup b of that launch reads steps b, b + 256, ...; workgroups are dealt to the eight XCDs round-robin,
 * so step s is read through the L2 of XCD s % 8 (what cq_nn_attention_decode's prefetch_piece_bytes wants to know).
 * No counterpart in the reference. */
int64_t cq_qmatmul_stream_step_bytes(int w_dtype, int64_t k, int64_t n);
int cq_qmatmul_forward(int w_dtype, const void *w_dev, const void *x_dev, int x_dtype, void *dst_dev, int dst_dtype,
                       int64_t m, int64_t k, int64_t n, void *workspace_dev, int64_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------------------------------------
 * cq_qmatmul_forward without a workspace argument and without any allocation.  No counterpart in the reference (its
 * scratch is a grow-only buffer that the host allocates, fast_mmvq.rs:44-81): this entry point is for callers that
 * cannot allocate device memory — code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The workspace is a fixed array of CQ_STATIC_WORKSPACE_BYTES inside the library's device code (one copy per GPU, held
 * until the process ends; its address is looked up on the first call made with a device current, by this entry point or by
 * cq_static_workspace_bytes(): the lookup may load the library's code object, so make one of the two calls on every device
 * eagerly before the entry point is used under stream capture).  Results are those
 * of cq_qmatmul_forward bit for bit (same kernels).  A call whose cq_qmatmul_workspace_bytes() exceeds the array
 * returns CQ_ERR_RANGE and enqueues nothing.  All calls on one GPU share the array: calls that may overlap on one GPU
 * (different streams, different threads) race; serialize them or use cq_qmatmul_forward with separate workspaces.
 * ------------------------------------------------------------------------------------------- */
#define CQ_STATIC_WORKSPACE_BYTES (32ll << 20)
int64_t cq_static_workspace_bytes(void);
int cq_qmatmul_forward_static(int w_dtype, const void *w_dev, const void *x_dev, int x_dtype, void *dst_dev, int dst_dtype,
                              int64_t m, int64_t k, int64_t n, void *stream);

/* ---------------------------------------------------------------------------------------------
 * QTensor::indexed_moe_forward (mod.rs:758-784 -> cuda.rs:505-622 ->
 * candle-kernels/src/quantized.cu:4670-4845):
 *   w [num_experts, n, k] blocks, x [batch, input_dim1, k] f32 with input_dim1 == topk or 1,
 *   ids [batch, topk] u32  ->  out [batch, topk, n] f32,
 *   out[b, t, :] = W[ids[b, t]] . x[b, input_dim1 == 1 ? 0 : t, :].
 * Up to 256 pairs (512 for short rows, see cq_moe_direct_pairs) each pair is its own fused matvec; beyond, pairs are grouped by expert on the device and an expert's
 * rows are streamed once per 32 of its pairs as a batched matvec (Q4K / Q5K experts with rows of up to 4096 elements that see at
 * most 64 pairs each on average), once per tile of 32 or 128 pairs on the matrix cores (K-quant experts; integer-exact) or once per
 * 8 pairs by the matvec kernel (the other formats).  The reference takes Q2K-Q6K and Q8_0 experts (cuda.rs:543-548).
 * An id >= num_experts leaves its output row zero-filled.
 * ------------------------------------------------------------------------------------------- */
int64_t cq_indexed_moe_workspace_bytes(int w_dtype, int64_t num_experts, int64_t n, int64_t k, int64_t batch, int64_t topk, int64_t input_dim1);
int cq_indexed_moe_forward(int w_dtype, const void *w_dev, const float *x_dev, const uint32_t *ids_dev, float *out_dev,
                           int64_t num_experts, int64_t n, int64_t k, int64_t batch, int64_t topk, int64_t input_dim1,
                           void *workspace_dev, int64_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------------------------------------
 * candle_nn::moe::moe_gemm_gguf (candle-nn/src/moe.rs:169-337 -> ffi.rs:25-56 ->
 * candle-kernels/src/moe/moe_gguf.cu:149-216 and moe_wmma_gguf.cu:354-422):
 *   for m < size_m: tok = sorted_token_ids[m], e = expert_ids[m] (pairs with e outside
 *   [0, num_experts) are skipped); in_row = topk_weights ? tok : tok / topk;
 *   out[tok, :] = (topk_weights ? topk_weights[tok] : 1) * W[e] . x[in_row, :]
 *   x [size_m or size_m/topk, k] f32, out [size_m, n] f32, sorted_token_ids / expert_ids int32 [size_m]
 *   (both device pointers), topk_weights f32 [size_m] device pointer or NULL.
 * `is_prefill` does not change the result: the number of pairs selects the kernel (as for cq_indexed_moe_forward
 * above), and every path quantizes the activations like candle's CPU path.
 * ------------------------------------------------------------------------------------------- */
int64_t cq_moe_gemm_workspace_bytes(int w_dtype, int64_t num_experts, int64_t topk, int64_t size_m, int64_t n, int64_t k, int has_topk_weights);
int cq_moe_gemm_gguf(int w_dtype, const float *x_dev, const void *w_dev, const int32_t *sorted_token_ids_dev,
                     const int32_t *expert_ids_dev, const float *topk_weights_dev, float *out_dev,
                     int64_t num_experts, int64_t topk, int64_t size_m, int64_t n, int64_t k, int is_prefill,
                     void *workspace_dev, int64_t workspace_bytes, void *stream);

/* Two moe_gemm_gguf calls without topk_weights over the same x and the same pairs — the gate and up matmuls of
 * FusedMoeGGUF::forward (candle-transformers/src/fused_moe.rs:263-276) — as one call: out_a = x W_a^T, out_b = x W_b^T per
 * pair, results identical to two cq_moe_gemm_gguf calls.  With more than 256 pairs on K-quant experts the pairs are
 * grouped by expert and the activations quantized once for both (Q4_K / Q5_K experts that see at most 64 pairs each on average, rows
 * up to 4096 elements: both tensors in one launch, every expert a batched matvec over its own pairs); otherwise it is the two
 * calls.  w_a / w_b [num_experts, n, k] of one format; workspace as cq_moe_gemm_workspace_bytes(..., has_topk_weights = 0).
 * CQ_ERR_ALIGN when such experts are not 16-byte aligned (a later cq_moe_gemm_gguf_down_after_pair tells from the shape
 * alone how this call grouped its pairs). */
int cq_moe_gemm_gguf_pair(int w_dtype, const float *x_dev, const void *w_a_dev, const void *w_b_dev, const int32_t *sorted_token_ids_dev,
                          const int32_t *expert_ids_dev, float *out_a_dev, float *out_b_dev, int64_t num_experts, int64_t topk, int64_t size_m,
                          int64_t n, int64_t k, int is_prefill, void *workspace_dev, int64_t workspace_bytes, void *stream);

/* The gate and up matmuls of FusedMoeGGUF::forward with its activation (candle-transformers/src/fused_moe.rs:263-281: two
 * moe_gemm_gguf calls without topk_weights, then up * silu(gate)) in one launch, for decode-sized calls:
 *   out[tok, :] = silu(W_gate[e] . x[tok / topk, :]) * (W_up[e] . x[tok / topk, :])
 * w_gate / w_up [num_experts, n, k] of one format.  CQ_ERR_RANGE (use the two calls and cq_nn_silu_mul) when
 * cq_moe_direct_pairs() is 0 for the call or k is longer than one wave step per row (4096 for K-quants, 2048 for Q4_0 / Q8_0).
 * Needs no workspace. */
int cq_moe_gemm_gguf_swiglu(int w_dtype, const float *x_dev, const void *w_gate_dev, const void *w_up_dev, const int32_t *sorted_token_ids_dev,
                            const int32_t *expert_ids_dev, float *out_dev, int64_t num_experts, int64_t topk, int64_t size_m, int64_t n,
                            int64_t k, void *stream);

/* The down projection of an expert MLP (fused_moe.rs:281-294: silu(gate) * up, then moe_gemm_gguf with the routing weights)
 * right after cq_moe_gemm_gguf_pair on the SAME workspace, pair list and expert count, for calls that bucket their pairs by
 * expert (more pairs than cq_moe_direct_pairs takes; K-quant experts; k and k_pair multiples of 256): the grouping the pair
 * call left in the workspace is used again (no second grouping pass), and silu(gate) * up is evaluated inside the activation
 * quantizer (the f32 product is never written).  out[p, :] = topk_weights[p] * W_down[e_p] . quantize(silu(gate[p]) * up[p]) for
 * pair p; gate / up: [size_m, k] f32 as the pair call wrote them (k = its n), k_pair = the pair call's k.  Bit-identical to
 * cq_nn_silu_mul + cq_moe_gemm_gguf.  CQ_ERR_RANGE (nothing enqueued) when the pair call did not bucket its pairs for the
 * matrix-core kernels or this call's quantized rows do not fit in front of that call's tables: the caller then takes the two
 * separate calls.  Nothing else may use the workspace between the two calls.  No counterpart in the reference, which sorts the
 * pairs once on the host side (fused_moe.rs:249-260) and passes the sorted list to all three calls. */
int cq_moe_gemm_gguf_down_after_pair(int w_dtype, const float *gate_dev, const float *up_dev, const void *w_down_dev, const float *topk_weights_dev,
                                     float *out_dev, int64_t num_experts, int64_t topk, int64_t size_m, int64_t n, int64_t k, int64_t k_pair,
                                     void *workspace_dev, int64_t workspace_bytes, void *stream);

/* 1 when a MoE call of size_m pairs runs every pair as its own fused matvec (no grouping by expert, so the order of the
 * pairs does not matter and a caller may skip its sort): up to 256 pairs always, up to 512 for rows of at most 32 units
 * (k <= 2048 for K-quants, 1024 otherwise) while size_m <= 3 * num_experts.  No counterpart in the reference, which always
 * sorts (fused_moe.rs:249-260). */
int cq_moe_direct_pairs(int w_dtype, int64_t num_experts, int64_t size_m, int64_t k);

#ifdef __cplusplus
}
#endif
#endif /* CANDLE_HIP_QUANT_H */
