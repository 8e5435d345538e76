/*
 * candle_hip_nn.h — C ABI of the f32 decoder glue that sits between the quantized matmuls of candle's
 * quantized llama (candle-transformers/src/models/quantized_llama.rs:191-266, 568-596).
 *
 * Same library (libcandle_hip_quant.so) and same conventions as candle_hip_quant.h: device pointers,
 * caller-owned buffers, nothing allocated or synchronized, everything enqueued on `stream`
 * (a hipStream_t passed as void*), status codes from enum cq_status.
 *
 * Position and token arguments exist in two forms so that one decode step can be captured in a HIP
 * graph and replayed: `pos` is a host integer, `pos_dev` an optional device int32 that is ADDED to it
 * when not NULL; cq_nn_argmax can write the chosen token and advance the device position itself.
 */
#ifndef CANDLE_HIP_NN_H
#define CANDLE_HIP_NN_H

#include <stdint.h>

#include "candle_hip_quant.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Number of floats in a "sum of squares" partials buffer: a producer of a residual row leaves sum(row^2) as
 * this many partial sums (unused slots zero), the fused rms-norm consumer adds them in a fixed order. */
#define CQ_NN_PARTIALS 256

/* out[r, :] = table[ids[r], :] — candle_nn::Embedding::forward (candle-nn/src/embedding.rs), used as
 * tok_embeddings in quantized_llama.rs:577.  table [vocab, dim] f32, dim % 4 == 0, 16-byte aligned.
 * An id outside [0, vocab) yields a zero row (the reference returns an error from index_select).
 * sumsq_partials_dev (optional, rows == 1 only): receives sum(out[0, :]^2) as CQ_NN_PARTIALS partials. */
int cq_nn_embedding(const float *table_dev, const int32_t *ids_dev, float *out_dev, int64_t rows, int64_t dim, int64_t vocab,
                    float *sumsq_partials_dev, void *stream);

/* Residual add + RMS norm: s = x (+ delta when delta_dev != NULL); sum_out = s (when sum_out_dev != NULL,
 * may alias x_dev); out = s / sqrt(mean(s^2) + eps) * weight.
 * candle_nn::ops::rms_norm CPU kernel (candle-nn/src/ops.rs:499-510) preceded by the `(attn + residual)`
 * / `(x + residual)` adds of quantized_llama.rs:584-591.  rows x dim, dim % 4 == 0. */
int cq_nn_rms_norm(const float *x_dev, const float *delta_dev, const float *weight_dev, float *sum_out_dev, float *out_dev, int64_t rows,
                   int64_t dim, float eps, void *stream);

/* Interleaved rotary embedding of q (in place) and k, and KV-cache append:
 * candle_nn::rotary_emb::rope_i (candle-nn/src/rotary_emb.rs:52-70) as called from
 * LayerWeights::apply_rotary_emb (quantized_llama.rs:174-189), followed by the Tensor::cat of
 * quantized_llama.rs:222-233 done as a write into a preallocated cache.
 * Row r has absolute position p = pos + *pos_dev + r.  q [rows, n_head*head_dim] (row stride q_stride),
 * k, v [rows, n_kv_head*head_dim]; caches [n_kv_head, ctx, head_dim]; cos, sin [>= p_max+1, head_dim/2]. */
int cq_nn_rope_i_kv(float *q_dev, const float *k_dev, const float *v_dev, float *k_cache_dev, float *v_cache_dev, const float *cos_dev,
                    const float *sin_dev, const int32_t *pos_dev, int64_t pos, int64_t rows, int64_t n_head, int64_t n_kv_head, int64_t head_dim,
                    int64_t ctx, int64_t q_stride, int64_t k_stride, int64_t v_stride, void *stream);

/* Causal grouped-query attention of `rows` new queries over the cache (quantized_llama.rs:246-261:
 * repeat_kv, q k^T / sqrt(d), mask, softmax_last_dim, . v, transpose back to [rows, n_head*head_dim]).
 * Query row r attends keys [0, pos + *pos_dev + r].  max_kv_len bounds pos + *pos_dev + rows and fixes
 * the launch geometry (keys are processed in splits of 128; more than one split needs the workspace).
 * head_dim 64 or 128; n_head / n_kv_head in {1, 2, 4, 8}. */
int64_t cq_nn_attention_workspace_bytes(int64_t rows, int64_t n_head, int64_t head_dim, int64_t max_kv_len);
int cq_nn_attention(const float *q_dev, int64_t q_stride, const float *k_cache_dev, const float *v_cache_dev, float *out_dev,
                    const int32_t *pos_dev, int64_t pos, int64_t rows, int64_t n_head, int64_t n_kv_head, int64_t head_dim, int64_t ctx,
                    int64_t max_kv_len, float scale, void *workspace_dev, int64_t workspace_bytes, void *stream);

/* One decode step (a single new token at position p = pos + *pos_dev) of the three calls above:
 * rope_i on q and on the new k, append of the new k and v to the cache at p, attention of the rotated q over keys
 * [0, p].  q [n_head*head_dim], k_new / v_new [n_kv_head*head_dim] are the raw projection outputs (16-byte aligned;
 * q is not modified).  partials_dev is CQ_NN_ATTD_HEADER_BYTES of arrival counters followed by per-split records
 * { acc[head_dim], m, l, 0, 0 } for every head ([n_head][splits][head_dim + 4] floats, splits =
 * cq_nn_attention_decode_splits(max_kv_len): splits of 64 keys while 32 of them cover max_kv_len, i.e. up to 2048 keys, else
 * of 128 keys; at most 32, i.e. max_kv_len <= 4096, MAX_SEQ_LEN of quantized_llama.rs:27; -1 beyond).  When out_dev != NULL the
 * workgroup of each kv head that finishes last merges that head group's splits into out_dev [n_head*head_dim] (same
 * launch, same arithmetic as a separate merge), and only the splits that hold keys at position p take part: a launch laid
 * out for a long context costs what the existing keys cost, the result does not depend on max_kv_len (splits of one length),
 * and the records of the other splits are left untouched.  With out_dev == NULL every split writes its record (empty ones
 * included) and the merge is left to cq_nn_qmatmul_residual_attn (up to 16 splits), which takes the address of the records
 * (partials_dev + CQ_NN_ATTD_HEADER_BYTES).
 * The counters (one int per kv head, n_kv_head <= 64) must be zero before the first call with a buffer, and every call
 * leaves them zero; they sit in front of the records so that one buffer serves calls of any max_kv_len.
 * Key rows of the cache beyond p, up to the end of the last split of max_kv_len (never beyond ctx), are read before the
 * position is known and masked afterwards: whatever they hold, NaN included, does not reach the result.
 * prefetch_dev / prefetch_bytes (optional, 16-byte aligned): a byte range that extra read-only workgroups of this
 * otherwise latency-bound launch pull into the caches, e.g. the weights of the kernels that follow.  With
 * prefetch_piece_bytes > 0 (a multiple of 16; n_kv_head == 8) the range is taken as pieces of that size and piece p is read by
 * a workgroup on XCD p % 8: with the piece = cq_qmatmul_stream_step_bytes() of the weight that starts at prefetch_dev, every
 * piece lands in the L2 of the XCD whose workgroup will stream it (the L2s of the eight XCDs are separate, and what one holds
 * survives the kernel boundary).
 * No counterpart in the reference, which runs these as separate tensor ops (quantized_llama.rs:217-261). */
#define CQ_NN_ATTD_HEADER_BYTES 256
int64_t cq_nn_attention_decode_workspace_bytes(int64_t n_head, int64_t head_dim, int64_t max_kv_len);
int64_t cq_nn_attention_decode_splits(int64_t max_kv_len);
int cq_nn_attention_decode(const float *q_dev, const float *k_new_dev, const float *v_new_dev, float *k_cache_dev, float *v_cache_dev,
                           const float *cos_dev, const float *sin_dev, float *out_dev, const int32_t *pos_dev, int64_t pos, int64_t n_head,
                           int64_t n_kv_head, int64_t head_dim, int64_t ctx, int64_t max_kv_len, float scale, void *partials_dev,
                           int64_t partials_bytes, const void *prefetch_dev, int64_t prefetch_bytes, int64_t prefetch_piece_bytes, void *stream);

/* out = silu(gate) * up with silu(v) = v / (1 + exp(-v)): Mlp::forward, quantized_llama.rs:56-63
 * (candle_nn::ops::silu, candle-core/src/op.rs Silu::f32).  gate/up rows may be strided views of one buffer. */
int cq_nn_silu_mul(const float *gate_dev, const float *up_dev, float *out_dev, int64_t rows, int64_t dim, int64_t gate_stride, int64_t up_stride,
                   void *stream);

/* dst [m, n] = QMatMul::forward(silu(gate) * up) for m rows: Mlp::forward's feed_forward_w2 (quantized_llama.rs:56-63) with
 * the activation folded into the activation quantizer, so the f32 product [m, k] is never written.  Results are those of
 * cq_nn_silu_mul followed by cq_qmatmul_forward (same arithmetic; for m <= 2 that pair quantizes inside the matvec kernel
 * instead).  k % 256 == 0 (else CQ_ERR_RANGE: use the two calls); gate/up rows may be strided views of one buffer
 * (strides in floats, multiples of 4); workspace as cq_qmatmul_workspace_bytes(w_dtype, m, k, n). */
int cq_nn_qmatmul_swiglu_rows(int w_dtype, const void *w_dev, const float *gate_dev, const float *up_dev, int64_t gate_stride, int64_t up_stride,
                              float *dst_dev, int64_t m, int64_t k, int64_t n, void *workspace_dev, int64_t workspace_bytes, void *stream);

/* Single-row (decode) fusions of the glue into the quantized matvec kernel.  No counterpart in the reference,
 * which runs these as separate tensor ops; results equal the unfused sequence up to f32 summation order.
 *
 * cq_nn_qmatmul_norm:      dst[n] = QMatMul(w).forward(rms_norm(x, norm_weight, eps)) for one row x[k]
 *                          (quantized_llama.rs:581-582 / :588-589 / :593-596); sum(x^2) is read from sumsq_partials.
 * cq_nn_qmatmul_residual:  residual[n] += QMatMul(w).forward(up ? silu(x) * up : x) for one row x[k]
 *                          (attention_wo + residual add :264,:584, or Mlp :56-63 + residual add :590-591);
 *                          sumsq_partials_out receives sum(residual^2) of the updated row. */
int cq_nn_qmatmul_norm(int w_dtype, const void *w_dev, const float *x_dev, const float *sumsq_partials_dev, const float *norm_weight_dev,
                       float eps, float *dst_dev, int64_t k, int64_t n, void *stream);
int cq_nn_qmatmul_residual(int w_dtype, const void *w_dev, const float *x_dev, const float *up_dev, float *residual_dev,
                           float *sumsq_partials_out_dev, int64_t k, int64_t n, void *stream);
/* cq_nn_qmatmul_norm for feed_forward_w1 and feed_forward_w3 at once with the activation of Mlp::forward
 * (quantized_llama.rs:56-63) as epilogue: dst[ffn] = silu(W1 . xn) * (W3 . xn).  Both tensors [ffn, k] in the same
 * format.  CQ_ERR_RANGE when k is longer than one wave step per row (k > 4096 for K-quants, > 2048 for Q4_0 / Q8_0). */
int cq_nn_qmatmul_norm_swiglu(int w_dtype, const void *w1_dev, const void *w3_dev, const float *x_dev, const float *sumsq_partials_dev,
                              const float *norm_weight_dev, float eps, float *dst_dev, int64_t k, int64_t ffn, void *stream);
/* cq_nn_qmatmul_norm for two weight tensors of (possibly different) K-quant formats over the same row in one launch,
 * e.g. attention_wq|attention_wk (Q4_K) and attention_wv (Q6_K) of a Q4_K_M file.  CQ_ERR_DTYPE for other formats. */
int cq_nn_qmatmul_norm_pair(int w_dtype_a, const void *w_a_dev, int64_t n_a, float *dst_a_dev, int w_dtype_b, const void *w_b_dev, int64_t n_b,
                            float *dst_b_dev, const float *x_dev, const float *sumsq_partials_dev, const float *norm_weight_dev, float eps,
                            int64_t k, void *stream);
/* cq_nn_qmatmul_residual whose input row is the attention output still in the per-split partials of
 * cq_nn_attention_decode (out_dev == NULL there; attn_partials_dev = that call's partials_dev + CQ_NN_ATTD_HEADER_BYTES,
 * the first record): the merge of the splits is the matvec's prologue.
 * CQ_ERR_RANGE (use the merge kernel + cq_nn_qmatmul_residual instead) when k = n_head*head_dim is longer than one
 * wave step per row (k > 4096 for K-quants, > 2048 for Q4_0 / Q8_0), splits > 16, or head_dim is not a power of 2. */
int cq_nn_qmatmul_residual_attn(int w_dtype, const void *w_dev, const float *attn_partials_dev, int64_t splits, int64_t head_dim,
                                float *residual_dev, float *sumsq_partials_out_dev, int64_t k, int64_t n, void *stream);

/* A long-row matvec split along K, for feed_forward_w2 of a decode step (Mlp::forward, quantized_llama.rs:56-63, and the
 * residual add :590-591 it feeds).  Quantizing a 14336-element activation row in every workgroup costs more than
 * streaming the weights those workgroups read, so the row is cut into cq_nn_qmatmul_split_planes(w_dtype, k) equal
 * slices of whole blocks (the fewest, from 2 to CQ_NN_MAX_PLANES, of at most 4096 elements for K-quants and 2048 for
 * Q4_0 / Q8_0: 4 x 3584 for k = 14336 K-quants; 0 = not available for this k), each workgroup quantizes one slice
 * (bit-identical: Q8_K / Q8_0 blocks are independent), and
 *   planes[s][n] = W[:, slice s] . quantize((up ? silu(x) * up : x)[slice s]).
 * The residual row x[n] is not touched; until the planes are merged into it every reader adds them in the fixed order
 * ((x + planes[0]) + planes[1]) + ...:
 *   cq_nn_qmatmul_norm_merge / _norm_pair_merge   cq_nn_qmatmul_norm / _norm_pair over that sum (sum(x^2) computed
 *                                                 in the kernel; CQ_ERR_RANGE when k is longer than one wave step per row);
 *   cq_nn_qmatmul_residual_merge / _residual_attn_merge   cq_nn_qmatmul_residual / _residual_attn that first add the
 *                                                 planes to the residual row, so the row leaves merged (n_planes = 0:
 *                                                 the plain call). */
#define CQ_NN_MAX_PLANES 4
int64_t cq_nn_qmatmul_split_planes(int w_dtype, int64_t k);
int cq_nn_qmatmul_split(int w_dtype, const void *w_dev, const float *x_dev, const float *up_dev, float *planes_dev, int64_t k, int64_t n,
                        void *stream);
int cq_nn_qmatmul_norm_merge(int w_dtype, const void *w_dev, const float *x_dev, const float *planes_dev, int64_t n_planes,
                             const float *norm_weight_dev, float eps, float *dst_dev, int64_t k, int64_t n, void *stream);
int cq_nn_qmatmul_norm_pair_merge(int w_dtype_a, const void *w_a_dev, int64_t n_a, float *dst_a_dev, int w_dtype_b, const void *w_b_dev,
                                  int64_t n_b, float *dst_b_dev, const float *x_dev, const float *planes_dev, int64_t n_planes,
                                  const float *norm_weight_dev, float eps, int64_t k, void *stream);
int cq_nn_qmatmul_residual_merge(int w_dtype, const void *w_dev, const float *x_dev, const float *up_dev, float *residual_dev,
                                 float *sumsq_partials_out_dev, const float *planes_dev, int64_t n_planes, int64_t k, int64_t n, void *stream);
int cq_nn_qmatmul_residual_attn_merge(int w_dtype, const void *w_dev, const float *attn_partials_dev, int64_t splits, int64_t head_dim,
                                      float *residual_dev, float *sumsq_partials_out_dev, const float *planes_dev, int64_t n_planes, int64_t k,
                                      int64_t n, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Cooperative decode launches: several of the dependent single-row calls above as ONE launch of 256 workgroups whose phases
 * are separated by a barrier across the launch instead of a kernel boundary; a workgroup that waits has already requested
 * the first weight steps of the next phase, so the HBM keeps streaming across the hand-over.  Results are bit-identical to
 * the chain of calls they replace.  No counterpart in the reference (quantized_llama.rs:56-63, 191-266, 584-591 are tensor ops).
 *
 * sync_dev: cq_nn_coop_sync_bytes() bytes, 128-byte aligned, zero before the first use and owned by these calls afterwards
 * (counters that only grow).  Word CQ_NN_COOP_ERR_WORD is the error word: every wait inside the kernels is bounded (4 ms), and a
 * workgroup that gives up sets it, stops waiting and finishes; the step's results are then invalid.  A caller checks the word
 * when it next synchronizes (at the latest before it uses a sampled token), and after an error clears all of sync_dev and
 * repeats the step through the chain of calls.
 * The launch needs all of its workgroups resident at once: CQ_ERR_RANGE on a device with fewer than 256 compute units, and for
 * formats or shapes without a cooperative kernel (use the chain of calls).  Another process computing on the same GPU can make
 * the waits expire.
 *
 * cq_nn_decode_mlp   residual[hidden] += W2 . q(silu(W1 . xn) * (W3 . xn)), xn = q(rms_norm(residual) * norm_weight)
 *                    = cq_nn_qmatmul_norm_swiglu followed by cq_nn_qmatmul_residual (Mlp::forward and the add of :590-591).
 *                    sumsq_partials_dev: sum(residual^2) in, and of the updated row out; h_dev [ffn]: scratch for the activation.
 *                    W1 / W3 Q4_K, W2 Q4_K or Q6_K; hidden <= 4096.
 * ------------------------------------------------------------------------------------------- */
#define CQ_NN_COOP_ERR_WORD 1056
int64_t cq_nn_coop_sync_bytes(void);
int cq_nn_decode_mlp(int w13_dtype, const void *w1_dev, const void *w3_dev, int w2_dtype, const void *w2_dev, float *residual_dev,
                     float *sumsq_partials_dev, const float *norm_weight_dev, float eps, float *h_dev, int64_t hidden, int64_t ffn, void *sync_dev,
                     void *stream);

/* Greedy sampling (LogitsProcessor with Sampling::ArgMax, candle-examples/examples/quantized/main.rs:603-604):
 * token_out[0] = index of the largest logit (lowest index on ties).  Optional bookkeeping for graph replay:
 * history_dev[*counter_dev] = token; *counter_dev += 1; *pos_dev += 1.
 * workspace_dev (optional, CQ_NN_ARGMAX_WORKSPACE bytes): lets long rows be scanned by many workgroups. */
#define CQ_NN_ARGMAX_WORKSPACE 1024
int cq_nn_argmax(const float *logits_dev, int64_t n, int32_t *token_out_dev, int32_t *history_dev, int32_t *counter_dev, int32_t *pos_dev,
                 void *workspace_dev, void *stream);
/* cq_nn_argmax (workspace_dev required) followed, in its last kernel, by the embedding lookup of the chosen token
 * (cq_nn_embedding for one row: out_dev[0 .. dim) = table_dev[token, :], sumsq_partials_dev as there), so that a greedy
 * decode loop (main.rs:616-690) finds the next step's input row in place and the step starts with its first matmul. */
int cq_nn_argmax_embed(const float *logits_dev, int64_t n, int32_t *token_out_dev, int32_t *history_dev, int32_t *counter_dev, int32_t *pos_dev,
                       void *workspace_dev, const float *table_dev, float *out_dev, int64_t dim, int64_t vocab, float *sumsq_partials_dev,
                       void *stream);

/* ---------------------------------------------------------------------------------------------
 * Routing glue of FusedMoeGGUF::forward (candle-transformers/src/fused_moe.rs:222-301) around the three
 * cq_moe_gemm_gguf calls (candle_hip_quant.h):
 * cq_nn_moe_route  router_logits = x . router_w^T (bias-free f32 Linear :233), softmax over the experts (:235-236),
 *                  topk_ids = the topk largest probabilities in descending order (:238-241; equal values: lower
 *                  expert first, as candle's stable descending arg_sort leaves them, candle-core/src/sort.rs:48-53),
 *                  topk_weights = those probabilities, divided by their sum when norm_topk_prob (:243-247).
 *                  x [tokens, hidden], router_w [num_experts, hidden], topk_ids u32 / topk_weights f32 [tokens, topk];
 *                  logits_dev [tokens, num_experts] f32 receives the router logits (two launches: the dot products
 *                  spread over tokens x num_experts/16 workgroups — num_experts/4 for few tokens — then softmax + top-k
 *                  per token, in the registers of one wave when num_experts <= 256).
 *                  num_experts <= 1024, topk <= 64, tokens <= 65535 per call.
 * cq_nn_moe_sort   (expert_ids, sorted_token_ids) = topk_ids.flatten().sort_last_dim(ascending) (:249-260): n_pairs =
 *                  tokens * topk entries each.  The order of the pairs of one expert is unspecified, as it is with
 *                  candle's unstable sort (candle-core/src/sort.rs:282-297); nothing downstream depends on it.
 * cq_nn_moe_sum    out[t, :] = sum over the topk rows y[t * topk + j, :] in slot order (:296).
 * silu(gate) * up between the calls (:281) is cq_nn_silu_mul with rows = n_pairs.
 * ------------------------------------------------------------------------------------------- */
int cq_nn_moe_route(const float *x_dev, const float *router_w_dev, uint32_t *topk_ids_dev, float *topk_weights_dev, float *logits_dev,
                    int64_t tokens, int64_t hidden, int64_t num_experts, int64_t topk, int norm_topk_prob, void *stream);
int cq_nn_moe_sort(const uint32_t *topk_ids_dev, int32_t *expert_ids_dev, int32_t *sorted_token_ids_dev, int64_t n_pairs, int64_t num_experts,
                   void *stream);
int cq_nn_moe_sum(const float *y_dev, float *out_dev, int64_t tokens, int64_t topk, int64_t dim, void *stream);

#ifdef __cplusplus
}
#endif
#endif
