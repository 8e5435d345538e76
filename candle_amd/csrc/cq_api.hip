// extern "C" boundary of the library: argument validation and dispatch to the kernel launchers.
// Declarations and the reference interfaces they replace are in include/candle_hip_quant.h.
#include "cq_device.h"
#include "cq_launch.h"
#include "../../include/candle_hip_nn.h"

#include <mutex>

// Workspace of cq_qmatmul_forward_static: device memory that belongs to the library's code object, so the entry point
// needs no allocation.  Each GPU the library runs on holds its own copy until the process ends.  In host code the
// name of the array is not a device address: every use goes through the per-device address that hipGetSymbolAddress
// returns (static_workspace below).
static __device__ __align__(256) uint8_t scratch[CQ_STATIC_WORKSPACE_BYTES];

namespace {

constexpr int STATIC_WS_MAX_DEVICES = 64;
std::mutex static_ws_mutex;
void *static_ws_ptr[STATIC_WS_MAX_DEVICES];   // per device, filled on the first call made with that device current

// device address of `scratch` on the current device; 0 = ok, else the hipError_t / CQ_ERR_RANGE
int static_workspace(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= STATIC_WS_MAX_DEVICES) return CQ_ERR_RANGE;
    std::lock_guard<std::mutex> g(static_ws_mutex);
    if (!static_ws_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        static_ws_ptr[dev] = p;
    }
    *out = static_ws_ptr[dev];
    return CQ_OK;
}

inline bool aligned(const void *p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// weight formats of the matmul-family entry points: every one has matvec and matrix-core kernels
inline bool matmul_weight_dtype(int dt) { return cq_has_mfma(dt); }

inline bool block_dtype(int dt) { return matmul_weight_dtype(dt) || dt == CQ_Q8K; }
// every GGUF block format can be stored and dequantized; the matmul-family and quantize entry points take fewer
inline bool storage_dtype(int dt) { return block_dtype(dt) || dt == CQ_Q8_1; }

inline bool float_dtype(int dt) { return dt == CQ_F32 || dt == CQ_F16 || dt == CQ_BF16; }

inline int64_t float_size(int dt) { return dt == CQ_F32 ? 4 : 2; }

// shared checks of the (w_dtype, k, n, rows) tuple of the matmul-family entry points
// expert formats of the MoE entry points: the reference's (Q2K ... Q6K, Q8_0: candle-core/src/quantized/cuda.rs:543-548,
// candle-nn/src/moe.rs:210-215) plus Q4_0
inline bool moe_weight_dtype(int dt) {
    return dt == CQ_Q8_0 || dt == CQ_Q2K || dt == CQ_Q3K || dt == CQ_Q4K || dt == CQ_Q5K || dt == CQ_Q6K || dt == CQ_Q4_0;
}

inline int check_mm_shape(int w_dtype, int64_t k, int64_t n, int64_t rows) {
    if (!matmul_weight_dtype(w_dtype)) return CQ_ERR_DTYPE;
    if (k <= 0 || n < 0 || rows < 0) return CQ_ERR_SHAPE;
    if (k % cq_block_size(w_dtype) != 0) return CQ_ERR_SHAPE;
    if (k > (1 << 24) || n > 0x7fffffffLL || rows > 0x7fffffffLL) return CQ_ERR_RANGE;
    return CQ_OK;
}

inline int check_weight_ptr(int w_dtype, const void *w) {
    if (!w) return CQ_ERR_NULL;
    if (!aligned(w, (w_dtype == CQ_Q4K || w_dtype == CQ_Q5K) ? 16 : 2)) return CQ_ERR_ALIGN;
    return CQ_OK;
}

}  // namespace

extern "C" {

const char *cq_status_string(int status) {
    switch (status) {
        case CQ_OK: return "ok";
        case CQ_ERR_DTYPE: return "dtype not supported by this entry point";
        case CQ_ERR_SHAPE: return "invalid shape (k must be a positive multiple of the block size, sizes must be non-negative)";
        case CQ_ERR_ALIGN: return "pointer alignment requirement not met";
        case CQ_ERR_NULL: return "required pointer is NULL";
        case CQ_ERR_WORKSPACE: return "workspace too small";
        case CQ_ERR_RANGE: return "size exceeds what this entry point supports";
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

int64_t cq_block_size(int dtype) {
    switch (dtype) {
        case CQ_F32: case CQ_F16: case CQ_BF16: return 1;
        case CQ_Q4_0: case CQ_Q4_1: case CQ_Q5_0: case CQ_Q5_1: case CQ_Q8_0: case CQ_Q8_1: return 32;
        case CQ_Q2K: case CQ_Q3K: case CQ_Q4K: case CQ_Q5K: case CQ_Q6K: case CQ_Q8K: return 256;
    }
    return 0;
}

int64_t cq_type_size(int dtype) {
    switch (dtype) {
        case CQ_F32: return 4;
        case CQ_F16: case CQ_BF16: return 2;
        case CQ_Q4_0: return 18;
        case CQ_Q4_1: return 20;
        case CQ_Q5_0: return 22;
        case CQ_Q5_1: return 24;
        case CQ_Q8_0: return 34;
        case CQ_Q8_1: return 36;
        case CQ_Q2K: return 84;
        case CQ_Q3K: return 110;
        case CQ_Q4K: return 144;
        case CQ_Q5K: return 176;
        case CQ_Q6K: return 210;
        case CQ_Q8K: return 292;
    }
    return 0;
}

int64_t cq_storage_bytes(int dtype, int64_t elem_count) {
    int64_t bs = cq_block_size(dtype);
    if (bs == 0 || elem_count < 0 || elem_count % bs != 0) return -1;
    return elem_count / bs * cq_type_size(dtype);
}

int cq_dequantize(int dtype, const void *blocks_dev, void *out_dev, int64_t elem_count, int out_dtype, void *stream) {
    if (!storage_dtype(dtype)) return CQ_ERR_DTYPE;
    if (out_dtype != CQ_F32 && out_dtype != CQ_F16) return CQ_ERR_DTYPE;
    if (elem_count < 0 || elem_count % cq_block_size(dtype) != 0) return CQ_ERR_SHAPE;
    if (elem_count == 0) return CQ_OK;
    if (!blocks_dev || !out_dev) return CQ_ERR_NULL;
    if (!aligned(blocks_dev, 2) || !aligned(out_dev, 16)) return CQ_ERR_ALIGN;
    return cq_dequantize_launch(dtype, blocks_dev, out_dev, elem_count, out_dtype, (hipStream_t)stream);
}

int cq_embedding(int dtype, const void *blocks_dev, const uint32_t *ids_dev, float *out_dev, int64_t n_ids, int64_t rows, int64_t hidden,
                 void *stream) {
    if (!storage_dtype(dtype)) return CQ_ERR_DTYPE;
    if (n_ids < 0 || rows <= 0 || hidden <= 0 || hidden % cq_block_size(dtype) != 0) return CQ_ERR_SHAPE;
    if (rows > 0x7fffffffLL || hidden > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (n_ids == 0) return CQ_OK;
    if (!blocks_dev || !ids_dev || !out_dev) return CQ_ERR_NULL;
    if (!aligned(blocks_dev, 2) || !aligned(ids_dev, 4) || !aligned(out_dev, 16)) return CQ_ERR_ALIGN;
    return cq_embedding_launch(dtype, blocks_dev, ids_dev, out_dev, n_ids, rows, hidden, (hipStream_t)stream);
}

int cq_quantize(int dtype, const float *x_dev, void *blocks_dev, int64_t elem_count, void *stream) {
    if (!storage_dtype(dtype)) return CQ_ERR_DTYPE;
    if (elem_count < 0 || elem_count % cq_block_size(dtype) != 0) return CQ_ERR_SHAPE;
    if (elem_count == 0) return CQ_OK;
    if (!x_dev || !blocks_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 4) || !aligned(blocks_dev, 2)) return CQ_ERR_ALIGN;
    return cq_quantize_launch(dtype, x_dev, blocks_dev, elem_count, (hipStream_t)stream);
}

int64_t cq_act_scratch_bytes(int w_dtype, int64_t k, int64_t rows) {
    if (!block_dtype(w_dtype) || k <= 0 || rows < 0 || k % cq_block_size(w_dtype) != 0) return -1;
    return cq_act_layout(w_dtype, k, rows).total;
}

int cq_quantize_act(int w_dtype, const void *x_dev, int x_dtype, void *scratch_dev, int64_t k, int64_t rows, void *stream) {
    if (!block_dtype(w_dtype) || !float_dtype(x_dtype)) return CQ_ERR_DTYPE;
    if (k <= 0 || rows < 0 || k % cq_block_size(w_dtype) != 0) return CQ_ERR_SHAPE;
    if (rows == 0) return CQ_OK;
    if (!x_dev || !scratch_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(scratch_dev, 256)) return CQ_ERR_ALIGN;
    return cq_quantize_act_launch(w_dtype, x_dev, x_dtype, scratch_dev, k, rows, (hipStream_t)stream);
}

int cq_matvec(int w_dtype, const void *w_dev, const void *act_scratch_dev, void *dst_dev, int dst_dtype,
              int64_t k, int64_t n, int64_t rows, int64_t stride_dst, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, rows);
    if (rc) return rc;
    if (!float_dtype(dst_dtype)) return CQ_ERR_DTYPE;
    if (rows > CQ_MATVEC_MAX_ROWS) return CQ_ERR_RANGE;
    if (stride_dst < n) return CQ_ERR_SHAPE;
    if (n == 0 || rows == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!act_scratch_dev || !dst_dev) return CQ_ERR_NULL;
    if (!aligned(act_scratch_dev, 256) || !aligned(dst_dev, float_size(dst_dtype))) return CQ_ERR_ALIGN;
    return cq_matvec_launch(w_dtype, w_dev, act_scratch_dev, dst_dev, dst_dtype, k, n, rows, stride_dst, (hipStream_t)stream);
}

int cq_matmul(int w_dtype, const void *w_dev, const void *act_scratch_dev, float *dst_dev,
              int64_t k, int64_t n, int64_t rows, int64_t stride_dst, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, rows);
    if (rc) return rc;
    if (stride_dst < n) return CQ_ERR_SHAPE;
    if (n == 0 || rows == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!act_scratch_dev || !dst_dev) return CQ_ERR_NULL;
    if (!aligned(act_scratch_dev, 256) || !aligned(dst_dev, 4)) return CQ_ERR_ALIGN;
    return cq_matmul_launch(w_dtype, w_dev, act_scratch_dev, dst_dev, k, n, rows, stride_dst, (hipStream_t)stream);
}

int64_t cq_qmatmul_workspace_bytes(int w_dtype, int64_t m, int64_t k, int64_t n) {
    if (check_mm_shape(w_dtype, k, n, m)) return -1;
    int64_t bytes = cq_act_layout(w_dtype, k, m).total;
    // the batched matvec lays the rows out as matrix operands, 16 row slots whatever the batch
    const int64_t batch_ws = cq_matvec_batch_workspace(w_dtype, k, m);
    if (batch_ws > bytes) bytes = batch_ws;
    const int64_t mid_ws = cq_matvec_batch_mid_workspace(w_dtype, k, m);
    if (mid_ws > bytes) bytes = mid_ws;
    // the MFMA path writes f32 and converts afterwards when the caller wants f16 / bf16; small grids split K into
    // partial planes that a second kernel adds up
    if (m > CQ_MATVEC_MAX_ROWS || cq_use_mfma(w_dtype, m, k)) {
        bytes += cq_align256(m * n * 4);
        const int sp = cq_qmm_splits(k, n, m);
        if (sp > 1) bytes += cq_align256((int64_t)sp * m * n * 4);
    }
    return bytes;
}

int cq_qmatmul_forward(int w_dtype, const void *w_dev, const void *x_dev, int x_dtype, void *dst_dev, int dst_dtype,
                       int64_t m, int64_t k, int64_t n, void *workspace_dev, int64_t workspace_bytes, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, m);
    if (rc) return rc;
    if (!float_dtype(x_dtype) || !float_dtype(dst_dtype)) return CQ_ERR_DTYPE;
    if (m == 0 || n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!x_dev || !dst_dev || !workspace_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(workspace_dev, 256) || !aligned(dst_dev, float_size(dst_dtype))) return CQ_ERR_ALIGN;
    if (workspace_bytes < cq_qmatmul_workspace_bytes(w_dtype, m, k, n)) return CQ_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    // decode: one kernel quantizes the activations into LDS and streams W (no scratch traffic)
    // (Q4_1, Q5_0, Q5_1, Q2K, Q3K have the fused instance for f32 activations only)
    if (m <= 2 && (cq_full_matvec(w_dtype) || x_dtype == CQ_F32))
        return cq_matvec_fused_launch(w_dtype, w_dev, x_dev, x_dtype, dst_dev, dst_dtype, k, n, m, n, s);
    // 3..16 rows of Q4_K: one small kernel quantizes the rows, then the weights are read once at streaming speed with the rows
    // as the second operand of the int8 matrix cores
    if (m >= 3 && cq_matvec_batch_takes(w_dtype, w_dev, k, n, m))
        return cq_matvec_batch_launch(w_dtype, w_dev, x_dev, x_dtype, workspace_dev, dst_dev, dst_dtype, k, n, m, n, s);
    // 17..64 rows of Q4_K (rows of up to 4096 elements): the same formulation, the rows in sets of 16
    if (m > 16 && cq_matvec_batch_mid_takes(w_dtype, w_dev, x_dev, x_dtype, dst_dtype, k, n, m))
        return cq_matvec_batch_mid_launch(w_dtype, w_dev, (const float *)x_dev, nullptr, k, 0, workspace_dev, (float *)dst_dev, k, n, m, s);
    // 3..8 rows: every workgroup re-quantizing all rows costs more than one small kernel that does it once
    if (m <= CQ_MATVEC_MAX_ROWS && !cq_use_mfma(w_dtype, m, k)) {
        if ((rc = cq_quantize_act_launch(w_dtype, x_dev, x_dtype, workspace_dev, k, m, s))) return rc;
        return cq_matvec_launch(w_dtype, w_dev, workspace_dev, dst_dev, dst_dtype, k, n, m, n, s);
    }
    if ((rc = cq_quantize_act_launch(w_dtype, x_dev, x_dtype, workspace_dev, k, m, s))) return rc;
    float *tmp = (float *)((uint8_t *)workspace_dev + cq_act_layout(w_dtype, k, m).total);
    float *split_ws = cq_qmm_splits(k, n, m) > 1 ? (float *)((uint8_t *)tmp + cq_align256(m * n * 4)) : nullptr;
    if (dst_dtype == CQ_F32)
        return cq_matmul_launch(w_dtype, w_dev, workspace_dev, (float *)dst_dev, k, n, m, n, s, split_ws);
    if ((rc = cq_matmul_launch(w_dtype, w_dev, workspace_dev, tmp, k, n, m, n, s, split_ws))) return rc;
    return cq_convert_f32_launch(tmp, dst_dev, dst_dtype, m * n, s);
}

int64_t cq_static_workspace_bytes(void) {
    // also looks the array's address up for the current device (when one can be used), so that a caller who asks for the
    // size before capturing a graph has the one-time lookup, which may load the code object, behind it
    void *ws = nullptr;
    (void)static_workspace(&ws);
    return CQ_STATIC_WORKSPACE_BYTES;
}

int cq_qmatmul_forward_static(int w_dtype, const void *w_dev, const void *x_dev, int x_dtype, void *dst_dev, int dst_dtype,
                              int64_t m, int64_t k, int64_t n, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, m);
    if (rc) return rc;
    // nothing is enqueued for a call that does not fit: the caller falls back to cq_qmatmul_forward with its own workspace
    if (cq_qmatmul_workspace_bytes(w_dtype, m, k, n) > CQ_STATIC_WORKSPACE_BYTES) return CQ_ERR_RANGE;
    void *ws = nullptr;
    if ((rc = static_workspace(&ws))) return rc;
    // every byte of the workspace that a kernel of this call reads has been written by an earlier kernel of the same
    // call (quantized activations, then K-split planes, then the f32 result awaiting conversion), so what the previous
    // call left there needs no clearing
    return cq_qmatmul_forward(w_dtype, w_dev, x_dev, x_dtype, dst_dev, dst_dtype, m, k, n, ws, CQ_STATIC_WORKSPACE_BYTES, stream);
}

int cq_nn_qmatmul_swiglu_rows(int w_dtype, const void *w_dev, const float *gate_dev, const float *up_dev, int64_t gate_stride, int64_t up_stride,
                              float *dst_dev, int64_t m, int64_t k, int64_t n, void *workspace_dev, int64_t workspace_bytes, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, m);
    if (rc) return rc;
    if (k % 256) return CQ_ERR_RANGE;
    if (gate_stride < k || up_stride < k || gate_stride % 4 || up_stride % 4) return CQ_ERR_SHAPE;
    if (m == 0 || n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!gate_dev || !up_dev || !dst_dev || !workspace_dev) return CQ_ERR_NULL;
    if (!aligned(gate_dev, 16) || !aligned(up_dev, 16) || !aligned(workspace_dev, 256) || !aligned(dst_dev, 4)) return CQ_ERR_ALIGN;
    if (workspace_bytes < cq_qmatmul_workspace_bytes(w_dtype, m, k, n)) return CQ_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    if (m >= 3 && cq_matvec_batch_takes(w_dtype, w_dev, k, n, m))          // the kernel cq_qmatmul_forward takes for these shapes
        return cq_matvec_batch_swiglu_launch(w_dtype, w_dev, gate_dev, up_dev, gate_stride, up_stride, workspace_dev, dst_dev, CQ_F32, k, n, m, n, s);
    if (m > 16 && cq_matvec_batch_mid_takes(w_dtype, w_dev, gate_dev, CQ_F32, CQ_F32, k, n, m))
        return cq_matvec_batch_mid_launch(w_dtype, w_dev, gate_dev, up_dev, gate_stride, up_stride, workspace_dev, dst_dev, k, n, m, s);
    if ((rc = cq_quantize_act_swiglu_launch(w_dtype, gate_dev, up_dev, gate_stride, up_stride, workspace_dev, k, m, s))) return rc;
    if (m <= CQ_MATVEC_MAX_ROWS && !cq_use_mfma(w_dtype, m, k)) return cq_matvec_launch(w_dtype, w_dev, workspace_dev, dst_dev, CQ_F32, k, n, m, n, s);
    float *tmp = (float *)((uint8_t *)workspace_dev + cq_act_layout(w_dtype, k, m).total);
    float *split_ws = cq_qmm_splits(k, n, m) > 1 ? (float *)((uint8_t *)tmp + cq_align256(m * n * 4)) : nullptr;
    return cq_matmul_launch(w_dtype, w_dev, workspace_dev, dst_dev, k, n, m, n, s, split_ws);
}

int64_t cq_indexed_moe_workspace_bytes(int w_dtype, int64_t num_experts, int64_t n, int64_t k, int64_t batch, int64_t topk,
                                       int64_t input_dim1) {
    if (!moe_weight_dtype(w_dtype) || check_mm_shape(w_dtype, k, n, batch) || num_experts <= 0 || topk <= 0) return -1;
    if (input_dim1 != 1 && input_dim1 != topk) return -1;
    return cq_moe_workspace_bytes_impl(w_dtype, num_experts, batch * topk, batch * input_dim1, k);
}

int cq_indexed_moe_forward(int w_dtype, const void *w_dev, const float *x_dev, const uint32_t *ids_dev, float *out_dev,
                           int64_t num_experts, int64_t n, int64_t k, int64_t batch, int64_t topk, int64_t input_dim1,
                           void *workspace_dev, int64_t workspace_bytes, void *stream) {
    int rc = moe_weight_dtype(w_dtype) ? check_mm_shape(w_dtype, k, n, batch) : (int)CQ_ERR_DTYPE;
    if (rc) return rc;
    if (num_experts <= 0 || topk <= 0) return CQ_ERR_SHAPE;
    if (input_dim1 != 1 && input_dim1 != topk) return CQ_ERR_SHAPE;
    if (num_experts > (1 << 20) || batch * topk > 0x7fffffffLL) return CQ_ERR_RANGE;
    if (batch == 0 || n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!x_dev || !ids_dev || !out_dev || !workspace_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(ids_dev, 4) || !aligned(out_dev, 4) || !aligned(workspace_dev, 256)) return CQ_ERR_ALIGN;
    if (workspace_bytes < cq_indexed_moe_workspace_bytes(w_dtype, num_experts, n, k, batch, topk, input_dim1)) return CQ_ERR_WORKSPACE;
    MoeArgs a;
    a.w_dtype = w_dtype; a.w = w_dev; a.x = x_dev; a.out = out_dev;
    a.num_experts = num_experts; a.n = n; a.k = k;
    a.n_pairs = batch * topk; a.x_rows = batch * input_dim1;
    a.mode = MOE_INDEXED; a.ids_u32 = ids_dev; a.topk = topk; a.input_dim1 = input_dim1;
    a.sorted_token_ids = nullptr; a.expert_ids = nullptr; a.topk_weights = nullptr;
    a.prefill = 0;
    return cq_moe_launch(a, workspace_dev, (hipStream_t)stream);
}

int64_t cq_moe_gemm_workspace_bytes(int w_dtype, int64_t num_experts, int64_t topk, int64_t size_m, int64_t n, int64_t k,
                                    int has_topk_weights) {
    if (!moe_weight_dtype(w_dtype) || check_mm_shape(w_dtype, k, n, size_m) || num_experts <= 0 || topk <= 0) return -1;
    if (!has_topk_weights && size_m % topk != 0) return -1;
    int64_t x_rows = has_topk_weights ? size_m : size_m / topk;
    return cq_moe_workspace_bytes_impl(w_dtype, num_experts, size_m, x_rows, k);
}

int cq_moe_gemm_gguf(int w_dtype, const float *x_dev, const void *w_dev, const int32_t *sorted_token_ids_dev,
                     const int32_t *expert_ids_dev, const float *topk_weights_dev, float *out_dev,
                     int64_t num_experts, int64_t topk, int64_t size_m, int64_t n, int64_t k, int is_prefill,
                     void *workspace_dev, int64_t workspace_bytes, void *stream) {
    int rc = moe_weight_dtype(w_dtype) ? check_mm_shape(w_dtype, k, n, size_m) : (int)CQ_ERR_DTYPE;
    if (rc) return rc;
    if (num_experts <= 0 || topk <= 0) return CQ_ERR_SHAPE;
    if (!topk_weights_dev && size_m % topk != 0) return CQ_ERR_SHAPE;
    if (num_experts > (1 << 20)) return CQ_ERR_RANGE;
    if (size_m == 0 || n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!x_dev || !sorted_token_ids_dev || !expert_ids_dev || !out_dev || !workspace_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(sorted_token_ids_dev, 4) || !aligned(expert_ids_dev, 4) || !aligned(out_dev, 4) ||
        !aligned(workspace_dev, 256) || (topk_weights_dev && !aligned(topk_weights_dev, 4)))
        return CQ_ERR_ALIGN;
    if (workspace_bytes < cq_moe_gemm_workspace_bytes(w_dtype, num_experts, topk, size_m, n, k, topk_weights_dev != nullptr))
        return CQ_ERR_WORKSPACE;
    MoeArgs a;
    a.w_dtype = w_dtype; a.w = w_dev; a.x = x_dev; a.out = out_dev;
    a.num_experts = num_experts; a.n = n; a.k = k;
    a.n_pairs = size_m; a.x_rows = topk_weights_dev ? size_m : size_m / topk;
    a.mode = MOE_SORTED; a.ids_u32 = nullptr; a.topk = topk; a.input_dim1 = 0;
    a.sorted_token_ids = sorted_token_ids_dev; a.expert_ids = expert_ids_dev; a.topk_weights = topk_weights_dev;
    a.prefill = is_prefill;
    return cq_moe_launch(a, workspace_dev, (hipStream_t)stream);
}

int cq_moe_gemm_gguf_pair(int w_dtype, const float *x_dev, const void *w_a_dev, const void *w_b_dev, const int32_t *sorted_token_ids_dev,
                          const int32_t *expert_ids_dev, float *out_a_dev, float *out_b_dev, int64_t num_experts, int64_t topk, int64_t size_m,
                          int64_t n, int64_t k, int is_prefill, void *workspace_dev, int64_t workspace_bytes, void *stream) {
    int rc = moe_weight_dtype(w_dtype) ? check_mm_shape(w_dtype, k, n, size_m) : (int)CQ_ERR_DTYPE;
    if (rc) return rc;
    if (num_experts <= 0 || topk <= 0 || size_m % topk != 0) return CQ_ERR_SHAPE;
    if (num_experts > (1 << 20)) return CQ_ERR_RANGE;
    if (size_m == 0 || n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_a_dev)) || (rc = check_weight_ptr(w_dtype, w_b_dev))) return rc;
    if (!x_dev || !sorted_token_ids_dev || !expert_ids_dev || !out_a_dev || !out_b_dev || !workspace_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(sorted_token_ids_dev, 4) || !aligned(expert_ids_dev, 4) || !aligned(out_a_dev, 4) ||
        !aligned(out_b_dev, 4) || !aligned(workspace_dev, 256))
        return CQ_ERR_ALIGN;
    if (workspace_bytes < cq_moe_gemm_workspace_bytes(w_dtype, num_experts, topk, size_m, n, k, 0)) return CQ_ERR_WORKSPACE;
    MoeArgs a;
    a.w_dtype = w_dtype; a.w = w_a_dev; a.x = x_dev; a.out = out_a_dev;
    a.w_b = w_b_dev; a.out_b = out_b_dev;
    a.num_experts = num_experts; a.n = n; a.k = k;
    a.n_pairs = size_m; a.x_rows = size_m / topk;
    a.mode = MOE_SORTED; a.ids_u32 = nullptr; a.topk = topk; a.input_dim1 = 0;
    a.sorted_token_ids = sorted_token_ids_dev; a.expert_ids = expert_ids_dev; a.topk_weights = nullptr;
    a.prefill = is_prefill;
    return cq_moe_launch(a, workspace_dev, (hipStream_t)stream);
}

int cq_moe_gemm_gguf_down_after_pair(int w_dtype, const float *gate_dev, const float *up_dev, const void *w_down_dev, const float *topk_weights_dev,
                                     float *out_dev, int64_t num_experts, int64_t topk, int64_t size_m, int64_t n, int64_t k, int64_t k_pair,
                                     void *workspace_dev, int64_t workspace_bytes, void *stream) {
    int rc = moe_weight_dtype(w_dtype) ? check_mm_shape(w_dtype, k, n, size_m) : (int)CQ_ERR_DTYPE;
    if (rc) return rc;
    if (num_experts <= 0 || topk <= 0 || size_m % topk != 0 || k_pair <= 0) return CQ_ERR_SHAPE;
    if (num_experts > (1 << 20)) return CQ_ERR_RANGE;
    if (size_m == 0 || n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_down_dev))) return rc;
    if (!gate_dev || !up_dev || !topk_weights_dev || !out_dev || !workspace_dev) return CQ_ERR_NULL;
    if (!aligned(gate_dev, 16) || !aligned(up_dev, 16) || !aligned(topk_weights_dev, 4) || !aligned(out_dev, 4) || !aligned(workspace_dev, 256))
        return CQ_ERR_ALIGN;
    // the workspace is the one the gate / up call was given: at least what that call asked for
    if (workspace_bytes < cq_moe_gemm_workspace_bytes(w_dtype, num_experts, topk, size_m, k, k_pair, 0)) return CQ_ERR_WORKSPACE;
    return cq_moe_down_after_pair_launch(w_dtype, w_down_dev, gate_dev, up_dev, topk_weights_dev, out_dev, num_experts, topk, size_m, n, k, k_pair,
                                         workspace_dev, (hipStream_t)stream);
}

int cq_moe_direct_pairs(int w_dtype, int64_t num_experts, int64_t size_m, int64_t k) {
    if (!moe_weight_dtype(w_dtype) || num_experts <= 0 || size_m < 0 || k <= 0) return 0;
    return cq_moe_direct(w_dtype, num_experts, size_m, k) ? 1 : 0;
}

int cq_moe_gemm_gguf_swiglu(int w_dtype, const float *x_dev, const void *w_gate_dev, const void *w_up_dev, const int32_t *sorted_token_ids_dev,
                            const int32_t *expert_ids_dev, float *out_dev, int64_t num_experts, int64_t topk, int64_t size_m, int64_t n,
                            int64_t k, void *stream) {
    int rc = moe_weight_dtype(w_dtype) ? check_mm_shape(w_dtype, k, n, size_m) : (int)CQ_ERR_DTYPE;
    if (rc) return rc;
    if (num_experts <= 0 || topk <= 0 || size_m % topk != 0) return CQ_ERR_SHAPE;
    if (num_experts > (1 << 20) || !cq_moe_direct(w_dtype, num_experts, size_m, k)) return CQ_ERR_RANGE;
    if (size_m == 0 || n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_gate_dev)) || (rc = check_weight_ptr(w_dtype, w_up_dev))) return rc;
    if (!x_dev || !sorted_token_ids_dev || !expert_ids_dev || !out_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(sorted_token_ids_dev, 4) || !aligned(expert_ids_dev, 4) || !aligned(out_dev, 4)) return CQ_ERR_ALIGN;
    PairSource ps;
    ps.mode = MOE_SORTED; ps.ids_u32 = nullptr; ps.sorted_token_ids = sorted_token_ids_dev; ps.expert_ids = expert_ids_dev;
    ps.topk_weights = nullptr; ps.topk = (int)topk; ps.input_dim1 = 0;
    ps.n_pairs = (int)size_m; ps.num_experts = (int)num_experts; ps.x_rows = (int)(size_m / topk);
    return cq_moe_pairs_swiglu_launch(w_dtype, w_gate_dev, w_up_dev, x_dev, out_dev, ps, k, n, (hipStream_t)stream);
}

// ---- single-row decoder fusions, declared in include/candle_hip_nn.h ----
int cq_nn_qmatmul_norm(int w_dtype, const void *w_dev, const float *x_dev, const float *sumsq_partials_dev, const float *norm_weight_dev,
                       float eps, float *dst_dev, int64_t k, int64_t n, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, 1);
    if (rc) return rc;
    if (n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!x_dev || !sumsq_partials_dev || !norm_weight_dev || !dst_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(norm_weight_dev, 16) || !aligned(sumsq_partials_dev, 4) || !aligned(dst_dev, 4)) return CQ_ERR_ALIGN;
    return cq_matvec_norm_launch(w_dtype, w_dev, x_dev, sumsq_partials_dev, norm_weight_dev, eps, dst_dev, k, n, (hipStream_t)stream);
}

int cq_nn_qmatmul_residual_merge(int w_dtype, const void *w_dev, const float *x_dev, const float *up_dev, float *residual_dev,
                                 float *sumsq_partials_out_dev, const float *planes_dev, int64_t n_planes, int64_t k, int64_t n, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, 1);
    if (rc) return rc;
    if (n_planes < 0 || n_planes > CQ_NN_MAX_PLANES) return CQ_ERR_RANGE;
    if (n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!x_dev || !residual_dev || !sumsq_partials_out_dev || (n_planes > 0 && !planes_dev)) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(up_dev, 16) || !aligned(residual_dev, 4) || !aligned(sumsq_partials_out_dev, 4) || !aligned(planes_dev, 4))
        return CQ_ERR_ALIGN;
    return cq_matvec_residual_launch(w_dtype, w_dev, x_dev, up_dev, residual_dev, sumsq_partials_out_dev, planes_dev, n_planes, k, n,
                                     (hipStream_t)stream);
}

int cq_nn_qmatmul_residual(int w_dtype, const void *w_dev, const float *x_dev, const float *up_dev, float *residual_dev,
                           float *sumsq_partials_out_dev, int64_t k, int64_t n, void *stream) {
    return cq_nn_qmatmul_residual_merge(w_dtype, w_dev, x_dev, up_dev, residual_dev, sumsq_partials_out_dev, nullptr, 0, k, n, stream);
}

int cq_nn_qmatmul_norm_swiglu(int w_dtype, const void *w1_dev, const void *w3_dev, const float *x_dev, const float *sumsq_partials_dev,
                              const float *norm_weight_dev, float eps, float *dst_dev, int64_t k, int64_t ffn, void *stream) {
    int rc = check_mm_shape(w_dtype, k, ffn, 1);
    if (rc) return rc;
    if (ffn == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w1_dev)) || (rc = check_weight_ptr(w_dtype, w3_dev))) return rc;
    if (!x_dev || !sumsq_partials_dev || !norm_weight_dev || !dst_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(norm_weight_dev, 16) || !aligned(sumsq_partials_dev, 4) || !aligned(dst_dev, 4)) return CQ_ERR_ALIGN;
    return cq_matvec_norm_swiglu_launch(w_dtype, w1_dev, w3_dev, x_dev, sumsq_partials_dev, norm_weight_dev, eps, dst_dev, k, ffn,
                                        (hipStream_t)stream);
}

int cq_nn_qmatmul_norm_pair(int w_dtype_a, const void *w_a_dev, int64_t n_a, float *dst_a_dev, int w_dtype_b, const void *w_b_dev, int64_t n_b,
                            float *dst_b_dev, const float *x_dev, const float *sumsq_partials_dev, const float *norm_weight_dev, float eps,
                            int64_t k, void *stream) {
    int rc = check_mm_shape(w_dtype_a, k, n_a, 1);
    if (rc || (rc = check_mm_shape(w_dtype_b, k, n_b, 1))) return rc;
    if ((rc = check_weight_ptr(w_dtype_a, w_a_dev)) || (rc = check_weight_ptr(w_dtype_b, w_b_dev))) return rc;
    if (!x_dev || !sumsq_partials_dev || !norm_weight_dev || !dst_a_dev || !dst_b_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(norm_weight_dev, 16) || !aligned(sumsq_partials_dev, 4) || !aligned(dst_a_dev, 4) || !aligned(dst_b_dev, 4))
        return CQ_ERR_ALIGN;
    return cq_matvec_norm_pair_launch(w_dtype_a, w_a_dev, n_a, dst_a_dev, w_dtype_b, w_b_dev, n_b, dst_b_dev, x_dev, sumsq_partials_dev,
                                      norm_weight_dev, eps, k, (hipStream_t)stream);
}

int64_t cq_nn_qmatmul_split_planes(int w_dtype, int64_t k) { return cq_matvec_ksplit_planes(w_dtype, k); }

int cq_nn_qmatmul_split(int w_dtype, const void *w_dev, const float *x_dev, const float *up_dev, float *planes_dev, int64_t k, int64_t n,
                        void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, 1);
    if (rc) return rc;
    if (cq_matvec_ksplit_planes(w_dtype, k) == 0) return CQ_ERR_RANGE;
    if (n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!x_dev || !planes_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || (up_dev && !aligned(up_dev, 16)) || !aligned(planes_dev, 16)) return CQ_ERR_ALIGN;
    return cq_matvec_ksplit_launch(w_dtype, w_dev, x_dev, up_dev, planes_dev, k, n, (hipStream_t)stream);
}

int cq_nn_qmatmul_norm_merge(int w_dtype, const void *w_dev, const float *x_dev, const float *planes_dev, int64_t n_planes,
                             const float *norm_weight_dev, float eps, float *dst_dev, int64_t k, int64_t n, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, 1);
    if (rc) return rc;
    if (n_planes < 1 || n_planes > CQ_NN_MAX_PLANES) return CQ_ERR_RANGE;
    if (n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!x_dev || !norm_weight_dev || !dst_dev || !planes_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(norm_weight_dev, 16) || !aligned(planes_dev, 16) || !aligned(dst_dev, 4)) return CQ_ERR_ALIGN;
    return cq_matvec_norm_merge_launch(w_dtype, w_dev, x_dev, planes_dev, n_planes, norm_weight_dev, eps, dst_dev, k, n, (hipStream_t)stream);
}

int cq_nn_qmatmul_norm_pair_merge(int w_dtype_a, const void *w_a_dev, int64_t n_a, float *dst_a_dev, int w_dtype_b, const void *w_b_dev,
                                  int64_t n_b, float *dst_b_dev, const float *x_dev, const float *planes_dev, int64_t n_planes,
                                  const float *norm_weight_dev, float eps, int64_t k, void *stream) {
    int rc = check_mm_shape(w_dtype_a, k, n_a, 1);
    if (rc || (rc = check_mm_shape(w_dtype_b, k, n_b, 1))) return rc;
    if (n_planes < 1 || n_planes > CQ_NN_MAX_PLANES) return CQ_ERR_RANGE;
    if ((rc = check_weight_ptr(w_dtype_a, w_a_dev)) || (rc = check_weight_ptr(w_dtype_b, w_b_dev))) return rc;
    if (!x_dev || !norm_weight_dev || !dst_a_dev || !dst_b_dev || !planes_dev) return CQ_ERR_NULL;
    if (!aligned(x_dev, 16) || !aligned(norm_weight_dev, 16) || !aligned(planes_dev, 16) || !aligned(dst_a_dev, 4) || !aligned(dst_b_dev, 4))
        return CQ_ERR_ALIGN;
    return cq_matvec_norm_pair_merge_launch(w_dtype_a, w_a_dev, n_a, dst_a_dev, w_dtype_b, w_b_dev, n_b, dst_b_dev, x_dev, planes_dev, n_planes,
                                            norm_weight_dev, eps, k, (hipStream_t)stream);
}

int cq_nn_qmatmul_residual_attn_merge(int w_dtype, const void *w_dev, const float *attn_partials_dev, int64_t splits, int64_t head_dim,
                                      float *residual_dev, float *sumsq_partials_out_dev, const float *planes_dev, int64_t n_planes, int64_t k,
                                      int64_t n, void *stream) {
    int rc = check_mm_shape(w_dtype, k, n, 1);
    if (rc) return rc;
    if (n_planes < 0 || n_planes > CQ_NN_MAX_PLANES) return CQ_ERR_RANGE;
    if (n == 0) return CQ_OK;
    if ((rc = check_weight_ptr(w_dtype, w_dev))) return rc;
    if (!attn_partials_dev || !residual_dev || !sumsq_partials_out_dev || (n_planes > 0 && !planes_dev)) return CQ_ERR_NULL;
    if (!aligned(attn_partials_dev, 16) || !aligned(residual_dev, 4) || !aligned(sumsq_partials_out_dev, 4) || !aligned(planes_dev, 4))
        return CQ_ERR_ALIGN;
    return cq_matvec_residual_attn_launch(w_dtype, w_dev, attn_partials_dev, splits, head_dim, residual_dev, sumsq_partials_out_dev, planes_dev,
                                          n_planes, k, n, (hipStream_t)stream);
}

int cq_nn_qmatmul_residual_attn(int w_dtype, const void *w_dev, const float *attn_partials_dev, int64_t splits, int64_t head_dim,
                                float *residual_dev, float *sumsq_partials_out_dev, int64_t k, int64_t n, void *stream) {
    return cq_nn_qmatmul_residual_attn_merge(w_dtype, w_dev, attn_partials_dev, splits, head_dim, residual_dev, sumsq_partials_out_dev, nullptr, 0,
                                             k, n, stream);
}

}  // extern "C"
