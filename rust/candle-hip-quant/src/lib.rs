//! `QHipStorage`: GGUF blocks in the HBM of an MI355X and the quantized-matmul path over them, with the method set of
//! candle-core's `QCudaStorage` (candle-core/src/quantized/cuda.rs:586-1008; the minimal surface is
//! candle-core/src/quantized/dummy_cuda.rs:10-105), so that `QStorage` can carry a `Hip` variant whose arms forward
//! one to one.  Every method is one or two calls into the C ABI of `ffi`; the library never allocates, so output
//! buffers and the workspace come from `hip::HipDevice`.
//!
//! Results follow candle's CPU `QMatMul::forward` (activations quantized to Q8_K / Q8_0 / Q8_1 like
//! candle-core/src/quantized/k_quants.rs does), not the q8_1 arithmetic of the CUDA kernels.
pub mod ffi;
pub mod hip;

use candle_core::quantized::{GgmlDType, GgmlType};
use candle_core::{CpuStorage, DType, Layout, Result, Shape};
use core::ffi::{c_int, c_void};
use hip::{HipDevice, HipSlice, HipStorage, HipStorageSlice};

/// GGUF type code of a block format (`GgmlDType::to_u32`, candle-core/src/quantized/mod.rs:323-342): the `dtype`
/// argument of every entry point.
fn code(dtype: GgmlDType) -> c_int {
    (match dtype {
        GgmlDType::F32 => 0,
        GgmlDType::F16 => 1,
        GgmlDType::Q4_0 => 2,
        GgmlDType::Q4_1 => 3,
        GgmlDType::Q5_0 => 6,
        GgmlDType::Q5_1 => 7,
        GgmlDType::Q8_0 => 8,
        GgmlDType::Q8_1 => 9,
        GgmlDType::Q2K => 10,
        GgmlDType::Q3K => 11,
        GgmlDType::Q4K => 12,
        GgmlDType::Q5K => 13,
        GgmlDType::Q6K => 14,
        GgmlDType::Q8K => 15,
        GgmlDType::BF16 => 30,
    }) as c_int
}

/// Status of an entry point: 0 = ok, negative = argument error (`CQ_ERR_*`), positive = the `hipError_t` of the launch.
fn check(what: &str, status: c_int) -> Result<()> {
    if status == 0 {
        return Ok(());
    }
    let s = unsafe { std::ffi::CStr::from_ptr(ffi::cq_status_string(status)) };
    candle_core::bail!("{what}: {} (status {status})", s.to_string_lossy())
}

fn is_block_format(dtype: GgmlDType) -> bool {
    !matches!(dtype, GgmlDType::F32 | GgmlDType::F16 | GgmlDType::BF16)
}

pub struct QHipStorage {
    data: HipSlice<u8>,
    // bytes of blocks; no tail padding (the kernels read [ptr, ptr + len) only, unlike cuda.rs:624-637)
    len: usize,
    dtype: GgmlDType,
    device: HipDevice,
}

impl QHipStorage {
    /// cuda.rs:624-637.
    pub fn zeros(device: &HipDevice, el_count: usize, dtype: GgmlDType) -> Result<Self> {
        let len = el_count.div_ceil(dtype.block_size()) * dtype.type_size();
        Ok(Self { data: device.alloc_zeros::<u8>(len)?, len, dtype, device: device.clone() })
    }

    pub fn dtype(&self) -> GgmlDType {
        self.dtype
    }

    pub fn device(&self) -> &HipDevice {
        &self.device
    }

    pub fn storage_size_in_bytes(&self) -> usize {
        self.len
    }

    /// cuda.rs:887-889.
    pub fn device_ptr(&self) -> Result<*const u8> {
        Ok(self.data.device_ptr() as *const u8)
    }

    /// cuda.rs:880-885: device -> host copy of the block bytes.
    pub fn data(&self) -> Result<Vec<u8>> {
        self.device.memcpy_dtov(&self.data, self.len)
    }

    fn dequantize_to(&self, elem_count: usize, out_dtype: DType) -> Result<HipStorage> {
        if elem_count.div_ceil(self.dtype.block_size()) * self.dtype.type_size() > self.len {
            candle_core::bail!("dequantize: {elem_count} elements exceed the storage of {} bytes", self.len)
        }
        if !is_block_format(self.dtype) {
            candle_core::bail!("dequantize: {:?} storage holds plain values, not blocks", self.dtype)
        }
        let mut out = unsafe { HipStorage::alloc_float(&self.device, out_dtype, elem_count)? };
        let out_code = if out_dtype == DType::F16 { 1 } else { 0 };
        check("cq_dequantize", unsafe {
            ffi::cq_dequantize(code(self.dtype), self.data.device_ptr(), out.float_ptr_mut(), elem_count as i64, out_code, self.device.stream())
        })?;
        Ok(out)
    }

    /// cuda.rs:647-698: `GgmlType::to_float` of every block, on the GPU, bit for bit.
    pub fn dequantize(&self, elem_count: usize) -> Result<HipStorage> {
        self.dequantize_to(elem_count, DType::F32)
    }

    /// cuda.rs:700-702.
    pub fn dequantize_f16(&self, elem_count: usize) -> Result<HipStorage> {
        self.dequantize_to(elem_count, DType::F16)
    }

    /// cuda.rs:704-725 copies to the host and quantizes there; here `GgmlType::from_float` runs on the GPU and writes the
    /// same bytes.
    pub fn quantize(&mut self, src: &HipStorage) -> Result<()> {
        let src = match &src.slice {
            HipStorageSlice::F32(data) => data,
            _ => candle_core::bail!("only f32 can be quantized"),
        };
        if src.len() % self.dtype.block_size() != 0 {
            candle_core::bail!("quantize: {} elements are not a whole number of {:?} blocks", src.len(), self.dtype)
        }
        let len = src.len() / self.dtype.block_size() * self.dtype.type_size();
        if len != self.len {
            self.data = unsafe { self.device.alloc::<u8>(len)? };
            self.len = len;
        }
        check("cq_quantize", unsafe {
            ffi::cq_quantize(code(self.dtype), src.device_ptr() as *const f32, self.data.device_ptr_mut(), src.len() as i64, self.device.stream())
        })
    }

    /// cuda.rs:784-806: the source is on the host; it is uploaded and quantized on the GPU.
    pub fn quantize_onto(&mut self, src: &CpuStorage) -> Result<()> {
        let host = src.as_slice::<f32>()?;
        let dev = self.device.memcpy_stod(host)?;
        let dev = HipStorage { slice: HipStorageSlice::F32(dev), device: self.device.clone() };
        self.quantize(&dev)
    }

    /// cuda.rs:727-753.  Importance-weighted quantization has no GPU kernel: like the reference it runs candle's CPU
    /// quantizer and uploads the blocks.
    pub fn quantize_imatrix(&mut self, src: &HipStorage, imatrix_weights: &[f32], n_per_row: usize) -> Result<()> {
        let host = self.device.memcpy_dtov(src.as_f32()?, src.as_f32()?.len())?;
        self.quantize_imatrix_onto(&CpuStorage::F32(host), imatrix_weights, n_per_row)
    }

    /// cuda.rs:755-782.
    pub fn quantize_imatrix_onto(&mut self, src: &CpuStorage, imatrix_weights: &[f32], n_per_row: usize) -> Result<()> {
        let src_len = src.as_slice::<f32>()?.len();
        let mut cpu = candle_core::Device::Cpu.qzeros(src_len, self.dtype)?;
        cpu.quantize_imatrix(&candle_core::Storage::Cpu(src.clone()), imatrix_weights, n_per_row)?;
        let bytes = cpu.data()?;
        self.data = self.device.memcpy_stod(&bytes)?;
        self.len = bytes.len();
        Ok(())
    }

    /// cuda.rs:812-844: rows `ids` of a quantized [rows, hidden] table, dequantized to f32.
    pub fn embedding(&self, rows: usize, hidden: usize, ids: &HipStorage, ids_l: &Layout) -> Result<HipStorage> {
        if !ids_l.is_contiguous() {
            candle_core::bail!("quantized embedding requires contiguous ids")
        }
        if hidden % self.dtype.block_size() != 0 {
            candle_core::bail!("quantized embedding hidden size {hidden} is not divisible by block size {}", self.dtype.block_size())
        }
        let expected_size = rows * hidden * self.dtype.type_size() / self.dtype.block_size();
        if self.storage_size_in_bytes() != expected_size {
            candle_core::bail!("quantized tensor has {} bytes, expected {expected_size}", self.storage_size_in_bytes())
        }
        let ids_s = ids.as_u32()?;
        let n_ids = ids_l.shape().elem_count();
        let mut out = unsafe { self.device.alloc::<f32>(n_ids * hidden)? };
        check("cq_embedding", unsafe {
            ffi::cq_embedding(code(self.dtype), self.data.device_ptr(), ids_s.device_ptr_at(ids_l.start_offset()) as *const u32,
                              out.device_ptr_mut() as *mut f32, n_ids as i64, rows as i64, hidden as i64, self.device.stream())
        })?;
        Ok(HipStorage { slice: HipStorageSlice::F32(out), device: self.device.clone() })
    }

    /// `QMatMul::forward` on a quantized weight (cuda.rs:846-878; shape rules of candle-core/src/quantized/mod.rs:899-927):
    /// activations [.., k] of f32 / f16 / bf16 against the [n, k] weight, result [.., n] in the activations' type.  One
    /// call quantizes the activations the CPU way and runs the matvec (up to 8 rows) or matrix-core kernel.
    pub fn fwd(&self, self_shape: &Shape, storage: &HipStorage, layout: &Layout) -> Result<(HipStorage, Shape)> {
        if !layout.is_contiguous() {
            candle_core::bail!("input tensor is not contiguous {layout:?}")
        }
        let (n, k) = self_shape.dims2()?;
        let mut dst_dims = layout.shape().dims().to_vec();
        if dst_dims.len() < 2 {
            candle_core::bail!("input tensor has only one dimension {layout:?}")
        }
        let last_k = dst_dims.pop().unwrap();
        if last_k != k {
            candle_core::bail!("input tensor {layout:?} incompatible with {self_shape:?}")
        }
        let m: usize = dst_dims.iter().product();
        dst_dims.push(n);
        let (x_ptr, x_code) = storage.float_ptr_at(layout.start_offset())?;
        let need = unsafe { ffi::cq_qmatmul_workspace_bytes(code(self.dtype), m as i64, k as i64, n as i64) };
        if need < 0 {
            candle_core::bail!("no quantized matmul kernel for {:?} weights", self.dtype)
        }
        let mut out = unsafe { HipStorage::alloc_float(&self.device, storage.dtype(), m * n)? };
        // the guard is held until the launch is enqueued
        let ws = self.device.quant_workspace(need as usize)?;
        check("cq_qmatmul_forward", unsafe {
            ffi::cq_qmatmul_forward(code(self.dtype), self.data.device_ptr(), x_ptr, x_code, out.float_ptr_mut(), x_code,
                                    m as i64, k as i64, n as i64, ws.ptr(), need, self.device.stream())
        })?;
        drop(ws);
        Ok((out, dst_dims.into()))
    }

    /// cuda.rs:587-622: `self` [num_experts, n, k], `input` [batch, topk or 1, k] f32, `ids` [batch, topk] u32 ->
    /// [batch, topk, n] with `out[b, t] = W[ids[b, t]] . input[b, t or 0]`.
    pub fn indexed_moe_forward(&self, self_shape: &Shape, input: &HipStorage, input_l: &Layout, ids: &HipStorage, ids_l: &Layout)
                               -> Result<(HipStorage, Shape)> {
        if !matches!(self.dtype, GgmlDType::Q8_0 | GgmlDType::Q2K | GgmlDType::Q3K | GgmlDType::Q4K | GgmlDType::Q5K | GgmlDType::Q6K | GgmlDType::Q4_0) {
            candle_core::bail!("The given quantized dtype {:?} is not supported for indexed_moe_forward!", self.dtype)
        }
        if !input_l.is_contiguous() || !ids_l.is_contiguous() {
            candle_core::bail!("indexed_moe_forward requires contiguous input and ids")
        }
        let (e, n, k) = self_shape.dims3()?;
        let (batch, input_dim1, k1) = input_l.shape().dims3()?;
        let (batch1, topk) = ids_l.shape().dims2()?;
        assert!(batch == batch1, "batch dim not match!");
        if k1 != k {
            candle_core::bail!("input {:?} incompatible with {self_shape:?}", input_l.shape())
        }
        let x = input.as_f32()?;
        let ids = ids.as_u32()?;
        let need = unsafe {
            ffi::cq_indexed_moe_workspace_bytes(code(self.dtype), e as i64, n as i64, k as i64, batch as i64, topk as i64, input_dim1 as i64)
        };
        if need < 0 {
            candle_core::bail!("indexed_moe_forward: unsupported shape (input dim 1 must be topk or 1)")
        }
        let mut out = unsafe { self.device.alloc::<f32>(batch * topk * n)? };
        let ws = self.device.quant_workspace(need as usize)?;
        check("cq_indexed_moe_forward", unsafe {
            ffi::cq_indexed_moe_forward(code(self.dtype), self.data.device_ptr(), x.device_ptr_at(input_l.start_offset()) as *const f32,
                                        ids.device_ptr_at(ids_l.start_offset()) as *const u32, out.device_ptr_mut() as *mut f32,
                                        e as i64, n as i64, k as i64, batch as i64, topk as i64, input_dim1 as i64, ws.ptr(), need,
                                        self.device.stream())
        })?;
        drop(ws);
        Ok((HipStorage { slice: HipStorageSlice::F32(out), device: self.device.clone() }, (batch, topk, n).into()))
    }
}

/// cuda.rs:989-1008: upload raw blocks (what `QStorage::from_data` ends in for a GGUF tensor).
pub fn load_quantized<T: GgmlType + Send + Sync + 'static>(device: &HipDevice, data: &[T]) -> Result<QHipStorage> {
    let bytes = unsafe { std::slice::from_raw_parts(data.as_ptr() as *const u8, core::mem::size_of_val(data)) };
    let inner = device.memcpy_stod(bytes)?;
    Ok(QHipStorage { data: inner, len: bytes.len(), dtype: T::DTYPE, device: device.clone() })
}

/// `candle_nn::moe::moe_gemm_gguf` (candle-nn/src/moe.rs:169-337) on device buffers: expert-grouped quantized matmul
/// over router-sorted (token, expert) pairs.
///
/// * `input`: [size_m / topk, k] f32 when `topk_weights` is `None` (one row per token: gate / up), else [size_m, k] (one row
///   per pair: down);
/// * `weights`: [num_experts, n, k] blocks;  `sorted_token_ids`, `experts_ids`: `size_m` i32 each, the flattened expert
///   list sorted ascending and the matching pair permutation (candle-transformers/src/fused_moe.rs:249-260);
/// * returns [size_m, n] f32, row `sorted_token_ids[i]` = `W[experts_ids[i]] . x`, scaled by `topk_weights` when given.
///
/// The reference's `dtype` argument picks the activation type of its prefill kernel; here both paths quantize the f32
/// activations the CPU way, so there is none.
#[allow(clippy::too_many_arguments)]
pub fn moe_gemm_gguf(input: &HipSlice<f32>, input_rows: usize, weights: &QHipStorage, weights_shape: &Shape, topk_weights: Option<&HipSlice<f32>>,
                     sorted_token_ids: &HipSlice<u32>, experts_ids: &HipSlice<u32>, topk: usize, is_prefill: bool) -> Result<HipSlice<f32>> {
    let (num_experts, size_n, size_k) = weights_shape.dims3()?;
    let size_m = if topk_weights.is_none() { input_rows * topk } else { input_rows };
    if input.len() != input_rows * size_k {
        candle_core::bail!("input of {} elements and weight {weights_shape:?} last dim mismatch!", input.len())
    }
    if sorted_token_ids.len() < size_m || experts_ids.len() < size_m {
        candle_core::bail!("moe_gemm_gguf: {size_m} pairs but {} / {} ids", sorted_token_ids.len(), experts_ids.len())
    }
    let dev = weights.device();
    let wcode = code(weights.dtype());
    let need = unsafe {
        ffi::cq_moe_gemm_workspace_bytes(wcode, num_experts as i64, topk as i64, size_m as i64, size_n as i64, size_k as i64,
                                         topk_weights.is_some() as c_int)
    };
    if need < 0 {
        candle_core::bail!("moe_gemm_gguf: unsupported shape or expert format {:?}", weights.dtype())
    }
    let mut out = unsafe { dev.alloc::<f32>(size_m * size_n)? };
    let tw: *const f32 = topk_weights.map_or(std::ptr::null(), |t| t.device_ptr() as *const f32);
    let ws = dev.quant_workspace(need as usize)?;
    check("cq_moe_gemm_gguf", unsafe {
        ffi::cq_moe_gemm_gguf(wcode, input.device_ptr() as *const f32, weights.data.device_ptr(), sorted_token_ids.device_ptr() as *const i32,
                              experts_ids.device_ptr() as *const i32, tw, out.device_ptr_mut() as *mut f32, num_experts as i64,
                              topk as i64, size_m as i64, size_n as i64, size_k as i64, is_prefill as c_int, ws.ptr(), need, dev.stream())
    })?;
    drop(ws);
    Ok(out)
}

/// `cq_qmatmul_forward` for callers that cannot allocate device memory (HIP graph capture, serving loops): the
/// workspace is an array inside the library, one per GPU.  Calls that need more than `cq_static_workspace_bytes()` fail;
/// calls that overlap on one GPU race on the array, so keep a lock around it.
///
/// # Safety
/// `x` and `dst` are device pointers to `m * k` and `m * n` elements of the types coded by `x_code` / `dst_code`.
#[allow(clippy::too_many_arguments)]
pub unsafe fn qmatmul_forward_static(weights: &QHipStorage, x: *const c_void, x_code: c_int, dst: *mut c_void, dst_code: c_int, m: usize, k: usize,
                                     n: usize, stream: *mut c_void) -> Result<()> {
    check("cq_qmatmul_forward_static",
          ffi::cq_qmatmul_forward_static(code(weights.dtype()), weights.data.device_ptr(), x, x_code, dst, dst_code, m as i64, k as i64, n as i64, stream))
}
