//! The device plumbing the quantized path needs, and nothing more: a device handle with one stream, typed device
//! buffers, an activation/result storage and the grow-only workspace of the library calls.  It stands where
//! `CudaDevice` / `CudaSlice` / `CudaStorage` stand for `QCudaStorage` (candle-core/src/cuda_backend/device.rs,
//! candle-core/src/quantized/cuda.rs:16-23).
use candle_core::{DType, Error, Result};
use core::ffi::{c_char, c_int, c_void};
use std::marker::PhantomData;
use std::sync::{Arc, Mutex, MutexGuard};

#[allow(non_camel_case_types)]
type hipError_t = c_int;
const HIP_MEMCPY_HOST_TO_DEVICE: c_int = 1;
const HIP_MEMCPY_DEVICE_TO_HOST: c_int = 2;

extern "C" {
    fn hipSetDevice(device: c_int) -> hipError_t;
    fn hipMalloc(ptr: *mut *mut c_void, size: usize) -> hipError_t;
    fn hipFree(ptr: *mut c_void) -> hipError_t;
    fn hipMemcpyAsync(dst: *mut c_void, src: *const c_void, size: usize, kind: c_int, stream: *mut c_void) -> hipError_t;
    fn hipMemsetAsync(dst: *mut c_void, value: c_int, size: usize, stream: *mut c_void) -> hipError_t;
    fn hipStreamCreate(stream: *mut *mut c_void) -> hipError_t;
    fn hipStreamDestroy(stream: *mut c_void) -> hipError_t;
    fn hipStreamSynchronize(stream: *mut c_void) -> hipError_t;
    fn hipGetErrorString(err: hipError_t) -> *const c_char;
}

pub(crate) fn hip_check(what: &str, e: hipError_t) -> Result<()> {
    if e == 0 {
        return Ok(());
    }
    let s = unsafe { std::ffi::CStr::from_ptr(hipGetErrorString(e)) };
    Err(Error::Msg(format!("{what}: {} (hipError_t {e})", s.to_string_lossy())).bt())
}

struct DeviceInner {
    ordinal: usize,
    stream: *mut c_void,
    // scratch of the library calls: one grow-only buffer, handed out under the lock, which the caller keeps until
    // its launch is enqueued (the guard of fast_mmvq.rs:44-81); every call of a device goes to its one stream, so
    // consecutive calls may share the buffer
    workspace: Mutex<Workspace>,
}
unsafe impl Send for DeviceInner {}
unsafe impl Sync for DeviceInner {}

impl Drop for DeviceInner {
    fn drop(&mut self) {
        unsafe {
            let _ = hipStreamSynchronize(self.stream);
            let w = self.workspace.get_mut().unwrap();
            for p in w.retired.drain(..).chain(std::iter::once(w.ptr)) {
                if !p.is_null() {
                    let _ = hipFree(p);
                }
            }
            let _ = hipStreamDestroy(self.stream);
        }
    }
}

pub struct Workspace {
    ptr: *mut c_void,
    len: usize,
    // outgrown buffers stay allocated until the device goes: a HIP graph captured earlier may still replay into them
    retired: Vec<*mut c_void>,
}

/// The workspace pointer, valid while the guard is alive.
pub struct WorkspaceGuard<'a> {
    guard: MutexGuard<'a, Workspace>,
}
impl WorkspaceGuard<'_> {
    pub fn ptr(&self) -> *mut c_void {
        self.guard.ptr
    }
    pub fn len(&self) -> usize {
        self.guard.len
    }
    pub fn is_empty(&self) -> bool {
        self.guard.len == 0
    }
}

#[derive(Clone)]
pub struct HipDevice {
    inner: Arc<DeviceInner>,
}

impl std::fmt::Debug for HipDevice {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "HipDevice({})", self.inner.ordinal)
    }
}

impl HipDevice {
    pub fn new(ordinal: usize) -> Result<Self> {
        hip_check("hipSetDevice", unsafe { hipSetDevice(ordinal as c_int) })?;
        let mut stream = std::ptr::null_mut();
        hip_check("hipStreamCreate", unsafe { hipStreamCreate(&mut stream) })?;
        let workspace = Mutex::new(Workspace { ptr: std::ptr::null_mut(), len: 0, retired: Vec::new() });
        Ok(Self { inner: Arc::new(DeviceInner { ordinal, stream, workspace }) })
    }
    pub fn ordinal(&self) -> usize {
        self.inner.ordinal
    }
    pub fn same_device(&self, rhs: &Self) -> bool {
        self.inner.ordinal == rhs.inner.ordinal
    }
    /// `hipStream_t` every call of this device is enqueued on.
    pub fn stream(&self) -> *mut c_void {
        self.inner.stream
    }
    pub fn synchronize(&self) -> Result<()> {
        hip_check("hipStreamSynchronize", unsafe { hipStreamSynchronize(self.inner.stream) })
    }
    fn bind(&self) -> Result<()> {
        hip_check("hipSetDevice", unsafe { hipSetDevice(self.inner.ordinal as c_int) })
    }

    /// Uninitialized device memory for `len` elements.
    ///
    /// # Safety
    /// The contents are undefined until written.
    pub unsafe fn alloc<T: Copy>(&self, len: usize) -> Result<HipSlice<T>> {
        self.bind()?;
        let mut ptr = std::ptr::null_mut();
        let bytes = (len * std::mem::size_of::<T>()).max(16);
        hip_check("hipMalloc", hipMalloc(&mut ptr, bytes))?;
        Ok(HipSlice { ptr, len, device: self.clone(), _t: PhantomData })
    }
    pub fn alloc_zeros<T: Copy>(&self, len: usize) -> Result<HipSlice<T>> {
        let s = unsafe { self.alloc::<T>(len)? };
        hip_check("hipMemsetAsync", unsafe { hipMemsetAsync(s.ptr, 0, len * std::mem::size_of::<T>(), self.inner.stream) })?;
        Ok(s)
    }
    pub fn memcpy_htod<T: Copy>(&self, src: &[T], dst: &mut HipSlice<T>) -> Result<()> {
        if src.len() > dst.len {
            candle_core::bail!("memcpy_htod: {} elements into a buffer of {}", src.len(), dst.len)
        }
        let bytes = std::mem::size_of_val(src);
        hip_check("hipMemcpyAsync", unsafe {
            hipMemcpyAsync(dst.ptr, src.as_ptr() as *const c_void, bytes, HIP_MEMCPY_HOST_TO_DEVICE, self.inner.stream)
        })?;
        // the source is pageable host memory the caller may drop: wait for the copy
        self.synchronize()
    }
    pub fn memcpy_stod<T: Copy>(&self, src: &[T]) -> Result<HipSlice<T>> {
        let mut dst = unsafe { self.alloc::<T>(src.len())? };
        self.memcpy_htod(src, &mut dst)?;
        Ok(dst)
    }
    pub fn memcpy_dtov<T: Copy + Default>(&self, src: &HipSlice<T>, len: usize) -> Result<Vec<T>> {
        if len > src.len {
            candle_core::bail!("memcpy_dtov: {len} elements out of a buffer of {}", src.len)
        }
        let mut out = vec![T::default(); len];
        hip_check("hipMemcpyAsync", unsafe {
            hipMemcpyAsync(out.as_mut_ptr() as *mut c_void, src.ptr, len * std::mem::size_of::<T>(), HIP_MEMCPY_DEVICE_TO_HOST, self.inner.stream)
        })?;
        self.synchronize()?;
        Ok(out)
    }

    /// The device's scratch buffer, at least `bytes` long and 256-byte aligned (hipMalloc aligns further).  Hold the
    /// guard until the call that uses the pointer has been enqueued.
    pub fn quant_workspace(&self, bytes: usize) -> Result<WorkspaceGuard<'_>> {
        let mut w = self.inner.workspace.lock().map_err(|_| Error::Msg("workspace lock poisoned".into()))?;
        if w.len < bytes {
            self.bind()?;
            let want = bytes.max(1 << 20).max(2 * w.len);
            let mut ptr = std::ptr::null_mut();
            hip_check("hipMalloc", unsafe { hipMalloc(&mut ptr, want) })?;
            let old = std::mem::replace(&mut w.ptr, ptr);
            if !old.is_null() {
                w.retired.push(old);
            }
            w.len = want;
        }
        Ok(WorkspaceGuard { guard: w })
    }
}

/// `len` elements of `T` in device memory, freed on drop (after the device's stream has drained).
pub struct HipSlice<T> {
    ptr: *mut c_void,
    len: usize,
    device: HipDevice,
    _t: PhantomData<T>,
}
unsafe impl<T: Send> Send for HipSlice<T> {}
unsafe impl<T: Sync> Sync for HipSlice<T> {}

impl<T> HipSlice<T> {
    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    pub fn device(&self) -> &HipDevice {
        &self.device
    }
    pub fn device_ptr(&self) -> *const c_void {
        self.ptr
    }
    pub fn device_ptr_mut(&mut self) -> *mut c_void {
        self.ptr
    }
    /// Device address of element `offset`.
    pub fn device_ptr_at(&self, offset: usize) -> *const c_void {
        (self.ptr as usize + offset * std::mem::size_of::<T>()) as *const c_void
    }
}

impl<T> Drop for HipSlice<T> {
    fn drop(&mut self) {
        // kernels enqueued on the device's stream may still read or write the buffer
        let _ = self.device.synchronize();
        unsafe {
            let _ = hipFree(self.ptr);
        }
    }
}

/// The activation / result tensors of the quantized path: what `CudaStorageSlice` is to `QCudaStorage`, restricted to
/// the element types the kernels take (f32, f16, bf16 activations; u32 ids).
pub enum HipStorageSlice {
    F32(HipSlice<f32>),
    F16(HipSlice<u16>),
    BF16(HipSlice<u16>),
    U32(HipSlice<u32>),
}

pub struct HipStorage {
    pub slice: HipStorageSlice,
    pub device: HipDevice,
}

impl HipStorage {
    pub fn dtype(&self) -> DType {
        match &self.slice {
            HipStorageSlice::F32(_) => DType::F32,
            HipStorageSlice::F16(_) => DType::F16,
            HipStorageSlice::BF16(_) => DType::BF16,
            HipStorageSlice::U32(_) => DType::U32,
        }
    }
    pub fn device(&self) -> &HipDevice {
        &self.device
    }
    pub fn as_f32(&self) -> Result<&HipSlice<f32>> {
        match &self.slice {
            HipStorageSlice::F32(s) => Ok(s),
            _ => candle_core::bail!("expected an f32 tensor, got {:?}", self.dtype()),
        }
    }
    pub fn as_u32(&self) -> Result<&HipSlice<u32>> {
        match &self.slice {
            HipStorageSlice::U32(s) => Ok(s),
            _ => candle_core::bail!("expected a u32 tensor, got {:?}", self.dtype()),
        }
    }
    /// (device address of element `offset`, the GGUF type code the C ABI uses for the element type)
    pub fn float_ptr_at(&self, offset: usize) -> Result<(*const c_void, c_int)> {
        match &self.slice {
            HipStorageSlice::F32(s) => Ok((s.device_ptr_at(offset), 0)),
            HipStorageSlice::F16(s) => Ok((s.device_ptr_at(offset), 1)),
            HipStorageSlice::BF16(s) => Ok((s.device_ptr_at(offset), 30)),
            HipStorageSlice::U32(_) => candle_core::bail!("expected f32, f16 or bf16 activations, got u32"),
        }
    }
    /// An uninitialized tensor of `len` elements of a float type.
    ///
    /// # Safety
    /// The contents are undefined until a kernel has written them.
    pub unsafe fn alloc_float(device: &HipDevice, dtype: DType, len: usize) -> Result<Self> {
        let slice = match dtype {
            DType::F32 => HipStorageSlice::F32(device.alloc::<f32>(len)?),
            DType::F16 => HipStorageSlice::F16(device.alloc::<u16>(len)?),
            DType::BF16 => HipStorageSlice::BF16(device.alloc::<u16>(len)?),
            dt => candle_core::bail!("no quantized matmul for {dt:?} activations"),
        };
        Ok(Self { slice, device: device.clone() })
    }
    pub fn float_ptr_mut(&mut self) -> *mut c_void {
        match &mut self.slice {
            HipStorageSlice::F32(s) => s.device_ptr_mut(),
            HipStorageSlice::F16(s) | HipStorageSlice::BF16(s) => s.device_ptr_mut(),
            HipStorageSlice::U32(s) => s.device_ptr_mut(),
        }
    }
}
