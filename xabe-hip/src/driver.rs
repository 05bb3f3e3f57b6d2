//! cudarc-shaped owners of HIP objects: the method names `xabe-engine` already calls on `CudaContext`,
//! `CudaStream` and `CudaSlice<T>` (crates/xabe-engine/src/block/moe.rs:94-102 and its 28 sibling files), over the HIP
//! runtime.  No arithmetic; every call is one HIP runtime call.
use std::ffi::{c_int, c_void};
use std::marker::PhantomData;
use std::sync::Arc;

#[allow(non_camel_case_types)]
type hipError_t = c_int;
const HIP_MEMCPY_HOST_TO_DEVICE: c_int = 1;
const HIP_MEMCPY_DEVICE_TO_HOST: c_int = 2;
const HIP_MEMCPY_DEVICE_TO_DEVICE: c_int = 3;
const HIP_STREAM_NON_BLOCKING: u32 = 1;

#[link(name = "amdhip64")]
extern "C" {
    fn hipSetDevice(device: c_int) -> hipError_t;
    fn hipMalloc(ptr: *mut *mut c_void, bytes: usize) -> hipError_t;
    fn hipFree(ptr: *mut c_void) -> hipError_t;
    fn hipMemsetAsync(dst: *mut c_void, value: c_int, bytes: usize, stream: *mut c_void) -> hipError_t;
    fn hipMemcpyAsync(dst: *mut c_void, src: *const c_void, bytes: usize, kind: c_int, stream: *mut c_void) -> hipError_t;
    fn hipStreamCreateWithFlags(stream: *mut *mut c_void, flags: u32) -> hipError_t;
    fn hipStreamDestroy(stream: *mut c_void) -> hipError_t;
    fn hipStreamSynchronize(stream: *mut c_void) -> hipError_t;
    fn hipGetErrorString(e: hipError_t) -> *const std::ffi::c_char;
}

/// cudarc's `DriverError`: the runtime's status and its text.
#[derive(Debug, Clone)]
pub struct DriverError(pub i32, pub String);
impl std::fmt::Display for DriverError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "HIP error {}: {}", self.0, self.1)
    }
}
impl std::error::Error for DriverError {}

fn check(e: hipError_t) -> Result<(), DriverError> {
    if e == 0 {
        return Ok(());
    }
    let text = unsafe { std::ffi::CStr::from_ptr(hipGetErrorString(e)) }.to_string_lossy().into_owned();
    Err(DriverError(e, text))
}

/// One device (cudarc: `CudaContext::new(ordinal)`).
pub struct HipContext {
    ordinal: usize,
}
impl HipContext {
    pub fn new(ordinal: usize) -> Result<Arc<Self>, DriverError> {
        check(unsafe { hipSetDevice(ordinal as c_int) })?;
        Ok(Arc::new(Self { ordinal }))
    }
    pub fn ordinal(&self) -> usize {
        self.ordinal
    }
    /// Make this device current on the calling thread (cudarc: `bind_to_thread`).
    pub fn bind_to_thread(&self) -> Result<(), DriverError> {
        check(unsafe { hipSetDevice(self.ordinal as c_int) })
    }
    /// A stream of the default priority (every stream this stack makes is: streams of different priorities have hung
    /// on the target machines).
    pub fn new_stream(self: &Arc<Self>) -> Result<Arc<HipStream>, DriverError> {
        self.bind_to_thread()?;
        let mut raw = std::ptr::null_mut();
        check(unsafe { hipStreamCreateWithFlags(&mut raw, HIP_STREAM_NON_BLOCKING) })?;
        Ok(Arc::new(HipStream { raw, ctx: self.clone() }))
    }
    /// The legacy default stream (cudarc: `default_stream`).  The library's handles are meant for explicit streams.
    pub fn default_stream(self: &Arc<Self>) -> Arc<HipStream> {
        Arc::new(HipStream { raw: std::ptr::null_mut(), ctx: self.clone() })
    }
}

pub struct HipStream {
    raw: *mut c_void,
    ctx: Arc<HipContext>,
}
unsafe impl Send for HipStream {}
unsafe impl Sync for HipStream {}
impl HipStream {
    /// The `hipStream_t`, as the C ABI takes it.
    pub fn raw(&self) -> *mut c_void {
        self.raw
    }
    pub fn context(&self) -> &Arc<HipContext> {
        &self.ctx
    }
    pub fn synchronize(&self) -> Result<(), DriverError> {
        check(unsafe { hipStreamSynchronize(self.raw) })
    }
    pub fn alloc_zeros<T: Copy>(self: &Arc<Self>, len: usize) -> Result<HipSlice<T>, DriverError> {
        let mut s = unsafe { self.alloc::<T>(len)? };
        self.memset_zeros(&mut s)?;
        Ok(s)
    }
    /// Uninitialised device memory (cudarc: `unsafe fn alloc`).
    pub unsafe fn alloc<T: Copy>(self: &Arc<Self>, len: usize) -> Result<HipSlice<T>, DriverError> {
        self.ctx.bind_to_thread()?;
        let mut ptr = std::ptr::null_mut();
        if len > 0 {
            check(unsafe { hipMalloc(&mut ptr, len * std::mem::size_of::<T>()) })?;
        }
        Ok(HipSlice { ptr, len, _stream: self.clone(), _t: PhantomData })
    }
    pub fn memset_zeros<T: Copy>(&self, dst: &mut HipSlice<T>) -> Result<(), DriverError> {
        if dst.len == 0 {
            return Ok(());
        }
        check(unsafe { hipMemsetAsync(dst.ptr, 0, dst.num_bytes(), self.raw) })
    }
    pub fn clone_htod<T: Copy>(self: &Arc<Self>, src: &[T]) -> Result<HipSlice<T>, DriverError> {
        let mut dst = unsafe { self.alloc::<T>(src.len())? };
        self.memcpy_htod(src, &mut dst)?;
        Ok(dst)
    }
    /// (pageable source: the runtime stages the copy, so `src` may be dropped when this returns)
    pub fn memcpy_htod<T: Copy>(&self, src: &[T], dst: &mut HipSlice<T>) -> Result<(), DriverError> {
        assert!(src.len() <= dst.len, "memcpy_htod: {} elements into a slice of {}", src.len(), dst.len);
        if src.is_empty() {
            return Ok(());
        }
        check(unsafe {
            hipMemcpyAsync(dst.ptr, src.as_ptr().cast(), std::mem::size_of_val(src), HIP_MEMCPY_HOST_TO_DEVICE, self.raw)
        })?;
        self.synchronize()
    }
    pub fn clone_dtoh<T: Copy + Default>(&self, src: &HipSlice<T>) -> Result<Vec<T>, DriverError> {
        let mut out = vec![T::default(); src.len];
        self.memcpy_dtoh(src, &mut out)?;
        Ok(out)
    }
    pub fn memcpy_dtoh<T: Copy>(&self, src: &HipSlice<T>, dst: &mut [T]) -> Result<(), DriverError> {
        assert!(dst.len() >= src.len, "memcpy_dtoh: {} elements into a buffer of {}", src.len, dst.len());
        if src.len == 0 {
            return Ok(());
        }
        check(unsafe {
            hipMemcpyAsync(dst.as_mut_ptr().cast(), src.ptr, src.num_bytes(), HIP_MEMCPY_DEVICE_TO_HOST, self.raw)
        })?;
        self.synchronize()
    }
    pub fn memcpy_dtod<T: Copy>(&self, src: &HipSlice<T>, dst: &mut HipSlice<T>) -> Result<(), DriverError> {
        assert!(src.len <= dst.len);
        if src.len == 0 {
            return Ok(());
        }
        check(unsafe { hipMemcpyAsync(dst.ptr, src.ptr, src.num_bytes(), HIP_MEMCPY_DEVICE_TO_DEVICE, self.raw) })
    }
}
impl Drop for HipStream {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { hipStreamDestroy(self.raw) };
        }
    }
}

/// Owned device memory, freed on drop (cudarc: `CudaSlice<T>`).  A buffer handed to a captured graph must outlive
/// the graph, as with cudarc (docs/TOOLCHAIN.md:107-142 of the reference).
pub struct HipSlice<T> {
    ptr: *mut c_void,
    len: usize,
    _stream: Arc<HipStream>,
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
    pub fn num_bytes(&self) -> usize {
        self.len * std::mem::size_of::<T>()
    }
    pub fn as_ptr(&self) -> *const T {
        self.ptr as *const T
    }
    pub fn as_mut_ptr(&mut self) -> *mut T {
        self.ptr as *mut T
    }
}
impl<T> Drop for HipSlice<T> {
    fn drop(&mut self) {
        if !self.ptr.is_null() {
            unsafe { hipFree(self.ptr) };
        }
    }
}

/// A borrowed view of library-owned device memory (what `MoeBuffers`' accessors hand out).
pub struct HipView<'a, T> {
    pub(crate) ptr: *const T,
    pub(crate) len: usize,
    pub(crate) _owner: PhantomData<&'a ()>,
}
impl<T: Copy + Default> HipView<'_, T> {
    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    pub fn as_ptr(&self) -> *const T {
        self.ptr
    }
    /// Copy to the host on `stream` (synchronises it).
    pub fn to_host(&self, stream: &HipStream) -> Result<Vec<T>, DriverError> {
        let mut out = vec![T::default(); self.len];
        if self.len > 0 {
            check(unsafe {
                hipMemcpyAsync(out.as_mut_ptr().cast(), self.ptr.cast(), self.len * std::mem::size_of::<T>(),
                               HIP_MEMCPY_DEVICE_TO_HOST, stream.raw())
            })?;
            stream.synchronize()?;
        }
        Ok(out)
    }
}
