//! An owning handle on one device's library context, and device buffers that free themselves.
use crate::error::{Result, RocmKernelError, Status};
use crate::ffi;
use core::ffi::{c_int, c_void};
use std::ffi::CStr;
use std::sync::Arc;

/// One `hodu_rocm_ctx` (one device, one stream).  The library serialises calls on a context internally and never
/// calls back, so sharing it between threads is sound.
pub struct Context {
    raw: *mut ffi::hodu_rocm_ctx,
    device: usize,
}
unsafe impl Send for Context {}
unsafe impl Sync for Context {}

impl Context {
    pub fn new(device: usize) -> Result<Arc<Self>> {
        let mut raw = core::ptr::null_mut();
        let rc = unsafe { ffi::hodu_rocm_ctx_create(device as c_int, &mut raw) };
        if rc != ffi::HODU_ROCM_OK || raw.is_null() {
            return Err(RocmKernelError::new(Status::from_code(rc), format!("hodu_rocm_ctx_create({device}) failed")));
        }
        Ok(Arc::new(Self { raw, device }))
    }
    pub fn device_id(&self) -> usize { self.device }
    pub fn raw(&self) -> *mut ffi::hodu_rocm_ctx { self.raw }

    /// status code -> error carrying the library's message for this thread
    pub fn check(&self, rc: c_int) -> Result<()> {
        if rc == ffi::HODU_ROCM_OK {
            return Ok(());
        }
        let msg = unsafe {
            let p = ffi::hodu_rocm_last_error(self.raw);
            if p.is_null() { String::new() } else { CStr::from_ptr(p).to_string_lossy().into_owned() }
        };
        Err(RocmKernelError::new(Status::from_code(rc), msg))
    }

    /// uninitialised device memory, like CpuDevice::allocate (crates/hodu_core/src/be_cpu/device.rs:19-24): a kernel
    /// writes every element of its output
    pub fn alloc(self: &Arc<Self>, bytes: usize) -> Result<DeviceBuf> {
        let mut p: *mut c_void = core::ptr::null_mut();
        self.check(unsafe { ffi::hodu_rocm_alloc(self.raw, bytes.max(1), &mut p) })?;
        Ok(DeviceBuf { ctx: Arc::clone(self), ptr: p, bytes })
    }
    pub fn upload(self: &Arc<Self>, host: &[u8]) -> Result<DeviceBuf> {
        let buf = self.alloc(host.len())?;
        if !host.is_empty() {
            self.check(unsafe { ffi::hodu_rocm_memcpy_h2d(self.raw, buf.ptr, host.as_ptr() as *const c_void, host.len()) })?;
        }
        Ok(buf)
    }
    /// synchronises the context's stream (the only other synchronising call is `sync`)
    pub fn download(&self, buf: &DeviceBuf) -> Result<Vec<u8>> {
        let mut out = vec![0u8; buf.bytes];
        if buf.bytes != 0 {
            self.check(unsafe { ffi::hodu_rocm_memcpy_d2h(self.raw, out.as_mut_ptr() as *mut c_void, buf.ptr, buf.bytes) })?;
        }
        Ok(out)
    }
    pub fn sync(&self) -> Result<()> { self.check(unsafe { ffi::hodu_rocm_sync(self.raw) }) }
    /// Products of f8e4m3 / f8e5m2 / bf16 / f16 in the CPU backend's arithmetic (the running sum re-rounded to the dtype
    /// after every multiply and add): byte for byte what `hodu_cpu_matmul_<dt>` stores, at a scalar loop's speed.  For
    /// tests that compare devices bit for bit; off by default.
    pub fn set_reference_sums(&self, on: bool) -> Result<()> {
        self.check(unsafe { ffi::hodu_rocm_ctx_set_reference_sums(self.raw, on as c_int) })
    }
}

impl Drop for Context {
    fn drop(&mut self) {
        unsafe { ffi::hodu_rocm_ctx_destroy(self.raw) };
    }
}

/// One `hodu_rocm_alloc` allocation; freed on drop.  Views of a tensor share it through `Arc<BackendStorage>`.
pub struct DeviceBuf {
    ctx: Arc<Context>,
    ptr: *mut c_void,
    bytes: usize,
}
unsafe impl Send for DeviceBuf {}
unsafe impl Sync for DeviceBuf {}

impl DeviceBuf {
    pub fn as_ptr(&self) -> *const c_void { self.ptr }
    pub fn as_mut_ptr(&self) -> *mut c_void { self.ptr }
    pub fn len_bytes(&self) -> usize { self.bytes }
    pub fn context(&self) -> &Arc<Context> { &self.ctx }
}
impl Drop for DeviceBuf {
    fn drop(&mut self) {
        unsafe { ffi::hodu_rocm_free(self.ctx.raw(), self.ptr) };
    }
}
