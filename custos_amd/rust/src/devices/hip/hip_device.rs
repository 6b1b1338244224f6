use core::cell::Cell;
use core::ffi::{CStr, c_void};
use std::ffi::CString;

use super::api::*;

/// An error reported by `libcustos_hip.so`: HIP's `hipError_t` numbers below 10000, the
/// library's own (`CUSTOS_HIP_ERR_*`) above, with the message of `custos_hip_last_error`.
#[derive(Debug, Clone, PartialEq, Eq)]
pub struct HipError {
    pub code: i32,
    pub msg: String,
}

impl core::fmt::Display for HipError {
    fn fmt(&self, f: &mut core::fmt::Formatter<'_>) -> core::fmt::Result {
        write!(f, "HIP device error {}: {}", self.code, self.msg)
    }
}

impl std::error::Error for HipError {}

pub type HipResult<T> = Result<T, HipError>;

/// Turns a status of the library into a `Result`, with the message the handle holds for it.
#[inline]
pub fn check(handle: *mut HipDeviceHandle, code: i32) -> HipResult<()> {
    if code == 0 {
        return Ok(());
    }
    let msg = unsafe { CStr::from_ptr(custos_hip_last_error(handle)) };
    Err(HipError { code, msg: msg.to_string_lossy().into_owned() })
}

std::thread_local! {
    static CURRENT: Cell<*mut HipDeviceHandle> = const { Cell::new(core::ptr::null_mut()) };
}

/// The handle of the device this thread created last and has not dropped; what a deserialised
/// [`HipPtr`](super::HipPtr) is allocated on.
pub fn current_handle() -> Option<*mut HipDeviceHandle> {
    let handle = CURRENT.with(|c| c.get());
    (!handle.is_null()).then_some(handle)
}

/// Arguments of a caller-written kernel (`AsCudaCvoidPtr`, `src/devices/cuda/kernel_launch.rs:29-78`):
/// a pointer to the value and its size in bytes (a recorded launch keeps a copy of the value).
pub trait AsHipKernelArg {
    fn as_kernel_arg(&self) -> (*mut c_void, usize);
}

impl<T> AsHipKernelArg for super::HipPtr<T> {
    #[inline]
    fn as_kernel_arg(&self) -> (*mut c_void, usize) {
        (&self.ptr as *const u64 as *mut c_void, 8)
    }
}

impl<T: crate::number::Number> AsHipKernelArg for T {
    #[inline]
    fn as_kernel_arg(&self) -> (*mut c_void, usize) {
        (self as *const T as *mut c_void, core::mem::size_of::<T>())
    }
}

/// State of one `HIP` device (`CudaDevice`, `src/devices/cuda/cuda_device.rs:14-31`): the library's
/// handle, which owns the streams, the kernel cache, the allocation pool and the graphs.
pub struct HipDevice {
    pub handle: *mut HipDeviceHandle,
    /// The graph of the last lazy run; the next run keeps it if it records the same program.
    #[cfg(feature = "lazy")]
    pub graph: Cell<*mut HipGraph>,
    /// Whether `LazyRun::run` waits for the stream (the reference does, `cuda/lazy.rs:42-43`).
    /// Off by default: a run returns once its graph is queued, and `read`, `write`, `sync`,
    /// dropping a buffer or the device, and an allocation during the next recording are
    /// ordered behind it or wait for it, so a program sees the same values either way.
    pub run_waits: Cell<bool>,
}

impl HipDevice {
    pub fn new(idx: usize) -> crate::Result<Self> {
        let mut handle = core::ptr::null_mut();
        let code = unsafe { custos_hip_device_create(idx as i32, &mut handle) };
        check(core::ptr::null_mut(), code)?;
        CURRENT.with(|c| c.set(handle));
        Ok(HipDevice {
            handle,
            #[cfg(feature = "lazy")]
            graph: Cell::new(core::ptr::null_mut()),
            run_waits: Cell::new(false),
        })
    }

    /// Turns a status into a `Result`, with the library's message for this device.
    #[inline]
    pub fn check(&self, code: i32) -> HipResult<()> {
        check(self.handle, code)
    }

    /// The kernel of an expression text (`fn_cache`, `src/devices/cuda/kernel_cache.rs:45-61`):
    /// looked up by its text, then by its structure; compiled once.
    pub fn compile(&self, kind: i32, dtype: i32, src: &str, markers: &[&CStr]) -> HipResult<*mut HipKernel> {
        let src = CString::new(src).expect("expression text contains a NUL byte");
        let markers: Vec<_> = markers.iter().map(|m| m.as_ptr()).collect();
        let mut kernel = core::ptr::null_mut();
        self.check(unsafe {
            custos_hip_expr_compile(
                self.handle,
                kind,
                dtype,
                src.as_ptr(),
                markers.as_ptr(),
                markers.len() as i32,
                &mut kernel,
            )
        })?;
        Ok(kernel)
    }

    /// Waits until the compute stream has drained (`Stream::sync`).
    #[inline]
    pub fn sync(&self) -> HipResult<()> {
        self.check(unsafe { custos_hip_sync(self.handle) })
    }

    fn source_kernel(&self, src: &str, fn_name: &str) -> HipResult<*mut HipKernel> {
        let src = CString::new(src).expect("kernel source contains a NUL byte");
        let fn_name = CString::new(fn_name).expect("kernel name contains a NUL byte");
        let mut kernel = core::ptr::null_mut();
        self.check(unsafe { custos_hip_source_compile(self.handle, src.as_ptr(), fn_name.as_ptr(), &mut kernel) })?;
        Ok(kernel)
    }

    /// Launches a caller-written HIP kernel over `len` work items, workgroup size chosen by the
    /// library (`CudaDevice::launch_kernel1d`, `src/devices/cuda/cuda_device.rs:85-100`).
    pub fn launch_kernel1d(&self, len: usize, src: &str, fn_name: &str, args: &[&dyn AsHipKernelArg]) -> crate::Result<()> {
        let kernel = self.source_kernel(src, fn_name)?;
        let (params, sizes): (Vec<_>, Vec<_>) = args.iter().map(|a| a.as_kernel_arg()).unzip();
        self.check(unsafe {
            custos_hip_source_launch1d(self.handle, kernel, len, params.as_ptr(), sizes.as_ptr(), params.len() as i32)
        })?;
        Ok(())
    }

    /// Launches a caller-written HIP kernel (`CudaDevice::launch_kernel`, `cuda_device.rs:102-112`).
    pub fn launch_kernel(
        &self,
        src: &str,
        fn_name: &str,
        grid: [u32; 3],
        blocks: [u32; 3],
        shared_mem_bytes: u32,
        args: &[&dyn AsHipKernelArg],
    ) -> crate::Result<()> {
        let kernel = self.source_kernel(src, fn_name)?;
        let (params, sizes): (Vec<_>, Vec<_>) = args.iter().map(|a| a.as_kernel_arg()).unzip();
        self.check(unsafe {
            custos_hip_source_launch(
                self.handle,
                kernel,
                grid.as_ptr(),
                blocks.as_ptr(),
                shared_mem_bytes,
                params.as_ptr(),
                sizes.as_ptr(),
                params.len() as i32,
            )
        })?;
        Ok(())
    }
}

impl Drop for HipDevice {
    fn drop(&mut self) {
        CURRENT.with(|c| {
            if c.get() == self.handle {
                c.set(core::ptr::null_mut());
            }
        });
        // graphs, kernels, pooled allocations and streams go with the handle
        unsafe { custos_hip_device_destroy(self.handle) };
    }
}
