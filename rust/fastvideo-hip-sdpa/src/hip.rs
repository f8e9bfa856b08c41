//! The few HIP runtime calls the shims need (libamdhip64): stream-ordered allocation and copies.
use std::ffi::{c_char, c_int, c_void, CStr};

pub type HipStream = *mut c_void;

pub const HIP_MEMCPY_HOST_TO_DEVICE: c_int = 1;
pub const HIP_MEMCPY_DEVICE_TO_HOST: c_int = 2;
pub const HIP_MEMCPY_DEVICE_TO_DEVICE: c_int = 3;

extern "C" {
    pub fn hipMalloc(ptr: *mut *mut c_void, bytes: usize) -> c_int;
    pub fn hipFree(ptr: *mut c_void) -> c_int;
    pub fn hipMallocAsync(ptr: *mut *mut c_void, bytes: usize, stream: HipStream) -> c_int;
    pub fn hipFreeAsync(ptr: *mut c_void, stream: HipStream) -> c_int;
    pub fn hipMemcpyAsync(dst: *mut c_void, src: *const c_void, bytes: usize, kind: c_int, stream: HipStream) -> c_int;
    pub fn hipStreamSynchronize(stream: HipStream) -> c_int;
    pub fn hipGetErrorString(code: c_int) -> *const c_char;
}

pub fn error_string(code: c_int) -> String {
    // SAFETY: hipGetErrorString returns a pointer to a static NUL-terminated string for every code.
    unsafe { CStr::from_ptr(hipGetErrorString(code)) }.to_string_lossy().into_owned()
}
