//! What a failed call of the kernel library looks like on the Rust side: the library's status code and the message it
//! left for the calling thread (`hodu_rocm_last_error`).  hodu_core turns it into `HoduError::RocmKernelError(String)`.
use core::ffi::c_int;

/// the status codes of include/hodu_rocm_kernels.h, plus one for a kernel name this crate does not know
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum Status {
    InvalidArg,
    /// no kernel takes the request: the caller may fall back (e.g. attention -> three launches)
    Unsupported,
    Hip,
    OutOfMemory,
    /// internal scratch could not be obtained (stream under capture, or the no-alloc entry point beyond its limit)
    Scratch,
    UnknownKernel,
    Other(c_int),
}

impl Status {
    pub fn from_code(rc: c_int) -> Self {
        match rc {
            1 => Status::InvalidArg,
            2 => Status::Unsupported,
            3 => Status::Hip,
            4 => Status::OutOfMemory,
            5 => Status::Scratch,
            other => Status::Other(other),
        }
    }
}

#[derive(Debug, Clone)]
pub struct RocmKernelError {
    pub status: Status,
    pub message: String,
}

impl RocmKernelError {
    pub fn new(status: Status, message: impl Into<String>) -> Self {
        Self { status, message: message.into() }
    }
    pub fn is_unsupported(&self) -> bool {
        self.status == Status::Unsupported
    }
}

impl core::fmt::Display for RocmKernelError {
    fn fmt(&self, f: &mut core::fmt::Formatter<'_>) -> core::fmt::Result {
        write!(f, "hodu_rocm_kernels [{:?}]: {}", self.status, self.message)
    }
}
impl std::error::Error for RocmKernelError {}

pub type Result<T> = core::result::Result<T, RocmKernelError>;
