//! Error type of the ROCm kernel crate (same shape as CudaKernelError, crates/hodu_cuda_kernels/src/error.rs:7-18).
use std::fmt;

#[derive(Debug, Clone)]
pub enum RocmKernelError {
    /// no kernel of that name
    InvalidKernel(String),
    /// HODU_ROCM_INVALID_ARG: bad metadata or arguments
    InvalidInput(String),
    /// HODU_ROCM_UNSUPPORTED: no kernel takes the request (the caller may fall back)
    Unsupported(String),
    /// HODU_ROCM_HIP_ERROR: a HIP call failed
    LaunchError(String),
    /// HODU_ROCM_OOM, or HODU_ROCM_SCRATCH (internal scratch could not be obtained)
    MemoryError(String),
    Message(String),
}

impl fmt::Display for RocmKernelError {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        match self {
            Self::InvalidKernel(m) => write!(f, "invalid kernel: {m}"),
            Self::InvalidInput(m) => write!(f, "invalid input: {m}"),
            Self::Unsupported(m) => write!(f, "unsupported: {m}"),
            Self::LaunchError(m) => write!(f, "launch error: {m}"),
            Self::MemoryError(m) => write!(f, "memory error: {m}"),
            Self::Message(m) => write!(f, "{m}"),
        }
    }
}
impl std::error::Error for RocmKernelError {}
pub type Result<T> = std::result::Result<T, RocmKernelError>;
