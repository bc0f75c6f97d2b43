//! MI355X (gfx950) kernels for hodu's matmul / dot / to_dtype / contiguous path, through the C ABI of
//! `include/hodu_rocm_kernels.h`.  Layout of the crate follows hodu_cpu_kernels: raw declarations (`ffi`), an error
//! type (`error`), an owning context with device buffers (`context`), and name-dispatched safe wrappers (`kernels`).
pub mod context;
pub mod error;
pub mod ffi;
pub mod kernels;

pub use context::{Context, DeviceBuf};
pub use error::{Result, RocmKernelError, Status};
