//! ROCm (MI355X, gfx950) backend: device + storage over the hodu_rocm_kernels crate.  Feature `rocm`.
//! Sibling of be_cuda; real for the matmul / dot / to_dtype / contiguous path (and `sum`, which the matmul VJP's
//! sum_to_shape needs), `NotImplemented` elsewhere.
pub mod device;
pub mod storage;
