//! Device storage with deferred casts.
//!
//! `dtype` is what the rest of hodu sees; `physical` is what the bytes in HBM are.  `to_dtype(F8E4M3 -> BF16)` and
//! `to_dtype(I8 -> I32)` of a contiguous tensor return a storage that SHARES the buffer with `physical` left as it was:
//! no kernel runs, and the product that consumes it reads the one-byte elements and widens them in registers
//! (`hodu_rocm_{matmul,dot}_bf16_f8e4m3w`, `_i32_i8i8`).  Strides and offsets are in elements either way, so views
//! of such a storage stay valid.  Any other consumer materialises the cast first.
pub mod ops_matrix;

use crate::{
    be::storage::BackendStorageT,
    be_cpu::storage::CpuStorage,
    be_rocm::device::RocmDevice,
    error::{HoduError, HoduResult},
    op_metadatas,
    ops::{Op, ReduceOp},
    scalar::Scalar,
    types::{DType, Device, Layout, Shape},
};
use hodu_rocm_kernels::{kernels, DeviceBuf};
use std::sync::Arc;

#[derive(Clone)]
pub struct RocmStorage {
    pub(crate) device: Arc<RocmDevice>,
    pub(crate) buf: Arc<DeviceBuf>,
    pub(crate) dtype: DType,    // logical
    pub(crate) physical: DType, // of the bytes in `buf`
    pub(crate) len: usize,      // elements in `buf`
}

impl From<hodu_rocm_kernels::RocmKernelError> for HoduError {
    fn from(e: hodu_rocm_kernels::RocmKernelError) -> Self {
        HoduError::RocmKernelError(e.to_string()) // new variant beside CudaKernelError (error.rs:300-306)
    }
}

macro_rules! not_on_rocm {
    ($what:literal) => {
        Err(HoduError::NotImplemented(concat!($what, " on Device::ROCm").into()))
    };
}

impl RocmStorage {
    pub(crate) fn plain(device: Arc<RocmDevice>, buf: Arc<DeviceBuf>, dtype: DType, len: usize) -> Self {
        Self { device, buf, dtype, physical: dtype, len }
    }
    pub fn is_deferred(&self) -> bool {
        self.physical != self.dtype
    }
    /// to_device from the CPU: raw little-endian element bytes, unchanged (tensor/bytes.rs:90-180)
    pub fn from_cpu_storage(cpu: &CpuStorage, device_id: usize) -> HoduResult<Self> {
        let device = RocmDevice::get(device_id)?;
        let bytes = cpu.to_bytes();
        let len = bytes.len() / cpu.dtype().size_in_bytes();
        let buf = device.ctx.upload(&bytes)?;
        Ok(Self::plain(device, Arc::new(buf), cpu.dtype(), len))
    }
    /// the storage with its deferred cast carried out (a real `hodu_rocm_cast` over the whole buffer), or a clone
    pub(crate) fn materialised(&self) -> HoduResult<Self> {
        if !self.is_deferred() {
            return Ok(self.clone());
        }
        let flat = Layout::from_shape(&Shape::new(&[self.len]));
        let out = self.device.ctx.alloc(self.len * self.dtype.size_in_bytes())?;
        kernels::call_ops_cast(&self.device.ctx, self.physical as u8, self.dtype as u8, &self.buf, &out,
                               &op_metadatas::cast_metadata(&flat))?;
        Ok(Self::plain(self.device.clone(), Arc::new(out), self.dtype, self.len))
    }
}

impl BackendStorageT for RocmStorage {
    type BackendDevice = RocmDevice;

    fn dtype(&self) -> DType {
        self.dtype
    }
    fn device(&self) -> Device {
        Device::ROCm(self.device.id)
    }
    fn backend_device(&self) -> &RocmDevice {
        &self.device
    }
    fn to_cpu_storage(&self) -> HoduResult<CpuStorage> {
        let real = self.materialised()?;
        let bytes = real.device.ctx.download(&real.buf)?; // synchronises the stream
        CpuStorage::from_bytes(&bytes, real.dtype)
    }

    fn call_ops_matmul(&self, rhs: &Self, ll: &Layout, rl: &Layout, op: Op) -> HoduResult<Self> {
        ops_matrix::call_ops_matmul(self, rhs, ll, rl, op, &[])
    }
    fn call_ops_dot(&self, rhs: &Self, ll: &Layout, rl: &Layout, op: Op) -> HoduResult<Self> {
        ops_matrix::call_ops_dot(self, rhs, ll, rl, op, &[])
    }

    fn to_dtype(&self, layout: &Layout, target: DType) -> HoduResult<Self> {
        if self.is_deferred() {
            return self.materialised()?.to_dtype(layout, target);
        }
        if self.dtype == target {
            return self.contiguous(layout);
        }
        // the two casts the products consume in place: defer them when the result would alias the buffer exactly
        let fusable = matches!((self.dtype, target), (DType::F8E4M3, DType::BF16) | (DType::I8, DType::I32));
        if fusable && layout.is_contiguous() && layout.offset() == 0 && layout.size() == self.len {
            return Ok(Self { dtype: target, ..self.clone() });
        }
        let out = self.device.ctx.alloc(layout.size() * target.size_in_bytes())?;
        kernels::call_ops_cast(&self.device.ctx, self.dtype as u8, target as u8, &self.buf, &out,
                               &op_metadatas::cast_metadata(layout))?;
        Ok(Self::plain(self.device.clone(), Arc::new(out), target, layout.size()))
    }

    fn contiguous(&self, layout: &Layout) -> HoduResult<Self> {
        if self.is_deferred() {
            return self.materialised()?.contiguous(layout);
        }
        // already dense from element 0: share the buffer (be_cpu/storage.rs:723-725 clones the Vec)
        if layout.is_contiguous() && layout.offset() == 0 && layout.size() == self.len {
            return Ok(self.clone());
        }
        let out = self.device.ctx.alloc(layout.size() * self.dtype.size_in_bytes())?;
        kernels::call_ops_contiguous(&self.device.ctx, self.dtype as u8, &self.buf, &out,
                                     &op_metadatas::contiguous_metadata(layout))?;
        Ok(Self::plain(self.device.clone(), Arc::new(out), self.dtype, layout.size()))
    }

    /// Sum only: what sum_to_shape of the matmul VJP launches (tensor/gradient/vjp_matrix.rs:17-67)
    fn call_ops_reduce(&self, layout: &Layout, dims: &[usize], keep_dim: bool, op: Op) -> HoduResult<Self> {
        if !matches!(op, Op::Reduce(ReduceOp::Sum)) {
            return not_on_rocm!("reduce ops other than sum");
        }
        let real = self.materialised()?;
        let md = op_metadatas::reduce_metadata(layout, dims, keep_dim);
        let out_len: usize = layout.size() / dims.iter().map(|&d| layout.shape()[d]).product::<usize>().max(1);
        let out = real.device.ctx.alloc(out_len * real.dtype.size_in_bytes())?;
        kernels::call_ops_sum(&real.device.ctx, real.dtype as u8, &real.buf, &out, &md)?;
        Ok(Self::plain(real.device.clone(), Arc::new(out), real.dtype, out_len))
    }

    // ---- everything else: not on this path --------------------------------------------------------------------
    fn const_set(&mut self, _: Scalar, _: &Layout) -> HoduResult<()> { not_on_rocm!("const_set") }
    fn call_ops_binary(&self, _: &Self, _: &Layout, _: &Layout, _: Op) -> HoduResult<Self> { not_on_rocm!("binary ops") }
    fn call_ops_binary_logical(&self, _: &Self, _: &Layout, _: &Layout, _: Op) -> HoduResult<Self> { not_on_rocm!("logical binary ops") }
    fn call_ops_bitwise_binary(&self, _: &Self, _: &Layout, _: &Layout, _: Op) -> HoduResult<Self> { not_on_rocm!("bitwise binary ops") }
    fn call_ops_bitwise_unary(&self, _: &Layout, _: Op) -> HoduResult<Self> { not_on_rocm!("bitwise unary ops") }
    fn call_ops_bitwise_unary_scalar(&self, _: &Layout, _: u32, _: Op) -> HoduResult<Self> { not_on_rocm!("bitwise shifts") }
    fn call_ops_cmp(&self, _: &Self, _: &Layout, _: &Layout, _: Op) -> HoduResult<Self> { not_on_rocm!("comparisons") }
    fn call_ops_cmp_scalar(&self, _: &Layout, _: Scalar, _: Op) -> HoduResult<Self> { not_on_rocm!("scalar comparisons") }
    fn call_ops_unary(&self, _: &Layout, _: Op) -> HoduResult<Self> { not_on_rocm!("unary ops") }
    fn call_ops_unary_logical(&self, _: &Layout, _: Op) -> HoduResult<Self> { not_on_rocm!("logical unary ops") }
    fn call_ops_unary_scalar(&self, _: &Layout, _: Scalar, _: Op) -> HoduResult<Self> { not_on_rocm!("scalar unary ops") }
    fn call_ops_det(&self, _: &Layout) -> HoduResult<Self> { not_on_rocm!("det") }
    fn call_ops_inv(&self, _: &Layout) -> HoduResult<Self> { not_on_rocm!("inv") }
    fn call_ops_trace(&self, _: &Layout) -> HoduResult<Self> { not_on_rocm!("trace") }
    fn call_ops_concat(&self, _: &[&Self], _: &[&Layout], _: usize, _: Op) -> HoduResult<Self> { not_on_rocm!("concat") }
    fn call_ops_split(&self, _: &Layout, _: usize, _: usize, _: usize, _: Op) -> HoduResult<Self> { not_on_rocm!("split") }
    fn call_ops_index_select(&self, _: &Layout, _: &Self, _: &Layout, _: usize, _: Op) -> HoduResult<Self> { not_on_rocm!("index_select") }
    fn call_ops_index_put(&self, _: &Layout, _: &Self, _: &Layout, _: &Self, _: &Layout, _: usize, _: Op) -> HoduResult<Self> { not_on_rocm!("index_put") }
    fn call_ops_gather(&self, _: &Layout, _: &Self, _: &Layout, _: usize, _: Op) -> HoduResult<Self> { not_on_rocm!("gather") }
    fn call_ops_scatter(&self, _: &Layout, _: &Self, _: &Layout, _: &Self, _: &Layout, _: usize, _: Op) -> HoduResult<Self> { not_on_rocm!("scatter") }
    fn call_ops_onehot(&self, _: &Layout, _: usize, _: usize, _: DType, _: Op) -> HoduResult<Self> { not_on_rocm!("onehot") }
    fn call_nonzero(&self, _: &Layout) -> HoduResult<(Self, usize)> { not_on_rocm!("nonzero") }
    fn call_unique(&self, _: &Layout) -> HoduResult<(Self, Self, Self, usize)> { not_on_rocm!("unique") }
    fn call_compress(&self, _: &Layout, _: &Self, _: &Layout, _: Option<usize>) -> HoduResult<(Self, usize)> { not_on_rocm!("compress") }
    fn call_ops_conv(&self, _: &Layout, _: &Self, _: &Layout, _: &[usize], _: &[usize], _: &[usize], _: Op) -> HoduResult<Self> { not_on_rocm!("conv") }
    fn call_ops_conv_grad_weight(&self, _: &Layout, _: &Self, _: &Layout, _: &Shape, _: &[usize], _: &[usize], _: &[usize], _: Op) -> HoduResult<Self> { not_on_rocm!("conv_grad_weight") }
    fn call_ops_reduce_window(&self, _: &Layout, _: &[usize], _: &[usize], _: &[usize], _: Op) -> HoduResult<Self> { not_on_rocm!("reduce_window") }
    fn call_ops_resize(&self, _: &Layout, _: &[usize], _: crate::op_params::ResizeMode, _: crate::op_params::ResizeCoordTransform,
                       _: crate::op_params::ResizeNearestMode) -> HoduResult<Self> { not_on_rocm!("resize") }
    fn call_ops_pad(&self, _: &Layout, _: &[usize], _: &[usize], _: Scalar, _: Op) -> HoduResult<Self> { not_on_rocm!("pad") }
    fn call_ops_cumsum(&self, _: &Layout, _: usize) -> HoduResult<Self> { not_on_rocm!("cumsum") }
    fn call_ops_cumprod(&self, _: &Layout, _: usize) -> HoduResult<Self> { not_on_rocm!("cumprod") }
    fn call_topk(&self, _: &Layout, _: usize, _: usize, _: usize, _: bool, _: bool) -> HoduResult<(Self, Self)> { not_on_rocm!("topk") }
    fn call_ops_einsum(&self, _: &[&Self], _: &[&Layout], _: &crate::einsum::ParsedEinsum) -> HoduResult<Self> { not_on_rocm!("einsum") }
    fn call_ops_flip(&self, _: &Layout, _: &[usize]) -> HoduResult<Self> { not_on_rocm!("flip") }
}
