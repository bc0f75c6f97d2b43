//! call_ops_matmul / call_ops_dot for RocmStorage (the shape of be_cuda/storage/ops_matrix.rs:10-190 and
//! be_cpu/storage/ops_matrix.rs:24-321): output shape from the layouts, hodu's own metadata encoder, kernel picked by
//! the (logical, physical) dtypes of the two operands, an uninitialised contiguous output.
use crate::{
    be_rocm::storage::RocmStorage,
    error::{HoduError, HoduResult},
    op_metadatas,
    ops::{MatrixOp, Op},
    types::{DType, Layout, Shape},
};
use hodu_rocm_kernels::{ffi::hodu_rocm_epilogue_step, kernels, kernels::Kernel};
use std::sync::Arc;

/// which entry point serves a product of these two storages
fn pick(op: &str, lhs: &RocmStorage, rhs: &RocmStorage) -> HoduResult<(Kernel, RocmStorage, RocmStorage)> {
    if lhs.dtype != rhs.dtype {
        return Err(HoduError::DTypeMismatch { expected: lhs.dtype, got: rhs.dtype });
    }
    let name = |suffix: &str| Kernel(crate::cache::kernel::get_kernel_name(format!("hodu_rocm_{op}_{suffix}")));
    match (lhs.dtype, lhs.physical, rhs.physical) {
        // x.matmul(w8.to_dtype(bf16)): the weight's bytes are still f8e4m3, widened between LDS and the matrix cores
        (DType::BF16, DType::BF16, DType::F8E4M3) => Ok((name("bf16_f8e4m3w"), lhs.clone(), rhs.clone())),
        // a8.to_dtype(i32).matmul(b8.to_dtype(i32)): the i8 matrix instruction, exact in i32
        (DType::I32, DType::I8, DType::I8) => Ok((name("i32_i8i8"), lhs.clone(), rhs.clone())),
        // any other combination with a pending cast: carry it out, then the plain kernel
        (dt, _, _) => Ok((name(&dt.to_string()), lhs.materialised()?, rhs.materialised()?)),
    }
}

pub fn call_ops_matmul(lhs: &RocmStorage, rhs: &RocmStorage, ll: &Layout, rl: &Layout, op: Op,
                       steps: &[hodu_rocm_epilogue_step]) -> HoduResult<RocmStorage> {
    if !matches!(op, Op::Matrix(MatrixOp::Matmul)) {
        return Err(HoduError::BackendError("call_ops_matmul expects Matmul op".to_string()));
    }
    let (ls, rs) = (ll.shape(), rl.shape());
    let (ln, rn) = (ls.ndim(), rs.ndim());
    // batch dims of the (already broadcast) left operand, then [M, N]
    let mut dims: Vec<usize> = (0..ln - 2).map(|i| ls[i]).collect();
    dims.push(ls[ln - 2]);
    dims.push(rs[rn - 1]);
    let out_layout = Layout::from_shape(&Shape::new(&dims));
    let md = op_metadatas::matmul_metadata(ll, rl, &out_layout)?;
    let (kernel, l, r) = pick("matmul", lhs, rhs)?;
    let out = l.device.ctx.alloc(out_layout.size() * l.dtype.size_in_bytes())?;
    kernels::call_ops_matmul(kernel, &l.device.ctx, &l.buf, &r.buf, &out, &md, steps)?;
    Ok(RocmStorage::plain(l.device.clone(), Arc::new(out), l.dtype, out_layout.size()))
}

pub fn call_ops_dot(lhs: &RocmStorage, rhs: &RocmStorage, ll: &Layout, rl: &Layout, op: Op,
                    steps: &[hodu_rocm_epilogue_step]) -> HoduResult<RocmStorage> {
    if !matches!(op, Op::Matrix(MatrixOp::Dot)) {
        return Err(HoduError::BackendError("call_ops_dot expects Dot op".to_string()));
    }
    let md = op_metadatas::dot_metadata(ll, rl)?; // [M, K, N, ls_m, ls_k, rs_k, rs_n, l_off, r_off]
    let out_len = ll.shape()[0] * rl.shape()[1];
    let (kernel, l, r) = pick("dot", lhs, rhs)?;
    let out = l.device.ctx.alloc(out_len * l.dtype.size_in_bytes())?;
    kernels::call_ops_dot(kernel, &l.device.ctx, &l.buf, &r.buf, &out, &md, steps)?;
    Ok(RocmStorage::plain(l.device.clone(), Arc::new(out), l.dtype, out_len))
}
