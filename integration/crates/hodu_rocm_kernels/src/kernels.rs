//! Name-dispatched wrappers in the shape of hodu_cpu_kernels::call_ops_matmul / call_ops_dot / call_ops_cast
//! (crates/hodu_cpu_kernels/src/kernels/ops_matrix.rs:56-68, :102-114; ops_cast.rs:70-81): a `Kernel` is a static
//! name "hodu_rocm_<op>_<dtype>", the metadata is hodu's `&[usize]`, a non-zero status becomes an error.
use crate::context::{Context, DeviceBuf};
use crate::error::{Result, RocmKernelError, Status};
use crate::ffi::{self, ProductExFn, ProductFn};
use core::ffi::c_int;

#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub struct Kernel(pub &'static str);

macro_rules! ops {
    ($($name:ident),+) => { $(
        pub mod $name {
            use super::Kernel;
            pub const F8E4M3: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_f8e4m3"));
            pub const F8E5M2: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_f8e5m2"));
            pub const BF16: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_bf16"));
            pub const F16: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_f16"));
            pub const F32: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_f32"));
            pub const F64: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_f64"));
            pub const U8: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_u8"));
            pub const U16: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_u16"));
            pub const U32: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_u32"));
            pub const U64: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_u64"));
            pub const I8: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_i8"));
            pub const I16: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_i16"));
            pub const I32: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_i32"));
            pub const I64: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_i64"));
            /// logical bf16 x bf16 -> bf16 with the right operand still stored as f8e4m3 (a deferred to_dtype)
            pub const BF16_F8E4M3W: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_bf16_f8e4m3w"));
            /// logical i32 x i32 -> i32 with both operands still stored as i8
            pub const I32_I8I8: Kernel = Kernel(concat!("hodu_rocm_", stringify!($name), "_i32_i8i8"));
        }
    )+ };
}
ops!(matmul, dot);

macro_rules! product_table {
    ($op:ident; $($dt:ident),*) => { paste::paste! {
        fn [<$op _fn>](name: &str) -> Option<ProductFn> {
            match name {
                $( concat!("hodu_rocm_", stringify!($op), "_", stringify!($dt)) => Some(ffi::[<hodu_rocm_ $op _ $dt>] as ProductFn), )*
                _ => None,
            }
        }
    } };
}
product_table!(matmul; f8e4m3, f8e5m2, bf16, f16, f32, f64, u8, u16, u32, u64, i8, i16, i32, i64, bf16_f8e4m3w, i32_i8i8);
product_table!(dot; f8e4m3, f8e5m2, bf16, f16, f32, f64, u8, u16, u32, u64, i8, i16, i32, i64, bf16_f8e4m3w, i32_i8i8);

macro_rules! product_ex_table {
    ($op:ident; $($dt:ident),*) => { paste::paste! {
        fn [<$op _ex_fn>](name: &str) -> Option<ProductExFn> {
            match name {
                $( concat!("hodu_rocm_", stringify!($op), "_", stringify!($dt)) => Some(ffi::[<hodu_rocm_ $op _ $dt _ex>] as ProductExFn), )*
                _ => None,
            }
        }
    } };
}
product_ex_table!(matmul; bf16, f16, f32, f64, u8, u16, u32, u64, i8, i16, i32, i64, bf16_f8e4m3w, i32_i8i8);
product_ex_table!(dot; bf16, f16, f32, f64, u8, u16, u32, u64, i8, i16, i32, i64, bf16_f8e4m3w, i32_i8i8);

fn run_product(ctx: &Context, plain: Option<ProductFn>, ex: Option<ProductExFn>, kernel: Kernel, lhs: &DeviceBuf,
               rhs: &DeviceBuf, out: &DeviceBuf, metadata: &[usize], steps: &[ffi::hodu_rocm_epilogue_step]) -> Result<()> {
    let rc = if steps.is_empty() {
        let f = plain.ok_or_else(|| RocmKernelError::new(Status::UnknownKernel, kernel.0))?;
        unsafe { f(ctx.raw(), lhs.as_ptr(), rhs.as_ptr(), out.as_mut_ptr(), metadata.as_ptr(), metadata.len()) }
    } else {
        let f = ex.ok_or_else(|| RocmKernelError::new(Status::UnknownKernel, format!("{} takes no fused steps", kernel.0)))?;
        unsafe { f(ctx.raw(), lhs.as_ptr(), rhs.as_ptr(), out.as_mut_ptr(), metadata.as_ptr(), metadata.len(), steps.as_ptr(), steps.len()) }
    };
    ctx.check(rc)
}

/// Batched matrix product with broadcast batch dims; `metadata` = op_metadatas::matmul_metadata (unchanged).
/// `steps`: element-wise kernels the caller would launch on the output next, fused into the store (may be empty).
pub fn call_ops_matmul(kernel: Kernel, ctx: &Context, lhs: &DeviceBuf, rhs: &DeviceBuf, out: &DeviceBuf, metadata: &[usize],
                       steps: &[ffi::hodu_rocm_epilogue_step]) -> Result<()> {
    run_product(ctx, matmul_fn(kernel.0), matmul_ex_fn(kernel.0), kernel, lhs, rhs, out, metadata, steps)
}

/// 2-D product; `metadata` = op_metadatas::dot_metadata.
pub fn call_ops_dot(kernel: Kernel, ctx: &Context, lhs: &DeviceBuf, rhs: &DeviceBuf, out: &DeviceBuf, metadata: &[usize],
                    steps: &[ffi::hodu_rocm_epilogue_step]) -> Result<()> {
    run_product(ctx, dot_fn(kernel.0), dot_ex_fn(kernel.0), kernel, lhs, rhs, out, metadata, steps)
}

/// to_dtype: `src` / `dst` are hodu's own `DType as u8` discriminants (types/dtype.rs:6-28); metadata = cast_metadata.
pub fn call_ops_cast(ctx: &Context, src: u8, dst: u8, input: &DeviceBuf, out: &DeviceBuf, metadata: &[usize]) -> Result<()> {
    ctx.check(unsafe { ffi::hodu_rocm_cast(ctx.raw(), src as c_int, dst as c_int, input.as_ptr(), out.as_mut_ptr(), metadata.as_ptr(), metadata.len()) })
}

/// strided gather into a contiguous buffer; metadata = contiguous_metadata.
pub fn call_ops_contiguous(ctx: &Context, dtype: u8, input: &DeviceBuf, out: &DeviceBuf, metadata: &[usize]) -> Result<()> {
    ctx.check(unsafe { ffi::hodu_rocm_contiguous(ctx.raw(), dtype as c_int, input.as_ptr(), out.as_mut_ptr(), metadata.as_ptr(), metadata.len()) })
}

/// ReduceOp::Sum (what sum_to_shape of the matmul VJP needs); metadata = reduce_metadata.
pub fn call_ops_sum(ctx: &Context, dtype: u8, input: &DeviceBuf, out: &DeviceBuf, metadata: &[usize]) -> Result<()> {
    ctx.check(unsafe { ffi::hodu_rocm_sum(ctx.raw(), dtype as c_int, input.as_ptr(), out.as_mut_ptr(), metadata.as_ptr(), metadata.len()) })
}

/// An `attn_mask` (crates/hodu_nn/src/modules/attention.rs:50-56) read in place: one byte per element (`dtype`: hodu's
/// discriminant of BOOL, U8 or I8; anything else goes through `call_ops_cast` to BOOL first), 0 = masked out.
/// `layout` = [nd, strides over the masked tensor's shape.., offset] in elements, stride 0 where the mask is broadcast
/// (`Layout::broadcast_to(shape)` gives exactly these strides).
pub struct MaskArg<'a> {
    pub buf: &'a DeviceBuf,
    pub dtype: u8,
    pub layout: &'a [usize],
}

/// Tensor::softmax (tensor/ops/normalization.rs:4-21) as one kernel; metadata = reduce_metadata of the input layout with
/// the softmax dim as the one reduced dim (keep_dim).  `causal` folds attention's is_causal mask in (last dim only);
/// with `mask` the softmax runs along the last dim over masked_fill(mask.eq_scalar(0), get_neg_inf(dtype)).
pub fn call_ops_softmax(ctx: &Context, dtype: u8, input: &DeviceBuf, out: &DeviceBuf, metadata: &[usize], causal: bool,
                        mask: Option<MaskArg>) -> Result<()> {
    let rc = match mask {
        None => unsafe {
            ffi::hodu_rocm_softmax(ctx.raw(), dtype as c_int, input.as_ptr(), out.as_mut_ptr(), metadata.as_ptr(), metadata.len(),
                                   causal as c_int)
        },
        Some(m) => unsafe {
            ffi::hodu_rocm_softmax_masked(ctx.raw(), dtype as c_int, input.as_ptr(), out.as_mut_ptr(), metadata.as_ptr(),
                                          metadata.len(), causal as c_int, m.buf.as_ptr(), m.dtype as c_int, m.layout.as_ptr(),
                                          m.layout.len())
        },
    };
    ctx.check(rc)
}

/// scaled_dot_product_attention (attention.rs:25-70, without dropout) as one kernel.  metadata: [nb, batch_shape..,
/// Sq, Sk, D, q_strides (nb + 2).., k_strides.., v_strides.., q_off, k_off, v_off]; `scale`: the scalar in `dtype`'s
/// storage (what mul_scalar would receive); a mask's layout runs over [batch.., Sq, Sk].  Ok(false): the kernel does
/// not take this call (dtype, head dim, alignment) and nothing was launched -- the caller runs the three launches
/// (call_ops_matmul with a MUL_SCALAR step, call_ops_softmax, call_ops_matmul).
pub fn call_ops_attention(ctx: &Context, dtype: u8, q: &DeviceBuf, k: &DeviceBuf, v: &DeviceBuf, out: &DeviceBuf,
                          metadata: &[usize], scale: &[u8], causal: bool, mask: Option<MaskArg>) -> Result<bool> {
    let rc = match mask {
        None => unsafe {
            ffi::hodu_rocm_attention(ctx.raw(), dtype as c_int, q.as_ptr(), k.as_ptr(), v.as_ptr(), out.as_mut_ptr(),
                                     metadata.as_ptr(), metadata.len(), scale.as_ptr() as *const core::ffi::c_void, causal as c_int)
        },
        Some(m) => unsafe {
            ffi::hodu_rocm_attention_masked(ctx.raw(), dtype as c_int, q.as_ptr(), k.as_ptr(), v.as_ptr(), out.as_mut_ptr(),
                                            metadata.as_ptr(), metadata.len(), scale.as_ptr() as *const core::ffi::c_void,
                                            causal as c_int, m.buf.as_ptr(), m.dtype as c_int, m.layout.as_ptr(), m.layout.len())
        },
    };
    match ctx.check(rc) {
        Ok(()) => Ok(true),
        Err(e) if e.is_unsupported() => Ok(false),
        Err(e) => Err(e),
    }
}
