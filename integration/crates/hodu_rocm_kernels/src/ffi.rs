//! Raw declarations of include/hodu_rocm_kernels.h.  `metadata` is always a HOST pointer to hodu's own `usize`
//! descriptor (op_metadatas.rs: matmul :192-291, dot :464-506, cast / contiguous :1615-1656, reduce :525-586),
//! read during the call only; data pointers are device pointers of the same context.
#![allow(non_camel_case_types)]
use core::ffi::{c_char, c_int, c_void};

#[repr(C)]
pub struct hodu_rocm_ctx {
    _private: [u8; 0],
}

pub const HODU_ROCM_OK: c_int = 0;
pub const HODU_ROCM_INVALID_ARG: c_int = 1;
pub const HODU_ROCM_UNSUPPORTED: c_int = 2;
pub const HODU_ROCM_HIP_ERROR: c_int = 3;
pub const HODU_ROCM_OOM: c_int = 4;
pub const HODU_ROCM_SCRATCH: c_int = 5;

pub const HODU_ROCM_EPI_ADD_ROW: c_int = 1;
pub const HODU_ROCM_EPI_MUL_SCALAR: c_int = 2;
pub const HODU_ROCM_EPI_RELU: c_int = 3;

/// one element-wise step fused into a product's store (Linear's add(bias), attention's mul_scalar, ReLU)
#[repr(C)]
#[derive(Clone, Copy)]
pub struct hodu_rocm_epilogue_step {
    pub op: c_int,
    pub vector: *const c_void, // ADD_ROW: device storage of the bias, in the output dtype
    pub stride: usize,         // ADD_ROW: element stride along the output's last axis (0 = one value)
    pub offset: usize,         // ADD_ROW: element offset of the bias layout
    pub scalar: [u8; 8],       // MUL_SCALAR: the scalar in the output dtype, low bytes first
}

pub type ProductFn = unsafe extern "C" fn(*mut hodu_rocm_ctx, *const c_void, *const c_void, *mut c_void, *const usize, usize) -> c_int;
pub type ProductExFn = unsafe extern "C" fn(
    *mut hodu_rocm_ctx, *const c_void, *const c_void, *mut c_void, *const usize, usize, *const hodu_rocm_epilogue_step, usize,
) -> c_int;

#[link(name = "hodu_rocm_kernels")]
extern "C" {
    pub fn hodu_rocm_ctx_create(device: c_int, ctx: *mut *mut hodu_rocm_ctx) -> c_int;
    pub fn hodu_rocm_ctx_destroy(ctx: *mut hodu_rocm_ctx) -> c_int;
    pub fn hodu_rocm_alloc(ctx: *mut hodu_rocm_ctx, bytes: usize, dptr: *mut *mut c_void) -> c_int;
    pub fn hodu_rocm_free(ctx: *mut hodu_rocm_ctx, dptr: *mut c_void) -> c_int;
    pub fn hodu_rocm_memcpy_h2d(ctx: *mut hodu_rocm_ctx, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn hodu_rocm_memcpy_d2h(ctx: *mut hodu_rocm_ctx, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn hodu_rocm_memcpy_d2d(ctx: *mut hodu_rocm_ctx, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn hodu_rocm_sync(ctx: *mut hodu_rocm_ctx) -> c_int;
    pub fn hodu_rocm_last_error(ctx: *mut hodu_rocm_ctx) -> *const c_char;
    pub fn hodu_rocm_ctx_set_reference_sums(ctx: *mut hodu_rocm_ctx, on: c_int) -> c_int;

    pub fn hodu_rocm_cast(ctx: *mut hodu_rocm_ctx, src_dtype: c_int, dst_dtype: c_int, input: *const c_void,
                          out: *mut c_void, metadata: *const usize, metadata_len: usize) -> c_int;
    pub fn hodu_rocm_contiguous(ctx: *mut hodu_rocm_ctx, dtype: c_int, input: *const c_void, out: *mut c_void,
                                metadata: *const usize, metadata_len: usize) -> c_int;
    pub fn hodu_rocm_sum(ctx: *mut hodu_rocm_ctx, dtype: c_int, input: *const c_void, out: *mut c_void,
                         metadata: *const usize, metadata_len: usize) -> c_int;
    pub fn hodu_rocm_softmax(ctx: *mut hodu_rocm_ctx, dtype: c_int, input: *const c_void, out: *mut c_void,
                             metadata: *const usize, metadata_len: usize, causal: c_int) -> c_int;

    // attn_mask (attention.rs:50-56) folded in: one byte per element, 0 = masked out, read through its own strides
    pub fn hodu_rocm_softmax_masked(ctx: *mut hodu_rocm_ctx, dtype: c_int, input: *const c_void, out: *mut c_void,
                                    metadata: *const usize, metadata_len: usize, causal: c_int, mask: *const c_void,
                                    mask_dtype: c_int, mask_layout: *const usize, mask_layout_len: usize) -> c_int;

    pub fn hodu_rocm_attention(ctx: *mut hodu_rocm_ctx, dtype: c_int, q: *const c_void, k: *const c_void, v: *const c_void,
                               out: *mut c_void, metadata: *const usize, metadata_len: usize, scale: *const c_void,
                               causal: c_int) -> c_int;
    pub fn hodu_rocm_attention_masked(ctx: *mut hodu_rocm_ctx, dtype: c_int, q: *const c_void, k: *const c_void,
                                      v: *const c_void, out: *mut c_void, metadata: *const usize, metadata_len: usize,
                                      scale: *const c_void, causal: c_int, mask: *const c_void, mask_dtype: c_int,
                                      mask_layout: *const usize, mask_layout_len: usize) -> c_int;

    // deferred casts fused into the product: bf16 x f8e4m3 bytes -> bf16, i8 x i8 -> i32
    pub fn hodu_rocm_matmul_bf16_f8e4m3w(ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
                                         metadata: *const usize, metadata_len: usize) -> c_int;
    pub fn hodu_rocm_dot_bf16_f8e4m3w(ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
                                      metadata: *const usize, metadata_len: usize) -> c_int;
    pub fn hodu_rocm_matmul_i32_i8i8(ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
                                     metadata: *const usize, metadata_len: usize) -> c_int;
    pub fn hodu_rocm_dot_i32_i8i8(ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
                                  metadata: *const usize, metadata_len: usize) -> c_int;
    /// hodu_rocm_dot_bf16_f8e4m3w for callers that may not allocate (graph capture, decode loops)
    pub fn hodu_rocm_dot_bf16_f8e4m3w_noalloc(ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void,
                                              out: *mut c_void, metadata: *const usize, metadata_len: usize) -> c_int;
    pub fn hodu_rocm_matmul_bf16_f8e4m3w_ex(ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
        metadata: *const usize, metadata_len: usize, steps: *const hodu_rocm_epilogue_step, n_steps: usize) -> c_int;
    pub fn hodu_rocm_dot_bf16_f8e4m3w_ex(ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
        metadata: *const usize, metadata_len: usize, steps: *const hodu_rocm_epilogue_step, n_steps: usize) -> c_int;
}

/// one (matmul, dot) pair per dtype, plain and with fused steps -- generated the way hodu_cpu_kernels declares its
/// kernels (crates/hodu_cpu_kernels/src/kernels/ops_matrix.rs:123-147)
macro_rules! declare_products {
    ($($dt:ident),*) => { paste::paste! {
        #[link(name = "hodu_rocm_kernels")]
        extern "C" { $(
            pub fn [<hodu_rocm_matmul_ $dt>](ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void,
                out: *mut c_void, metadata: *const usize, metadata_len: usize) -> c_int;
            pub fn [<hodu_rocm_dot_ $dt>](ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void,
                out: *mut c_void, metadata: *const usize, metadata_len: usize) -> c_int;
        )* }
    } };
}
declare_products!(f8e4m3, f8e5m2, bf16, f16, f32, f64, u8, u16, u32, u64, i8, i16, i32, i64);

macro_rules! declare_products_ex {
    ($($dt:ident),*) => { paste::paste! {
        #[link(name = "hodu_rocm_kernels")]
        extern "C" { $(
            pub fn [<hodu_rocm_matmul_ $dt _ex>](ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
                metadata: *const usize, metadata_len: usize, steps: *const hodu_rocm_epilogue_step, n_steps: usize) -> c_int;
            pub fn [<hodu_rocm_dot_ $dt _ex>](ctx: *mut hodu_rocm_ctx, lhs: *const c_void, rhs: *const c_void, out: *mut c_void,
                metadata: *const usize, metadata_len: usize, steps: *const hodu_rocm_epilogue_step, n_steps: usize) -> c_int;
        )* }
    } };
}
// (the 8-bit float dtypes take no fused steps)
declare_products_ex!(bf16, f16, f32, f64, u8, u16, u32, u64, i8, i16, i32, i64, i32_i8i8);
