/*
 * hodu_rocm_kernels.h -- C ABI of the MI355X (gfx950) matmul / dot / to_dtype / contiguous backend.
 *
 * This is the seam a `crates/hodu_rocm_kernels` FFI crate binds, a sibling of
 * crates/hodu_cpu_kernels (plain C ABI) and crates/hodu_cuda_kernels.  Every compute entry point
 * mirrors one reference kernel symbol:
 *
 *   hodu_cpu_matmul_<dt>(lhs, rhs, out, metadata)      kernels/ops_matrix.h:56-69
 *   hodu_cpu_dot_<dt>(lhs, rhs, out, metadata)         kernels/ops_matrix.h:97-110
 *   hodu_cpu_cast_<a>_to_<b>(in, out, metadata)        kernels/ops_cast.h:41-88
 *   hodu_cpu_contiguous_<dt>(in, out, metadata)        kernels/ops_memory.h:44
 *
 * with three differences forced by the device: (1) a context handle comes first; (2) operand
 * pointers are DEVICE pointers while `metadata` stays a HOST array of size_t in exactly the
 * reference's formats (crates/hodu_core/src/op_metadatas.rs:192-291, :464-506, :1615-1656) and
 * is parsed on the host -- it is never copied to the device (the CUDA sibling re-uploads it on
 * every call, crates/hodu_cuda_kernels/src/kernels/ops_matrix.rs:372-374); (3) every call
 * returns a status instead of void (the CPU kernels have no error channel,
 * crates/hodu_cpu_kernels/src/kernels/ops_matrix.rs:56-68).
 *
 * Contract shared by all compute calls
 *   - strides and offsets are in ELEMENTS; stride 0 broadcasts; operands may be transposed,
 *     sliced or batch-broadcast views and are consumed in place (no contiguous copy);
 *   - `out` is caller-allocated, contiguous, uninitialised (crates/hodu_core/src/be_cpu/device.rs:19-24)
 *     and every element of it is written; it must not alias an input; inputs may alias each other;
 *   - launches are asynchronous on the context's stream; hodu_rocm_sync and hodu_rocm_memcpy_d2h
 *     synchronise;
 *   - the library keeps no caller pointer after the call returns and never calls back.
 */
#ifndef HODU_ROCM_KERNELS_H
#define HODU_ROCM_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hodu_rocm_ctx hodu_rocm_ctx;

/* status codes (0 = ok).  Maps onto CudaKernelError::{InvalidInput, InvalidKernel, LaunchError,
 * MemoryError} of crates/hodu_cuda_kernels/src/error.rs:7-18. */
enum {
    HODU_ROCM_OK = 0,
    HODU_ROCM_INVALID_ARG = 1, /* null pointer, malformed or inconsistent metadata */
    HODU_ROCM_UNSUPPORTED = 2, /* dtype / rank outside what the device implements */
    HODU_ROCM_HIP_ERROR = 3,   /* a HIP runtime call failed; see hodu_rocm_last_error */
    HODU_ROCM_OOM = 4,         /* device allocation failed */
    HODU_ROCM_SCRATCH = 5      /* the call may not allocate (the entry point that allocates nothing, or a stream under
                                  graph capture) and its kernels need more scratch than is there */
};

/* dtype ids, equal to hodu's repr(u8) DType (crates/hodu_core/src/types/dtype.rs:6-28) */
enum {
    HODU_BOOL = 0, HODU_F8E4M3 = 1, HODU_F8E5M2 = 2, HODU_BF16 = 3, HODU_F16 = 4, HODU_F32 = 5,
    HODU_F64 = 6, HODU_U8 = 7, HODU_U16 = 8, HODU_U32 = 9, HODU_U64 = 10, HODU_I8 = 11,
    HODU_I16 = 12, HODU_I32 = 13, HODU_I64 = 14
};

/* ---- runtime (replaces what cudarc gives the CUDA sibling: context, stream, slices;
 *      crates/hodu_core/src/be_cuda/device.rs:20-65, be_cuda/storage.rs:165-173) ---------------- */
int hodu_rocm_device_count(int *count);
int hodu_rocm_ctx_create(int device, hodu_rocm_ctx **ctx);
int hodu_rocm_ctx_destroy(hodu_rocm_ctx *ctx);
int hodu_rocm_alloc(hodu_rocm_ctx *ctx, size_t bytes, void **dptr);
int hodu_rocm_free(hodu_rocm_ctx *ctx, void *dptr);
int hodu_rocm_memcpy_h2d(hodu_rocm_ctx *ctx, void *dst_device, const void *src_host, size_t bytes);
int hodu_rocm_memcpy_d2h(hodu_rocm_ctx *ctx, void *dst_host, const void *src_device, size_t bytes);
int hodu_rocm_memcpy_d2d(hodu_rocm_ctx *ctx, void *dst_device, const void *src_device, size_t bytes);
int hodu_rocm_memset(hodu_rocm_ctx *ctx, void *dptr, int byte, size_t bytes);
int hodu_rocm_sync(hodu_rocm_ctx *ctx);
/* message of the last failing call made on this context by the calling thread ("" if none) */
const char *hodu_rocm_last_error(hodu_rocm_ctx *ctx);
/* device facts for roofline reporting: name (<=255 chars), compute units, clock (kHz), memory bytes */
int hodu_rocm_device_info(hodu_rocm_ctx *ctx, char *name, size_t name_len, int *compute_units,
                          int *clock_khz, size_t *total_mem);
/* HIP-event stopwatch on the context's stream (the stream the kernels run on) */
int hodu_rocm_timer_create(hodu_rocm_ctx *ctx, void **timer);
int hodu_rocm_timer_start(hodu_rocm_ctx *ctx, void *timer);
int hodu_rocm_timer_stop(hodu_rocm_ctx *ctx, void *timer, float *elapsed_ms); /* synchronises */
int hodu_rocm_timer_destroy(hodu_rocm_ctx *ctx, void *timer);
/* name of the kernel family the last matmul/dot call on this context dispatched to (diagnostics) */
const char *hodu_rocm_last_kernel(hodu_rocm_ctx *ctx);
/* The reference's own arithmetic for products of the narrow float dtypes, for a caller that needs hodu's CPU bytes.
 * hodu_cpu_matmul_<dt> / hodu_cpu_dot_<dt> for f8e4m3, f8e5m2, bf16 and f16 keep the running sum in the narrow type,
 * sum = add(sum, mul(a, b)) with both results narrowed by the type's routine (kernels/ops_matrix.c:196-240, :351-354,
 * :556-600, :713-716; t_bf16.h:27-55, t_f16.h:27-84, t_f8e4m3.h:27-101, t_f8e5m2.h:27-100).  With `on` != 0 every
 * later product of those four dtypes on this context (plain and _ex, and the bf16_f8e4m3w kind as this library's
 * cast of the weight followed by the bf16 product) is computed that way, k ascending, and stores the reference's bytes
 * bit for bit -- at the rate of one scalar loop per output element.  Off (the default) they accumulate in f32 and
 * round once, which is what the rest of this header documents.  Other dtypes are not affected: integers and f64 are
 * the reference's arithmetic already, f32 goes to a BLAS there.                                                   */
int hodu_rocm_ctx_set_reference_sums(hodu_rocm_ctx *ctx, int on);
/* ---- matmul / dot: lhs, rhs and out share one dtype (utils/valid.rs:50-76) -------------------- *
 * replaces hodu_cpu_matmul_<dt> (kernels/ops_matrix.c:70, :221) and hodu_cpu_dot_<dt>
 * (kernels/ops_matrix.c:423, :581).  Narrow floats accumulate in f32 and round once on store.   */
#define HODU_ROCM_DECL_PRODUCT(dt)                                                               \
    int hodu_rocm_matmul_##dt(hodu_rocm_ctx *ctx, const void *lhs, const void *rhs, void *out,   \
                              const size_t *metadata, size_t metadata_len);                      \
    int hodu_rocm_dot_##dt(hodu_rocm_ctx *ctx, const void *lhs, const void *rhs, void *out,      \
                           const size_t *metadata, size_t metadata_len);
HODU_ROCM_DECL_PRODUCT(f8e4m3)
HODU_ROCM_DECL_PRODUCT(f8e5m2)
HODU_ROCM_DECL_PRODUCT(bf16)
HODU_ROCM_DECL_PRODUCT(f16)
HODU_ROCM_DECL_PRODUCT(f32)
HODU_ROCM_DECL_PRODUCT(f64)
HODU_ROCM_DECL_PRODUCT(u8)
HODU_ROCM_DECL_PRODUCT(u16)
HODU_ROCM_DECL_PRODUCT(u32)
HODU_ROCM_DECL_PRODUCT(u64)
HODU_ROCM_DECL_PRODUCT(i8)
HODU_ROCM_DECL_PRODUCT(i16)
HODU_ROCM_DECL_PRODUCT(i32)
HODU_ROCM_DECL_PRODUCT(i64)

/* ---- fused to_dtype + matmul / dot ------------------------------------------------------------ *
 * `x.matmul(w8.to_dtype(bf16))`: Tensor::to_dtype (tensor/ops/cast_memory.rs:11-38) followed by
 * Tensor::matmul (tensor/ops/matrix.rs:13-92) without materialising the cast.  The logical dtype
 * contract of the product is unchanged (bf16 x bf16 -> bf16, i32 x i32 -> i32); only the physical
 * storage of the named operand differs, and its metadata strides/offsets count ITS elements.
 *   _bf16_f8e4m3w : lhs bf16, rhs stored f8e4m3 (OCP E4M3FN), out bf16
 *   _i32_i8i8     : lhs and rhs stored i8 (sign-extended), out i32, wrap-around i32 arithmetic   */
int hodu_rocm_matmul_bf16_f8e4m3w(hodu_rocm_ctx *ctx, const void *lhs_bf16, const void *rhs_f8e4m3,
                                  void *out_bf16, const size_t *metadata, size_t metadata_len);
int hodu_rocm_dot_bf16_f8e4m3w(hodu_rocm_ctx *ctx, const void *lhs_bf16, const void *rhs_f8e4m3,
                               void *out_bf16, const size_t *metadata, size_t metadata_len);
int hodu_rocm_matmul_i32_i8i8(hodu_rocm_ctx *ctx, const void *lhs_i8, const void *rhs_i8,
                              void *out_i32, const size_t *metadata, size_t metadata_len);
int hodu_rocm_dot_i32_i8i8(hodu_rocm_ctx *ctx, const void *lhs_i8, const void *rhs_i8,
                           void *out_i32, const size_t *metadata, size_t metadata_len);

/* ---- the one entry point that allocates nothing ------------------------------------------------- *
 * No counterpart in the reference.  It exists for callers that cannot allocate device memory while they call:
 * code under HIP graph capture, tight decode loops, harnesses that forbid hipMalloc.  Same arguments, same result
 * (bit for bit) as hodu_rocm_dot_bf16_f8e4m3w, whose kernels for M <= 16 cut K across workgroups and keep partial
 * sums and arrival counters in a workspace the context allocates and grows on demand; here that scratch is a
 * file-scope device array inside the library (16 KiB of counters + HODU_ROCM_NOALLOC_PARTIAL_BYTES of partial
 * sums; every GPU the library runs on holds one copy until the process ends) and the call makes no hipMalloc /
 * hipFree.  A product whose kernel would need more partial-sum space than that returns HODU_ROCM_SCRATCH with a
 * message naming both sizes (C3's M = 256 cut four ways needs 16 MiB; M <= 16 against any weight up to
 * N x slices <= 131072 fits).  All calls on one GPU share the array and it keeps what the last call left: a call
 * whose kernel counts arrivals zeroes the counters first (one small kernel in front of it, never a memset: the call
 * may be under capture), a call whose kernel uses no scratch (M <= 4) launches nothing extra.  Calls that overlap
 * on one GPU -- two contexts, i.e. two streams -- race on the array; calls on one context are ordered by its
 * stream.  No fused steps. */
#define HODU_ROCM_NOALLOC_PARTIAL_BYTES ((size_t)8 << 20)
int hodu_rocm_dot_bf16_f8e4m3w_noalloc(hodu_rocm_ctx *ctx, const void *lhs_bf16, const void *rhs_f8e4m3,
                                       void *out_bf16, const size_t *metadata, size_t metadata_len);

/* ---- matmul / dot with the caller's next element-wise kernels fused into the store -------------- *
 * The reference's callers of the product launch an element-wise kernel on its output straight away:
 *   Linear::forward (crates/hodu_nn/src/modules/linear.rs:40-46): matmul, then add(bias)
 *       -> hodu_cpu_add_<dt> (kernels/ops_binary.c:208-262 and the native-type macro above it)
 *   scaled_dot_product_attention (crates/hodu_nn/src/modules/attention.rs:37): matmul, then mul_scalar
 *       -> hodu_cpu_mul_scalar_<dt> (kernels/ops_unary.c:138-200, :352-386)
 *   ReLU after a Linear (crates/hodu_nn/src/modules/activation.rs:8-17): relu
 *       -> hodu_cpu_relu_<dt> (kernels/ops_unary.c:648-697, :1404, :1484)
 * The _ex entry points apply up to HODU_ROCM_MAX_EPILOGUE_STEPS such steps, in order, to every output element
 * before it is stored.  Each step takes the value the plain product would have stored (already rounded to the
 * output dtype) and uses the reference kernel's arithmetic for that dtype -- bf16 adds in f32 and truncates,
 * f16 narrows through the reference's own routine, integers wrap --, so the result equals running the plain
 * entry point followed by the reference's kernels bit for bit, with one pass over the output instead of
 * 1 + 2 per step.  n_steps == 0 is the plain product.  The f8 dtypes have no _ex form.
 *   ADD_ROW:    out[.., m, n] += vector[offset + n * stride]; `vector` is device storage of the output dtype.
 *               This is what Tensor::add makes of a bias: broadcast_tensors2 (tensor/ops/binary.rs:21) gives the
 *               operand the output's shape with stride 0 on every axis but the last; pass that last stride
 *               (0 allowed: one value for all columns) and the layout's offset.
 *   MUL_SCALAR: out *= scalar; `scalar` holds the value in the output dtype, as the reference kernel's
 *               `const void *scalar` argument points to it (low bytes first).
 *   RELU:       out = out > 0 ? out : 0 (floating dtypes only; NaN and -0 become +0 as in the reference).      */
enum {
    HODU_ROCM_EPI_ADD_ROW = 1,
    HODU_ROCM_EPI_MUL_SCALAR = 2,
    HODU_ROCM_EPI_RELU = 3
};
#define HODU_ROCM_MAX_EPILOGUE_STEPS 3
typedef struct hodu_rocm_epilogue_step {
    int op;
    const void *vector;
    size_t stride;
    size_t offset;
    unsigned char scalar[8];
} hodu_rocm_epilogue_step;
#define HODU_ROCM_DECL_PRODUCT_EX(dt)                                                                        \
    int hodu_rocm_matmul_##dt##_ex(hodu_rocm_ctx *ctx, const void *lhs, const void *rhs, void *out,          \
                                   const size_t *metadata, size_t metadata_len,                              \
                                   const hodu_rocm_epilogue_step *steps, size_t n_steps);                    \
    int hodu_rocm_dot_##dt##_ex(hodu_rocm_ctx *ctx, const void *lhs, const void *rhs, void *out,             \
                                const size_t *metadata, size_t metadata_len,                                 \
                                const hodu_rocm_epilogue_step *steps, size_t n_steps);
HODU_ROCM_DECL_PRODUCT_EX(bf16)
HODU_ROCM_DECL_PRODUCT_EX(f16)
HODU_ROCM_DECL_PRODUCT_EX(f32)
HODU_ROCM_DECL_PRODUCT_EX(f64)
HODU_ROCM_DECL_PRODUCT_EX(u8)
HODU_ROCM_DECL_PRODUCT_EX(u16)
HODU_ROCM_DECL_PRODUCT_EX(u32)
HODU_ROCM_DECL_PRODUCT_EX(u64)
HODU_ROCM_DECL_PRODUCT_EX(i8)
HODU_ROCM_DECL_PRODUCT_EX(i16)
HODU_ROCM_DECL_PRODUCT_EX(i32)
HODU_ROCM_DECL_PRODUCT_EX(i64)
HODU_ROCM_DECL_PRODUCT_EX(bf16_f8e4m3w) /* vector / scalar in bf16 */
HODU_ROCM_DECL_PRODUCT_EX(i32_i8i8)     /* vector / scalar in i32 */
/* ---- casts and strided gather ------------------------------------------------------------------ *
 * replaces hodu_cpu_cast_<src>_to_<dst> (kernels/ops_cast.c:53, table :108-388) and
 * hodu_cpu_contiguous_<dt> (kernels/ops_memory.c:36).  One entry point taking dtype ids stands
 * for the 225 + 15 symbols; a Rust wrapper maps the kernel-name string to the two ids the way
 * crates/hodu_cpu_kernels/src/kernels/ops_cast.rs:70-81 maps it to a function pointer.           */
int hodu_rocm_cast(hodu_rocm_ctx *ctx, int src_dtype, int dst_dtype, const void *in, void *out,
                   const size_t *metadata, size_t metadata_len);
int hodu_rocm_contiguous(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out,
                         const size_t *metadata, size_t metadata_len);

/* ---- sum over dims (the reduce that the matmul gradient needs) ----------------------------------- *
 * replaces hodu_cpu_sum_<dt> (kernels/ops_reduce.c:47-118 macro, instantiations :127-130, :133-237, :345-352) for
 * the use Tensor::sum_to_shape makes of it on a matmul's gradients when an operand was broadcast
 * (tensor/gradient/vjp_matrix.rs:41-43, tensor/ops/reduce.rs:19-50).  metadata is reduce_metadata
 * (op_metadatas.rs:525-586): [nd, shape.., strides.., offset, out_nd, out_shape.., n_reduce, reduce_dims..,
 * keep_dim, reduce_size]; any strided input, output contiguous in out_shape.  Narrow floats and f32 accumulate in
 * f32 and round once on store, f64 in f64, integers wrap.  One entry point taking the dtype id, as for the casts. */
int hodu_rocm_sum(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const size_t *metadata,
                  size_t metadata_len);

/* ---- softmax along one dim (the step between attention's two products) ------------------------------ *
 * Tensor::softmax (crates/hodu_core/src/tensor/ops/normalization.rs:4-21) is max(keep_dim), sub, exp, sum(keep_dim),
 * div in the reference: five kernels (hodu_cpu_max_<dt>, _sub_, _exp_, _sum_, _div_), five passes, a rounding to the
 * storage type after each.  This is the same function as one kernel with one rounding: elements widened to f32 (f64
 * stays f64), exp and sum in that type, RNE on store.  metadata: reduce_metadata (op_metadatas.rs:525-586) of the
 * input layout with the softmax dim as the one reduced dim -- what the reference hands its max / sum kernels; the
 * output is contiguous in the INPUT's shape.  Any dim (dense rows of the last dim up to 4096 long stay in registers,
 * longer ones take two passes; another dim gets a thread per position of the other dims).  causal != 0 (last dim of
 * a matrix only) treats entries j > i of every [.., Sq, Sk] matrix as -inf before the softmax:
 * scaled_dot_product_attention's masked_fill with create_causal_mask (crates/hodu_nn/src/modules/attention.rs:40-48,
 * :73-86) without building the mask.  dtypes: bf16, f16, f32, f64. */
int hodu_rocm_softmax(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const size_t *metadata,
                      size_t metadata_len, int causal);

/* The same along the last dim with scaled_dot_product_attention's attn_mask (crates/hodu_nn/src/modules/attention.rs:
 * 50-56: masked_fill(mask.eq_scalar(0), get_neg_inf(dtype)) in front of the softmax) folded in; causal as above, both
 * may be given.  mask: device storage of a bool / u8 / i8 tensor, 0 = masked out; mask_layout (host): [nd, strides
 * (nd).., offset] in elements over the INPUT's shape, stride 0 where the mask is broadcast (a [B, 1, 1, Sk] padding
 * mask, a [Sq, Sk] mask shared by every head) -- the mask is read in place, never expanded.  Masked scores count as
 * what the reference fills them with: -inf in f32 / f64, the dtype's rounding of -65504 in f16 / bf16 (:88-96), so a
 * masked entry of a row that has an open one is an exact zero, a row masked entirely is uniform (16-bit types) or NaN
 * (f32 / f64).  A mask of another dtype is cast by the caller with hodu_rocm_cast to bool (x != 0: -0.0 masks, a NaN attends, as eq_scalar(0) has it). */
int hodu_rocm_softmax_masked(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const size_t *metadata,
                             size_t metadata_len, int causal, const void *mask, int mask_dtype,
                             const size_t *mask_layout, size_t mask_layout_len);

/* ---- attention as one kernel --------------------------------------------------------------------------- *
 * out = softmax(q k^T * scale [causal]) v for q [batch.., Sq, D], k and v [batch.., Sk, D]: what
 * scaled_dot_product_attention (crates/hodu_nn/src/modules/attention.rs:25-70) computes with a batched matmul,
 * mul_scalar, masked_fill, the five softmax kernels and a second batched matmul, without attn_mask and dropout.  The
 * scores never leave the chip: scores and probabilities stay in f32 (the reference rounds them to the storage type
 * after every kernel), the output is rounded once.  Takes bf16 / f16, D = 64 or 128, dense head dims, rows / offsets /
 * batch strides that are multiples of 8 elements, a positive finite scale (the row maximum is taken before the scale
 * is applied); returns HODU_ROCM_UNSUPPORTED otherwise, and the caller runs the
 * three launches (hodu_rocm_matmul_<dt>_ex with MUL_SCALAR, hodu_rocm_softmax, hodu_rocm_matmul_<dt>).
 * metadata (this library's own): [nb, batch_shape (nb).., Sq, Sk, D, q_strides (nb + 2).., k_strides (nb + 2)..,
 * v_strides (nb + 2).., q_off, k_off, v_off], strides and offsets in elements, batch dims already broadcast (stride
 * 0 where an operand lacks the dim).  scale: the scalar in `dtype` (what mul_scalar receives); causal != 0 masks
 * key j > query i.  out: contiguous [batch.., Sq, D]. */
int hodu_rocm_attention(hodu_rocm_ctx *ctx, int dtype, const void *q, const void *k, const void *v, void *out,
                        const size_t *metadata, size_t metadata_len, const void *scale, int causal);

/* The same with scaled_dot_product_attention's attn_mask (crates/hodu_nn/src/modules/attention.rs:50-56:
 * masked_fill(mask.eq_scalar(0), get_neg_inf(dtype)) over the scaled scores) as part of the one kernel.  mask, mask_dtype:
 * as for hodu_rocm_softmax_masked; mask_layout (host): [nd, strides (nd).., offset] in elements over the SCORES' shape
 * [batch.., Sq, Sk] (nd = nb + 2), stride 0 where the mask is broadcast -- read in place, never expanded.  A masked
 * score counts as what the reference fills it with in a 16-bit type (:88-96: the dtype's rounding of -65504, a finite
 * value), the causal mask likewise when both are given: a row with an open key gives its masked keys weight exp(fill -
 * max) = 0, a row masked entirely is the uniform average over all Sk keys, as in the reference.  Same conditions and
 * the same HODU_ROCM_UNSUPPORTED as hodu_rocm_attention; the caller's other path is hodu_rocm_matmul_<dt>_ex with
 * MUL_SCALAR, hodu_rocm_softmax_masked, hodu_rocm_matmul_<dt>. */
int hodu_rocm_attention_masked(hodu_rocm_ctx *ctx, int dtype, const void *q, const void *k, const void *v, void *out,
                               const size_t *metadata, size_t metadata_len, const void *scale, int causal,
                               const void *mask, int mask_dtype, const size_t *mask_layout, size_t mask_layout_len);

#ifdef __cplusplus
}
#endif
#endif /* HODU_ROCM_KERNELS_H */
