// Internal declarations shared by the translation units of libhodu_rocm_kernels.so.
#pragma once

#include <hip/hip_runtime.h>

#include <mutex>

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <string>

#include "hodu_rocm_kernels.h"

namespace hodu {

// ------------------------------------------------------------------------------------------------
// context
// ------------------------------------------------------------------------------------------------
struct Workspace {
    void *ptr = nullptr;
    size_t bytes = 0;
};

}  // namespace hodu

struct hodu_rocm_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t props{};
    hodu::Workspace workspace;  // split-K partial sums; grown on demand, owned by the context
    int *arrival = nullptr;     // kArrivalSlots zeroed counters for kernels whose last workgroup finishes a reduction
    // The counters `arrival` points at may hold something other than zeros (fresh memory; a launch that failed part
    // way; the shared static array, which keeps what the last call on this GPU left): ensure_arrival zeroes them, by
    // a kernel in stream order, before the next kernel that counts on them -- and only then.
    bool arrival_stale = false;
    // Set for the duration of a call that must not allocate: `workspace` and `arrival` then point into the
    // device's static scratch array, and a kernel that needs more than it holds is refused instead of grown.
    bool fixed_scratch = false;
    void *static_scratch = nullptr;  // this device's copy of the static scratch array (hipGetSymbolAddress)
    bool reference_sums = false;  // narrow-float products re-round after every multiply and add, as the reference's do
    const char *last_kernel = "";
    int force_tile = -1;    // testing hook: pins the MFMA tile size
    int force_splits = -1;  // testing hook: pins the number of K ranges of the pipelined kernels (1 = never split)
    char kernel_name[96] = {0};  // storage for a composed last_kernel name
    // kernels whose dynamic-LDS limit has been raised on THIS context's device (the attribute belongs to a
    // function on a device; a second context on another device has to set it again).  A fixed open-addressed
    // table: recording a kernel allocates nothing, so entry points that must not allocate can share it.
    static constexpr int kLdsSlots = 1024;
    const void *lds_configured[kLdsSlots] = {};
    // every entry point that launches kernels holds this for the call: the workspace, the arrival counters, the
    // testing hooks and last_kernel belong to the context, and launches of one context go to one stream anyway
    std::recursive_mutex mu;
};

namespace hodu {

// per-thread error text (any host thread may call into one context)
void set_error(const char *fmt, ...);
const char *get_error();
void clear_error();

int fail(int code, const char *fmt, ...);

#define HODU_HIP(expr)                                                                         \
    do {                                                                                       \
        hipError_t _e = (expr);                                                                \
        if (_e != hipSuccess)                                                                  \
            return ::hodu::fail(_e == hipErrorOutOfMemory ? HODU_ROCM_OOM : HODU_ROCM_HIP_ERROR, \
                                "%s: %s", #expr, hipGetErrorString(_e));                       \
    } while (0)

// raises a kernel's dynamic-LDS limit once per context (called with ctx->mu held, like every launch)
inline int ensure_dynamic_lds(hodu_rocm_ctx *ctx, const void *kernel, int bytes) {
    constexpr int N = hodu_rocm_ctx::kLdsSlots;
    unsigned h = (unsigned)(((uintptr_t)kernel >> 4) * 2654435761u) % N;
    for (int probe = 0; probe < N; probe++, h = (h + 1) % N) {
        if (ctx->lds_configured[h] == kernel) return HODU_ROCM_OK;
        if (ctx->lds_configured[h] == nullptr) break;
    }
    HODU_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    if (ctx->lds_configured[h] == nullptr) ctx->lds_configured[h] = kernel;  // a full table only repeats the call
    return HODU_ROCM_OK;
}

// grows ctx->workspace to at least `bytes` (refused, with an error text, while ctx->fixed_scratch is set and the
// static scratch is smaller, or while the context's stream is being captured into a graph and it would have to grow)
int ensure_workspace(hodu_rocm_ctx *ctx, size_t bytes);
// allocates ctx->arrival (once) and zeroes the counters whenever ctx->arrival_stale says they may not be zero; a
// kernel that uses a counter leaves it at zero again, so a launch that runs to completion keeps them clean.  Every
// kernel that counts arrivals calls this right before its launch.
constexpr int kArrivalSlots = 4096;
int ensure_arrival(hodu_rocm_ctx *ctx);

// The static scratch array of the entry point that allocates nothing: kArrivalSlots counters, then partial sums.
constexpr size_t kStaticArrivalBytes = (size_t)kArrivalSlots * sizeof(int);
constexpr size_t kStaticPartialBytes = (size_t)8 << 20;
constexpr size_t kStaticScratchBytes = kStaticArrivalBytes + kStaticPartialBytes;

inline size_t dtype_size(int dt) {
    static const size_t sz[15] = {1, 1, 1, 2, 2, 4, 8, 1, 2, 4, 8, 1, 2, 4, 8};
    return (dt >= 0 && dt < 15) ? sz[dt] : 0;
}

// ------------------------------------------------------------------------------------------------
// parsed product problem: `batches` independent (M x K)(K x N) products
// ------------------------------------------------------------------------------------------------
constexpr int kMaxBatchDims = 16;  // the reference kernels index batch_indices[16] (ops_matrix.c:152)
constexpr int kKernelBatchDims = 4; // innermost merged batch dims a single launch decomposes

struct Product {
    long M = 0, N = 0, K = 0;
    long a_m = 0, a_k = 0, b_k = 0, b_n = 0;  // element strides of the two matrix dims
    long a_off = 0, b_off = 0;                // element offsets
    // batch space after merging: up to kMaxBatchDims dims, innermost last; stride 0 = broadcast
    int nb = 0;
    long bshape[kMaxBatchDims] = {};
    long a_bs[kMaxBatchDims] = {};
    long b_bs[kMaxBatchDims] = {};
    long batches = 1;
};

// Validates and converts the reference's metadata vectors.  Returns a status code.
int parse_matmul_metadata(const size_t *md, size_t len, Product *p);
int parse_dot_metadata(const size_t *md, size_t len, Product *p);

struct Strided {
    long n = 0;
    int nd = 0;
    long shape[16];
    long strides[16];
    long offset = 0;
    bool contiguous = false;  // reference rule: extent-1 dims do not constrain (utils.h:16-27)
};
int parse_cast_metadata(const size_t *md, size_t len, Strided *s);

// Element-wise steps applied to every output of a product before it is stored: what the callers of the product
// run next in the reference as kernels of their own (hodu_nn/src/modules/linear.rs:40-46: matmul, then add(bias);
// attention.rs:37: matmul, then mul_scalar).  A step works on the value the product alone would have stored, with
// the arithmetic of the reference's element-wise kernel for the output dtype, so the fused result equals the two
// launches' bit for bit.
enum EpilogueOp {
    EPI_ADD_ROW = 1,     // + vec[n * stride]: a vector along the output's last axis (ops_binary.c, add)
    EPI_MUL_SCALAR = 2,  // * scalar (ops_unary.c, mul_scalar; the scalar in the output dtype)
    EPI_RELU = 3         // x > 0 ? x : 0 (ops_unary.c, relu; floating dtypes only)
};
constexpr int kMaxEpilogueSteps = 3;
struct DevEpilogueStep {
    int op;
    const void *vec;            // device pointer, already offset to element 0 of the vector
    long stride;                // elements between consecutive entries of the vector
    unsigned long long scalar;  // bit pattern of the scalar, in the output dtype, in the low bytes
};
struct DevEpilogue {
    int n;  // 0: store the product as it is
    DevEpilogueStep step[kMaxEpilogueSteps];
};

// What one launch needs to know about a product; passed by value as a kernel argument.
struct DevProduct {
    int M, N, K;
    long a_m, a_k, b_k, b_n;
    long a_off, b_off;
    int nb;                        // batch dims decomposed by the kernel (<= kKernelBatchDims)
    int bshape[kKernelBatchDims];  // innermost last
    long a_bs[kKernelBatchDims];
    long b_bs[kKernelBatchDims];
    long batches;                  // product of bshape
    DevEpilogue epi;
};

// ------------------------------------------------------------------------------------------------
// kernel families (each in its own .hip file)
// ------------------------------------------------------------------------------------------------
// "kind" of a product = (lhs storage, rhs storage, out) triple
enum ProductKind {
    PK_SAME = 0,     // all three share `dtype`
    PK_BF16_F8W = 1, // bf16 x f8e4m3 -> bf16
    PK_I32_I8I8 = 2  // i8 x i8 -> i32
};

// Each launcher handles one DevProduct whose output starts at `c` (batches * M * N elements).
// generic strided kernel: every dtype, any strides; slow, always correct
int launch_generic(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c,
                   const DevProduct &g);
// the reference's narrow-type running sum (gemm_refsum.hip): returns HODU_ROCM_UNSUPPORTED for dtypes it is not for
int launch_reference_sums(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c,
                          const DevProduct &g);
// MFMA tile kernel: returns HODU_ROCM_UNSUPPORTED (without setting an error) when it has no variant
int launch_mfma(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c,
                const DevProduct &g);
// bandwidth-bound small-M path: returns HODU_ROCM_UNSUPPORTED when not applicable
int launch_gemv(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g);
// small f32 products straight from memory into the matrix cores (a 32 x 32 tile per workgroup, K cut four ways inside
// it): returns HODU_ROCM_UNSUPPORTED when the product is not f32 or is large enough for the tiled kernels
int launch_small_f32(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g);
// f64 products on the f64 matrix-core instruction, operands straight from memory: returns HODU_ROCM_UNSUPPORTED for
// other dtypes
int launch_gemm_f64(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g);
int launch_skinny(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c,
                  const DevProduct &g);
// [1, K] x [K, 1] with a long K (reduce.hip)
int launch_inner_product(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g);
// at most 16 rows against a row-dense right operand (gemv_rows.hip)
int launch_gemv_rows(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g);

// A sum over some dims of a strided tensor, as the reference's reduce metadata describes it: the dims that stay
// (in input order: that is the row-major order of the output, kept extent-1 dims included or not) and the dims
// that are summed, each list with extents and element strides, adjacent dims merged where the strides allow.
struct Reduction {
    long n_out = 1;       // output elements
    long reduce_size = 1; // inputs per output
    int kept_n = 0, red_n = 0;
    long kept_shape[16], kept_stride[16];
    long red_shape[16], red_stride[16];
    long offset = 0;
};
int parse_reduce_metadata(const size_t *md, size_t len, Reduction *r);
int launch_sum(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const Reduction &r);
// softmax over the one reduced dim of `r`; dim_is_last: it is the tensor's last dim; causal: entries j > i of every
// [sq, len] matrix count as -inf
int launch_softmax(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const Reduction &r, long inner,
                   int causal, long sq);

// softmax along the last dim with an attention mask (one byte per element, 0 = masked, own strides over the input's
// shape) applied the way the reference's masked_fill + softmax applies it; causal as above
int launch_softmax_masked(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const void *mask, int nd,
                          const long *shape, const long *in_strides, long in_off, const long *mask_strides, long mask_off,
                          int causal);

// One fused attention call: q [batch.., sq, d], k and v [batch.., sk, d] (batch dims already broadcast, last dim
// dense), out contiguous [batch.., sq, d]
struct AttentionArgs {
    long sq = 0, sk = 0, d = 0;
    long q_row = 0, k_row = 0, v_row = 0;  // element strides between rows
    int nb = 0;
    long bshape[16];
    long q_bs[16], k_bs[16], v_bs[16];
    long q_off = 0, k_off = 0, v_off = 0;
    long batches = 1;
    float scale = 1.f;
    bool causal = false;
};
int parse_attention_metadata(const size_t *md, size_t len, AttentionArgs *a);
// an attn_mask read in place: one byte per element, strides (0 where broadcast) over [batch.., Sq, Sk]
struct AttentionMask {
    const void *ptr = nullptr;
    long bs[16];
    long row = 0, key = 0, off = 0;
};
// HODU_ROCM_UNSUPPORTED without an error text when the fused kernel does not take the call
int launch_attention(hodu_rocm_ctx *ctx, int dtype, const void *q, const void *k, const void *v, void *out,
                     const AttentionArgs &a, const AttentionMask *mask = nullptr);

int launch_cast(hodu_rocm_ctx *ctx, int src, int dst, const void *in, void *out, const Strided &s);
int launch_gather(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const Strided &s);

}  // namespace hodu
