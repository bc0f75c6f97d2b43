// extern "C" compute entry points: metadata parsing, kernel-family selection, launch.
#include "common.hpp"

#include <cstring>

namespace hodu {
namespace {

int check_ptrs(const char *op, hodu_rocm_ctx *ctx, const void *a, const void *b, const void *out) {
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "%s: context is null", op);
    if (!a || !b || !out) return fail(HODU_ROCM_INVALID_ARG, "%s: null operand pointer", op);
    if (out == a || out == b) return fail(HODU_ROCM_INVALID_ARG, "%s: out aliases an input", op);
    return HODU_ROCM_OK;
}

// the bandwidth-bound families for few rows on the left
int dispatch_few_rows(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    int rc = launch_inner_product(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    rc = launch_gemv(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    rc = launch_skinny(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    return launch_gemv_rows(ctx, kind, dtype, a, b, c, g);
}

// Picks the kernel family for one launch-sized product.
int dispatch_one(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c,
                 const DevProduct &g) {
    if (ctx->reference_sums) {
        const int rc = launch_reference_sums(ctx, kind, dtype, a, b, c, g);
        if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    }
    // A matrix times a vector, [M, K] x [K, 1] (what Tensor::matmul makes of a 2-D and a 1-D tensor,
    // crates/hodu_core/src/tensor/ops/matrix.rs:50-66), is the transposed problem of one row against the matrix as
    // the weight, [1, K] x [K, M], and the [M, 1] output is the same memory as [1, M]: the few-rows kernels take it.
    // Fused steps go along: they are element-wise, and a vector added along an output row of one element is that one
    // element for every output (stride 0 in the transposed problem).
    if (g.N == 1 && g.M > 1 && g.batches == 1 && kind == PK_SAME && ctx->force_tile < 0) {
        DevProduct t = g;
        t.M = 1; t.N = g.M;
        t.a_m = g.b_n; t.a_k = g.b_k; t.a_off = g.b_off;
        t.b_k = g.a_k; t.b_n = g.a_m; t.b_off = g.a_off;
        for (int i = 0; i < t.epi.n; i++)
            if (t.epi.step[i].op == HODU_ROCM_EPI_ADD_ROW) t.epi.step[i].stride = 0;
        const int rc = dispatch_few_rows(ctx, kind, dtype, b, a, c, t);
        if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    }
    int rc = ctx->force_tile >= 0 ? HODU_ROCM_UNSUPPORTED : launch_inner_product(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    rc = ctx->force_tile == 30 ? HODU_ROCM_UNSUPPORTED : launch_gemv(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    rc = launch_skinny(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    if (ctx->force_tile < 0) {  // (a pinned tile variant means the caller wants that kernel)
        rc = launch_gemv_rows(ctx, kind, dtype, a, b, c, g);
        if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    }
    rc = launch_small_f32(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    rc = launch_gemm_f64(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    rc = launch_mfma(ctx, kind, dtype, a, b, c, g);
    if (rc != HODU_ROCM_UNSUPPORTED) return rc;
    ctx->last_kernel = "generic";
    return launch_generic(ctx, kind, dtype, a, b, c, g);
}

size_t out_elem_size(int kind, int dtype) {
    if (kind == PK_BF16_F8W) return 2;
    if (kind == PK_I32_I8I8) return 4;
    return dtype_size(dtype);
}

// Splits a parsed product into launches: the innermost kKernelBatchDims merged batch dims go to
// the kernel, any further outer dims are walked here.
int run_product_launches(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const Product &p,
                         const DevEpilogue &epi) {
    HODU_HIP(hipSetDevice(ctx->device));
    if (p.M > 0x7FFFFFFFL || p.N > 0x7FFFFFFFL || p.K > 0x7FFFFFFFL)
        return fail(HODU_ROCM_UNSUPPORTED, "matrix extent exceeds 2^31-1");
    if (p.batches == 0 || p.M == 0 || p.N == 0) return HODU_ROCM_OK;  // empty output: nothing to write

    DevProduct g{};
    g.epi = epi;
    g.M = (int)p.M; g.N = (int)p.N; g.K = (int)p.K;
    g.a_m = p.a_m; g.a_k = p.a_k; g.b_k = p.b_k; g.b_n = p.b_n;
    const int inner = p.nb < kKernelBatchDims ? p.nb : kKernelBatchDims;
    const int outer = p.nb - inner;
    g.nb = inner;
    g.batches = 1;
    for (int d = 0; d < inner; d++) {
        if (p.bshape[outer + d] > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "batch extent exceeds 2^31-1");
        g.bshape[d] = (int)p.bshape[outer + d];
        g.a_bs[d] = p.a_bs[outer + d];
        g.b_bs[d] = p.b_bs[outer + d];
        g.batches *= p.bshape[outer + d];
    }
    long outer_count = 1;
    for (int d = 0; d < outer; d++) outer_count *= p.bshape[d];
    const size_t out_step = (size_t)g.batches * (size_t)p.M * (size_t)p.N * out_elem_size(kind, dtype);
    for (long o = 0; o < outer_count; o++) {
        long rem = o, ao = p.a_off, bo = p.b_off;
        for (int d = outer - 1; d >= 0; d--) {
            const long i = rem % p.bshape[d];
            rem /= p.bshape[d];
            ao += i * p.a_bs[d];
            bo += i * p.b_bs[d];
        }
        g.a_off = ao; g.b_off = bo;
        int rc = dispatch_one(ctx, kind, dtype, a, b, (char *)c + (size_t)o * out_step, g);
        if (rc != HODU_ROCM_OK) return rc;
    }
    return HODU_ROCM_OK;
}

int run_product(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const Product &p,
                const DevEpilogue &epi) {
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    const int rc = run_product_launches(ctx, kind, dtype, a, b, c, p, epi);
    // A launch that failed may have left arrival counters half counted (a kernel cut along K puts its counter back
    // to zero only when its last workgroup finishes): zero them before the next kernel that relies on them.
    if (rc == HODU_ROCM_HIP_ERROR || rc == HODU_ROCM_OOM) ctx->arrival_stale = true;
    return rc;
}

// Validates the caller's fused steps for an output of `dtype` and turns them into what the kernels read.
int build_epilogue(const char *op, int kind, int dtype, const void *out, const hodu_rocm_epilogue_step *steps, size_t n,
                   DevEpilogue *epi) {
    *epi = DevEpilogue{};
    if (n == 0) return HODU_ROCM_OK;
    if (!steps) return fail(HODU_ROCM_INVALID_ARG, "%s: %zu fused steps but the step array is null", op, n);
    if (n > (size_t)kMaxEpilogueSteps)
        return fail(HODU_ROCM_INVALID_ARG, "%s: %zu fused steps, at most %d", op, n, kMaxEpilogueSteps);
    const int out_dtype = kind == PK_BF16_F8W ? HODU_BF16 : kind == PK_I32_I8I8 ? HODU_I32 : dtype;
    if (out_dtype == HODU_F8E4M3 || out_dtype == HODU_F8E5M2 || out_dtype == HODU_BOOL)
        return fail(HODU_ROCM_UNSUPPORTED, "%s: fused steps are not defined for dtype id %d", op, out_dtype);
    const bool floating = out_dtype == HODU_BF16 || out_dtype == HODU_F16 || out_dtype == HODU_F32 || out_dtype == HODU_F64;
    const size_t es = dtype_size(out_dtype);
    for (size_t i = 0; i < n; i++) {
        DevEpilogueStep &d = epi->step[i];
        d = DevEpilogueStep{};
        d.op = steps[i].op;
        switch (steps[i].op) {
        case HODU_ROCM_EPI_ADD_ROW:
            if (!steps[i].vector) return fail(HODU_ROCM_INVALID_ARG, "%s: step %zu adds a null vector", op, i);
            if (steps[i].vector == out) return fail(HODU_ROCM_INVALID_ARG, "%s: step %zu reads the output buffer", op, i);
            if (steps[i].stride > 0x7FFFFFFFFFFFL || steps[i].offset > 0x7FFFFFFFFFFFL)
                return fail(HODU_ROCM_INVALID_ARG, "%s: step %zu stride/offset out of range", op, i);
            d.vec = (const char *)steps[i].vector + steps[i].offset * es;
            d.stride = (long)steps[i].stride;
            break;
        case HODU_ROCM_EPI_MUL_SCALAR:
            memcpy(&d.scalar, steps[i].scalar, es);  // low bytes; the rest stays zero
            break;
        case HODU_ROCM_EPI_RELU:
            if (!floating) return fail(HODU_ROCM_INVALID_ARG, "%s: relu is defined for floating dtypes only", op);
            break;
        default: return fail(HODU_ROCM_INVALID_ARG, "%s: step %zu has unknown op %d", op, i, steps[i].op);
        }
    }
    epi->n = (int)n;
    return HODU_ROCM_OK;
}

int matmul_entry(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const size_t *md,
                 size_t len, const hodu_rocm_epilogue_step *steps = nullptr, size_t n_steps = 0) {
    clear_error();
    int rc = check_ptrs("matmul", ctx, a, b, c);
    if (rc) return rc;
    Product p;
    rc = parse_matmul_metadata(md, len, &p);
    if (rc) return rc;
    DevEpilogue epi;
    rc = build_epilogue("matmul", kind, dtype, c, steps, n_steps, &epi);
    if (rc) return rc;
    return run_product(ctx, kind, dtype, a, b, c, p, epi);
}

int dot_entry(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const size_t *md,
              size_t len, const hodu_rocm_epilogue_step *steps = nullptr, size_t n_steps = 0) {
    clear_error();
    int rc = check_ptrs("dot", ctx, a, b, c);
    if (rc) return rc;
    Product p;
    rc = parse_dot_metadata(md, len, &p);
    if (rc) return rc;
    DevEpilogue epi;
    rc = build_epilogue("dot", kind, dtype, c, steps, n_steps, &epi);
    if (rc) return rc;
    return run_product(ctx, kind, dtype, a, b, c, p, epi);
}

}  // namespace
}  // namespace hodu

using namespace hodu;

extern "C" {

#define HODU_ROCM_DEF_PRODUCT(dt, ID)                                                                          \
    int hodu_rocm_matmul_##dt(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md,     \
                              size_t n) {                                                                      \
        return matmul_entry(ctx, PK_SAME, ID, l, r, o, md, n);                                                 \
    }                                                                                                          \
    int hodu_rocm_dot_##dt(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md,        \
                           size_t n) {                                                                         \
        return dot_entry(ctx, PK_SAME, ID, l, r, o, md, n);                                                    \
    }
HODU_ROCM_DEF_PRODUCT(f8e4m3, HODU_F8E4M3)
HODU_ROCM_DEF_PRODUCT(f8e5m2, HODU_F8E5M2)
HODU_ROCM_DEF_PRODUCT(bf16, HODU_BF16)
HODU_ROCM_DEF_PRODUCT(f16, HODU_F16)
HODU_ROCM_DEF_PRODUCT(f32, HODU_F32)
HODU_ROCM_DEF_PRODUCT(f64, HODU_F64)
HODU_ROCM_DEF_PRODUCT(u8, HODU_U8)
HODU_ROCM_DEF_PRODUCT(u16, HODU_U16)
HODU_ROCM_DEF_PRODUCT(u32, HODU_U32)
HODU_ROCM_DEF_PRODUCT(u64, HODU_U64)
HODU_ROCM_DEF_PRODUCT(i8, HODU_I8)
HODU_ROCM_DEF_PRODUCT(i16, HODU_I16)
HODU_ROCM_DEF_PRODUCT(i32, HODU_I32)
HODU_ROCM_DEF_PRODUCT(i64, HODU_I64)

int hodu_rocm_matmul_bf16_f8e4m3w(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md,
                                  size_t n) {
    return matmul_entry(ctx, PK_BF16_F8W, HODU_BF16, l, r, o, md, n);
}
int hodu_rocm_dot_bf16_f8e4m3w(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md,
                               size_t n) {
    return dot_entry(ctx, PK_BF16_F8W, HODU_BF16, l, r, o, md, n);
}
int hodu_rocm_matmul_i32_i8i8(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md,
                              size_t n) {
    return matmul_entry(ctx, PK_I32_I8I8, HODU_I32, l, r, o, md, n);
}
int hodu_rocm_dot_i32_i8i8(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md, size_t n) {
    return dot_entry(ctx, PK_I32_I8I8, HODU_I32, l, r, o, md, n);
}

int hodu_rocm_ctx_set_reference_sums(hodu_rocm_ctx *ctx, int on) {
    clear_error();
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "set_reference_sums: context is null");
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    ctx->reference_sums = on != 0;
    return HODU_ROCM_OK;
}

// The one entry point that allocates nothing: hodu_rocm_dot_bf16_f8e4m3w with the partial sums and arrival counters
// of its split-K kernels in the device's static scratch array instead of the context's workspace.  For the length
// of the call the context's workspace / counters are pointed at that array and marked fixed, so a kernel choice that
// needs more is refused (ensure_workspace) rather than grown.  The array is shared by every call on this GPU and
// keeps whatever the last one left, so its counters are marked stale: the kernel that counts on them zeroes them first
// (ensure_arrival, one small launch), and a product whose kernel uses no counter -- the M <= 4 decode shapes -- pays
// nothing for them.
int hodu_rocm_dot_bf16_f8e4m3w_noalloc(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md,
                                       size_t n) {
    clear_error();
    int rc = check_ptrs("dot", ctx, l, r, o);
    if (rc) return rc;
    Product p;
    rc = parse_dot_metadata(md, n, &p);
    if (rc) return rc;
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    if (!ctx->static_scratch) return fail(HODU_ROCM_HIP_ERROR, "dot: the static scratch is not set up on this context");
    const Workspace saved_ws = ctx->workspace;
    int *const saved_arrival = ctx->arrival;
    ctx->workspace.ptr = (char *)ctx->static_scratch + kStaticArrivalBytes;
    ctx->workspace.bytes = kStaticPartialBytes;
    ctx->arrival = (int *)ctx->static_scratch;
    const bool saved_stale = ctx->arrival_stale;
    ctx->fixed_scratch = true;
    ctx->arrival_stale = true;
    rc = run_product(ctx, PK_BF16_F8W, HODU_BF16, l, r, o, p, DevEpilogue{});
    ctx->workspace = saved_ws;
    ctx->arrival = saved_arrival;
    ctx->arrival_stale = saved_stale;
    ctx->fixed_scratch = false;
    return rc;
}

#define HODU_ROCM_DEF_PRODUCT_EX(dt, KIND, ID)                                                                  \
    int hodu_rocm_matmul_##dt##_ex(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md, \
                                   size_t n, const hodu_rocm_epilogue_step *steps, size_t n_steps) {           \
        return matmul_entry(ctx, KIND, ID, l, r, o, md, n, steps, n_steps);                                    \
    }                                                                                                          \
    int hodu_rocm_dot_##dt##_ex(hodu_rocm_ctx *ctx, const void *l, const void *r, void *o, const size_t *md,    \
                                size_t n, const hodu_rocm_epilogue_step *steps, size_t n_steps) {              \
        return dot_entry(ctx, KIND, ID, l, r, o, md, n, steps, n_steps);                                       \
    }
HODU_ROCM_DEF_PRODUCT_EX(bf16, PK_SAME, HODU_BF16)
HODU_ROCM_DEF_PRODUCT_EX(f16, PK_SAME, HODU_F16)
HODU_ROCM_DEF_PRODUCT_EX(f32, PK_SAME, HODU_F32)
HODU_ROCM_DEF_PRODUCT_EX(f64, PK_SAME, HODU_F64)
HODU_ROCM_DEF_PRODUCT_EX(u8, PK_SAME, HODU_U8)
HODU_ROCM_DEF_PRODUCT_EX(u16, PK_SAME, HODU_U16)
HODU_ROCM_DEF_PRODUCT_EX(u32, PK_SAME, HODU_U32)
HODU_ROCM_DEF_PRODUCT_EX(u64, PK_SAME, HODU_U64)
HODU_ROCM_DEF_PRODUCT_EX(i8, PK_SAME, HODU_I8)
HODU_ROCM_DEF_PRODUCT_EX(i16, PK_SAME, HODU_I16)
HODU_ROCM_DEF_PRODUCT_EX(i32, PK_SAME, HODU_I32)
HODU_ROCM_DEF_PRODUCT_EX(i64, PK_SAME, HODU_I64)
HODU_ROCM_DEF_PRODUCT_EX(bf16_f8e4m3w, PK_BF16_F8W, HODU_BF16)
HODU_ROCM_DEF_PRODUCT_EX(i32_i8i8, PK_I32_I8I8, HODU_I32)

int hodu_rocm_cast(hodu_rocm_ctx *ctx, int src, int dst, const void *in, void *out, const size_t *md, size_t len) {
    clear_error();
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "cast: context is null");
    if (!in || !out) return fail(HODU_ROCM_INVALID_ARG, "cast: null operand pointer");
    if (in == out) return fail(HODU_ROCM_INVALID_ARG, "cast: out aliases the input");
    if (dtype_size(src) == 0 || dtype_size(dst) == 0)
        return fail(HODU_ROCM_UNSUPPORTED, "cast: unknown dtype id (%d -> %d)", src, dst);
    Strided s;
    int rc = parse_cast_metadata(md, len, &s);
    if (rc) return rc;
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    return launch_cast(ctx, src, dst, in, out, s);
}

int hodu_rocm_sum(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const size_t *md, size_t len) {
    clear_error();
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "sum: context is null");
    if (!in || !out) return fail(HODU_ROCM_INVALID_ARG, "sum: null operand pointer");
    if (in == out) return fail(HODU_ROCM_INVALID_ARG, "sum: out aliases the input");
    if (dtype_size(dtype) == 0 || dtype == HODU_BOOL) return fail(HODU_ROCM_UNSUPPORTED, "sum: dtype id %d has no sum kernel", dtype);
    Reduction r;
    int rc = parse_reduce_metadata(md, len, &r);
    if (rc) return rc;
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    return launch_sum(ctx, dtype, in, out, r);
}

int hodu_rocm_softmax(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const size_t *md, size_t len, int causal) {
    clear_error();
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "softmax: context is null");
    if (!in || !out) return fail(HODU_ROCM_INVALID_ARG, "softmax: null operand pointer");
    if (in == out) return fail(HODU_ROCM_INVALID_ARG, "softmax: out aliases the input");
    Reduction r;
    int rc = parse_reduce_metadata(md, len, &r);
    if (rc) return rc;
    const size_t nd = md[0], out_nd = md[2 + 2 * nd], n_red = md[3 + 2 * nd + out_nd];
    if (n_red != 1) return fail(HODU_ROCM_INVALID_ARG, "softmax: exactly one dim, got %zu", n_red);
    const size_t dim = md[4 + 2 * nd + out_nd];
    if (dim >= nd) return fail(HODU_ROCM_INVALID_ARG, "softmax: dim %zu of a %zu-d tensor", dim, nd);
    const bool last = dim + 1 == nd;
    if (causal && (!last || nd < 2)) return fail(HODU_ROCM_INVALID_ARG, "softmax: the causal mask needs the last dim of a matrix");
    long inner = 1;  // extents after the softmax dim
    for (size_t d = dim + 1; d < nd; d++) inner *= (long)md[1 + d];
    if (inner == 0) return HODU_ROCM_OK;
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    return launch_softmax(ctx, dtype, in, out, r, inner, causal ? 1 : 0, nd >= 2 ? (long)md[1 + nd - 2] : 1);
}

int hodu_rocm_softmax_masked(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const size_t *md, size_t len,
                             int causal, const void *mask, int mask_dtype, const size_t *mask_layout, size_t mask_layout_len) {
    clear_error();
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "softmax: context is null");
    if (!in || !out || !mask) return fail(HODU_ROCM_INVALID_ARG, "softmax: null operand pointer");
    if (in == out || mask == out) return fail(HODU_ROCM_INVALID_ARG, "softmax: out aliases an input");
    if (mask_dtype != HODU_BOOL && mask_dtype != HODU_U8 && mask_dtype != HODU_I8)
        return fail(HODU_ROCM_UNSUPPORTED, "softmax: the mask is one byte per element (bool, u8 or i8), got dtype id %d", mask_dtype);
    Reduction r;
    int rc = parse_reduce_metadata(md, len, &r);
    if (rc) return rc;
    const size_t nd = md[0], out_nd = md[2 + 2 * nd], n_red = md[3 + 2 * nd + out_nd];
    if (nd < 1 || n_red != 1 || md[4 + 2 * nd + out_nd] + 1 != nd)
        return fail(HODU_ROCM_INVALID_ARG, "softmax: a mask applies to the last dim of the input");
    if (!mask_layout || mask_layout_len != nd + 2 || mask_layout[0] != nd)
        return fail(HODU_ROCM_INVALID_ARG, "softmax: the mask layout is [nd, strides (nd).., offset] over the input's %zu dims", nd);
    long shape[16], in_strides[16], mask_strides[16];
    for (size_t d = 0; d < nd; d++) {
        if (mask_layout[1 + d] > 0x7FFFFFFFFFFFL) return fail(HODU_ROCM_INVALID_ARG, "softmax: mask stride %zu out of range", d);
        shape[d] = (long)md[1 + d];
        in_strides[d] = (long)md[1 + nd + d];
        mask_strides[d] = (long)mask_layout[1 + d];
    }
    if (mask_layout[1 + nd] > 0x7FFFFFFFFFFFL) return fail(HODU_ROCM_INVALID_ARG, "softmax: mask offset out of range");
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    return launch_softmax_masked(ctx, dtype, in, out, mask, (int)nd, shape, in_strides, (long)md[1 + 2 * nd], mask_strides,
                                 (long)mask_layout[1 + nd], causal ? 1 : 0);
}

static int attention_entry(hodu_rocm_ctx *ctx, int dtype, const void *q, const void *k, const void *v, void *out,
                           const size_t *md, size_t len, const void *scale, int causal, const void *mask, int mask_dtype,
                           const size_t *mask_layout, size_t mask_layout_len, bool masked) {
    clear_error();
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "attention: context is null");
    if (!q || !k || !v || !out || !scale) return fail(HODU_ROCM_INVALID_ARG, "attention: null pointer");
    if (out == q || out == k || out == v) return fail(HODU_ROCM_INVALID_ARG, "attention: out aliases an input");
    AttentionArgs a;
    int rc = parse_attention_metadata(md, len, &a);
    if (rc) return rc;
    AttentionMask m;
    if (masked) {
        if (!mask) return fail(HODU_ROCM_INVALID_ARG, "attention: null mask pointer");
        if (mask == out) return fail(HODU_ROCM_INVALID_ARG, "attention: out aliases the mask");
        if (mask_dtype != HODU_BOOL && mask_dtype != HODU_U8 && mask_dtype != HODU_I8)
            return fail(HODU_ROCM_UNSUPPORTED, "attention: the mask is one byte per element (bool, u8 or i8), got dtype id %d", mask_dtype);
        const size_t nd = (size_t)a.nb + 2;
        if (!mask_layout || mask_layout_len != nd + 2 || mask_layout[0] != nd)
            return fail(HODU_ROCM_INVALID_ARG, "attention: the mask layout is [nd, strides (nd).., offset] over the %zu dims of the scores", nd);
        for (size_t i = 1; i < nd + 2; i++)
            if (mask_layout[i] > 0x7FFFFFFFFFFFL) return fail(HODU_ROCM_INVALID_ARG, "attention: mask layout[%zu] out of range", i);
        m.ptr = mask;
        for (int d = 0; d < a.nb; d++) m.bs[d] = (long)mask_layout[1 + d];
        m.row = (long)mask_layout[1 + a.nb];
        m.key = (long)mask_layout[2 + a.nb];
        m.off = (long)mask_layout[1 + nd];
    }
    if (dtype == HODU_BF16) {
        uint16_t h;
        memcpy(&h, scale, 2);
        uint32_t u = (uint32_t)h << 16;
        memcpy(&a.scale, &u, 4);
    } else if (dtype == HODU_F16) {
        _Float16 h;
        memcpy(&h, scale, 2);
        a.scale = (float)h;
    } else {
        return fail(HODU_ROCM_UNSUPPORTED, "attention: the fused kernel takes bf16 and f16 (dtype id %d)", dtype);
    }
    a.causal = causal != 0;
    if (a.batches == 0 || a.sq == 0) return HODU_ROCM_OK;
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    rc = launch_attention(ctx, dtype, q, k, v, out, a, masked ? &m : nullptr);
    if (rc == HODU_ROCM_UNSUPPORTED)
        return fail(HODU_ROCM_UNSUPPORTED, "attention: the fused kernel needs head dim 64 or 128, at most %d batch dims, 16-byte aligned rows and a positive finite scale",
                    kKernelBatchDims);
    return rc;
}

int hodu_rocm_attention(hodu_rocm_ctx *ctx, int dtype, const void *q, const void *k, const void *v, void *out,
                        const size_t *md, size_t len, const void *scale, int causal) {
    return attention_entry(ctx, dtype, q, k, v, out, md, len, scale, causal, nullptr, 0, nullptr, 0, false);
}

int hodu_rocm_attention_masked(hodu_rocm_ctx *ctx, int dtype, const void *q, const void *k, const void *v, void *out,
                               const size_t *md, size_t len, const void *scale, int causal, const void *mask, int mask_dtype,
                               const size_t *mask_layout, size_t mask_layout_len) {
    return attention_entry(ctx, dtype, q, k, v, out, md, len, scale, causal, mask, mask_dtype, mask_layout, mask_layout_len, true);
}

int hodu_rocm_contiguous(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const size_t *md, size_t len) {
    clear_error();
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "contiguous: context is null");
    if (!in || !out) return fail(HODU_ROCM_INVALID_ARG, "contiguous: null operand pointer");
    if (in == out) return fail(HODU_ROCM_INVALID_ARG, "contiguous: out aliases the input");
    if (dtype_size(dtype) == 0) return fail(HODU_ROCM_UNSUPPORTED, "contiguous: unknown dtype id %d", dtype);
    Strided s;
    int rc = parse_cast_metadata(md, len, &s);
    if (rc) return rc;
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    return launch_gather(ctx, dtype, in, out, s);
}

}  // extern "C"
