// Test and measurement hooks: libhodu_rocm_debug.so, declared in include/hodu_rocm_debug.h.  Nothing here is part
// of what a hodu_rocm_kernels crate would bind; the hooks sit on top of the public entry points of
// libhodu_rocm_kernels.so (include/hodu_rocm_kernels.h) and of the context structure the two libraries share.
#include <cstring>

#include "common.hpp"
#include "hodu_rocm_debug.h"

using namespace hodu;

namespace {

typedef int (*product_fn)(hodu_rocm_ctx *, const void *, const void *, void *, const size_t *, size_t);
typedef int (*product_ex_fn)(hodu_rocm_ctx *, const void *, const void *, void *, const size_t *, size_t,
                             const hodu_rocm_epilogue_step *, size_t);

// the public entry point a (format, kind, dtype) triple names; nullptr if there is none
product_fn plain_entry(int is_matmul, int kind, int dtype) {
    if (kind == PK_BF16_F8W) return is_matmul ? hodu_rocm_matmul_bf16_f8e4m3w : hodu_rocm_dot_bf16_f8e4m3w;
    if (kind == PK_I32_I8I8) return is_matmul ? hodu_rocm_matmul_i32_i8i8 : hodu_rocm_dot_i32_i8i8;
    switch (dtype) {
#define HODU_CASE(ID, dt) case ID: return is_matmul ? hodu_rocm_matmul_##dt : hodu_rocm_dot_##dt;
    HODU_CASE(HODU_F8E4M3, f8e4m3) HODU_CASE(HODU_F8E5M2, f8e5m2) HODU_CASE(HODU_BF16, bf16) HODU_CASE(HODU_F16, f16)
    HODU_CASE(HODU_F32, f32) HODU_CASE(HODU_F64, f64) HODU_CASE(HODU_U8, u8) HODU_CASE(HODU_U16, u16)
    HODU_CASE(HODU_U32, u32) HODU_CASE(HODU_U64, u64) HODU_CASE(HODU_I8, i8) HODU_CASE(HODU_I16, i16)
    HODU_CASE(HODU_I32, i32) HODU_CASE(HODU_I64, i64)
#undef HODU_CASE
    default: return nullptr;
    }
}
product_ex_fn ex_entry(int is_matmul, int kind, int dtype) {
    if (kind == PK_BF16_F8W) return is_matmul ? hodu_rocm_matmul_bf16_f8e4m3w_ex : hodu_rocm_dot_bf16_f8e4m3w_ex;
    if (kind == PK_I32_I8I8) return is_matmul ? hodu_rocm_matmul_i32_i8i8_ex : hodu_rocm_dot_i32_i8i8_ex;
    switch (dtype) {
#define HODU_CASE(ID, dt) case ID: return is_matmul ? hodu_rocm_matmul_##dt##_ex : hodu_rocm_dot_##dt##_ex;
    HODU_CASE(HODU_BF16, bf16) HODU_CASE(HODU_F16, f16) HODU_CASE(HODU_F32, f32) HODU_CASE(HODU_F64, f64)
    HODU_CASE(HODU_U8, u8) HODU_CASE(HODU_U16, u16) HODU_CASE(HODU_U32, u32) HODU_CASE(HODU_U64, u64)
    HODU_CASE(HODU_I8, i8) HODU_CASE(HODU_I16, i16) HODU_CASE(HODU_I32, i32) HODU_CASE(HODU_I64, i64)
#undef HODU_CASE
    default: return nullptr;
    }
}

// `iters` calls of `once(i)` between two HIP events on the context's stream; with `graph` the calls are captured
// once (after one call outside the capture, so that workspaces exist and code objects are loaded) and replayed as
// one graph launch inside the timed region
template <class F> int timed_loop(hodu_rocm_ctx *ctx, bool graph, int iters, float *elapsed_ms, F once) {
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    hipEvent_t t0 = nullptr, t1 = nullptr;
    hipGraph_t g = nullptr;
    hipGraphExec_t exec = nullptr;
    int rc = HODU_ROCM_OK;
    hipError_t e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    if (e == hipSuccess && graph) {
        rc = once(0);
        if (rc == HODU_ROCM_OK) e = hipStreamSynchronize(ctx->stream);
        if (rc == HODU_ROCM_OK && e == hipSuccess) {
            e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
            if (e == hipSuccess) {
                for (int i = 0; i < iters && rc == HODU_ROCM_OK; i++) rc = once(i);
                const hipError_t ce = hipStreamEndCapture(ctx->stream, &g);  // always: the stream must leave capture
                if (e == hipSuccess) e = ce;
            }
        }
        if (rc == HODU_ROCM_OK && e == hipSuccess) e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
        if (rc == HODU_ROCM_OK && e == hipSuccess) e = hipGraphLaunch(exec, ctx->stream);  // one untimed replay
        if (rc == HODU_ROCM_OK && e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    }
    if (rc == HODU_ROCM_OK && e == hipSuccess) e = hipEventRecord(t0, ctx->stream);
    if (rc == HODU_ROCM_OK && e == hipSuccess) {
        if (graph) e = hipGraphLaunch(exec, ctx->stream);
        else
            for (int i = 0; i < iters && rc == HODU_ROCM_OK; i++) rc = once(i);
    }
    if (rc == HODU_ROCM_OK && e == hipSuccess) e = hipEventRecord(t1, ctx->stream);
    if (rc == HODU_ROCM_OK && e == hipSuccess) e = hipEventSynchronize(t1);
    if (rc == HODU_ROCM_OK && e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, t0, t1);
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (g) (void)hipGraphDestroy(g);
    if (rc) return rc;
    if (e != hipSuccess) return fail(HODU_ROCM_HIP_ERROR, "timed loop: %s", hipGetErrorString(e));
    return HODU_ROCM_OK;
}

int time_product_impl(bool graph, hodu_rocm_ctx *ctx, int is_matmul, int kind, int dtype, const void *lhs,
                      const void *const *rhs_list, size_t n_rhs, void *out, const size_t *md, size_t len, int iters,
                      float *elapsed_ms, const hodu_rocm_epilogue_step *steps = nullptr, size_t n_steps = 0) {
    clear_error();
    if (!ctx || !rhs_list || n_rhs == 0 || !elapsed_ms || iters <= 0)
        return fail(HODU_ROCM_INVALID_ARG, "time_product: bad argument");
    if (kind < PK_SAME || kind > PK_I32_I8I8) return fail(HODU_ROCM_INVALID_ARG, "time_product: kind %d", kind);
    const product_fn plain = n_steps == 0 ? plain_entry(is_matmul, kind, dtype) : nullptr;
    const product_ex_fn ex = n_steps != 0 ? ex_entry(is_matmul, kind, dtype) : nullptr;
    if (!plain && !ex) return fail(HODU_ROCM_UNSUPPORTED, "time_product: no entry point for dtype id %d", dtype);
    return timed_loop(ctx, graph, iters, elapsed_ms, [&](int i) {
        const void *rhs = rhs_list[(size_t)i % n_rhs];
        return plain ? plain(ctx, lhs, rhs, out, md, len) : ex(ctx, lhs, rhs, out, md, len, steps, n_steps);
    });
}

}  // namespace

extern "C" {

int hodu_rocm_debug_force_tile(hodu_rocm_ctx *ctx, int tile) {
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "context is null");
    const bool ok = tile == -1 || (tile >= 0 && tile <= 3) || (tile >= 10 && tile <= 16) || tile == 30 || tile == 31 ||
                    (tile >= 32 && tile <= 34) || (tile >= 35 && tile <= 39) || (tile >= 40 && tile <= 43);
    if (!ok) return fail(HODU_ROCM_INVALID_ARG, "tile %d not in -1..3, 10..16, 30..39, 40..43", tile);
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    ctx->force_tile = tile;
    return HODU_ROCM_OK;
}

int hodu_rocm_debug_scratch_state(hodu_rocm_ctx *ctx, size_t *workspace_bytes, int *arrival_allocated, int *in_fixed_mode) {
    if (!ctx || !workspace_bytes || !arrival_allocated || !in_fixed_mode) return fail(HODU_ROCM_INVALID_ARG, "null argument");
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    *workspace_bytes = ctx->workspace.ptr ? ctx->workspace.bytes : 0;
    *arrival_allocated = ctx->arrival != nullptr;
    *in_fixed_mode = ctx->fixed_scratch || (ctx->static_scratch && ctx->arrival == (int *)ctx->static_scratch);
    return HODU_ROCM_OK;
}

int hodu_rocm_debug_force_splitk(hodu_rocm_ctx *ctx, int splits) {
    if (!ctx) return fail(HODU_ROCM_INVALID_ARG, "context is null");
    if (splits < -1 || splits == 0 || splits > 64) return fail(HODU_ROCM_INVALID_ARG, "splits %d not in -1, 1..64", splits);
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    ctx->force_splits = splits;
    return HODU_ROCM_OK;
}

int hodu_rocm_debug_time_product(hodu_rocm_ctx *ctx, int is_matmul, int kind, int dtype, const void *lhs,
                                 const void *const *rhs_list, size_t n_rhs, void *out, const size_t *md, size_t len,
                                 int iters, float *elapsed_ms) {
    return time_product_impl(false, ctx, is_matmul, kind, dtype, lhs, rhs_list, n_rhs, out, md, len, iters, elapsed_ms);
}

int hodu_rocm_debug_time_product_graph(hodu_rocm_ctx *ctx, int is_matmul, int kind, int dtype, const void *lhs,
                                       const void *const *rhs_list, size_t n_rhs, void *out, const size_t *md,
                                       size_t len, int iters, float *elapsed_ms) {
    return time_product_impl(true, ctx, is_matmul, kind, dtype, lhs, rhs_list, n_rhs, out, md, len, iters, elapsed_ms);
}

int hodu_rocm_debug_time_product_ex(hodu_rocm_ctx *ctx, int is_matmul, int kind, int dtype, const void *lhs,
                                    const void *const *rhs_list, size_t n_rhs, void *out, const size_t *md, size_t len,
                                    const hodu_rocm_epilogue_step *steps, size_t n_steps, int iters, float *elapsed_ms) {
    return time_product_impl(false, ctx, is_matmul, kind, dtype, lhs, rhs_list, n_rhs, out, md, len, iters, elapsed_ms,
                             steps, n_steps);
}

int hodu_rocm_debug_time_noalloc(hodu_rocm_ctx *ctx, const void *lhs, const void *const *rhs_list, size_t n_rhs,
                                 void *out, const size_t *md, size_t len, int iters, int graph, float *elapsed_ms) {
    clear_error();
    if (!ctx || !rhs_list || n_rhs == 0 || !elapsed_ms || iters <= 0)
        return fail(HODU_ROCM_INVALID_ARG, "time_noalloc: bad argument");
    return timed_loop(ctx, graph != 0, iters, elapsed_ms, [&](int i) {
        return hodu_rocm_dot_bf16_f8e4m3w_noalloc(ctx, lhs, rhs_list[(size_t)i % n_rhs], out, md, len);
    });
}

int hodu_rocm_debug_time_cast(hodu_rocm_ctx *ctx, int src, int dst, const void *const *in_list, void *const *out_list,
                              size_t n_buffers, const size_t *md, size_t len, int iters, float *elapsed_ms) {
    clear_error();
    if (!ctx || !in_list || !out_list || n_buffers == 0 || !elapsed_ms || iters < 1)
        return fail(HODU_ROCM_INVALID_ARG, "time_cast: bad argument");
    return timed_loop(ctx, false, iters, elapsed_ms, [&](int i) {
        const size_t j = (size_t)i % n_buffers;
        return src == dst ? hodu_rocm_contiguous(ctx, src, in_list[j], out_list[j], md, len)
                          : hodu_rocm_cast(ctx, src, dst, in_list[j], out_list[j], md, len);
    });
}

int hodu_rocm_debug_time_sum(hodu_rocm_ctx *ctx, int dtype, const void *const *in_list, void *const *out_list,
                             size_t n_buffers, const size_t *md, size_t len, int iters, float *elapsed_ms) {
    clear_error();
    if (!ctx || !in_list || !out_list || n_buffers == 0 || !elapsed_ms || iters < 1)
        return fail(HODU_ROCM_INVALID_ARG, "time_sum: bad argument");
    return timed_loop(ctx, false, iters, elapsed_ms, [&](int i) {
        const size_t j = (size_t)i % n_buffers;
        return hodu_rocm_sum(ctx, dtype, in_list[j], out_list[j], md, len);
    });
}

}  // extern "C"
