// Test infrastructure: what the plain kernels' translation units need from runtime.cpp when they are compiled for the
// host against tests/emu/hip/hip_runtime.h -- the error text, a host-memory workspace, a context to hand to the real
// entry points of api.cpp -- and UNSUPPORTED stand-ins for the kernel families that need the matrix cores or
// LDS-DMA and therefore have no CPU build (the long inner product of reduce.hip does).  "Device" pointers are host pointers here.
#include <cstdarg>
#include <cstdlib>

#include "common.hpp"

namespace hodu {
namespace {
thread_local char g_error[512] = "";
}
void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
const char *get_error() { return g_error; }
void clear_error() { g_error[0] = 0; }
int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}
int ensure_workspace(hodu_rocm_ctx *ctx, size_t bytes) {
    if (ctx->workspace.bytes >= bytes) return HODU_ROCM_OK;
    free(ctx->workspace.ptr);
    ctx->workspace.ptr = malloc(bytes);
    ctx->workspace.bytes = ctx->workspace.ptr ? bytes : 0;
    return ctx->workspace.ptr ? HODU_ROCM_OK : fail(HODU_ROCM_OOM, "workspace of %zu bytes", bytes);
}
int ensure_arrival(hodu_rocm_ctx *) { return fail(HODU_ROCM_UNSUPPORTED, "no arrival counters in the CPU build"); }

#define NO_CPU_BUILD(name) \
    int name(hodu_rocm_ctx *, int, int, const void *, const void *, void *, const DevProduct &) { return HODU_ROCM_UNSUPPORTED; }
NO_CPU_BUILD(launch_mfma)
NO_CPU_BUILD(launch_gemv)
NO_CPU_BUILD(launch_small_f32)
NO_CPU_BUILD(launch_gemm_f64)
NO_CPU_BUILD(launch_skinny)
NO_CPU_BUILD(launch_gemv_rows)
int launch_attention(hodu_rocm_ctx *, int, const void *, const void *, const void *, void *, const AttentionArgs &) {
    return HODU_ROCM_UNSUPPORTED;
}
}  // namespace hodu

extern "C" {
hodu_rocm_ctx *emu_ctx_create(void) { return new hodu_rocm_ctx; }
void emu_ctx_destroy(hodu_rocm_ctx *ctx) {
    if (ctx) free(ctx->workspace.ptr);
    delete ctx;
}
const char *emu_last_kernel(hodu_rocm_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }
const char *emu_last_error(void) { return hodu::get_error(); }
// how often a kernel reached an instruction that has no CPU stand-in (must stay 0 for a result to mean anything)
int emu_unsupported_hits(void) { return emu::no_such_instruction_hits(); }
}
