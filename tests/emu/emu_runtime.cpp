// Test infrastructure: what the plain kernels' translation units need from runtime.cpp when they are compiled for the
// host against tests/emu/hip/hip_runtime.h -- the error text, a host-memory workspace, a context to hand to the real
// entry points of api.cpp -- and UNSUPPORTED stand-ins for the kernel families that need the matrix cores or
// LDS-DMA and therefore have no CPU build (the long inner product of reduce.hip does).  "Device" pointers are host pointers here.
#include <cstdarg>
#include <cstdlib>
#include <cstring>

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
#ifdef EMU_WITH_MFMA
int ensure_arrival(hodu_rocm_ctx *ctx) {
    if (!ctx->arrival) ctx->arrival = (int *)calloc(kArrivalSlots, sizeof(int));
    if (ctx->arrival && ctx->arrival_stale) memset(ctx->arrival, 0, kArrivalSlots * sizeof(int));
    ctx->arrival_stale = false;
    return ctx->arrival ? HODU_ROCM_OK : fail(HODU_ROCM_OOM, "arrival counters");
}
#else
int ensure_arrival(hodu_rocm_ctx *) { return fail(HODU_ROCM_UNSUPPORTED, "no arrival counters in the CPU build"); }
#endif

#define NO_CPU_BUILD(name) \
    int name(hodu_rocm_ctx *, int, int, const void *, const void *, void *, const DevProduct &) { return HODU_ROCM_UNSUPPORTED; }
#ifndef EMU_WITH_MFMA
NO_CPU_BUILD(launch_mfma)
NO_CPU_BUILD(launch_gemv)
NO_CPU_BUILD(launch_small_f32)
NO_CPU_BUILD(launch_gemm_f64)
NO_CPU_BUILD(launch_skinny)
NO_CPU_BUILD(launch_gemv_rows)
#endif
int launch_attention(hodu_rocm_ctx *, int, const void *, const void *, const void *, void *, const AttentionArgs &) {
    return HODU_ROCM_UNSUPPORTED;
}
}  // namespace hodu

// LDS of the workgroup that is running (workgroups run one at a time): what HODU_DYNAMIC_LDS names in the kernels
namespace emu {
namespace {
alignas(256) char g_lds[kLdsBytes];
}
char *lds_base() { return g_lds; }
}  // namespace emu
// fills LDS with a pattern, so that a kernel that reads what it has not written does not find the last launch's data
extern "C" void emu_lds_fill(int byte) { memset(emu::lds_base(), byte, emu::kLdsBytes); }
#ifdef EMU_WITH_MFMA
// the model of LDS-DMA arrival (gfx950_insn_emu.hpp)
namespace emu {
int &dma_lazy() { static int model = 0; return model; }
}  // namespace emu
extern "C" void emu_dma_lazy(int model) { emu::dma_lazy() = model; }
#endif

extern "C" {
hodu_rocm_ctx *emu_ctx_create(void) { return new hodu_rocm_ctx; }
void emu_ctx_destroy(hodu_rocm_ctx *ctx) {
    if (ctx) {
        free(ctx->workspace.ptr);
        free(ctx->arrival);
    }
    delete ctx;
}
const char *emu_last_kernel(hodu_rocm_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }
// the testing hooks of the debug library, which has no CPU build
void emu_force_tile(hodu_rocm_ctx *ctx, int v) { ctx->force_tile = v; }
void emu_force_splitk(hodu_rocm_ctx *ctx, int v) { ctx->force_splits = v; }
const char *emu_last_error(void) { return hodu::get_error(); }
// how often a kernel reached an instruction that has no CPU stand-in (must stay 0 for a result to mean anything)
int emu_unsupported_hits(void) { return emu::no_such_instruction_hits(); }
const char *emu_unsupported_first(void) { return emu::no_such_instruction_first(); }
void emu_unsupported_reset(void) { emu::no_such_instruction_hits() = 0; }
}
