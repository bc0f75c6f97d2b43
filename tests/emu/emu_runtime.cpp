// Test infrastructure: the CPU build's own part -- the workgroup's LDS, guarded "device" memory, the switches of the
// instruction models.  Built twice.  In the library of all kernels (EMU_WITH_RUNTIME) the library's real runtime.cpp is compiled beside it, against
// the runtime API of tests/emu/hip/hip_runtime.h.  In the small library of the plain kernels (softmax, casts, sums,
// the generic and reference-sum products) this file also stands in for runtime.cpp -- error text, workspace, a bare
// context -- and every other kernel family's launcher answers UNSUPPORTED, which routes every product to the generic
// kernel.  "Device" pointers are host pointers here.
#include <sys/mman.h>

#include <cstdarg>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

#include "common.hpp"

// ---- LDS of the workgroup that is running (workgroups run one at a time): what HODU_DYNAMIC_LDS names in the kernels
namespace emu {
namespace {
alignas(256) char g_lds[kLdsBytes];
constexpr size_t kPage = 4096;
std::mutex g_alloc_mu;
std::map<void *, std::pair<void *, size_t>> g_allocs;  // pointer handed out -> (mapping, its length)
bool g_tight_end = true;
}  // namespace
char *lds_base() { return g_lds; }

void *device_alloc(size_t bytes) {
    const size_t body = (bytes + kPage - 1) / kPage * kPage + (bytes == 0 ? kPage : 0), total = body + 2 * kPage;
    char *base = (char *)mmap(nullptr, total, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
    if (base == MAP_FAILED) return nullptr;
    mprotect(base, kPage, PROT_NONE);
    mprotect(base + kPage + body, kPage, PROT_NONE);
    char *p = base + kPage + (g_tight_end && bytes != 0 ? body - (bytes + 15) / 16 * 16 : 0);
    std::lock_guard<std::mutex> hold(g_alloc_mu);
    g_allocs[p] = {base, total};
    return p;
}
bool device_free(void *p) {
    std::lock_guard<std::mutex> hold(g_alloc_mu);
    auto it = g_allocs.find(p);
    if (it == g_allocs.end()) return false;
    munmap(it->second.first, it->second.second);
    g_allocs.erase(it);
    return true;
}
#ifdef EMU_WITH_RUNTIME
int &dma_lazy() { static int model = 0; return model; }  // the model of LDS-DMA arrival (gfx950_insn_emu.hpp)
#endif
}  // namespace emu

#ifndef EMU_WITH_RUNTIME
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
int ensure_arrival(hodu_rocm_ctx *) { return fail(HODU_ROCM_UNSUPPORTED, "no arrival counters in the library of the plain kernels"); }

#define NOT_IN_THIS_LIBRARY(name) \
    int name(hodu_rocm_ctx *, int, int, const void *, const void *, void *, const DevProduct &) { return HODU_ROCM_UNSUPPORTED; }
NOT_IN_THIS_LIBRARY(launch_mfma)
NOT_IN_THIS_LIBRARY(launch_gemv)
NOT_IN_THIS_LIBRARY(launch_small_f32)
NOT_IN_THIS_LIBRARY(launch_gemm_f64)
NOT_IN_THIS_LIBRARY(launch_skinny)
NOT_IN_THIS_LIBRARY(launch_gemv_rows)
int launch_attention(hodu_rocm_ctx *, int, const void *, const void *, const void *, void *, const AttentionArgs &, const AttentionMask *) {
    return HODU_ROCM_UNSUPPORTED;
}
}  // namespace hodu

extern "C" {
hodu_rocm_ctx *emu_ctx_create(void) { return new hodu_rocm_ctx; }
void emu_ctx_destroy(hodu_rocm_ctx *ctx) {
    if (ctx) free(ctx->workspace.ptr);
    delete ctx;
}
}
#endif

extern "C" {
const char *emu_last_kernel(hodu_rocm_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }
const char *emu_last_error(void) { return hodu::get_error(); }
// fills LDS with a pattern, so that a kernel that reads what it has not written does not find the last launch's data
void emu_lds_fill(int byte) { memset(emu::lds_base(), byte, emu::kLdsBytes); }
// where an allocation touches its guard page: 1 its end (the default), 0 its start
void emu_alloc_tight(int end) { emu::g_tight_end = end != 0; }
// how often a kernel reached an instruction that has no CPU stand-in (must stay 0 for a result to mean anything)
int emu_unsupported_hits(void) { return emu::no_such_instruction_hits(); }
const char *emu_unsupported_first(void) { return emu::no_such_instruction_first(); }
void emu_unsupported_reset(void) { emu::no_such_instruction_hits() = 0; }
#ifdef EMU_WITH_RUNTIME
void emu_dma_lazy(int model) { emu::dma_lazy() = model; }
// the two probes of the debug library that are kernels written around inline assembly (clock_probe.hip) have no CPU build;
// the rest of it (csrc_debug/timing.cpp: hooks, scratch report, timing loops, graph replay) is compiled as it is
int hodu_rocm_debug_mfma_clock(hodu_rocm_ctx *, int, const void *, int, float *, double *, double *) {
    return hodu::fail(HODU_ROCM_UNSUPPORTED, "the matrix-core clock probe has no CPU build");
}
int hodu_rocm_debug_read_floor(hodu_rocm_ctx *, const void *const *, size_t, size_t, int, float *, float *) {
    return hodu::fail(HODU_ROCM_UNSUPPORTED, "the streaming-read probe has no CPU build");
}
#endif
}
