// Test infrastructure: what the kernels' translation units need from runtime.cpp when they are compiled for the host
// against tests/emu/hip/hip_runtime.h -- the error text, a host-memory workspace and arrival counters, a context to
// hand to the real entry points of api.cpp, the workgroup's LDS.  Built twice: as part of the small library of the
// plain kernels (softmax, casts, sums, the generic and reference-sum products), where every other kernel family's
// launcher answers UNSUPPORTED, and with EMU_WITH_MFMA as part of the library that holds all of them.  "Device"
// pointers are host pointers here.
#include <cstdarg>
#include <cstdlib>
#include <cstring>
#include <mutex>

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
int launch_attention(hodu_rocm_ctx *, int, const void *, const void *, const void *, void *, const AttentionArgs &) {
    return HODU_ROCM_UNSUPPORTED;
}
#endif
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

#ifdef EMU_WITH_MFMA
// The rest of the C ABI (runtime.cpp's part), so that code written against include/hodu_rocm_kernels.h -- the host
// mirror's compiled library -- links against this build as it does against the real one.  An allocation is host
// memory between two inaccessible pages, its last 16-byte unit ending where the second one begins.
#include <sys/mman.h>

#include <map>
namespace {
constexpr size_t kPage = 4096;
std::mutex g_alloc_mu;
std::map<void *, std::pair<void *, size_t>> g_allocs;  // pointer handed out -> (mapping, its length)
}  // namespace
extern "C" {
int hodu_rocm_device_count(int *count) {
    if (!count) return hodu::fail(HODU_ROCM_INVALID_ARG, "count is null");
    *count = 1;
    return HODU_ROCM_OK;
}
int hodu_rocm_ctx_create(int device, hodu_rocm_ctx **out) {
    if (!out) return hodu::fail(HODU_ROCM_INVALID_ARG, "ctx_create: out pointer is null");
    if (device != 0) return hodu::fail(HODU_ROCM_INVALID_ARG, "ctx_create: the CPU build has one device");
    *out = new hodu_rocm_ctx;
    return HODU_ROCM_OK;
}
int hodu_rocm_ctx_destroy(hodu_rocm_ctx *ctx) {
    if (ctx) {
        free(ctx->workspace.ptr);
        free(ctx->arrival);
    }
    delete ctx;
    return HODU_ROCM_OK;
}
int hodu_rocm_alloc(hodu_rocm_ctx *ctx, size_t bytes, void **dptr) {
    if (!ctx) return hodu::fail(HODU_ROCM_INVALID_ARG, "context is null");
    if (!dptr) return hodu::fail(HODU_ROCM_INVALID_ARG, "dptr is null");
    const size_t body = (bytes + kPage - 1) / kPage * kPage + (bytes == 0 ? kPage : 0), total = body + 2 * kPage;
    char *base = (char *)mmap(nullptr, total, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
    if (base == MAP_FAILED) return hodu::fail(HODU_ROCM_OOM, "alloc(%zu)", bytes);
    mprotect(base, kPage, PROT_NONE);
    mprotect(base + kPage + body, kPage, PROT_NONE);
    char *p = base + kPage + body - (bytes + 15) / 16 * 16;
    if (bytes == 0) p = base + kPage;
    std::lock_guard<std::mutex> hold(g_alloc_mu);
    g_allocs[p] = {base, total};
    *dptr = p;
    return HODU_ROCM_OK;
}
int hodu_rocm_free(hodu_rocm_ctx *ctx, void *dptr) {
    if (!ctx) return hodu::fail(HODU_ROCM_INVALID_ARG, "context is null");
    if (!dptr) return HODU_ROCM_OK;
    std::lock_guard<std::mutex> hold(g_alloc_mu);
    auto it = g_allocs.find(dptr);
    if (it == g_allocs.end()) return hodu::fail(HODU_ROCM_INVALID_ARG, "free: not an allocation of this library");
    munmap(it->second.first, it->second.second);
    g_allocs.erase(it);
    return HODU_ROCM_OK;
}
static int emu_copy(hodu_rocm_ctx *ctx, void *dst, const void *src, size_t bytes, const char *what) {
    if (!ctx) return hodu::fail(HODU_ROCM_INVALID_ARG, "context is null");
    if (bytes == 0) return HODU_ROCM_OK;
    if (!dst || !src) return hodu::fail(HODU_ROCM_INVALID_ARG, "%s: null pointer", what);
    memmove(dst, src, bytes);
    return HODU_ROCM_OK;
}
int hodu_rocm_memcpy_h2d(hodu_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) { return emu_copy(ctx, dst, src, bytes, "memcpy_h2d"); }
int hodu_rocm_memcpy_d2h(hodu_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) { return emu_copy(ctx, dst, src, bytes, "memcpy_d2h"); }
int hodu_rocm_memcpy_d2d(hodu_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) { return emu_copy(ctx, dst, src, bytes, "memcpy_d2d"); }
int hodu_rocm_memset(hodu_rocm_ctx *ctx, void *dptr, int byte, size_t bytes) {
    if (!ctx) return hodu::fail(HODU_ROCM_INVALID_ARG, "context is null");
    if (bytes == 0) return HODU_ROCM_OK;
    if (!dptr) return hodu::fail(HODU_ROCM_INVALID_ARG, "memset: null pointer");
    memset(dptr, byte, bytes);
    return HODU_ROCM_OK;
}
int hodu_rocm_sync(hodu_rocm_ctx *ctx) { return ctx ? HODU_ROCM_OK : hodu::fail(HODU_ROCM_INVALID_ARG, "context is null"); }
const char *hodu_rocm_last_error(hodu_rocm_ctx *) { return hodu::get_error(); }
const char *hodu_rocm_last_kernel(hodu_rocm_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }
}
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
