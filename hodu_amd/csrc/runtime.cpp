// Context, memory and timing entry points of the C ABI.
#include <cstdarg>
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

namespace {

// Scratch of the entry point that allocates nothing: arrival counters first, partial sums behind them.  Every GPU
// the library runs on holds its own copy of this array until the process ends.  In host code the NAME is only a
// handle for hipGetSymbolAddress; kernels and copies get the per-device address that call returns.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices] = {};  // per device: where that device keeps its copy of `scratch`

// with `device` current: the device's address of the static scratch array, looked up once per device
int static_scratch_of(int device, void **ptr) {
    if (device < 0 || device >= kMaxDevices) return fail(HODU_ROCM_UNSUPPORTED, "device id %d beyond %d", device, kMaxDevices);
    std::lock_guard<std::mutex> hold(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        void *p = nullptr;
        HODU_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(HODU_ROCM_HIP_ERROR, "hipGetSymbolAddress returned a null address for the static scratch");
        g_scratch_ptr[device] = p;
    }
    *ptr = g_scratch_ptr[device];
    return HODU_ROCM_OK;
}

__global__ __launch_bounds__(1024) void clear_words_kernel(int *__restrict__ p, int n) {
    const int i = blockIdx.x * 1024 + threadIdx.x;
    if (i < n) p[i] = 0;
}

bool stream_is_capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}

}  // namespace

int ensure_workspace(hodu_rocm_ctx *ctx, size_t bytes) {
    if (ctx->workspace.bytes >= bytes) return HODU_ROCM_OK;
    if (ctx->fixed_scratch)
        return fail(HODU_ROCM_SCRATCH,
                    "this product needs %zu bytes of partial sums; the static scratch of the entry point that "
                    "allocates nothing holds %zu", bytes, ctx->workspace.bytes);
    if (stream_is_capturing(ctx->stream))
        return fail(HODU_ROCM_SCRATCH, "the workspace would have to grow to %zu bytes while the stream is being "
                    "captured: run the product once outside the capture first", bytes);
    if (ctx->workspace.ptr) {
        HODU_HIP(hipStreamSynchronize(ctx->stream));
        HODU_HIP(hipFree(ctx->workspace.ptr));
        ctx->workspace = Workspace();
    }
    size_t want = bytes < ((size_t)64 << 20) ? ((size_t)64 << 20) : bytes;
    HODU_HIP(hipMalloc(&ctx->workspace.ptr, want));
    ctx->workspace.bytes = want;
    return HODU_ROCM_OK;
}

int ensure_arrival(hodu_rocm_ctx *ctx) {
    if (!ctx->arrival) {
        if (ctx->fixed_scratch) return fail(HODU_ROCM_HIP_ERROR, "static scratch is not set up on this context");
        if (stream_is_capturing(ctx->stream))
            return fail(HODU_ROCM_SCRATCH, "the arrival counters would be allocated while the stream is being "
                        "captured: run the product once outside the capture first");
        HODU_HIP(hipMalloc((void **)&ctx->arrival, kArrivalSlots * sizeof(int)));
        ctx->arrival_stale = true;
    }
    if (ctx->arrival_stale) {
        // by a kernel, in stream order (never a memset node: the caller may be capturing a graph)
        hipLaunchKernelGGL(clear_words_kernel, dim3((kArrivalSlots + 1023) / 1024), dim3(1024), 0, ctx->stream, ctx->arrival,
                           kArrivalSlots);
        HODU_HIP(hipGetLastError());
        ctx->arrival_stale = false;
    }
    return HODU_ROCM_OK;
}

}  // namespace hodu

using namespace hodu;

#define REQUIRE_CTX(ctx)                                                                        \
    do {                                                                                        \
        if (!(ctx)) return fail(HODU_ROCM_INVALID_ARG, "context is null");                      \
        HODU_HIP(hipSetDevice((ctx)->device));                                                  \
    } while (0)

extern "C" {

int hodu_rocm_device_count(int *count) {
    if (!count) return fail(HODU_ROCM_INVALID_ARG, "count is null");
    *count = 0;
    hipError_t e = hipGetDeviceCount(count);
    if (e != hipSuccess) {
        *count = 0;
        return fail(HODU_ROCM_HIP_ERROR, "hipGetDeviceCount: %s", hipGetErrorString(e));
    }
    return HODU_ROCM_OK;
}

int hodu_rocm_ctx_create(int device, hodu_rocm_ctx **out) {
    if (!out) return fail(HODU_ROCM_INVALID_ARG, "ctx out-pointer is null");
    *out = nullptr;
    int n = 0;
    HODU_HIP(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) return fail(HODU_ROCM_INVALID_ARG, "device %d of %d", device, n);
    HODU_HIP(hipSetDevice(device));
    hodu_rocm_ctx *ctx = new hodu_rocm_ctx();
    ctx->device = device;
    hipError_t e = hipGetDeviceProperties(&ctx->props, device);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete ctx;
        return fail(HODU_ROCM_HIP_ERROR, "context setup: %s", hipGetErrorString(e));
    }
    if (strncmp(ctx->props.gcnArchName, "gfx950", 6) != 0) {
        // the embedded code object is gfx950 only; any launch would fail with a less clear error
        char arch[64];
        snprintf(arch, sizeof(arch), "%s", ctx->props.gcnArchName);
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return fail(HODU_ROCM_UNSUPPORTED, "device %d is %s; this library carries gfx950 code only", device, arch);
    }
    // this device's address of the static scratch array (the device is current): kept for the entry point that
    // allocates nothing
    if (int rc = static_scratch_of(device, &ctx->static_scratch)) {
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return rc;
    }
    *out = ctx;
    return HODU_ROCM_OK;
}

int hodu_rocm_ctx_destroy(hodu_rocm_ctx *ctx) {
    if (!ctx) return HODU_ROCM_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->workspace.ptr) (void)hipFree(ctx->workspace.ptr);
    if (ctx->arrival) (void)hipFree(ctx->arrival);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return HODU_ROCM_OK;
}

int hodu_rocm_alloc(hodu_rocm_ctx *ctx, size_t bytes, void **dptr) {
    REQUIRE_CTX(ctx);
    if (!dptr) return fail(HODU_ROCM_INVALID_ARG, "dptr is null");
    *dptr = nullptr;
    hipError_t e = hipMalloc(dptr, bytes ? bytes : 1);
    if (e != hipSuccess) {
        *dptr = nullptr;
        return fail(e == hipErrorOutOfMemory ? HODU_ROCM_OOM : HODU_ROCM_HIP_ERROR, "hipMalloc(%zu): %s", bytes,
                    hipGetErrorString(e));
    }
    return HODU_ROCM_OK;
}

int hodu_rocm_free(hodu_rocm_ctx *ctx, void *dptr) {
    REQUIRE_CTX(ctx);
    if (!dptr) return HODU_ROCM_OK;
    HODU_HIP(hipStreamSynchronize(ctx->stream));  // kernels may still read it
    HODU_HIP(hipFree(dptr));
    return HODU_ROCM_OK;
}

int hodu_rocm_memcpy_h2d(hodu_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) {
    REQUIRE_CTX(ctx);
    if (bytes == 0) return HODU_ROCM_OK;
    if (!dst || !src) return fail(HODU_ROCM_INVALID_ARG, "memcpy_h2d: null pointer");
    HODU_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    HODU_HIP(hipStreamSynchronize(ctx->stream));  // src is pageable host memory owned by the caller
    return HODU_ROCM_OK;
}

int hodu_rocm_memcpy_d2h(hodu_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) {
    REQUIRE_CTX(ctx);
    if (bytes == 0) return HODU_ROCM_OK;
    if (!dst || !src) return fail(HODU_ROCM_INVALID_ARG, "memcpy_d2h: null pointer");
    HODU_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HODU_HIP(hipStreamSynchronize(ctx->stream));
    return HODU_ROCM_OK;
}

int hodu_rocm_memcpy_d2d(hodu_rocm_ctx *ctx, void *dst, const void *src, size_t bytes) {
    REQUIRE_CTX(ctx);
    if (bytes == 0) return HODU_ROCM_OK;
    if (!dst || !src) return fail(HODU_ROCM_INVALID_ARG, "memcpy_d2d: null pointer");
    HODU_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return HODU_ROCM_OK;
}

int hodu_rocm_memset(hodu_rocm_ctx *ctx, void *dptr, int byte, size_t bytes) {
    REQUIRE_CTX(ctx);
    if (bytes == 0) return HODU_ROCM_OK;
    if (!dptr) return fail(HODU_ROCM_INVALID_ARG, "memset: null pointer");
    HODU_HIP(hipMemsetAsync(dptr, byte, bytes, ctx->stream));
    return HODU_ROCM_OK;
}

int hodu_rocm_sync(hodu_rocm_ctx *ctx) {
    REQUIRE_CTX(ctx);
    HODU_HIP(hipStreamSynchronize(ctx->stream));
    return HODU_ROCM_OK;
}

const char *hodu_rocm_last_error(hodu_rocm_ctx *) { return get_error(); }

const char *hodu_rocm_last_kernel(hodu_rocm_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }

int hodu_rocm_device_info(hodu_rocm_ctx *ctx, char *name, size_t name_len, int *cus, int *clock_khz,
                          size_t *total_mem) {
    REQUIRE_CTX(ctx);
    if (name && name_len) snprintf(name, name_len, "%s (%s)", ctx->props.name, ctx->props.gcnArchName);
    if (cus) *cus = ctx->props.multiProcessorCount;
    if (clock_khz) *clock_khz = ctx->props.clockRate;
    if (total_mem) *total_mem = ctx->props.totalGlobalMem;
    return HODU_ROCM_OK;
}

struct hodu_timer {
    hipEvent_t start, stop;
};

int hodu_rocm_timer_create(hodu_rocm_ctx *ctx, void **timer) {
    REQUIRE_CTX(ctx);
    if (!timer) return fail(HODU_ROCM_INVALID_ARG, "timer is null");
    hodu_timer *t = new hodu_timer();
    hipError_t e = hipEventCreate(&t->start);
    if (e == hipSuccess) e = hipEventCreate(&t->stop);
    if (e != hipSuccess) {
        delete t;
        return fail(HODU_ROCM_HIP_ERROR, "hipEventCreate: %s", hipGetErrorString(e));
    }
    *timer = t;
    return HODU_ROCM_OK;
}

int hodu_rocm_timer_start(hodu_rocm_ctx *ctx, void *timer) {
    REQUIRE_CTX(ctx);
    if (!timer) return fail(HODU_ROCM_INVALID_ARG, "timer is null");
    HODU_HIP(hipEventRecord(((hodu_timer *)timer)->start, ctx->stream));
    return HODU_ROCM_OK;
}

int hodu_rocm_timer_stop(hodu_rocm_ctx *ctx, void *timer, float *ms) {
    REQUIRE_CTX(ctx);
    if (!timer || !ms) return fail(HODU_ROCM_INVALID_ARG, "timer or result is null");
    hodu_timer *t = (hodu_timer *)timer;
    HODU_HIP(hipEventRecord(t->stop, ctx->stream));
    HODU_HIP(hipEventSynchronize(t->stop));
    HODU_HIP(hipEventElapsedTime(ms, t->start, t->stop));
    return HODU_ROCM_OK;
}

int hodu_rocm_timer_destroy(hodu_rocm_ctx *ctx, void *timer) {
    REQUIRE_CTX(ctx);
    if (!timer) return HODU_ROCM_OK;
    hodu_timer *t = (hodu_timer *)timer;
    (void)hipEventDestroy(t->start);
    (void)hipEventDestroy(t->stop);
    delete t;
    return HODU_ROCM_OK;
}

}  // extern "C"
