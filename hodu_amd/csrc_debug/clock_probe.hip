// Measurement hook: what the matrix cores sustain when nothing else is in the way, and at which shader clock.
//
// A register-only loop of MFMAs (no LDS, no memory traffic inside the loop) on operand bits the caller supplies,
// two workgroups of four wavefronts on every compute unit.  One wavefront reads the shader-clock counter
// (s_memtime) and the constant 100 MHz counter (s_memrealtime) before and after its loop; their ratio is the clock
// the wavefront ran at.  On this part the clock under full MFMA load depends on the operand data (how many
// multiplier inputs toggle): the rate this probe reports for N(0,1) operands, not the datasheet peak, is what a
// GEMM kernel can approach.
#include "common.hpp"
#include "device_types.hpp"

#include <type_traits>

namespace hodu {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// KIND 0: v_mfma_f32_32x32x16_bf16; KIND 1: v_mfma_scale_f32_32x32x64_f8f6f4 on f8e4m3 with unit scales;
// KIND 2: v_mfma_f32_16x16x32_bf16 (half the flop per instruction of KIND 0, a quarter of the accumulator registers);
// KIND 3: v_mfma_scale_f32_16x16x128_f8f6f4, the same relation to KIND 1
typedef float f32x4_acc_t __attribute__((ext_vector_type(4)));
template <int KIND>
__global__ __launch_bounds__(256) void mfma_clock_kernel(const u32x4_t *__restrict__ operands, float *__restrict__ sink,
                                                        unsigned long long *__restrict__ clocks, int iters) {
    constexpr int NACC = 4;
    const int t = threadIdx.x;
    const u32x4_t a0 = operands[t], b0 = operands[256 + t], a1 = operands[512 + t], b1 = operands[768 + t];
    f32x16_t acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.f;
    if constexpr (KIND == 2) {
        // eight independent 16 x 16 accumulators, two instructions per accumulator and trip: the same flop per
        // trip as KIND 0
        f32x4_acc_t small[8];
#pragma unroll
        for (int i = 0; i < 8; i++) small[i] = f32x4_acc_t{0.f, 0.f, 0.f, 0.f};
        const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 8; i++)
                // (written out: left to the register allocator, the eight accumulators rotate through copies)
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(small[i]) : "v"(a0), "v"(b0));
        }
        const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) v += small[i][0] + small[i][1] + small[i][2] + small[i][3];
        sink[blockIdx.x * 256 + t] = v + a1.x + b1.x;
        if (blockIdx.x == 0 && t == 0) {
            clocks[0] = c1 - c0;
            clocks[1] = r1 - r0;
        }
        return;
    }
    if constexpr (KIND == 3) {
        // v_mfma_scale_f32_16x16x128_f8f6f4 on f8e4m3 with unit scales: eight accumulators, the flop per trip of KIND 1
        f32x4_acc_t small[8];
#pragma unroll
        for (int i = 0; i < 8; i++) small[i] = f32x4_acc_t{0.f, 0.f, 0.f, 0.f};
        const i32x8_t a = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
        const i32x8_t b = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
        const int unit = 0x7F7F7F7F;
        const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 8; i++)
                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]"
                             : "+v"(small[i]) : "v"(a), "v"(b), "v"(unit));
        }
        const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) v += small[i][0] + small[i][1] + small[i][2] + small[i][3];
        sink[blockIdx.x * 256 + t] = v;
        if (blockIdx.x == 0 && t == 0) {
            clocks[0] = c1 - c0;
            clocks[1] = r1 - r0;
        }
        return;
    }
    const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < NACC; i++) {
            if constexpr (KIND == 0) {
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a0), __builtin_bit_cast(bf16x8_t, b0),
                                                                 acc[i], 0, 0, 0);
            } else {
                const i32x8_t a = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                const i32x8_t b = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
                acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i], 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
            }
        }
    }
    const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    f32x16_t s = acc[0];
#pragma unroll
    for (int i = 1; i < NACC; i++) s += acc[i];
    float v = 0.f;
#pragma unroll
    for (int e = 0; e < 16; e++) v += s[e];
    sink[blockIdx.x * 256 + t] = v;
    if (blockIdx.x == 0 && t == 0) {
        clocks[0] = c1 - c0;
        clocks[1] = r1 - r0;
    }
}

// the simplest possible reader: every lane loads PER 16-byte vectors, all in flight at once, and folds them into a
// value that is (almost) never stored
template <int PER, bool NT>
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4_t *__restrict__ src, unsigned *__restrict__ sink, long n_vec) {
    const long base = (long)blockIdx.x * PER * 256 + threadIdx.x;
    u32x4_t v[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const long j = base + (long)i * 256;
        v[i] = u32x4_t{0u, 0u, 0u, 0u};
        if (j < n_vec) v[i] = NT ? __builtin_nontemporal_load(src + j) : src[j];
    }
    unsigned x = 0;
#pragma unroll
    for (int i = 0; i < PER; i++) x += v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    if (x == 0x9E3779B9u) sink[threadIdx.x] = x;
}

__global__ void empty_kernel() {}

}  // namespace
}  // namespace hodu

using namespace hodu;

// iters launches of a flat streaming read of `bytes` from each of `n_src` buffers in turn (more buffers than the
// Infinity Cache holds: the reads come from HBM), and iters launches of an empty kernel: what the memory system and
// the launch path allow a kernel of this size, before any arithmetic
extern "C" int hodu_rocm_debug_read_floor(hodu_rocm_ctx *ctx, const void *const *src_list, size_t n_src, size_t bytes, int iters,
                                          float *read_us, float *empty_us) {
    clear_error();
    if (!ctx || !src_list || n_src == 0 || bytes == 0 || bytes % 16 != 0 || iters <= 0 || !read_us || !empty_us)
        return fail(HODU_ROCM_INVALID_ARG, "read_floor: bad argument");
    for (size_t i = 0; i < n_src; i++)
        if (!src_list[i] || (uintptr_t)src_list[i] % 16 != 0) return fail(HODU_ROCM_INVALID_ARG, "read_floor: bad buffer %zu", i);
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    const long n_vec = (long)(bytes / 16);
    if ((n_vec + 4 * 256 - 1) / (4 * 256) > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "read_floor: buffer too large");
    unsigned *sink = nullptr;
    HODU_HIP(hipMalloc((void **)&sink, 256 * sizeof(unsigned)));
    hipEvent_t t0, t1;
    hipError_t e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    auto timed = [&](auto launch, float *us) {
        for (int i = 0; i < 3; i++) launch(i);
        if (e == hipSuccess) e = hipEventRecord(t0, ctx->stream);
        for (int i = 0; i < iters; i++) launch(i);
        if (e == hipSuccess) e = hipEventRecord(t1, ctx->stream);
        if (e == hipSuccess) e = hipEventSynchronize(t1);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
        *us = ms * 1e3f / (float)iters;
    };
    // the fastest of several shapes of the same read -- 4, 8 or 16 loads in flight per lane, plain and with the
    // non-temporal hint -- so that the figure is a floor of the memory system and not of one kernel shape
    *read_us = 1e30f;
    auto shape = [&](auto per_, auto nt_) {
        constexpr int PER = decltype(per_)::value;
        constexpr bool NT = decltype(nt_)::value;
        const unsigned blocks = (unsigned)((n_vec + PER * 256 - 1) / (PER * 256));
        float us = 0.f;
        timed([&](int i) {
            hipLaunchKernelGGL((stream_read_kernel<PER, NT>), dim3(blocks), dim3(256), 0, ctx->stream,
                               (const u32x4_t *)src_list[(size_t)i % n_src], sink, n_vec);
        }, &us);
        if (us < *read_us) *read_us = us;
    };
    shape(std::integral_constant<int, 8>{}, std::false_type{});
    shape(std::integral_constant<int, 8>{}, std::true_type{});
    shape(std::integral_constant<int, 4>{}, std::false_type{});
    shape(std::integral_constant<int, 16>{}, std::false_type{});
    shape(std::integral_constant<int, 16>{}, std::true_type{});
    timed([&](int) { hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, ctx->stream); }, empty_us);
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    (void)hipFree(sink);
    if (e != hipSuccess) return fail(HODU_ROCM_HIP_ERROR, "read_floor: %s", hipGetErrorString(e));
    return HODU_ROCM_OK;
}

extern "C" int hodu_rocm_debug_mfma_clock(hodu_rocm_ctx *ctx, int kind, const void *operands, int iters, float *elapsed_ms,
                                          double *tflops, double *shader_mhz) {
    clear_error();
    if (!ctx || !operands || iters <= 0 || !elapsed_ms || !tflops || !shader_mhz || kind < 0 || kind > 3)
        return fail(HODU_ROCM_INVALID_ARG, "mfma_clock: bad argument");
    std::lock_guard<std::recursive_mutex> hold(ctx->mu);
    HODU_HIP(hipSetDevice(ctx->device));
    const unsigned blocks = 2u * (unsigned)ctx->props.multiProcessorCount;
    float *sink = nullptr;
    unsigned long long *clocks = nullptr;
    HODU_HIP(hipMalloc((void **)&sink, (size_t)blocks * 256 * sizeof(float)));
    if (hipMalloc((void **)&clocks, 16) != hipSuccess) {
        (void)hipFree(sink);
        return fail(HODU_ROCM_OOM, "mfma_clock: out of memory");
    }
    auto launch = [&](int n) {
        if (kind == 0)
            hipLaunchKernelGGL(mfma_clock_kernel<0>, dim3(blocks), dim3(256), 0, ctx->stream, (const u32x4_t *)operands, sink, clocks, n);
        else if (kind == 3)
            hipLaunchKernelGGL(mfma_clock_kernel<3>, dim3(blocks), dim3(256), 0, ctx->stream, (const u32x4_t *)operands, sink, clocks, n);
        else if (kind == 2)
            hipLaunchKernelGGL(mfma_clock_kernel<2>, dim3(blocks), dim3(256), 0, ctx->stream, (const u32x4_t *)operands, sink, clocks, n);
        else
            hipLaunchKernelGGL(mfma_clock_kernel<1>, dim3(blocks), dim3(256), 0, ctx->stream, (const u32x4_t *)operands, sink, clocks, n);
    };
    hipEvent_t t0, t1;
    hipError_t e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    if (e == hipSuccess) {
        launch(iters / 10 + 1);  // warm-up: the clock settles
        launch(iters / 10 + 1);
        e = hipEventRecord(t0, ctx->stream);
        launch(iters);
        if (e == hipSuccess) e = hipEventRecord(t1, ctx->stream);
        if (e == hipSuccess) e = hipEventSynchronize(t1);
        if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, t0, t1);
    }
    unsigned long long h[2] = {0, 0};
    if (e == hipSuccess) e = hipMemcpy(h, clocks, 16, hipMemcpyDeviceToHost);
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    (void)hipFree(sink);
    (void)hipFree(clocks);
    if (e != hipSuccess) return fail(HODU_ROCM_HIP_ERROR, "mfma_clock: %s", hipGetErrorString(e));
    // flop per trip of the loop: four 32 x 32 x k x 2 instructions with k = 16 (bf16) or 64 (f8), or eight 16 x 16 x 32 x 2
    const double per_trip = kind == 0 ? 4 * 32768.0 : kind == 2 ? 8 * 16384.0 : kind == 3 ? 8 * 65536.0 : 4 * 131072.0;
    *tflops = (double)blocks * 4 /* wavefronts */ * (double)iters * per_trip / (*elapsed_ms * 1e-3) / 1e12;
    *shader_mhz = h[1] ? (double)h[0] / (double)h[1] * 100.0 : 0.0;
    return HODU_ROCM_OK;
}
