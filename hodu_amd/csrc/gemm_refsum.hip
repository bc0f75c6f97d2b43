// Products of the narrow float dtypes in the reference's own arithmetic, for a caller that needs hodu's CPU bytes.
//
// hodu_cpu_matmul_<dt> / hodu_cpu_dot_<dt> for f8e4m3, f8e5m2, bf16 and f16 keep the running sum in the narrow type:
//     sum = add(sum, mul(a, b)),  add / mul = narrow(widen(x) (+|*) widen(y))
// (crates/hodu_cpu_kernels/kernels/ops_matrix.c:196-240 and :351-354, :556-600 and :713-716; the scalar routines
// t_bf16.h:27-55, t_f16.h:27-84, t_f8e4m3.h:27-101, t_f8e5m2.h:27-100).  Every other kernel of this library adds
// exact products in f32 and rounds once; the two agree only by accident once K exceeds a few terms -- and for
// f8e4m3 not even on single products above 240, which the reference's decoder reads as infinity.
// hodu_rocm_ctx_set_reference_sums(ctx, 1) routes those four dtypes (and the bf16 x f8e4m3-weight kind, whose
// reference form is to_dtype(bf16) of the weight followed by the bf16 product) here: one thread per output element,
// k ascending, two narrowings per k, each a restatement of the reference's routine -- including what that routine
// does with values it was not written for (a subnormal f8 result ORs a negative mantissa into the exponent field).
// Outputs are the reference's bit for bit; the rate is that of a scalar loop per output (config 5 down: seconds).
#include "common.hpp"
#include "device_types.hpp"
#include "epilogue.hpp"

namespace hodu {
namespace {

// t_f8e4m3.h:27-50: exponent 15 is infinity (mantissa 0) or NaN, unlike the OCP format the hardware converts
__device__ __forceinline__ float ref_f8e4m3_to_f32(uint8_t b) {
    const uint32_t e = (b >> 3) & 15u, m = b & 7u;
    float v;
    if (e == 15u) {
        if (m != 0u) return __uint_as_float(0x7FC00000u);
        v = __uint_as_float(0x7F800000u);
    } else if (e == 0u) {
        v = ldexpf((float)m * 0.125f, -6);
    } else {
        v = ldexpf(1.0f + (float)m * 0.125f, (int)e - 7);
    }
    return (b & 0x80u) ? -v : v;
}
// t_f8e5m2.h:27-50
__device__ __forceinline__ float ref_f8e5m2_to_f32(uint8_t b) {
    const uint32_t e = (b >> 2) & 31u, m = b & 3u;
    float v;
    if (e == 31u) {
        if (m != 0u) return __uint_as_float(0x7FC00000u);
        v = __uint_as_float(0x7F800000u);
    } else if (e == 0u) {
        v = ldexpf((float)m * 0.25f, -14);
    } else {
        v = ldexpf(1.0f + (float)m * 0.25f, (int)e - 15);
    }
    return (b & 0x80u) ? -v : v;
}
// t_f8e4m3.h:52-85 and t_f8e5m2.h:52-84, one routine: MB mantissa bits, exponent bias BIAS, largest finite value
// LIMIT, smallest value kept TINY.  The last line is evaluated in 32 bits and cut to a byte, as there: with e == 0
// the mantissa term can be negative.
template <int MB, int BIAS, int EMAX> __device__ __forceinline__ uint8_t ref_f32_to_f8(float val, float limit, float tiny) {
#pragma clang fp contract(off)
    if (val == 0.0f) return 0;
    if (val != val) return 0x7F;
    const uint32_t sign = val < 0 ? 1u : 0u;
    val = fabsf(val);
    if (isinf(val) || val > limit) return (uint8_t)((sign << 7) | 0x7Fu);
    if (val < tiny) return (uint8_t)(sign << 7);
    int e;
    float m = frexpf(val, &e);
    e += BIAS - 1;
    if (e <= 0) {
        m = ldexpf(m, e);
        e = 0;
    } else if (e >= EMAX) {
        return (uint8_t)((sign << 7) | 0x7Fu);
    }
    int mb = (int)((m * 2.0f - 1.0f) * (float)(1 << MB) + 0.5f);
    if (mb > (1 << MB) - 1) mb = (1 << MB) - 1;
    return (uint8_t)((sign << 7) | (uint32_t)(e << MB) | (uint32_t)mb);
}

template <int DT> struct RefElem;
template <> struct RefElem<HODU_BF16> {
    typedef uint16_t T;
    static __device__ __forceinline__ float widen(T v) { return bf16_bits_to_f32(v); }
    static __device__ __forceinline__ T narrow(float w) { return (uint16_t)(__float_as_uint(w) >> 16); }
};
template <> struct RefElem<HODU_F16> {
    typedef uint16_t T;
    static __device__ __forceinline__ float widen(T v) { return f16_bits_to_f32(v); }
    static __device__ __forceinline__ T narrow(float w) { return ref_f32_to_f16(w); }
};
template <> struct RefElem<HODU_F8E4M3> {
    typedef uint8_t T;
    static __device__ __forceinline__ float widen(T v) { return ref_f8e4m3_to_f32(v); }
    static __device__ __forceinline__ T narrow(float w) { return ref_f32_to_f8<3, 7, 15>(w, 448.0f, 0.001953125f); }
};
template <> struct RefElem<HODU_F8E5M2> {
    typedef uint8_t T;
    static __device__ __forceinline__ float widen(T v) { return ref_f8e5m2_to_f32(v); }
    static __device__ __forceinline__ T narrow(float w) { return ref_f32_to_f8<2, 15, 31>(w, 57344.0f, 0.0000152587890625f); }
};
// the weight of the bf16 x f8e4m3 kind: to_dtype(bf16) widens it exactly, by the OCP reading of the byte (Rust's
// float8 type, not the C decoder above), before the bf16 product sees it
struct WeightF8 {
    typedef uint8_t T;
    static __device__ __forceinline__ float widen(T v) { return f8e4m3_to_f32(v); }
};

// E: the output's element (and the left operand's); EB: the right operand's storage and widening
template <class E, class EB, int OUT_DT, bool EPI>
__global__ __launch_bounds__(256) void reference_sum_kernel(const typename E::T *__restrict__ A, const typename EB::T *__restrict__ B,
                                                           typename E::T *__restrict__ C, DevProduct g, long total) {
#pragma clang fp contract(off)
    const long per_batch = (long)g.M * g.N;
    for (long idx = (long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long)gridDim.x * 256) {
        const long batch = idx / per_batch, rem = idx % per_batch;
        const long m = rem / g.N, n = rem % g.N;
        long ao, bo;
        batch_offsets(g, batch, ao, bo);
        const typename E::T *a = A + ao + m * g.a_m;
        const typename EB::T *b = B + bo + n * g.b_n;
        typename E::T sum = 0;
        for (long k = 0; k < g.K; k++) {
            const typename E::T p = E::narrow(E::widen(a[k * g.a_k]) * EB::widen(b[k * g.b_k]));
            sum = E::narrow(E::widen(sum) + E::widen(p));
        }
        if constexpr (EPI) sum = epilogue_apply_call<OUT_DT>(g.epi, sum, n);
        C[idx] = sum;
    }
}

template <class E, class EB, int OUT_DT>
int run(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    const long total = g.batches * (long)g.M * g.N;
    if (total <= 0) return HODU_ROCM_OK;
    const long want = (total + 255) / 256, cap = (long)ctx->props.multiProcessorCount * 64;
    const unsigned blocks = (unsigned)(want < cap ? want : cap);
    hipLaunchKernelGGL((reference_sum_kernel<E, EB, OUT_DT, false>), dim3(blocks), dim3(256), 0, ctx->stream, (const typename E::T *)a,
                       (const typename EB::T *)b, (typename E::T *)c, g, total);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}
template <class E, class EB, int OUT_DT>
int run_steps(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    if (g.epi.n == 0) return run<E, EB, OUT_DT>(ctx, a, b, c, g);
    const long total = g.batches * (long)g.M * g.N;
    if (total <= 0) return HODU_ROCM_OK;
    const long want = (total + 255) / 256, cap = (long)ctx->props.multiProcessorCount * 64;
    const unsigned blocks = (unsigned)(want < cap ? want : cap);
    hipLaunchKernelGGL((reference_sum_kernel<E, EB, OUT_DT, true>), dim3(blocks), dim3(256), 0, ctx->stream, (const typename E::T *)a,
                       (const typename EB::T *)b, (typename E::T *)c, g, total);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace

// UNSUPPORTED (no error text) for the dtypes whose reference arithmetic the other kernels already are: integers,
// f64, and f32, which the reference hands to a BLAS
int launch_reference_sums(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    if (kind == PK_BF16_F8W) {
        ctx->last_kernel = "reference_sums_bf16_f8w";
        return run_steps<RefElem<HODU_BF16>, WeightF8, HODU_BF16>(ctx, a, b, c, g);
    }
    if (kind != PK_SAME) return HODU_ROCM_UNSUPPORTED;
    switch (dtype) {
    case HODU_BF16:
        ctx->last_kernel = "reference_sums_bf16";
        return run_steps<RefElem<HODU_BF16>, RefElem<HODU_BF16>, HODU_BF16>(ctx, a, b, c, g);
    case HODU_F16:
        ctx->last_kernel = "reference_sums_f16";
        return run_steps<RefElem<HODU_F16>, RefElem<HODU_F16>, HODU_F16>(ctx, a, b, c, g);
    case HODU_F8E4M3:
        ctx->last_kernel = "reference_sums_f8e4m3";
        return run<RefElem<HODU_F8E4M3>, RefElem<HODU_F8E4M3>, HODU_F8E4M3>(ctx, a, b, c, g);
    case HODU_F8E5M2:
        ctx->last_kernel = "reference_sums_f8e5m2";
        return run<RefElem<HODU_F8E5M2>, RefElem<HODU_F8E5M2>, HODU_F8E5M2>(ctx, a, b, c, g);
    default: return HODU_ROCM_UNSUPPORTED;
    }
}

}  // namespace hodu
