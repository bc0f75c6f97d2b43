// Element-wise steps fused into the store of a product (DevEpilogue): the arithmetic of the reference's
// element-wise CPU kernels on ONE stored element, by output dtype.
//
//   add         crates/hodu_cpu_kernels/kernels/ops_binary.c:208-262 (IMPL_BINARY_OP_CONVERT: widen both operands to
//               f32, add, narrow with the type's own routine) and the native-type macro above it
//   mul_scalar  kernels/ops_unary.c:352-386 (IMPL_UNARY_WITH_SCALAR_CONVERT: the scalar arrives in the storage type and
//               is widened the same way) and :138-200 for the native types
//   relu        kernels/ops_unary.c:648-697, 1404, 1484: (x > 0) ? x : 0 in f32 -- NaN and -0 become +0
//
// Narrowing is the reference's: bf16 truncates (t_bf16.h:35-39), f16 goes through its frexp-based routine
// (t_f16.h), integers wrap in their own width.  The 8-bit float dtypes have no epilogue: the reference's narrowing
// routine for them does not survive subnormal inputs, the products here round them differently on purpose, and a
// fused step would have to pick one of the two.
#pragma once

#include <type_traits>

#include "device_types.hpp"

namespace hodu {

// the reference's f32 -> f16 (t_f16.h): round half up on the mantissa with a clamp instead of a carry, values
// below 2^-14 flush to zero
__device__ __forceinline__ uint16_t ref_f32_to_f16(float val) {
#pragma clang fp contract(off)
    if (val == 0.0f) return 0;
    if (val != val) return 0x7E00;
    const uint32_t sign = val < 0 ? 1u : 0u;
    val = fabsf(val);
    if (isinf(val) || val > 65504.0f) return (uint16_t)((sign << 15) | 0x7C00u);
    if (val < 0.00006103515625f) return (uint16_t)(sign << 15);
    int e;
    float m = frexpf(val, &e);
    e += 14;
    if (e <= 0) { m = ldexpf(m, e); e = 0; }
    else if (e >= 31) return (uint16_t)((sign << 15) | 0x7C00u);
    int mb = (int)((m * 2.0f - 1.0f) * 1024.0f + 0.5f);
    if (mb > 1023) mb = 1023;
    return (uint16_t)((sign << 15) | ((uint32_t)e << 10) | (uint32_t)mb);
}

template <int DT> struct EpiElem;  // T: stored type; W: type the reference computes in; U: T's bits

template <> struct EpiElem<HODU_BF16> {
    typedef uint16_t T; typedef float W; typedef uint16_t U;
    static constexpr bool floating = true;
    static __device__ __forceinline__ W widen(T v) { return bf16_bits_to_f32(v); }
    static __device__ __forceinline__ T narrow(W w) { return (uint16_t)(__float_as_uint(w) >> 16); }
};
template <> struct EpiElem<HODU_F16> {
    typedef uint16_t T; typedef float W; typedef uint16_t U;
    static constexpr bool floating = true;
    static __device__ __forceinline__ W widen(T v) { return f16_bits_to_f32(v); }
    static __device__ __forceinline__ T narrow(W w) { return ref_f32_to_f16(w); }
};
template <> struct EpiElem<HODU_F32> {
    typedef float T; typedef float W; typedef uint32_t U;
    static constexpr bool floating = true;
    static __device__ __forceinline__ W widen(T v) { return v; }
    static __device__ __forceinline__ T narrow(W w) { return w; }
};
template <> struct EpiElem<HODU_F64> {
    typedef double T; typedef double W; typedef uint64_t U;
    static constexpr bool floating = true;
    static __device__ __forceinline__ W widen(T v) { return v; }
    static __device__ __forceinline__ T narrow(W w) { return w; }
};
// integers: modular arithmetic in the unsigned type of the same width (what the reference's `TYPE x = a + b`
// comes to on two's-complement hardware)
#define HODU_EPI_INT(ID, S, UU)                                                      \
    template <> struct EpiElem<ID> {                                                 \
        typedef S T; typedef UU W; typedef UU U;                                     \
        static constexpr bool floating = false;                                      \
        static __device__ __forceinline__ W widen(T v) { return (UU)v; }             \
        static __device__ __forceinline__ T narrow(W w) { return (S)w; }             \
    };
HODU_EPI_INT(HODU_U8, uint8_t, uint8_t)
HODU_EPI_INT(HODU_U16, uint16_t, uint16_t)
HODU_EPI_INT(HODU_U32, uint32_t, uint32_t)
HODU_EPI_INT(HODU_U64, uint64_t, uint64_t)
HODU_EPI_INT(HODU_I8, int8_t, uint8_t)
HODU_EPI_INT(HODU_I16, int16_t, uint16_t)
HODU_EPI_INT(HODU_I32, int32_t, uint32_t)
HODU_EPI_INT(HODU_I64, int64_t, uint64_t)
#undef HODU_EPI_INT
// the 8-bit floats never carry an epilogue (the entry points refuse it): the value passes through
#define HODU_EPI_NONE(ID)                                                            \
    template <> struct EpiElem<ID> {                                                 \
        typedef uint8_t T; typedef uint8_t W; typedef uint8_t U;                     \
        static constexpr bool floating = false;                                      \
        static __device__ __forceinline__ W widen(T v) { return v; }                 \
        static __device__ __forceinline__ T narrow(W w) { return w; }                \
    };
HODU_EPI_NONE(HODU_F8E4M3)
HODU_EPI_NONE(HODU_F8E5M2)
#undef HODU_EPI_NONE

// a * b in the type the reference computes in.  Two 16-bit integers would be promoted to int, where 65535 * 65535
// overflows -- undefined, although every compiler in sight produces the wrapped product the reference's
// `uint16_t x = a * b` means; multiplied as unsigned the wrap is what the language says.
template <class W> __device__ __forceinline__ W epi_mul(W a, W b) {
    if constexpr (std::is_integral<W>::value && sizeof(W) == 2) return (W)((unsigned)a * (unsigned)b);
    else return (W)(a * b);
}

// v: the element the product alone would store at column n of its row; returns what the fused launch stores.
// e.n is the same for every lane, so a product without an epilogue pays one scalar compare per call.  The loop over
// the steps stays rolled and every step narrows in one place: the routine is inlined at every store site of every
// kernel, and the f16 narrowing alone is some fifty instructions.
template <int DT>
__device__ __forceinline__ typename EpiElem<DT>::T epilogue_apply(const DevEpilogue &e, typename EpiElem<DT>::T v, long n) {
#pragma clang fp contract(off)
    typedef EpiElem<DT> E;
    typedef typename E::T T;
    typedef typename E::W W;
    typedef typename E::U U;
#pragma unroll 1
    for (int i = 0; i < e.n; i++) {
        const DevEpilogueStep &s = e.step[i];
        const W x = E::widen(v);
        W r = x;
        if (s.op == EPI_ADD_ROW) {
            r = (W)(x + E::widen(static_cast<const T *>(s.vec)[n * s.stride]));
        } else if (s.op == EPI_MUL_SCALAR) {
            r = epi_mul<W>(x, E::widen(__builtin_bit_cast(T, (U)s.scalar)));
        } else if (E::floating) {  // EPI_RELU
            r = x > (W)0 ? x : (W)0;
        }
        v = E::narrow(r);
    }
    return v;
}

// For kernels in which a lane stores the same EPV neighbouring columns over and over (row after row of a tile): what
// the steps need per column is fetched once -- the vector's entries for those columns, the scalar, the ops -- and
// then applied to any number of EPV-wide pieces of rows.
template <int DT, int EPV> struct EpiPrepared {
    typename EpiElem<DT>::W k[kMaxEpilogueSteps][EPV];  // ADD_ROW: vector entries; MUL_SCALAR: k[i][0] is the scalar
    int op[kMaxEpilogueSteps];
    int n;  // number of steps
};

// n0: first of the lane's EPV columns; columns at or beyond N are clamped into the vector (their results are
// never stored)
template <int DT, int EPV>
__device__ __forceinline__ EpiPrepared<DT, EPV> epilogue_prepare(const DevEpilogue &e, int n0, int N) {
    typedef EpiElem<DT> E;
    typedef typename E::T T;
    typedef typename E::W W;
    typedef typename E::U U;
    EpiPrepared<DT, EPV> p;
    p.n = e.n;
#pragma unroll
    for (int i = 0; i < kMaxEpilogueSteps; i++) {
        p.op[i] = i < e.n ? e.step[i].op : 0;
#pragma unroll
        for (int k = 0; k < EPV; k++) p.k[i][k] = (W)0;
        if (p.op[i] == EPI_ADD_ROW) {
            const T *vec = static_cast<const T *>(e.step[i].vec);
            const long stride = e.step[i].stride;
#pragma unroll
            for (int k = 0; k < EPV; k++) {
                const int col = n0 + k < N ? n0 + k : N - 1;
                p.k[i][k] = E::widen(vec[col * stride]);
            }
        } else if (p.op[i] == EPI_MUL_SCALAR) {
            p.k[i][0] = E::widen(__builtin_bit_cast(T, (U)e.step[i].scalar));
        }
    }
    return p;
}

// v: EPV stored elements of one row, columns as prepared
template <int DT, int EPV>
__device__ __forceinline__ void epilogue_apply_prepared(const EpiPrepared<DT, EPV> &p, typename EpiElem<DT>::T *v) {
#pragma clang fp contract(off)
    typedef EpiElem<DT> E;
    typedef typename E::W W;
#pragma unroll
    for (int i = 0; i < kMaxEpilogueSteps; i++) {
        if (i >= p.n) break;
        W r[EPV];
#pragma unroll
        for (int k = 0; k < EPV; k++) r[k] = E::widen(v[k]);
        if (p.op[i] == EPI_ADD_ROW) {
#pragma unroll
            for (int k = 0; k < EPV; k++) r[k] = (W)(r[k] + p.k[i][k]);
        } else if (p.op[i] == EPI_MUL_SCALAR) {
#pragma unroll
            for (int k = 0; k < EPV; k++) r[k] = epi_mul<W>(r[k], p.k[i][0]);
        } else if (E::floating) {  // EPI_RELU
#pragma unroll
            for (int k = 0; k < EPV; k++) r[k] = r[k] > (W)0 ? r[k] : (W)0;
        }
#pragma unroll
        for (int k = 0; k < EPV; k++) v[k] = E::narrow(r[k]);
    }
}

// The same for G pieces at once (the same columns of G rows): the steps are the outer loop, so a launch's choice
// of operation is branched on once per step and group instead of once per step and piece, and each step is G * EPV
// independent operations.  Between steps a value is narrowed and widened again, exactly what storing it and loading
// it for the next step would do (for bf16 that is one AND).
template <int DT, int EPV, int G>
__device__ __forceinline__ void epilogue_apply_prepared_group(const EpiPrepared<DT, EPV> &p, typename EpiElem<DT>::T (&v)[G][EPV]) {
#pragma clang fp contract(off)
    typedef EpiElem<DT> E;
    typedef typename E::W W;
    W r[G][EPV];
#pragma unroll
    for (int q = 0; q < G; q++)
#pragma unroll
        for (int k = 0; k < EPV; k++) r[q][k] = E::widen(v[q][k]);
#pragma unroll
    for (int i = 0; i < kMaxEpilogueSteps; i++) {
        if (i >= p.n) break;
        if (p.op[i] == EPI_ADD_ROW) {
#pragma unroll
            for (int q = 0; q < G; q++)
#pragma unroll
                for (int k = 0; k < EPV; k++) r[q][k] = E::widen(E::narrow((W)(r[q][k] + p.k[i][k])));
        } else if (p.op[i] == EPI_MUL_SCALAR) {
#pragma unroll
            for (int q = 0; q < G; q++)
#pragma unroll
                for (int k = 0; k < EPV; k++) r[q][k] = E::widen(E::narrow(epi_mul<W>(r[q][k], p.k[i][0])));
        } else if (E::floating) {  // EPI_RELU
#pragma unroll
            for (int q = 0; q < G; q++)
#pragma unroll
                for (int k = 0; k < EPV; k++) r[q][k] = E::widen(E::narrow(r[q][k] > (W)0 ? r[q][k] : (W)0));
        }
    }
#pragma unroll
    for (int q = 0; q < G; q++)
#pragma unroll
        for (int k = 0; k < EPV; k++) v[q][k] = E::narrow(r[q][k]);
}

// the same behind a call, for kernels whose accumulator layout makes for hundreds of store sites per lane
template <int DT>
__device__ __attribute__((noinline)) typename EpiElem<DT>::T epilogue_apply_call(const DevEpilogue &e, typename EpiElem<DT>::T v,
                                                                                  long n) {
    return epilogue_apply<DT>(e, v, n);
}

}  // namespace hodu
