// Element traits shared by the kernels that handle every dtype (the generic product, the reduction): how an element
// is stored, which type it is accumulated in, and how an accumulator becomes a stored element again.
// Narrow floats (f8, bf16, f16) and f32 accumulate in f32 and round once on store (RNE; f8 saturates); f64 in f64;
// integers wrap: unsigned arithmetic of at least their own width, truncated on store.
#pragma once

#include "device_types.hpp"

namespace hodu {

template <int DT> struct Elem;

#define NATIVE_ELEM(ID, S, A)                                                                  \
    template <> struct Elem<ID> {                                                              \
        typedef S storage;                                                                     \
        typedef A acc;                                                                         \
        static constexpr int id = ID;                                                          \
        static __device__ __forceinline__ A load(S v) { return (A)v; }                         \
        static __device__ __forceinline__ S store(A v) { return (S)v; }                        \
    };
NATIVE_ELEM(HODU_F32, float, float)
NATIVE_ELEM(HODU_F64, double, double)
NATIVE_ELEM(HODU_U8, uint8_t, uint32_t)
NATIVE_ELEM(HODU_U16, uint16_t, uint32_t)
NATIVE_ELEM(HODU_U32, uint32_t, uint32_t)
NATIVE_ELEM(HODU_U64, uint64_t, uint64_t)
NATIVE_ELEM(HODU_I64, int64_t, uint64_t)
#undef NATIVE_ELEM

// signed integers: sign-extend into the unsigned accumulate type, then modular arithmetic
#define SIGNED_ELEM(ID, S)                                                                     \
    template <> struct Elem<ID> {                                                              \
        typedef S storage;                                                                     \
        typedef uint32_t acc;                                                                  \
        static constexpr int id = ID;                                                          \
        static __device__ __forceinline__ uint32_t load(S v) { return (uint32_t)(int32_t)v; }  \
        static __device__ __forceinline__ S store(uint32_t v) { return (S)v; }                 \
    };
SIGNED_ELEM(HODU_I8, int8_t)
SIGNED_ELEM(HODU_I16, int16_t)
SIGNED_ELEM(HODU_I32, int32_t)
#undef SIGNED_ELEM

template <> struct Elem<HODU_BF16> {
    static constexpr int id = HODU_BF16;
    typedef uint16_t storage;
    typedef float acc;
    static __device__ __forceinline__ float load(uint16_t v) { return bf16_bits_to_f32(v); }
    static __device__ __forceinline__ uint16_t store(float v) { return f32_to_bf16_bits_rne(v); }
};
template <> struct Elem<HODU_F16> {
    static constexpr int id = HODU_F16;
    typedef uint16_t storage;
    typedef float acc;
    static __device__ __forceinline__ float load(uint16_t v) { return f16_bits_to_f32(v); }
    static __device__ __forceinline__ uint16_t store(float v) { return f32_to_f16_bits_rne(v); }
};
template <> struct Elem<HODU_F8E4M3> {
    static constexpr int id = HODU_F8E4M3;
    typedef uint8_t storage;
    typedef float acc;
    static __device__ __forceinline__ float load(uint8_t v) { return f8e4m3_to_f32(v); }
    static __device__ __forceinline__ uint8_t store(float v) { return f32_to_f8e4m3_sat(v); }
};
template <> struct Elem<HODU_F8E5M2> {
    static constexpr int id = HODU_F8E5M2;
    typedef uint8_t storage;
    typedef float acc;
    static __device__ __forceinline__ float load(uint8_t v) { return f8e5m2_to_f32(v); }
    static __device__ __forceinline__ uint8_t store(float v) { return f32_to_f8e5m2_sat(v); }
};

}  // namespace hodu
