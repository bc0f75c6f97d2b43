// Device-side element types, vector types and scalar conversions for gfx950.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.hpp"

// The workgroup's dynamically sized LDS as a char array called `name`, 16-byte aligned.  (A macro so that a CPU build
// of the kernels for tests, where LDS is an ordinary array, can say it its own way: it defines the macro first.)
#ifndef HODU_DYNAMIC_LDS
#define HODU_DYNAMIC_LDS(name) extern __shared__ __align__(16) char name[]
#endif

namespace hodu {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x2_t __attribute__((ext_vector_type(2)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

// batch index -> element offsets of the two operands
__device__ __forceinline__ void batch_offsets(const DevProduct &g, long batch, long &ao, long &bo) {
    ao = g.a_off;
    bo = g.b_off;
    // (a batch index is below 2^31 -- a grid has no more workgroups than that -- and 32-bit unsigned division is a
    // fraction of the instructions of the 64-bit signed one)
    unsigned rest = (unsigned)batch;
#pragma unroll
    for (int d = kKernelBatchDims - 1; d >= 0; d--) {
        if (d < g.nb) {
            const unsigned extent = (unsigned)g.bshape[d], q = rest / extent;
            const long i = (long)(rest - q * extent);
            rest = q;
            ao += i * g.a_bs[d];
            bo += i * g.b_bs[d];
        }
    }
}

// ---- scalar conversions ---------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// round-to-nearest-even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_bits_rne(float f) {
    __bf16 h = (__bf16)f;
    return __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f32_to_f16_bits_rne(float f) {
    _Float16 h = (_Float16)f;
    return __builtin_bit_cast(uint16_t, h);
}

// OCP E4M3FN / E5M2 decode in hardware (v_cvt_f32_fp8 / v_cvt_f32_bf8)
__device__ __forceinline__ float f8e4m3_to_f32(uint8_t b) { return __builtin_amdgcn_cvt_f32_fp8((int)b, 0); }
__device__ __forceinline__ float f8e5m2_to_f32(uint8_t b) { return __builtin_amdgcn_cvt_f32_bf8((int)b, 0); }

// round-to-nearest-even, saturating to the largest finite value, NaN stays NaN
__device__ __forceinline__ uint8_t f32_to_f8e4m3_sat(float f) {
    f = (f != f) ? f : fminf(fmaxf(f, -448.0f), 448.0f);
    return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false) & 0xFF);
}
__device__ __forceinline__ uint8_t f32_to_f8e5m2_sat(float f) {
    f = (f != f) ? f : fminf(fmaxf(f, -57344.0f), 57344.0f);
    return (uint8_t)(__builtin_amdgcn_cvt_pk_bf8_f32(f, f, 0, false) & 0xFF);
}
// the same narrowing of four values into the four bytes of a dword (a first, in the low byte): the conversion
// instruction takes two values and fills the half of the dword it is told to
__device__ __forceinline__ float clamp_keep_nan(float f, float lim) { return (f != f) ? f : __builtin_amdgcn_fmed3f(f, -lim, lim); }
__device__ __forceinline__ uint32_t f32x4_to_f8e4m3_sat(float a, float b, float c, float d) {
    const int lo = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_keep_nan(a, 448.0f), clamp_keep_nan(b, 448.0f), 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(clamp_keep_nan(c, 448.0f), clamp_keep_nan(d, 448.0f), lo, true);
}
__device__ __forceinline__ uint32_t f32x4_to_f8e5m2_sat(float a, float b, float c, float d) {
    const int lo = __builtin_amdgcn_cvt_pk_bf8_f32(clamp_keep_nan(a, 57344.0f), clamp_keep_nan(b, 57344.0f), 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(clamp_keep_nan(c, 57344.0f), clamp_keep_nan(d, 57344.0f), lo, true);
}

}  // namespace hodu
