// LDS-staged MFMA tile kernel for gfx950, shared by the per-dtype translation units.
//
// Replaces the hot loops of hodu_cpu_matmul_<dt> / hodu_cpu_dot_<dt>
// (crates/hodu_cpu_kernels/kernels/ops_matrix.c:46-193, :399-549) for bf16, f16, f32, the fused
// f8e4m3-weight product and the fused i8 -> i32 product.
//
// Shape of the kernel
//   * one workgroup (WM x WN wavefronts of 64 lanes) owns a BM x BN output tile and walks K in
//     steps of 128 bytes of the compute type (64 bf16/f16, 128 i8, 32 f32);
//   * both operands are staged through LDS as rows of 16-byte chunks, each chunk holding
//     consecutive k of ONE row, so a lane's MFMA operand is a single ds_read_b128;
//   * global -> register -> LDS staging is double buffered (one barrier per K step): the global
//     loads of step t+1 are issued before the MFMAs of step t and written to the other LDS
//     buffer after them;
//   * the path from global memory to LDS is chosen per operand from its strides:
//       LM_K      k is the dense dim: 16-byte (8-byte for f8 storage) loads along k
//       LM_MN     the row dim (m of lhs / n of rhs) is dense: loads along the rows for 8 (16-bit
//                 and 8-bit types) or 4 (f32) consecutive k, transposed in registers with
//                 v_perm_b32 on the way to LDS -- a transposed view costs no extra HBM traffic
//       LM_MNU    the row dim is dense but its vectors are not 16-byte aligned, or the row count is no whole
//                 number of vectors (a [K, N] weight with an odd N): the LM_MN scheme with unaligned loads
//       LM_SCALAR anything else (odd strides, misaligned, ragged K): element loads with bounds
//     f8e4m3 storage is widened to bf16 in registers between the global load and the LDS store
//     (v_cvt_pk_f32_fp8 + v_perm_b32; exact, since e4m3 has 3 mantissa bits), so the weight is
//     read from HBM once, as bytes;
//   * accumulation is f32 (i32 for the i8 product) in MFMA accumulators; the result is rounded
//     once (RNE) on store.
#pragma once

#include "common.hpp"
#include "device_types.hpp"
#include "tile_walk.hpp"
#include "epilogue.hpp"

namespace hodu {
namespace mfma {

enum { CK_BF16 = 0, CK_F16 = 1, CK_I8 = 2, CK_F32 = 3 };  // compute kind (type held in LDS / fed to MFMA)
enum { SK_SAME = 0, SK_F8 = 1 };                         // operand storage: compute type, or f8e4m3 -> bf16
enum { LM_K = 0, LM_MN = 1, LM_SCALAR = 2, LM_MNU = 3 };
enum { OUT_BF16 = 0, OUT_F16 = 1, OUT_F32 = 2, OUT_I32 = 3, OUT_I8 = 6, OUT_U8 = 7 };  // (4, 5: the f8 outputs)

constexpr int ROW_BYTES = 128;   // bytes of compute type per LDS row per K step
constexpr int ROW_PITCH = 144;   // padded: 16 consecutive rows at one chunk hit 64 distinct banks
constexpr int CHUNKS = 8;        // 16-byte chunks per row

template <class To, class From> __device__ __forceinline__ To bitcast(const From &f) {
    static_assert(sizeof(To) == sizeof(From), "size");
    return __builtin_bit_cast(To, f);
}

template <int CK> struct Compute;
template <> struct Compute<CK_BF16> {
    static constexpr int ES = 2;
    typedef f32x4_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<bf16x8_t>(a), bitcast<bf16x8_t>(b), c, 0, 0, 0);
    }
};
template <> struct Compute<CK_F16> {
    static constexpr int ES = 2;
    typedef f32x4_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<f16x8_t>(a), bitcast<f16x8_t>(b), c, 0, 0, 0);
    }
};
template <> struct Compute<CK_I8> {
    static constexpr int ES = 1;
    typedef i32x4_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_i32_16x16x64_i8(bitcast<i32x4_t>(a), bitcast<i32x4_t>(b), c, 0, 0, 0);
    }
};
template <> struct Compute<CK_F32> {
    static constexpr int ES = 4;
    typedef f32x4_t acc_t;
    // a lane's chunk holds 4 consecutive k of its row; MFMA t consumes element t of every lane, so
    // the four lane groups cover k = t, 4+t, 8+t, 12+t -- the same assignment for both operands
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        const f32x4_t af = bitcast<f32x4_t>(a), bf = bitcast<f32x4_t>(b);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.x, bf.x, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.y, bf.y, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.z, bf.z, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.w, bf.w, c, 0, 0, 0);
    }
};

// 32x32 MFMA tiles for the tile kernels.  One 4-pass 16x16x32 MFMA can be issued by a wavefront only
// about every 28 cycles (measured: a single wavefront per SIMD sustains 56 % of the matrix-core peak
// with it), whereas the 8-pass 32x32x16 form keeps the pipe full from one wavefront and leaves issue
// slots for LDS and address instructions in between.
// Fragment: lane l supplies row (or column) l % 32 and the 16 bytes of k-half l / 32; a 64-byte
// slice of K therefore takes two MFMAs per tile, fed by chunks 2*s + (l / 32).
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
template <int CK> struct Compute32;
template <> struct Compute32<CK_BF16> {
    typedef f32x16_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bitcast<bf16x8_t>(a), bitcast<bf16x8_t>(b), c, 0, 0, 0);
    }
};
template <> struct Compute32<CK_F16> {
    typedef f32x16_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(bitcast<f16x8_t>(a), bitcast<f16x8_t>(b), c, 0, 0, 0);
    }
};
template <> struct Compute32<CK_I8> {
    typedef i32x16_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(bitcast<i32x4_t>(a), bitcast<i32x4_t>(b), c, 0, 0, 0);
    }
};
template <> struct Compute32<CK_F32> {
    typedef f32x16_t acc_t;
    // a lane's chunk holds 4 consecutive k; MFMA t consumes element t of both lane halves (k = t, 4 + t)
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        const f32x4_t af = bitcast<f32x4_t>(a), bf = bitcast<f32x4_t>(b);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.x, bf.x, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.y, bf.y, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.z, bf.z, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(af.w, bf.w, c, 0, 0, 0);
    }
};

// ------------------------------------------------------------------------------------------------
// LDS layouts.  Both give conflict-free ds_read_b128 for "16 lanes = 16 consecutive rows, one chunk".
// ------------------------------------------------------------------------------------------------
// Row-major with an XOR swizzle, in blocks of 8 rows (1 KB) separated by 128 bytes: chunk c of
// row r sits at slot c ^ (r % 8).  A block is exactly what one wavefront-wide 16-byte-per-lane
// LDS-DMA load writes (lane l -> byte 16*l), which is why there is no padding INSIDE a block; the
// swizzle is applied on the global-address side of that load.  Used by LM_K and LM_SCALAR.
constexpr int SWZ_BLOCK = 8 * ROW_BYTES + 128;
__device__ __forceinline__ int lds_swizzled(int row, int chunk) {
    return (row >> 3) * SWZ_BLOCK + (row & 7) * ROW_BYTES + ((chunk ^ (row & 7)) << 4);
}

// Written by LM_MN, where a lane owns the same chunk of G consecutive rows: rows are split by
// (row % G) into G sub-planes so that neighbouring lanes (row groups) write neighbouring 16 bytes.
template <int ROWS, int G> struct MnLayout {
    static constexpr int SUB = (ROWS / G) * 16 + (G == 8 ? 32 : 64);  // bytes per (row % G) sub-plane
    static constexpr int PLANE = G * SUB;                              // bytes per chunk index
    static __device__ __forceinline__ int at(int row, int chunk) {
        return chunk * PLANE + (row % G) * SUB + (row / G) * 16;
    }
};

// ------------------------------------------------------------------------------------------------
// operand description handed to the loaders
// ------------------------------------------------------------------------------------------------
struct Operand {
    const char *base;   // storage pointer, batch and view offset applied
    long row_stride;    // elements between consecutive rows (m of lhs, n of rhs)
    long k_stride;      // elements between consecutive k
    int rows;           // extent of the row dim (M or N)
    int K;
};

__device__ __forceinline__ u32x4_t zero4() { return u32x4_t{0u, 0u, 0u, 0u}; }
__device__ __forceinline__ u32x4_t ldg128(const char *p) { return *reinterpret_cast<const u32x4_t *>(p); }
__device__ __forceinline__ u32x2_t ldg64(const char *p) { return *reinterpret_cast<const u32x2_t *>(p); }
// 16 bytes from an address that is only known to be a multiple of 2 (one 16-byte load all the same)
typedef u32x4_t __attribute__((aligned(2))) u32x4_elem_aligned_t;
__device__ __forceinline__ u32x4_t ldg128_elem_aligned(const char *p) { return *reinterpret_cast<const u32x4_elem_aligned_t *>(p); }
// and the stores: BYTES at an address that is only known to be a multiple of ALIGN (the element size) -- one store
// instruction all the same, which is what an output with an odd row length needs ([.., 197, 197] scores)
template <int BYTES, int ALIGN> struct UnderAligned;
#define HODU_UNDER_ALIGNED(BYTES, ALIGN, BASE) \
    template <> struct UnderAligned<BYTES, ALIGN> { typedef BASE Base; typedef BASE __attribute__((aligned(ALIGN))) T; };
HODU_UNDER_ALIGNED(16, 1, u32x4_t)
HODU_UNDER_ALIGNED(16, 2, u32x4_t)
HODU_UNDER_ALIGNED(16, 4, u32x4_t)
HODU_UNDER_ALIGNED(8, 2, u32x2_t)
HODU_UNDER_ALIGNED(4, 1, uint32_t)
#undef HODU_UNDER_ALIGNED
template <int BYTES, int ALIGN> __device__ __forceinline__ void stg_elem_aligned(void *dst, const void *src) {
    typedef UnderAligned<BYTES, ALIGN> U;
    *reinterpret_cast<typename U::T *>(dst) = *reinterpret_cast<const typename U::Base *>(src);
}
__device__ __forceinline__ void lds_put(char *lds, int off, const u32x4_t &v) { *reinterpret_cast<u32x4_t *>(lds + off) = v; }
__device__ __forceinline__ u32x4_t lds_get(const char *lds, int off) { return *reinterpret_cast<const u32x4_t *>(lds + off); }

// 16 bytes per lane from global memory straight into LDS (global_load_lds_dwordx4): the wavefront
// writes 1 KB starting at `lds_block` (wave-uniform), lane l at byte 16*l
__device__ __forceinline__ void dma16(const char *gptr, char *lds_block) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gptr,
                                     (__attribute__((address_space(3))) void *)lds_block, 16, 0, 0);
}

// two f8e4m3 -> two bf16 packed (lo = first)
__device__ __forceinline__ uint32_t f8pair_to_bf16pair(uint32_t word, bool hi) {
    const f32x2_t f = hi ? __builtin_amdgcn_cvt_pk_f32_fp8((int)word, true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)word, false);
    return __builtin_amdgcn_perm(__float_as_uint(f.y), __float_as_uint(f.x), 0x07060302u);
}

// ------------------------------------------------------------------------------------------------
// Loader<LM, SK, CK, ROWS, NT>: stages one operand tile (ROWS rows x 128 bytes of compute type).
//   issue_full()   start moving a K step that lies fully inside K (no k checks, rows clamped): either
//                  LDS-DMA straight into `dst`, or global loads into registers
//   commit_full()  registers -> LDS for the register paths; nothing for the DMA path
//   tail()         the ragged last K step: guarded loads, zero fill, written to `dst` at once
//   at()           LDS byte offset of (row, chunk) for the fragment reads
// ------------------------------------------------------------------------------------------------
template <int LM, int SK, int CK, int ROWS, int NT> struct Loader;

// ---- k-dense, storage type == compute type: LDS-DMA, no registers, no LDS store instructions ----
template <int CK, int ROWS, int NT> struct Loader<LM_K, SK_SAME, CK, ROWS, NT> {
    static constexpr int ES = Compute<CK>::ES, EPC = 16 / ES;
    static constexpr int NW = NT / 64, BLOCKS = ROWS / 8;
    static constexpr int PER_WAVE = (BLOCKS + NW - 1) / NW;
    static constexpr int LDS_BYTES = BLOCKS * SWZ_BLOCK;
    static __device__ __forceinline__ int at(int row, int chunk) { return lds_swizzled(row, chunk); }
    __device__ __forceinline__ void issue_full(const Operand &op, int row0, int k0, int tid, char *dst) {
        const int lane = tid & 63, wave = tid >> 6;
        const int ri = lane >> 3, kc = (lane & 7) ^ ri;  // the swizzle, applied to the source address
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) {
            const int blk = i * NW + wave;
            if (BLOCKS % NW != 0 && blk >= BLOCKS) break;
            int grow = row0 + blk * 8 + ri;
            grow = grow < op.rows ? grow : op.rows - 1;
            dma16(op.base + ((long)grow * op.row_stride + k0 + kc * EPC) * ES, dst + blk * SWZ_BLOCK);
        }
    }
    __device__ __forceinline__ void commit_full(char *, int) const {}
    __device__ __forceinline__ void tail(const Operand &op, int row0, int k0, int tid, char *dst) {
        for (int c = tid; c < ROWS * CHUNKS; c += NT) {
            const int row = c >> 3, kc = c & 7;
            int grow = row0 + row;
            grow = grow < op.rows ? grow : op.rows - 1;
            const int k = k0 + kc * EPC;
            u32x4_t v = zero4();
            if (k < op.K) v = ldg128(op.base + ((long)grow * op.row_stride + k) * ES);
            lds_put(dst, lds_swizzled(row, kc), v);
        }
    }
};

// ---- k-dense f8e4m3 storage -> bf16 compute: one 8-byte load per chunk, widened at the LDS store --
template <int ROWS, int NT> struct Loader<LM_K, SK_F8, CK_BF16, ROWS, NT> {
    static constexpr int UNITS = ROWS * CHUNKS / NT;
    static_assert(ROWS * CHUNKS % NT == 0, "tile/threads");
    static constexpr int LDS_BYTES = (ROWS / 8) * SWZ_BLOCK;
    u32x2_t r[UNITS];
    static __device__ __forceinline__ int at(int row, int chunk) { return lds_swizzled(row, chunk); }
    static __device__ __forceinline__ u32x4_t widen(const u32x2_t &v) {
        return u32x4_t{f8pair_to_bf16pair(v.x, false), f8pair_to_bf16pair(v.x, true), f8pair_to_bf16pair(v.y, false),
                       f8pair_to_bf16pair(v.y, true)};
    }
    __device__ __forceinline__ void issue_full(const Operand &op, int row0, int k0, int tid, char *) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT, row = c >> 3, kc = c & 7;
            int grow = row0 + row;
            grow = grow < op.rows ? grow : op.rows - 1;
            r[u] = ldg64(op.base + (long)grow * op.row_stride + k0 + kc * 8);
        }
    }
    __device__ __forceinline__ void commit_full(char *dst, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT;
            lds_put(dst, lds_swizzled(c >> 3, c & 7), widen(r[u]));
        }
    }
    __device__ __forceinline__ void tail(const Operand &op, int row0, int k0, int tid, char *dst) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT, row = c >> 3, kc = c & 7;
            int grow = row0 + row;
            grow = grow < op.rows ? grow : op.rows - 1;
            const int k = k0 + kc * 8;
            r[u] = u32x2_t{0u, 0u};
            if (k < op.K) r[u] = ldg64(op.base + (long)grow * op.row_stride + k);
        }
        commit_full(dst, tid);
    }
};

// ---- row-dense operands: loads run along the rows for VK consecutive k, then a register transpose.
// RowDense<...> supplies the per-type pieces: VB bytes per load (RG rows), VK loads per unit, and
// transpose() turning the VK loaded vectors into RG chunks of 16 bytes (one per row).
template <int SK, int CK> struct RowDense;

// 16-bit storage: 8 loads of 8 rows (16 B) for 8 consecutive k
template <int CK> struct RowDenseHalf {
    static constexpr int RG = 8, VK = 8, SES = 2;
    typedef u32x4_t vec_t;
    static __device__ __forceinline__ vec_t zero() { return zero4(); }
    static __device__ __forceinline__ vec_t load(const char *p) { return ldg128(p); }
    static __device__ __forceinline__ void transpose(const vec_t (&v)[8], u32x4_t (&w)[8]) {
#pragma unroll
        for (int rr = 0; rr < 8; rr++) {
            // rows 2q, 2q+1 live in dword q of every k-vector
            const uint32_t sel = (rr & 1) ? 0x07060302u : 0x05040100u;
            w[rr].x = __builtin_amdgcn_perm(v[1][rr >> 1], v[0][rr >> 1], sel);
            w[rr].y = __builtin_amdgcn_perm(v[3][rr >> 1], v[2][rr >> 1], sel);
            w[rr].z = __builtin_amdgcn_perm(v[5][rr >> 1], v[4][rr >> 1], sel);
            w[rr].w = __builtin_amdgcn_perm(v[7][rr >> 1], v[6][rr >> 1], sel);
        }
    }
};
template <> struct RowDense<SK_SAME, CK_BF16> : RowDenseHalf<CK_BF16> {};
template <> struct RowDense<SK_SAME, CK_F16> : RowDenseHalf<CK_F16> {};

// f8e4m3 storage -> bf16: 8 loads of 8 rows (8 B) for 8 consecutive k; the widening conversion
// yields f32 pairs whose high halves are packed across k, so the transpose costs nothing extra
template <> struct RowDense<SK_F8, CK_BF16> {
    static constexpr int RG = 8, VK = 8, SES = 1;
    typedef u32x2_t vec_t;
    static __device__ __forceinline__ vec_t zero() { return u32x2_t{0u, 0u}; }
    static __device__ __forceinline__ vec_t load(const char *p) { return ldg64(p); }
    static __device__ __forceinline__ void transpose(const vec_t (&v)[8], u32x4_t (&w)[8]) {
#pragma unroll
        for (int p = 0; p < 4; p++) {      // k pair (2p, 2p+1)
#pragma unroll
            for (int q = 0; q < 4; q++) {  // row pair (2q, 2q+1): byte pair q of the 8-byte vector
                const uint32_t wa = q < 2 ? v[2 * p].x : v[2 * p].y;
                const uint32_t wb = q < 2 ? v[2 * p + 1].x : v[2 * p + 1].y;
                const f32x2_t fa = (q & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)wa, true)
                                           : __builtin_amdgcn_cvt_pk_f32_fp8((int)wa, false);
                const f32x2_t fb = (q & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)wb, true)
                                           : __builtin_amdgcn_cvt_pk_f32_fp8((int)wb, false);
                w[2 * q][p] = __builtin_amdgcn_perm(__float_as_uint(fb.x), __float_as_uint(fa.x), 0x07060302u);
                w[2 * q + 1][p] = __builtin_amdgcn_perm(__float_as_uint(fb.y), __float_as_uint(fa.y), 0x07060302u);
            }
        }
    }
};

// 8-bit storage: 16 loads of 8 rows (8 B) for 16 consecutive k, two-level byte transpose
template <> struct RowDense<SK_SAME, CK_I8> {
    static constexpr int RG = 8, VK = 16, SES = 1;
    typedef u32x2_t vec_t;
    static __device__ __forceinline__ vec_t zero() { return u32x2_t{0u, 0u}; }
    static __device__ __forceinline__ vec_t load(const char *p) { return ldg64(p); }
    static __device__ __forceinline__ void transpose(const vec_t (&v)[16], u32x4_t (&w)[8]) {
#pragma unroll
        for (int q = 0; q < 4; q++) {  // k quad (4q .. 4q+3) -> dword q of the output chunk
#pragma unroll
            for (int h = 0; h < 2; h++) {  // rows 4h .. 4h+3 live in dword h of every k-vector
                const uint32_t v0 = h ? v[4 * q].y : v[4 * q].x;
                const uint32_t v1 = h ? v[4 * q + 1].y : v[4 * q + 1].x;
                const uint32_t v2 = h ? v[4 * q + 2].y : v[4 * q + 2].x;
                const uint32_t v3 = h ? v[4 * q + 3].y : v[4 * q + 3].x;
                // level 1: interleave bytes of (k, k+1): [k.r0, k1.r0, k.r1, k1.r1] and rows 2, 3
                const uint32_t a01 = __builtin_amdgcn_perm(v1, v0, 0x05010400u);
                const uint32_t a23 = __builtin_amdgcn_perm(v1, v0, 0x07030602u);
                const uint32_t b01 = __builtin_amdgcn_perm(v3, v2, 0x05010400u);
                const uint32_t b23 = __builtin_amdgcn_perm(v3, v2, 0x07030602u);
                // level 2: [k0, k1, k2, k3] of one row
                w[4 * h + 0][q] = __builtin_amdgcn_perm(b01, a01, 0x05040100u);
                w[4 * h + 1][q] = __builtin_amdgcn_perm(b01, a01, 0x07060302u);
                w[4 * h + 2][q] = __builtin_amdgcn_perm(b23, a23, 0x05040100u);
                w[4 * h + 3][q] = __builtin_amdgcn_perm(b23, a23, 0x07060302u);
            }
        }
    }
};

// f32 storage: 4 loads of 4 rows (16 B) for 4 consecutive k; the transpose is register renaming
template <> struct RowDense<SK_SAME, CK_F32> {
    static constexpr int RG = 4, VK = 4, SES = 4;
    typedef u32x4_t vec_t;
    static __device__ __forceinline__ vec_t zero() { return zero4(); }
    static __device__ __forceinline__ vec_t load(const char *p) { return ldg128(p); }
    static __device__ __forceinline__ void transpose(const vec_t (&v)[4], u32x4_t (&w)[4]) {
#pragma unroll
        for (int rr = 0; rr < 4; rr++) w[rr] = u32x4_t{v[0][rr], v[1][rr], v[2][rr], v[3][rr]};
    }
};

template <int SK, int CK, int ROWS, int NT> struct Loader<LM_MN, SK, CK, ROWS, NT> {
    typedef RowDense<SK, CK> RD;
    static constexpr int RG = RD::RG, VK = RD::VK, SES = RD::SES;
    typedef MnLayout<ROWS, RG> L;
    static constexpr int GROUPS = ROWS / RG;
    static constexpr int TOTAL = GROUPS * CHUNKS;  // units: (row group, chunk)
    static constexpr int UNITS = (TOTAL + NT - 1) / NT;
    static constexpr int LDS_BYTES = CHUNKS * L::PLANE;
    typename RD::vec_t r[UNITS][VK];
    static __device__ __forceinline__ int at(int row, int chunk) { return L::at(row, chunk); }
    __device__ __forceinline__ void issue_full(const Operand &op, int row0, int k0, int tid, char *) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % GROUPS, kc = (id / GROUPS) % CHUNKS;  // ids past TOTAL wrap: harmless reloads
            int row = row0 + rg * RG;
            row = row < op.rows ? row : op.rows - RG;  // op.rows % RG == 0: the clamped vector is in range
#pragma unroll
            for (int j = 0; j < VK; j++)
                r[u][j] = RD::load(op.base + ((long)(k0 + kc * VK + j) * op.k_stride + row) * SES);
        }
    }
    __device__ __forceinline__ void commit_full(char *dst, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int rg = id % GROUPS, kc = id / GROUPS;
            u32x4_t w[RG];
            RD::transpose(r[u], w);
#pragma unroll
            for (int rr = 0; rr < RG; rr++) lds_put(dst, L::at(rg * RG + rr, kc), w[rr]);
        }
    }
    __device__ __forceinline__ void tail(const Operand &op, int row0, int k0, int tid, char *dst) {
        // same registers as the full path, guarded loads with zero fill
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % GROUPS, kc = (id / GROUPS) % CHUNKS;
            const int row = row0 + rg * RG;
#pragma unroll
            for (int j = 0; j < VK; j++) {
                const int k = k0 + kc * VK + j;
                r[u][j] = RD::zero();
                if (row < op.rows && k < op.K) r[u][j] = RD::load(op.base + ((long)k * op.k_stride + row) * SES);
            }
        }
        commit_full(dst, tid);
    }
};

// ---- anything else: element loads with full bounds checks ------------------------------------------
template <int SK, int CK> struct ScalarFetch;
template <> struct ScalarFetch<SK_SAME, CK_BF16> {
    static __device__ __forceinline__ uint32_t get(const char *p, long i) { return reinterpret_cast<const uint16_t *>(p)[i]; }
};
template <> struct ScalarFetch<SK_SAME, CK_F16> {
    static __device__ __forceinline__ uint32_t get(const char *p, long i) { return reinterpret_cast<const uint16_t *>(p)[i]; }
};
template <> struct ScalarFetch<SK_SAME, CK_I8> {
    static __device__ __forceinline__ uint32_t get(const char *p, long i) { return reinterpret_cast<const uint8_t *>(p)[i]; }
};
template <> struct ScalarFetch<SK_SAME, CK_F32> {
    static __device__ __forceinline__ uint32_t get(const char *p, long i) { return reinterpret_cast<const uint32_t *>(p)[i]; }
};
template <> struct ScalarFetch<SK_F8, CK_BF16> {
    static __device__ __forceinline__ uint32_t get(const char *p, long i) {
        return __float_as_uint(f8e4m3_to_f32(reinterpret_cast<const uint8_t *>(p)[i])) >> 16;
    }
};

// ---- row-dense, unaligned: the registers, the transpose and the LDS layout of LM_MN; every vector is fetched at
// whatever alignment it has (the hardware takes unaligned vector loads).  A vector of the last row group may reach
// past the row's end: the extra lanes belong to rows that do not exist and are never stored, so that is harmless as
// long as the bytes are inside the operand -- the next k-row's.  Where they would not be (the last k-row, or k-rows
// closer together than a vector) the vector is put together element by element.
template <class V> __device__ __forceinline__ V ldg_elem_aligned(const char *p) {
    typedef V __attribute__((aligned(1))) unaligned_t;
    return *reinterpret_cast<const unaligned_t *>(p);
}
template <int SK, int CK, int ROWS, int NT> struct Loader<LM_MNU, SK, CK, ROWS, NT> : Loader<LM_MN, SK, CK, ROWS, NT> {
    typedef Loader<LM_MN, SK, CK, ROWS, NT> Base;
    typedef RowDense<SK, CK> RD;
    static constexpr int RG = RD::RG, VK = RD::VK, SES = RD::SES, GROUPS = Base::GROUPS, UNITS = Base::UNITS;
    static __device__ __forceinline__ typename RD::vec_t fetch(const Operand &op, int k, int row) {
        if (row >= op.rows) row = 0;  // a group of the tile's overhang: any readable rows will do
        const char *p = op.base + ((long)k * op.k_stride + row) * SES;
        const bool past_end = row + RG > op.rows && (k == op.K - 1 || op.k_stride < RG);
        if (!past_end) return ldg_elem_aligned<typename RD::vec_t>(p);
        union { typename RD::vec_t v; unsigned char b[sizeof(typename RD::vec_t)]; } u;
        u.v = RD::zero();
        for (int e = 0; e < RG; e++)
            if (row + e < op.rows)
                for (int i = 0; i < SES; i++) u.b[e * SES + i] = (unsigned char)p[e * SES + i];
        return u.v;
    }
    __device__ __forceinline__ void issue_full(const Operand &op, int row0, int k0, int tid, char *) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % GROUPS, kc = (id / GROUPS) % CHUNKS;
#pragma unroll
            for (int j = 0; j < VK; j++) this->r[u][j] = fetch(op, k0 + kc * VK + j, row0 + rg * RG);
        }
    }
    __device__ __forceinline__ void tail(const Operand &op, int row0, int k0, int tid, char *dst) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % GROUPS, kc = (id / GROUPS) % CHUNKS;
#pragma unroll
            for (int j = 0; j < VK; j++) {
                const int k = k0 + kc * VK + j;
                this->r[u][j] = k < op.K ? fetch(op, k, row0 + rg * RG) : RD::zero();
            }
        }
        this->commit_full(dst, tid);
    }
};

template <int SK, int CK, int ROWS, int NT> struct Loader<LM_SCALAR, SK, CK, ROWS, NT> {
    static constexpr int ES = Compute<CK>::ES, EPC = 16 / ES;
    static constexpr int UNITS = ROWS * CHUNKS / NT;
    static constexpr int LDS_BYTES = (ROWS / 8) * SWZ_BLOCK;
    u32x4_t r[UNITS];
    static __device__ __forceinline__ int at(int row, int chunk) { return lds_swizzled(row, chunk); }
    __device__ __forceinline__ void issue_full(const Operand &op, int row0, int k0, int tid, char *) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT, row = c >> 3, kc = c & 7;
            const int grow = row0 + row;
            uint32_t w[4] = {0u, 0u, 0u, 0u};
            if constexpr (SK == SK_SAME) {
                // a k-dense row whose chunk lies inside K: one 16-byte load at whatever alignment the row has (the
                // hardware takes unaligned vector loads; only their element alignment is guaranteed here).  This is
                // the case of an odd K or row stride -- a [.., 197, 197] score matrix, K = 4100.
                if (grow < op.rows && op.k_stride == 1 && k0 + kc * EPC + EPC <= op.K) {
                    r[u] = ldg128_elem_aligned(op.base + ((long)grow * op.row_stride + k0 + kc * EPC) * ES);
                    continue;
                }
            }
            if (grow < op.rows) {
#pragma unroll
                for (int e = 0; e < EPC; e++) {
                    const int k = k0 + kc * EPC + e;
                    if (k < op.K) {
                        const uint32_t v = ScalarFetch<SK, CK>::get(op.base, (long)grow * op.row_stride + (long)k * op.k_stride);
                        w[(e * ES) >> 2] |= v << (((e * ES) & 3) * 8);
                    }
                }
            }
            r[u] = u32x4_t{w[0], w[1], w[2], w[3]};
        }
    }
    __device__ __forceinline__ void commit_full(char *dst, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT;
            lds_put(dst, lds_swizzled(c >> 3, c & 7), r[u]);
        }
    }
    __device__ __forceinline__ void tail(const Operand &op, int row0, int k0, int tid, char *dst) {
        issue_full(op, row0, k0, tid, dst);  // the scalar path is guarded throughout
        commit_full(dst, tid);
    }
};

// ------------------------------------------------------------------------------------------------
// output conversion
// ------------------------------------------------------------------------------------------------
template <int OUT> struct Out;
template <> struct Out<OUT_BF16> {
    static constexpr int DT = HODU_BF16;
    typedef uint16_t T;
    static __device__ __forceinline__ T cvt(float v) { return f32_to_bf16_bits_rne(v); }
};
template <> struct Out<OUT_F16> {
    static constexpr int DT = HODU_F16;
    typedef uint16_t T;
    static __device__ __forceinline__ T cvt(float v) { return f32_to_f16_bits_rne(v); }
};
template <> struct Out<OUT_F32> {
    static constexpr int DT = HODU_F32;
    typedef float T;
    static __device__ __forceinline__ T cvt(float v) { return v; }
};
template <> struct Out<OUT_I32> {
    static constexpr int DT = HODU_I32;
    typedef int32_t T;
    static __device__ __forceinline__ T cvt(int v) { return v; }
};

// i8 x i8 -> i8 and u8 x u8 -> u8 (hodu's own 8-bit integer products, which wrap): the low byte of the exact i32 sum.
// The matrix core reads the bytes as signed; for u8 that changes each factor by a multiple of 256, so the low byte of
// the sum is the same.
template <> struct Out<OUT_I8> {
    static constexpr int DT = HODU_I8;
    typedef int8_t T;
    static __device__ __forceinline__ T cvt(int v) { return (int8_t)v; }
};
template <> struct Out<OUT_U8> {
    static constexpr int DT = HODU_U8;
    typedef uint8_t T;
    static __device__ __forceinline__ T cvt(int v) { return (uint8_t)v; }
};

// accumulator -> stored element: the product's own rounding, then the fused element-wise steps for column n
template <int OUT, class A>
__device__ __forceinline__ typename Out<OUT>::T finish(const DevEpilogue &epi, A acc, long n) {
    return epilogue_apply<Out<OUT>::DT>(epi, Out<OUT>::cvt(acc), n);
}

// the same for the kernel below, which has TM x TN x 16 store sites per lane: the steps sit behind a call, in an
// instantiation of the kernel of its own (a call costs the kernel a stack, which the plain product should not pay)
template <int OUT, class A>
__device__ __forceinline__ typename Out<OUT>::T finish_call(const DevEpilogue &epi, A acc, long n) {
    const typename Out<OUT>::T v = Out<OUT>::cvt(acc);
    return epi.n == 0 ? v : epilogue_apply_call<Out<OUT>::DT>(epi, v, n);
}

// Stores the 32x32 accumulator tile of one wavefront.  With the operands swapped in the MFMA (the
// right operand's fragment in the A slot) a lane holds, for ONE output row m = m_base + l % 32, four
// runs of four consecutive columns n = n_base + 8*q + 4*(l / 32) + e.
template <int OUT, bool EPI, class acc_t>
__device__ __forceinline__ void store_tile32(typename Out<OUT>::T *Cb, const acc_t &acc, int m, int n_base, int lh,
                                             int M, int N, bool vec_ok, const DevEpilogue &epi) {
    typedef typename Out<OUT>::T out_t;
    if (m >= M) return;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int n = n_base + 8 * q + 4 * lh;
        out_t v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if constexpr (EPI) v[e] = finish_call<OUT>(epi, acc[4 * q + e], n + e < N ? n + e : N - 1);  // ragged: stay inside the vector
            else v[e] = Out<OUT>::cvt(acc[4 * q + e]);
        }
        out_t *dst = Cb + (long)m * N + n;
        struct alignas(sizeof(out_t) * 4) Quad { out_t q[4]; };
        if (vec_ok && n + 3 < N) {
            *reinterpret_cast<Quad *>(dst) = Quad{{v[0], v[1], v[2], v[3]}};
        } else if (n + 3 < N) {  // an odd row length: the same store at element alignment
            const Quad quad{{v[0], v[1], v[2], v[3]}};
            stg_elem_aligned<sizeof(out_t) * 4, sizeof(out_t)>(dst, &quad);
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < N) dst[e] = v[e];
        }
    }
}

// ------------------------------------------------------------------------------------------------
// the kernel
// ------------------------------------------------------------------------------------------------
template <int CK_, int SKA_, int SKB_, int OUT_, int BM_, int BN_, int WM_, int WN_, int LA_, int LB_> struct Config {
    static constexpr int CK = CK_, SKA = SKA_, SKB = SKB_, OUT = OUT_, BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    static constexpr int NT = WM * WN * 64;
    static constexpr int ES = Compute<CK>::ES;
    static constexpr int BK = ROW_BYTES / ES;
    static constexpr int SA_BYTES = SKA == SK_F8 ? 1 : ES, SB_BYTES = SKB == SK_F8 ? 1 : ES;
    typedef Loader<LA_, SKA, CK, BM, NT> LoaderA;
    typedef Loader<LB_, SKB, CK, BN, NT> LoaderB;
    static constexpr int A_BYTES = LoaderA::LDS_BYTES, B_BYTES = LoaderB::LDS_BYTES;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;  // 32x32 MFMA tiles per wave
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tiling");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
};

// maps the linear workgroup id to (batch, tile_m, tile_n): tile_walk.hpp
__device__ __forceinline__ void tile_of(long pid, long total, int tiles_m, int tiles_n, long &batch, int &tm, int &tn) {
    unsigned b, m, n;
    tile_walk((unsigned)pid, (unsigned)total, (unsigned)tiles_m, (unsigned)tiles_n, b, m, n);
    batch = b;
    tm = (int)m;
    tn = (int)n;
}

// One K step (128 bytes of K = four 32-byte slices) out of LDS.  The fragments of slice s+1 are read
// into a second register set while slice s multiplies.
template <class Cfg, class acc_t>
__device__ __forceinline__ void compute_stage(const char *As, const char *Bs, acc_t (&acc)[Cfg::TM][Cfg::TN], int a_row,
                                              int b_row, int lh) {
    typedef Compute32<Cfg::CK> Cmp;
    typedef typename Cfg::LoaderA LoaderA;
    typedef typename Cfg::LoaderB LoaderB;
    constexpr int TM = Cfg::TM, TN = Cfg::TN;
    u32x4_t af[2][TM], bf[2][TN];
#pragma unroll
    for (int i = 0; i < TM; i++) af[0][i] = lds_get(As, LoaderA::at(a_row + i * 32, lh));
#pragma unroll
    for (int j = 0; j < TN; j++) bf[0][j] = lds_get(Bs, LoaderB::at(b_row + j * 32, lh));
#pragma unroll
    for (int s = 0; s < 4; s++) {
        if (s + 1 < 4) {
#pragma unroll
            for (int i = 0; i < TM; i++) af[(s + 1) & 1][i] = lds_get(As, LoaderA::at(a_row + i * 32, 2 * (s + 1) + lh));
#pragma unroll
            for (int j = 0; j < TN; j++) bf[(s + 1) & 1][j] = lds_get(Bs, LoaderB::at(b_row + j * 32, 2 * (s + 1) + lh));
        }
        // operands swapped: the accumulator then holds, per lane, runs of 4 consecutive n of one m
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int i = 0; i < TM; i++) Cmp::mma(bf[s & 1][j], af[s & 1][i], acc[i][j]);
    }
}

// LDS-DMA loads are tracked by vmcnt; wait for them before the barrier that publishes the stage
__device__ __forceinline__ void wait_vm() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// steps_per_split > 0 (kernels without fused steps only): K is cut into ranges of that many K steps, one per
// blockIdx.y, and the range's sums go to partials[blockIdx.y] in the accumulate type; a second kernel adds them
template <class Cfg, bool EPI>
__global__ __launch_bounds__(Cfg::NT) void mfma_product_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                               typename Out<Cfg::OUT>::T *__restrict__ C,
                                                               DevProduct g, int tiles_m, int tiles_n, int steps_per_split,
                                                               void *__restrict__ partials) {
    HODU_DYNAMIC_LDS(smem);
    typedef typename Compute32<Cfg::CK>::acc_t acc_t;
    typedef typename Cfg::LoaderA LoaderA;
    typedef typename Cfg::LoaderB LoaderB;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, BK = Cfg::BK;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int lr = lane & 31, lh = lane >> 5;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    const Operand opA{A + ao * Cfg::SA_BYTES, g.a_m, g.a_k, g.M, g.K};
    const Operand opB{B + bo * Cfg::SB_BYTES, g.b_n, g.b_k, g.N, g.K};

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;

    LoaderA la;
    LoaderB lb;
    const int KT_full = g.K / BK;             // K steps that lie fully inside K
    const int KT_all = (g.K + BK - 1) / BK;   // plus the ragged one, if any
    int kt0 = 0, KT = KT_all;                 // this workgroup's range of K steps
    if constexpr (!EPI) {
        if (steps_per_split > 0) {
            kt0 = blockIdx.y * steps_per_split;
            KT = kt0 + steps_per_split < KT_all ? kt0 + steps_per_split : KT_all;
        }
    }
    if (kt0 < KT_full) {
        la.issue_full(opA, m0, kt0 * BK, tid, smem);
        lb.issue_full(opB, n0, kt0 * BK, tid, smem + Cfg::A_BYTES);
        la.commit_full(smem, tid);
        lb.commit_full(smem + Cfg::A_BYTES, tid);
        wait_vm();
    } else {
        la.tail(opA, m0, kt0 * BK, tid, smem);
        lb.tail(opB, n0, kt0 * BK, tid, smem + Cfg::A_BYTES);
    }
    __syncthreads();

    const int a_row = wave_m * TM * 32 + lr, b_row = wave_n * TN * 32 + lr;
    for (int kt = kt0; kt < KT; kt++) {
        char *cur = smem + ((kt - kt0) & 1) * Cfg::STAGE_BYTES;
        char *nxt = smem + ((kt - kt0 + 1) & 1) * Cfg::STAGE_BYTES;
        const bool more_full = kt + 1 < KT_full;
        if (more_full) {  // in flight while the matrix cores work on the current stage
            la.issue_full(opA, m0, (kt + 1) * BK, tid, nxt);
            lb.issue_full(opB, n0, (kt + 1) * BK, tid, nxt + Cfg::A_BYTES);
        }
        compute_stage<Cfg>(cur, cur + Cfg::A_BYTES, acc, a_row, b_row, lh);
        if (more_full) {
            la.commit_full(nxt, tid);
            lb.commit_full(nxt + Cfg::A_BYTES, tid);
        } else if (kt + 1 < KT) {  // the ragged last step: guarded loads, zero fill
            la.tail(opA, m0, (kt + 1) * BK, tid, nxt);
            lb.tail(opB, n0, (kt + 1) * BK, tid, nxt + Cfg::A_BYTES);
        }
        wait_vm();
        __syncthreads();
    }

    const bool vec_ok = (g.N & 3) == 0;
    if constexpr (!EPI) {
        if (steps_per_split > 0) {
            constexpr int ACC = Cfg::CK == CK_I8 ? OUT_I32 : OUT_F32;
            typedef typename Out<ACC>::T part_t;
            part_t *Pb = reinterpret_cast<part_t *>(partials) + ((long)blockIdx.y * g.batches + batch) * (long)g.M * g.N;
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    store_tile32<ACC, false>(Pb, acc[i][j], m0 + wave_m * TM * 32 + i * 32 + lr, n0 + wave_n * TN * 32 + j * 32, lh,
                                             g.M, g.N, vec_ok, g.epi);
            return;
        }
    }
    out_t *Cb = C + batch * (long)g.M * g.N;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
            store_tile32<Cfg::OUT, EPI>(Cb, acc[i][j], m0 + wave_m * TM * 32 + i * 32 + lr, n0 + wave_n * TN * 32 + j * 32, lh,
                                   g.M, g.N, vec_ok, g.epi);
}

// out[i] = round(partials[0][i] + partials[1][i] + ...), the slabs added in index order: bit-reproducible
template <int OUT, class part_t>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const part_t *__restrict__ partials,
                                                           typename Out<OUT>::T *__restrict__ out, long elems, int splits,
                                                           int N, DevEpilogue epi) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= elems) return;
    // column of element i + e, for the fused element-wise steps (rows are N long, outputs contiguous)
    long col[4] = {0, 0, 0, 0};
    if (epi.n != 0) {
        col[0] = i % N;
#pragma unroll
        for (int e = 1; e < 4; e++) col[e] = col[e - 1] + 1 == N ? 0 : col[e - 1] + 1;
    }
    if (i + 3 < elems) {
        struct alignas(16) Quad { part_t q[4]; };
        Quad s = *reinterpret_cast<const Quad *>(partials + i);
        for (int k = 1; k < splits; k++) {
            const Quad t = *reinterpret_cast<const Quad *>(partials + (long)k * elems + i);
#pragma unroll
            for (int e = 0; e < 4; e++) s.q[e] += t.q[e];
        }
        struct alignas(sizeof(typename Out<OUT>::T) * 4) OutQuad { typename Out<OUT>::T q[4]; };
        *reinterpret_cast<OutQuad *>(out + i) = OutQuad{{finish<OUT>(epi, s.q[0], col[0]), finish<OUT>(epi, s.q[1], col[1]),
                                                       finish<OUT>(epi, s.q[2], col[2]), finish<OUT>(epi, s.q[3], col[3])}};
    } else {
        for (long j = i; j < elems; j++) {
            part_t s = partials[j];
            for (int k = 1; k < splits; k++) s += partials[(long)k * elems + j];
            out[j] = finish<OUT>(epi, s, col[j - i]);
        }
    }
}


// ------------------------------------------------------------------------------------------------
// host side: load-mode selection and launch
// ------------------------------------------------------------------------------------------------
// `ses`: storage element bytes; `rowvec`: rows per vector load on the LM_MN path; `epc`: compute
// elements per 16-byte chunk (= storage elements per vector load on the LM_K path)
inline int pick_mode(const void *base, long off, long row_stride, long k_stride, long rows, long K, int ses, int epc,
                     int rowvec, const DevProduct &g, const long *bstrides) {
    auto aligned = [&](long elems, int bytes) { return (elems * ses) % bytes == 0; };
    const uintptr_t addr = (uintptr_t)base + (uintptr_t)off * ses;
    const int kbytes = epc * ses, rbytes = rowvec * ses;
    bool batch_k = true, batch_r = true;
    for (int d = 0; d < g.nb; d++) {
        batch_k = batch_k && aligned(bstrides[d], kbytes);
        batch_r = batch_r && aligned(bstrides[d], rbytes);
    }
    if ((k_stride == 1 || K == 1) && K % epc == 0 && addr % kbytes == 0 && (rows == 1 || aligned(row_stride, kbytes)) && batch_k)
        return LM_K;
    if ((row_stride == 1 || rows == 1) && rows % rowvec == 0 && addr % rbytes == 0 && (K == 1 || aligned(k_stride, rbytes)) && batch_r)
        return LM_MN;
    // row-dense without the alignment (storage type = compute type only; k-rows must not overlap)
    if (row_stride == 1 && rows > 1 && ses * epc == 16 && (K == 1 || k_stride >= rows)) return LM_MNU;
    return LM_SCALAR;
}

// splits > 1: K is cut into that many ranges of whole K steps (grid.y); the partial sums go through the context's
// workspace and splitk_reduce_kernel (which also applies the fused steps); batches * M * N must be a multiple of 4
template <class Cfg> int launch_config(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g,
                                       int splits = 1) {
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    const long elems = g.batches * (long)g.M * g.N;
    const int KT = (g.K + Cfg::BK - 1) / Cfg::BK;
    int per = 0;
    if (splits > 1 && elems % 4 == 0) {
        per = (KT + splits - 1) / splits;
        splits = (KT + per - 1) / per;
    }
    if (splits <= 1 || per == 0) {
        auto kernel = g.epi.n != 0 ? mfma_product_kernel<Cfg, true> : mfma_product_kernel<Cfg, false>;
        if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
        hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream, (const char *)a,
                           (const char *)b, (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n, 0, (void *)nullptr);
        HODU_HIP(hipGetLastError());
        return HODU_ROCM_OK;
    }
    auto kernel = mfma_product_kernel<Cfg, false>;
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    if (int rc = ensure_workspace(ctx, (size_t)splits * elems * 4)) return rc;
    void *partials = ctx->workspace.ptr;
    hipLaunchKernelGGL(kernel, dim3((unsigned)total, (unsigned)splits), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream,
                       (const char *)a, (const char *)b, (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n, per, partials);
    HODU_HIP(hipGetLastError());
    const unsigned blocks = (unsigned)((elems + 1023) / 1024);
    if (Cfg::CK == CK_I8)
        hipLaunchKernelGGL((splitk_reduce_kernel<Cfg::OUT, int32_t>), dim3(blocks), dim3(256), 0, ctx->stream,
                           (const int32_t *)partials, (typename Out<Cfg::OUT>::T *)c, elems, splits, g.N, g.epi);
    else
        hipLaunchKernelGGL((splitk_reduce_kernel<Cfg::OUT, float>), dim3(blocks), dim3(256), 0, ctx->stream,
                           (const float *)partials, (typename Out<Cfg::OUT>::T *)c, elems, splits, g.N, g.epi);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace mfma
}  // namespace hodu
