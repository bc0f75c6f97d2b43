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
//       LM_SCALAR anything else (odd strides, misaligned, ragged K): element loads with bounds
//     f8e4m3 storage is widened to bf16 in registers between the global load and the LDS store
//     (v_cvt_pk_f32_fp8 + v_perm_b32; exact, since e4m3 has 3 mantissa bits), so the weight is
//     read from HBM once, as bytes;
//   * accumulation is f32 (i32 for the i8 product) in MFMA accumulators; the result is rounded
//     once (RNE) on store.
#pragma once

#include "common.hpp"
#include "device_types.hpp"

namespace hodu {
namespace mfma {

enum { CK_BF16 = 0, CK_F16 = 1, CK_I8 = 2, CK_F32 = 3 };  // compute kind (type held in LDS / fed to MFMA)
enum { SK_SAME = 0, SK_F8 = 1 };                         // operand storage: compute type, or f8e4m3 -> bf16
enum { LM_K = 0, LM_MN = 1, LM_SCALAR = 2 };
enum { OUT_BF16 = 0, OUT_F16 = 1, OUT_F32 = 2, OUT_I32 = 3 };

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

// ------------------------------------------------------------------------------------------------
// LDS layouts.  Both give conflict-free ds_read_b128 for "16 lanes = 16 consecutive rows, one chunk".
// ------------------------------------------------------------------------------------------------
// row-major, padded: written by LM_K / LM_SCALAR (a lane owns one chunk)
__device__ __forceinline__ int lds_rowmajor(int row, int chunk) { return row * ROW_PITCH + chunk * 16; }

// written by LM_MN, where a lane owns the same chunk of G consecutive rows: rows are split by
// (row % G) into G sub-planes so that neighbouring lanes (row groups) write neighbouring 16 bytes
template <int ROWS, int G> struct MnLayout {
    static constexpr int SUB = (ROWS / G) * 16 + (G == 8 ? 32 : 64);  // bytes per (row % G) sub-plane
    static constexpr int PLANE = G * SUB;                              // bytes per chunk index
    static __device__ __forceinline__ int at(int row, int chunk) {
        return chunk * PLANE + (row % G) * SUB + (row / G) * 16;
    }
};

template <int ROWS, int G> constexpr int operand_lds_bytes() {
    return (ROWS * ROW_PITCH) > (CHUNKS * MnLayout<ROWS, G>::PLANE) ? (ROWS * ROW_PITCH)
                                                                  : (CHUNKS * MnLayout<ROWS, G>::PLANE);
}

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

// two f8e4m3 -> two bf16 packed (lo = first)
__device__ __forceinline__ uint32_t f8pair_to_bf16pair(uint32_t word, bool hi) {
    const f32x2_t f = hi ? __builtin_amdgcn_cvt_pk_f32_fp8((int)word, true) : __builtin_amdgcn_cvt_pk_f32_fp8((int)word, false);
    return __builtin_amdgcn_perm(__float_as_uint(f.y), __float_as_uint(f.x), 0x07060302u);
}

// ------------------------------------------------------------------------------------------------
// Loader<LM, SK, CK, ROWS, NT>: stages one operand tile (ROWS rows x 128 bytes of compute type)
//   load()  global -> registers (issued early)       store() registers -> LDS (after the MFMAs)
//   at()    LDS byte offset of (row, chunk) for the fragment reads
// ------------------------------------------------------------------------------------------------
template <int LM, int SK, int CK, int ROWS, int NT> struct Loader;

// ---- k-dense, storage type == compute type: one 16-byte load per chunk ---------------------------
template <int CK, int ROWS, int NT> struct Loader<LM_K, SK_SAME, CK, ROWS, NT> {
    static constexpr int ES = Compute<CK>::ES, EPC = 16 / ES;
    static constexpr int UNITS = ROWS * CHUNKS / NT;
    static_assert(ROWS * CHUNKS % NT == 0, "tile/threads");
    static constexpr int LDS_BYTES = ROWS * ROW_PITCH;
    u32x4_t r[UNITS];
    static __device__ __forceinline__ int at(int row, int chunk) { return lds_rowmajor(row, chunk); }
    __device__ __forceinline__ void load(const Operand &op, int row0, int k0, int tid) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT, row = c >> 3, kc = c & 7;
            int grow = row0 + row;
            grow = grow < op.rows ? grow : op.rows - 1;
            const int k = k0 + kc * EPC;
            r[u] = zero4();
            if (k < op.K) r[u] = *reinterpret_cast<const u32x4_t *>(op.base + ((long)grow * op.row_stride + k) * ES);
        }
    }
    __device__ __forceinline__ void store(char *lds, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT;
            *reinterpret_cast<u32x4_t *>(lds + lds_rowmajor(c >> 3, c & 7)) = r[u];
        }
    }
};

// ---- k-dense f8e4m3 storage -> bf16 compute: one 8-byte load per chunk, widened at the LDS store --
template <int ROWS, int NT> struct Loader<LM_K, SK_F8, CK_BF16, ROWS, NT> {
    static constexpr int UNITS = ROWS * CHUNKS / NT;
    static_assert(ROWS * CHUNKS % NT == 0, "tile/threads");
    static constexpr int LDS_BYTES = ROWS * ROW_PITCH;
    u32x2_t r[UNITS];
    static __device__ __forceinline__ int at(int row, int chunk) { return lds_rowmajor(row, chunk); }
    __device__ __forceinline__ void load(const Operand &op, int row0, int k0, int tid) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT, row = c >> 3, kc = c & 7;
            int grow = row0 + row;
            grow = grow < op.rows ? grow : op.rows - 1;
            const int k = k0 + kc * 8;
            r[u] = u32x2_t{0u, 0u};
            if (k < op.K) r[u] = *reinterpret_cast<const u32x2_t *>(op.base + (long)grow * op.row_stride + k);
        }
    }
    __device__ __forceinline__ void store(char *lds, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT;
            u32x4_t w;
            w.x = f8pair_to_bf16pair(r[u].x, false);
            w.y = f8pair_to_bf16pair(r[u].x, true);
            w.z = f8pair_to_bf16pair(r[u].y, false);
            w.w = f8pair_to_bf16pair(r[u].y, true);
            *reinterpret_cast<u32x4_t *>(lds + lds_rowmajor(c >> 3, c & 7)) = w;
        }
    }
};

// ---- row-dense 16-bit storage: 8 loads of 8 rows (16 B) for 8 consecutive k, 8x8 transpose ---------
template <int CK, int ROWS, int NT> struct Loader<LM_MN, SK_SAME, CK, ROWS, NT> {
    static_assert(Compute<CK>::ES == 2, "specialised below for 1- and 4-byte types");
    typedef MnLayout<ROWS, 8> L;
    static constexpr int TOTAL = ROWS;  // (ROWS/8 row groups) x 8 chunks
    static constexpr int UNITS = (TOTAL + NT - 1) / NT;
    static constexpr int LDS_BYTES = CHUNKS * L::PLANE;
    u32x4_t r[UNITS][8];
    static __device__ __forceinline__ int at(int row, int chunk) { return L::at(row, chunk); }
    __device__ __forceinline__ void load(const Operand &op, int row0, int k0, int tid) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % (ROWS / 8), kc = id / (ROWS / 8);
            const int row = row0 + rg * 8;
            const bool row_ok = (TOTAL % NT == 0 || id < TOTAL) && row < op.rows;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int k = k0 + kc * 8 + j;
                r[u][j] = zero4();
                if (row_ok && k < op.K)
                    r[u][j] = *reinterpret_cast<const u32x4_t *>(op.base + ((long)k * op.k_stride + row) * 2);
            }
        }
    }
    __device__ __forceinline__ void store(char *lds, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int rg = id % (ROWS / 8), kc = id / (ROWS / 8);
#pragma unroll
            for (int rr = 0; rr < 8; rr++) {
                // rows 2q, 2q+1 live in dword q of every k-vector
                const uint32_t sel = (rr & 1) ? 0x07060302u : 0x05040100u;
                u32x4_t w;
                w.x = __builtin_amdgcn_perm(r[u][1][rr >> 1], r[u][0][rr >> 1], sel);
                w.y = __builtin_amdgcn_perm(r[u][3][rr >> 1], r[u][2][rr >> 1], sel);
                w.z = __builtin_amdgcn_perm(r[u][5][rr >> 1], r[u][4][rr >> 1], sel);
                w.w = __builtin_amdgcn_perm(r[u][7][rr >> 1], r[u][6][rr >> 1], sel);
                *reinterpret_cast<u32x4_t *>(lds + L::at(rg * 8 + rr, kc)) = w;
            }
        }
    }
};

// ---- row-dense f8e4m3 storage -> bf16: 8 loads of 8 rows (8 B), widen + transpose ------------------
template <int ROWS, int NT> struct Loader<LM_MN, SK_F8, CK_BF16, ROWS, NT> {
    typedef MnLayout<ROWS, 8> L;
    static constexpr int TOTAL = ROWS;
    static constexpr int UNITS = (TOTAL + NT - 1) / NT;
    static constexpr int LDS_BYTES = CHUNKS * L::PLANE;
    u32x2_t r[UNITS][8];
    static __device__ __forceinline__ int at(int row, int chunk) { return L::at(row, chunk); }
    __device__ __forceinline__ void load(const Operand &op, int row0, int k0, int tid) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % (ROWS / 8), kc = id / (ROWS / 8);
            const int row = row0 + rg * 8;
            const bool row_ok = (TOTAL % NT == 0 || id < TOTAL) && row < op.rows;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int k = k0 + kc * 8 + j;
                r[u][j] = u32x2_t{0u, 0u};
                if (row_ok && k < op.K)
                    r[u][j] = *reinterpret_cast<const u32x2_t *>(op.base + (long)k * op.k_stride + row);
            }
        }
    }
    __device__ __forceinline__ void store(char *lds, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int rg = id % (ROWS / 8), kc = id / (ROWS / 8);
            uint32_t w[8][4];
#pragma unroll
            for (int p = 0; p < 4; p++) {      // k pair (2p, 2p+1)
#pragma unroll
                for (int q = 0; q < 4; q++) {  // row pair (2q, 2q+1): byte pair q of the 8-byte vector
                    const uint32_t wa = q < 2 ? r[u][2 * p].x : r[u][2 * p].y;
                    const uint32_t wb = q < 2 ? r[u][2 * p + 1].x : r[u][2 * p + 1].y;
                    const f32x2_t fa = (q & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)wa, true)
                                               : __builtin_amdgcn_cvt_pk_f32_fp8((int)wa, false);
                    const f32x2_t fb = (q & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)wb, true)
                                               : __builtin_amdgcn_cvt_pk_f32_fp8((int)wb, false);
                    w[2 * q][p] = __builtin_amdgcn_perm(__float_as_uint(fb.x), __float_as_uint(fa.x), 0x07060302u);
                    w[2 * q + 1][p] = __builtin_amdgcn_perm(__float_as_uint(fb.y), __float_as_uint(fa.y), 0x07060302u);
                }
            }
#pragma unroll
            for (int rr = 0; rr < 8; rr++)
                *reinterpret_cast<u32x4_t *>(lds + L::at(rg * 8 + rr, kc)) = u32x4_t{w[rr][0], w[rr][1], w[rr][2], w[rr][3]};
        }
    }
};

// ---- row-dense 8-bit storage: 16 loads of 8 rows (8 B) for 16 consecutive k, byte transpose --------
template <int ROWS, int NT> struct Loader<LM_MN, SK_SAME, CK_I8, ROWS, NT> {
    typedef MnLayout<ROWS, 8> L;
    static constexpr int TOTAL = ROWS;
    static constexpr int UNITS = (TOTAL + NT - 1) / NT;
    static constexpr int LDS_BYTES = CHUNKS * L::PLANE;
    u32x2_t r[UNITS][16];
    static __device__ __forceinline__ int at(int row, int chunk) { return L::at(row, chunk); }
    __device__ __forceinline__ void load(const Operand &op, int row0, int k0, int tid) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % (ROWS / 8), kc = id / (ROWS / 8);
            const int row = row0 + rg * 8;
            const bool row_ok = (TOTAL % NT == 0 || id < TOTAL) && row < op.rows;
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const int k = k0 + kc * 16 + j;
                r[u][j] = u32x2_t{0u, 0u};
                if (row_ok && k < op.K)
                    r[u][j] = *reinterpret_cast<const u32x2_t *>(op.base + (long)k * op.k_stride + row);
            }
        }
    }
    __device__ __forceinline__ void store(char *lds, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int rg = id % (ROWS / 8), kc = id / (ROWS / 8);
            uint32_t w[8][4];
#pragma unroll
            for (int q = 0; q < 4; q++) {  // k quad (4q .. 4q+3) -> dword q of the output chunk
#pragma unroll
                for (int h = 0; h < 2; h++) {  // rows 4h .. 4h+3 live in dword h of every k-vector
                    const uint32_t v0 = h ? r[u][4 * q].y : r[u][4 * q].x;
                    const uint32_t v1 = h ? r[u][4 * q + 1].y : r[u][4 * q + 1].x;
                    const uint32_t v2 = h ? r[u][4 * q + 2].y : r[u][4 * q + 2].x;
                    const uint32_t v3 = h ? r[u][4 * q + 3].y : r[u][4 * q + 3].x;
                    // level 1: interleave bytes of (k, k+1): [k.r0, k1.r0, k.r1, k1.r1] and rows 2,3
                    const uint32_t a01 = __builtin_amdgcn_perm(v1, v0, 0x05010400u);
                    const uint32_t a23 = __builtin_amdgcn_perm(v1, v0, 0x07030602u);
                    const uint32_t b01 = __builtin_amdgcn_perm(v3, v2, 0x05010400u);
                    const uint32_t b23 = __builtin_amdgcn_perm(v3, v2, 0x07030602u);
                    // level 2: [k0,k1,k2,k3] of one row
                    w[4 * h + 0][q] = __builtin_amdgcn_perm(b01, a01, 0x05040100u);
                    w[4 * h + 1][q] = __builtin_amdgcn_perm(b01, a01, 0x07060302u);
                    w[4 * h + 2][q] = __builtin_amdgcn_perm(b23, a23, 0x05040100u);
                    w[4 * h + 3][q] = __builtin_amdgcn_perm(b23, a23, 0x07060302u);
                }
            }
#pragma unroll
            for (int rr = 0; rr < 8; rr++)
                *reinterpret_cast<u32x4_t *>(lds + L::at(rg * 8 + rr, kc)) = u32x4_t{w[rr][0], w[rr][1], w[rr][2], w[rr][3]};
        }
    }
};

// ---- row-dense f32 storage: 4 loads of 4 rows (16 B) for 4 consecutive k, transpose by renaming ---
template <int ROWS, int NT> struct Loader<LM_MN, SK_SAME, CK_F32, ROWS, NT> {
    typedef MnLayout<ROWS, 4> L;
    static constexpr int TOTAL = (ROWS / 4) * CHUNKS;
    static constexpr int UNITS = (TOTAL + NT - 1) / NT;
    static constexpr int LDS_BYTES = CHUNKS * L::PLANE;
    u32x4_t r[UNITS][4];
    static __device__ __forceinline__ int at(int row, int chunk) { return L::at(row, chunk); }
    __device__ __forceinline__ void load(const Operand &op, int row0, int k0, int tid) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            const int rg = id % (ROWS / 4), kc = id / (ROWS / 4);
            const int row = row0 + rg * 4;
            const bool row_ok = (TOTAL % NT == 0 || id < TOTAL) && row < op.rows;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int k = k0 + kc * 4 + j;
                r[u][j] = zero4();
                if (row_ok && k < op.K)
                    r[u][j] = *reinterpret_cast<const u32x4_t *>(op.base + ((long)k * op.k_stride + row) * 4);
            }
        }
    }
    __device__ __forceinline__ void store(char *lds, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int id = tid + u * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int rg = id % (ROWS / 4), kc = id / (ROWS / 4);
#pragma unroll
            for (int rr = 0; rr < 4; rr++)
                *reinterpret_cast<u32x4_t *>(lds + L::at(rg * 4 + rr, kc)) =
                    u32x4_t{r[u][0][rr], r[u][1][rr], r[u][2][rr], r[u][3][rr]};
        }
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

template <int SK, int CK, int ROWS, int NT> struct Loader<LM_SCALAR, SK, CK, ROWS, NT> {
    static constexpr int ES = Compute<CK>::ES, EPC = 16 / ES;
    static constexpr int UNITS = ROWS * CHUNKS / NT;
    static constexpr int LDS_BYTES = ROWS * ROW_PITCH;
    u32x4_t r[UNITS];
    static __device__ __forceinline__ int at(int row, int chunk) { return lds_rowmajor(row, chunk); }
    __device__ __forceinline__ void load(const Operand &op, int row0, int k0, int tid) {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT, row = c >> 3, kc = c & 7;
            const int grow = row0 + row;
            uint32_t w[4] = {0u, 0u, 0u, 0u};
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
    __device__ __forceinline__ void store(char *lds, int tid) const {
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int c = tid + u * NT;
            *reinterpret_cast<u32x4_t *>(lds + lds_rowmajor(c >> 3, c & 7)) = r[u];
        }
    }
};

// ------------------------------------------------------------------------------------------------
// output conversion
// ------------------------------------------------------------------------------------------------
template <int OUT> struct Out;
template <> struct Out<OUT_BF16> {
    typedef uint16_t T;
    static __device__ __forceinline__ T cvt(float v) { return f32_to_bf16_bits_rne(v); }
};
template <> struct Out<OUT_F16> {
    typedef uint16_t T;
    static __device__ __forceinline__ T cvt(float v) { return f32_to_f16_bits_rne(v); }
};
template <> struct Out<OUT_F32> {
    typedef float T;
    static __device__ __forceinline__ T cvt(float v) { return v; }
};
template <> struct Out<OUT_I32> {
    typedef int32_t T;
    static __device__ __forceinline__ T cvt(int v) { return v; }
};

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
    static constexpr int TM = BM / WM / 16, TN = BN / WN / 16;  // 16x16 MFMA tiles per wave
    static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "wave tiling");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
};

// maps the linear workgroup id to (batch, tile_m, tile_n): ids that land on one XCD (id % 8) get
// neighbouring tiles, and tiles are walked in groups of 8 tile-rows so that the A and B panels a
// group shares stay in that XCD's L2
__device__ __forceinline__ void tile_of(long pid, long total, int tiles_m, int tiles_n, long &batch, int &tm, int &tn) {
    if (total % 8 == 0) pid = (pid % 8) * (total / 8) + pid / 8;
    const long per_batch = (long)tiles_m * tiles_n;
    batch = pid / per_batch;
    const int t = (int)(pid % per_batch);
    constexpr int GROUP = 8;
    const int width = GROUP * tiles_n;
    const int first_m = (t / width) * GROUP;
    const int gsize = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    tm = first_m + (t % width) % gsize;
    tn = (t % width) / gsize;
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_product_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                               typename Out<Cfg::OUT>::T *__restrict__ C,
                                                               DevProduct g, int tiles_m, int tiles_n) {
    extern __shared__ __align__(16) char smem[];
    typedef Compute<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Cfg::LoaderA LoaderA;
    typedef typename Cfg::LoaderB LoaderB;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, BK = Cfg::BK;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int lr = lane & 15, lg = lane >> 4;

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
        for (int j = 0; j < TN; j++) acc[i][j] = acc_t{0, 0, 0, 0};

    LoaderA la;
    LoaderB lb;
    const int KT = (g.K + BK - 1) / BK;
    if (KT > 0) {
        la.load(opA, m0, 0, tid);
        lb.load(opB, n0, 0, tid);
        la.store(smem, tid);
        lb.store(smem + Cfg::A_BYTES, tid);
    }
    __syncthreads();

    const int a_row = wave_m * TM * 16 + lr, b_row = wave_n * TN * 16 + lr;
    for (int kt = 0; kt < KT; kt++) {
        char *cur = smem + (kt & 1) * Cfg::STAGE_BYTES;
        char *nxt = smem + ((kt + 1) & 1) * Cfg::STAGE_BYTES;
        const bool more = kt + 1 < KT;
        if (more) {  // in flight while the matrix cores work on the current stage
            la.load(opA, m0, (kt + 1) * BK, tid);
            lb.load(opB, n0, (kt + 1) * BK, tid);
        }
        const char *As = cur, *Bs = cur + Cfg::A_BYTES;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            u32x4_t af[TM];
#pragma unroll
            for (int i = 0; i < TM; i++)
                af[i] = *reinterpret_cast<const u32x4_t *>(As + LoaderA::at(a_row + i * 16, s * 4 + lg));
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const u32x4_t bf = *reinterpret_cast<const u32x4_t *>(Bs + LoaderB::at(b_row + j * 16, s * 4 + lg));
                // operands swapped: the accumulator then holds, per lane, 4 consecutive n of one m
#pragma unroll
                for (int i = 0; i < TM; i++) Cmp::mma(bf, af[i], acc[i][j]);
            }
        }
        if (more) {
            la.store(nxt, tid);
            lb.store(nxt + Cfg::A_BYTES, tid);
        }
        __syncthreads();
    }

    out_t *Cb = C + batch * (long)g.M * g.N;
    const bool vec_ok = (g.N & 3) == 0;
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + wave_m * TM * 16 + i * 16 + lr;
        if (m >= g.M) continue;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + wave_n * TN * 16 + j * 16 + lg * 4;
            out_t v[4];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = Out<Cfg::OUT>::cvt(acc[i][j][e]);
            out_t *dst = Cb + (long)m * g.N + n;
            if (vec_ok && n + 3 < g.N) {
                struct alignas(sizeof(out_t) * 4) Quad { out_t q[4]; };
                *reinterpret_cast<Quad *>(dst) = Quad{{v[0], v[1], v[2], v[3]}};
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < g.N) dst[e] = v[e];
            }
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
    return LM_SCALAR;
}

template <class Cfg> int launch_config(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    static bool configured = false;  // benign race: the attribute call is idempotent
    auto kernel = mfma_product_kernel<Cfg>;
    if (!configured) {
        HODU_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     Cfg::LDS_BYTES));
        configured = true;
    }
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream, (const char *)a,
                       (const char *)b, (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

// One compute kind = 13 kernels: {KK, KM, MK, MM} x {256x256, 128x128, 64x64} tiles plus a scalar-load
// 64x64 kernel.  The tile is the largest that still yields at least one workgroup per compute unit.
template <int CK, int SKA, int SKB, int OUT>
int launch_kind(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g, const char *const names[13]) {
    constexpr int ES = Compute<CK>::ES, EPC = 16 / ES;
    constexpr int SA = SKA == SK_F8 ? 1 : ES, SB = SKB == SK_F8 ? 1 : ES;
    constexpr int ROWVEC = ES == 4 ? 4 : 8;
    const int la = pick_mode(a, g.a_off, g.a_m, g.a_k, g.M, g.K, SA, EPC, ROWVEC, g, g.a_bs);
    const int lb = pick_mode(b, g.b_off, g.b_n, g.b_k, g.N, g.K, SB, EPC, ROWVEC, g, g.b_bs);
    if (la == LM_SCALAR || lb == LM_SCALAR) {
        ctx->last_kernel = names[12];
        return launch_config<Config<CK, SKA, SKB, OUT, 64, 64, 2, 2, LM_SCALAR, LM_SCALAR>>(ctx, a, b, c, g);
    }
    const long cus = ctx->props.multiProcessorCount;
    auto tiles = [&](long bm, long bn) { return g.batches * ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn); };
    const int size = ctx->force_tile >= 0 ? ctx->force_tile : tiles(256, 256) >= cus ? 0 : tiles(128, 128) >= cus ? 1 : 2;
    const int combo = (la == LM_MN ? 2 : 0) + (lb == LM_MN ? 1 : 0);
    ctx->last_kernel = names[size * 4 + combo];
#define HODU_MFMA_CASE(SZ, CB, BM, BN, LA, LB)                                                             \
    if (size == SZ && combo == CB) return launch_config<Config<CK, SKA, SKB, OUT, BM, BN, 2, 2, LA, LB>>(ctx, a, b, c, g);
    HODU_MFMA_CASE(0, 0, 256, 256, LM_K, LM_K)
    HODU_MFMA_CASE(0, 1, 256, 256, LM_K, LM_MN)
    HODU_MFMA_CASE(0, 2, 256, 256, LM_MN, LM_K)
    HODU_MFMA_CASE(0, 3, 256, 256, LM_MN, LM_MN)
    HODU_MFMA_CASE(1, 0, 128, 128, LM_K, LM_K)
    HODU_MFMA_CASE(1, 1, 128, 128, LM_K, LM_MN)
    HODU_MFMA_CASE(1, 2, 128, 128, LM_MN, LM_K)
    HODU_MFMA_CASE(1, 3, 128, 128, LM_MN, LM_MN)
    HODU_MFMA_CASE(2, 0, 64, 64, LM_K, LM_K)
    HODU_MFMA_CASE(2, 1, 64, 64, LM_K, LM_MN)
    HODU_MFMA_CASE(2, 2, 64, 64, LM_MN, LM_K)
    HODU_MFMA_CASE(2, 3, 64, 64, LM_MN, LM_MN)
#undef HODU_MFMA_CASE
    return fail(HODU_ROCM_UNSUPPORTED, "no MFMA variant");
}

#define HODU_MFMA_NAMES(P)                                                                                 \
    {P "_256x256_KK", P "_256x256_KM", P "_256x256_MK", P "_256x256_MM", P "_128x128_KK", P "_128x128_KM", \
     P "_128x128_MK", P "_128x128_MM", P "_64x64_KK",   P "_64x64_KM",   P "_64x64_MK",   P "_64x64_MM",   \
     P "_64x64_scalar"}

}  // namespace mfma
}  // namespace hodu
