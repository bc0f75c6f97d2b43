// Software-pipelined MFMA tile kernel for products whose operands are vector-loadable (k-dense, or
// row-dense for the 8- and 16-bit types) and whose K is a multiple of 128 bytes.  Same MFMA
// instructions and the same results as the general kernel in gemm_mfma.hpp; what differs is how
// the K loop is fed and how the tile leaves:
//
//   * K advances 128 bytes per stage (64 bf16 / 128 i8 / 32 f32 = four MFMA k-slices).  Every DMA
//     request is one whole 128-byte cache line of one row: fetching rows in 64-byte halves feeds a
//     compute unit at 29 B/clk, whole lines at 47 B/clk (measured on the 4096 x 4096 x 14336 sweep);
//   * a ring of NST (2..4) stages of LDS, written by LDS-DMA only (global_load_lds_dwordx4: no staging
//     registers, no ds_write).  Behind the barrier of stage t the DMA of stage t + NST is issued into
//     the buffer stage t just vacated, spread between the MFMAs of the following two k-slices;
//   * a k-dense stage is rows of 128 bytes back to back; one wavefront-wide DMA instruction writes
//     8 rows.  The eight 16-byte chunks of a row are XOR-swizzled by (row >> 1) & 7 -- applied to the
//     SOURCE address of the DMA -- so that an MFMA fragment read (16 lanes = 16 rows, one chunk)
//     touches all 64 banks once without any padding;
//   * the MFMA fragments live in one register set that is refilled one k-slice ahead of its use, each
//     LDS read placed between the MFMAs of the previous slice in a pinned order, so that LDS and the
//     matrix cores run side by side instead of in alternating bursts;
//   * one bare s_barrier per stage, preceded by s_waitcnt vmcnt(n) lgkmcnt(0) with n = what the NST - 2
//     youngest stages' DMA amounts to (loads return in issue order): stage t+1 has landed, every
//     fragment read of stage t has returned, younger stages stay in flight;
//   * the epilogue stages each 32-row band of a wavefront's accumulators in LDS and stores whole rows.
//
// Row-dense operands (stride 1 along m or n: a [K, N] row-major right operand, a transposed left
// operand) take the same path.  A stage of such an operand is the stage's k-rows of the tile's ROWS
// contiguous elements, DMA'd as whole rows into a plain [k][ROWS] array whose 16-byte chunks are
// XOR-swizzled by (k % 4) << 2 (16-bit) or k % 8 (8-bit).  The MFMA fragment -- 16 bytes of
// consecutive k of ONE row per lane -- comes out of that k-major array through two LDS transpose
// reads (ds_read_b64_tr_b16 / _tr_b8: each hands a lane 4 or 8 consecutive k of its own column from
// the k-rows that 16 lanes read together), so no register-level transpose and no second LDS layout
// is needed.
//
// f8e4m3 right operands (the fused to_dtype of a weight) are DMA'd as the bytes they are and widened
// to bf16 between the fragment read and the MFMA (v_cvt_scalef32_pk_bf16_fp8, exact): no widened
// copy ever exists in LDS or HBM.  k-dense f8 rows still move as whole 128-byte lines, which is 128 k
// = two stages of the bf16 left operand, so the right operand's buffers each hold a PAIR of stages
// and are refilled one half per stage; row-dense f8 ([K, N] bytes) moves 64 k-rows per stage.
//
// Hazards.  The barrier in stage t is reached by a wavefront only after all its reads of stage t
// have RETURNED (lgkmcnt(0)) and its own share of stage t+1 has landed (vmcnt); past it, stage t's
// buffer is dead for everybody and stage t+1 is complete for everybody.  Past the end of K every
// stage still issues a full (re-fetching) list so that the in-flight count stays a constant; those
// land in buffers nobody reads, and the workgroup waits for them before it touches LDS again or ends.
#pragma once

#include <type_traits>

#include "agent_scope.hpp"
#include "gemm_mfma.hpp"
#include "gfx950_insn.hpp"

// Measurement builds only (never the library's): HODU_PIPE_STAMPS makes every workgroup record the 100 MHz
// real-time counter at a few points into the buffer whose address the third fused-step slot carries.
#ifdef HODU_PIPE_STAMPS
#define HODU_STAMP(i)                                                                                              \
    do {                                                                                                           \
        if (threadIdx.x == 0)                                                                                      \
            ((unsigned long long *)g.epi.step[2].vec)[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 8 + (i)] =   \
                __builtin_amdgcn_s_memrealtime();                                                                  \
    } while (0)
#else
#define HODU_STAMP(i) do { } while (0)
#endif

namespace hodu {
namespace mfma {

constexpr int P_ROW_BYTES = 128;   // == ROW_BYTES of the swizzled layout
constexpr int P_SLICES = 4;        // 32-byte k-slices (of the compute type) per stage

// s_waitcnt immediate for gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
constexpr int waitcnt_vm(int n) { return (n & 15) | 0x70 | 0xF00 | ((n >> 4) << 14); }
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | 0x70 | ((n >> 4) << 14); }

// Row-dense operand geometry for elements of SB bytes in memory feeding a compute type of ES bytes
// (SB == ES, or SB == 1 under ES == 2 for f8e4m3 storage); a "chunk" is 16 bytes of one k-row.
//   swizzle   chunk c of k-row k sits at slot c ^ swz(k); one transpose read takes its 16 lanes through
//             RPT consecutive k-rows, 32 (SB = 2) or 16 (SB = 1) bytes of each, and the swizzle puts those
//             rows into different banks
template <int SB, int ES> struct RowDenseGeom {
    static constexpr int RPT = SB == 2 ? 4 : 8;           // k-rows one transpose read covers
    static constexpr int EPC = 16 / SB;                    // elements per chunk
    static constexpr int STAGE_K = 128 / ES;               // k-rows per stage
    static constexpr int SLICE_K = 32 / ES;                // k per MFMA slice
    static constexpr int READS = (SLICE_K / 2) / RPT;      // transpose reads per fragment (8 or 16 k per lane)
    static __device__ __forceinline__ int swz(int k) { return SB == 2 ? (k & 3) << 2 : (k & 7); }
};

// k-dense LDS layout of the pipelined kernels: rows of 128 bytes back to back (no padding: it buys a deeper
// stage ring), 16-byte chunk c of row r at slot c ^ ((r >> 1) & 7).  The 16 rows one ds_read_b128 phase touches
// then spread over all 64 banks: bank group (of 16) = (r & 1) * 8 + (c ^ ((r >> 1) & 7)).
__device__ __forceinline__ int kd_slot(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

template <int CK_, int OUT_, int BM_, int BN_, int WM_, int WN_, int LA_ = LM_K, int LB_ = LM_K, int SKB_ = SK_SAME,
          int NST_ = 2>
struct PipeConfig {
    static constexpr int CK = CK_, OUT = OUT_, BM = BM_, BN = BN_, WM = WM_, WN = WN_, LA = LA_, LB = LB_, SKB = SKB_;
    static constexpr int NST = NST_;                       // stages of the LDS ring
    static constexpr int NT = WM * WN * 64, NW = WM * WN;
    static constexpr int ES = Compute<CK>::ES;
    static constexpr bool B_F8 = SKB == SK_F8;
    static constexpr int SB = B_F8 ? 1 : ES;               // bytes of a right-operand element in memory
    static constexpr bool B_PAIR = B_F8 && LB == LM_K;     // right-operand buffers hold two stages each
    static constexpr int BK = P_ROW_BYTES / ES;
    // k-dense: rows of 128 bytes; row-dense: [k-rows of a stage][ROWS]; both without gaps
    static constexpr int A_BYTES = BM * P_ROW_BYTES;
    static constexpr int B_BYTES = LB == LM_K ? BN * P_ROW_BYTES : (BK * BN * SB);
    static constexpr int LDS_BYTES = NST * (A_BYTES + B_BYTES);
    static constexpr int PA = (BM / 8) / NW;                                    // DMA instructions per wavefront: a stage of A,
    static constexpr int PB = (LB == LM_K ? BN / 8 : BK * BN * SB / 1024) / NW;  // a buffer of B,
    static constexpr int PBS = B_PAIR ? PB / 2 : PB;                            // what of B goes out per stage
    static constexpr int P = PA + PBS;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;  // 32x32 MFMA tiles per wave
    static_assert(NST >= 2 && NST <= 4, "ring depth");
    static_assert(!B_F8 || CK == CK_BF16, "f8e4m3 storage widens to bf16");
    static_assert((BM / 8) % NW == 0 && PB >= 1 && (!B_PAIR || PB % 2 == 0), "DMA split");
    static_assert((NST - 1) * (PA + PB) < 64, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
    static_assert(NW * 32 * (TN * 128 + 16) <= LDS_BYTES, "the epilogue stages a 32-row band per wavefront in LDS");
    static_assert((LA == LM_K || (ES <= 2 && BM >= 128)) && (LB == LM_K || (ES <= 2 && BN >= 128)),
                  "row-dense operands: 8- and 16-bit types, tiles of at least 128 rows");
};

// A pointer the compiler can hold in scalar registers (the base of dma16_sbase / dma16_imm): both halves through
// readfirstlane, which is free for a value that already is uniform and makes the "s" constraints of those
// instructions hold where the uniformity analysis gives up.
__device__ __forceinline__ const char *uniform_ptr(const char *p) {
    const unsigned long long v = (unsigned long long)(uintptr_t)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const char *)(uintptr_t)(((unsigned long long)hi << 32) | lo);
}

// 64 bits per lane through the LDS transpose.  Of the 16 lanes that execute together, lane s supplies the
// address of 8 consecutive bytes.
//   16-bit elements: lane i receives element (i % 4) of lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4 -- with lanes
//     4e..4e+3 pointing at 16 consecutive columns of k-row e, lane i gets column i of k-rows 0..3;
//   8-bit elements: lane i receives element (i % 8) of lanes i/8, 2 + i/8, .., 14 + i/8 -- with lanes 2e, 2e+1
//     pointing at 16 consecutive columns of k-row e, lane i gets column i of k-rows 0..7.
template <int SB> __device__ __forceinline__ u32x2_t lds_get_tr(const char *lds, int off) {
    if constexpr (SB == 2) {
        typedef short s16x4_t __attribute__((ext_vector_type(4)));
        typedef s16x4_t __attribute__((address_space(3))) * lds_ptr_t;
        return bitcast<u32x2_t>(__builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)(lds + off)));
    } else {
        typedef int i32x2_t __attribute__((ext_vector_type(2)));
        typedef i32x2_t __attribute__((address_space(3))) * lds_ptr_t;
        return bitcast<u32x2_t>(__builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr_t)(uintptr_t)(lds + off)));
    }
}
__device__ __forceinline__ u32x2_t lds_get64(const char *lds, int off) { return *reinterpret_cast<const u32x2_t *>(lds + off); }

// 8 f8e4m3 -> 8 bf16 (exact), two per instruction (v_cvt_scalef32_pk_bf16_fp8 with a unit scale)
__device__ __forceinline__ u32x4_t widen_f8x8(const u32x2_t &v) {
    return u32x4_t{bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.x, 1.0f, false)),
                   bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.x, 1.0f, true)),
                   bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.y, 1.0f, false)),
                   bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(v.y, 1.0f, true))};
}

// Epilogue for one band of a wavefront's tile (TN accumulator tiles side by side; 32 rows, or 16 with TS = 16): the values go through a
// wavefront-private patch of LDS so that they leave as whole rows -- 16 contiguous bytes per lane, a row of the
// band per 2..16 lanes -- instead of the accumulator layout's 8-byte pieces of 32 different rows per instruction
// (measured: 13 us of a 37 us launch spent storing a 256 x 256 bf16 tile that way).
//   acc layout (operands swapped): lane (lr, lh) holds row lr, columns 32*j + 8*q + 4*lh + e of the band.
// EPI: the values are final outputs and take the fused element-wise steps (partial sums of a K range do not).
// TS = 16: bands of 16 rows out of 16 x 16 accumulators, where lane (r = lane % 16, g = lane / 16) holds row r,
// columns 16*j + 4*g + e.
// What the fused steps need for the columns a lane stores in a band of TN tiles of TS columns (the same columns in
// every pass of every band of a wavefront's tile): fetched once per tile by the caller and handed to every band --
// fetched per band, a bias vector's entries cost a trip to memory eight times per tile (config 5 up with bias and
// ReLU: 46 us more than the plain product; once per tile: 28; with four passes' pieces taking each step together,
// one branch on the step's kind per group instead of per piece: 26).
template <int OUT, int TN, int TS>
__device__ __forceinline__ EpiPrepared<Out<OUT>::DT, 16 / (int)sizeof(typename Out<OUT>::T)> band_columns_prepare(const DevEpilogue &epi, int n_base,
                                                                                                                  int lane, int N) {
    constexpr int OS = sizeof(typename Out<OUT>::T), EPV = 16 / OS, CPR = TN * TS * OS / 16;
    const int n = n_base + (lane % CPR) * EPV;
    return epilogue_prepare<Out<OUT>::DT, EPV>(epi, n < N ? n : N - 1, N);
}

// an output type that narrows four accumulators into one dword at once (Out<OUT>::cvt4; the 8-bit floats)
template <class O, class = void> struct OutHasCvt4 : std::false_type {};
template <class O> struct OutHasCvt4<O, std::void_t<decltype(&O::cvt4)>> : std::true_type {};

template <int OUT, int TN, bool EPI, class acc_t, int TS = 32, bool READY = false>
__device__ __forceinline__ void store_band_via_lds(char *patch, typename Out<OUT>::T *Cb, const acc_t (&acc)[TN], int m_base,
                                                   int n_base, int lane, int M, int N, const DevEpilogue &epi,
                                                   const EpiPrepared<Out<OUT>::DT, 16 / (int)sizeof(typename Out<OUT>::T)> &ready) {
    typedef typename Out<OUT>::T out_t;
    constexpr int OS = sizeof(out_t), ROWB = TN * TS * OS, PITCH = ROWB + 16, EPV = 16 / OS;
    constexpr int CPR = ROWB / 16, RPP = 64 / CPR;  // 16-byte chunks per row, rows per pass of the wavefront
    static_assert((TS == 32 || TS == 16) && CPR <= 64 && TS % RPP == 0, "band geometry");
    struct alignas(OS * 4) Quad { out_t v[4]; };
    if constexpr (TS == 32) {
        const int lr = lane & 31, lh = lane >> 5;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                Quad w;
                if constexpr (OutHasCvt4<Out<OUT>>::value) {
                    const uint32_t bits = Out<OUT>::cvt4(acc[j][4 * q], acc[j][4 * q + 1], acc[j][4 * q + 2], acc[j][4 * q + 3]);
                    __builtin_memcpy(&w, &bits, 4);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) w.v[e] = Out<OUT>::cvt(acc[j][4 * q + e]);
                }
                *reinterpret_cast<Quad *>(patch + lr * PITCH + (j * 32 + 8 * q + 4 * lh) * OS) = w;
            }
    } else {
        const int r16 = lane & 15, g4 = lane >> 4;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            Quad w;
            if constexpr (OutHasCvt4<Out<OUT>>::value) {
                const uint32_t bits = Out<OUT>::cvt4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
                __builtin_memcpy(&w, &bits, 4);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) w.v[e] = Out<OUT>::cvt(acc[j][e]);
            }
            *reinterpret_cast<Quad *>(patch + r16 * PITCH + (j * 16 + 4 * g4) * OS) = w;
        }
    }
    // the same wavefront reads what it wrote: the LDS operations of one wavefront complete in order, and the
    // compiler is told not to move the differently-typed accesses across each other
    wave_lds_fence();
    const bool vec_ok = ((long)N * OS) % 16 == 0;
    // the fused element-wise steps work on the rounded values, here where a lane holds EPV neighbouring columns
    // of one row -- the same columns in every pass, so what the steps need for them is fetched once
    EpiPrepared<Out<OUT>::DT, EPV> prepared;
    if (EPI && epi.n != 0) {
        if constexpr (READY) {
            prepared = ready;
        } else {
            const int n = n_base + (lane % CPR) * EPV;
            prepared = epilogue_prepare<Out<OUT>::DT, EPV>(epi, n < N ? n : N - 1, N);
        }
    }
    auto patch_chunk = [&](int pass) {
        const int row = pass * RPP + lane / CPR, chunk = lane % CPR;
        return *reinterpret_cast<const u32x4_t *>(patch + row * PITCH + chunk * 16);
    };
    auto store_chunk = [&](int pass, u32x4_t v) {
        const int row = pass * RPP + lane / CPR, chunk = lane % CPR;
        const int m = m_base + row, n = n_base + chunk * EPV;
        if (m >= M || n >= N) return;
        out_t *dst = Cb + (long)m * N + n;
        if (vec_ok && n + EPV <= N) {
            *reinterpret_cast<u32x4_t *>(dst) = v;
        } else if (n + EPV <= N) {  // an odd row length: the same store at element alignment
            stg_elem_aligned<16, OS>(dst, &v);
        } else {
            const out_t *e = reinterpret_cast<const out_t *>(&v);
#pragma unroll
            for (int k = 0; k < EPV; k++)
                if (n + k < N) dst[k] = e[k];
        }
    };
    if (EPI && epi.n != 0) {
        // f16 stays rolled (nothing here indexes registers by `pass`): its narrowing routine is some fifty
        // instructions per element, inlined once per band this way instead of once per pass
        if constexpr (Out<OUT>::DT == HODU_F16) {
#pragma unroll 1
            for (int pass = 0; pass < TS / RPP; pass++) {
                u32x4_t v = patch_chunk(pass);
                epilogue_apply_prepared<Out<OUT>::DT, EPV>(prepared, reinterpret_cast<out_t *>(&v));
                store_chunk(pass, v);
            }
        } else {
            // up to four passes' pieces at a time: their steps are applied together
            constexpr int NP = TS / RPP, GRP = NP < 4 ? NP : 4;
            static_assert(NP % GRP == 0, "whole groups of passes");
#pragma unroll
            for (int p0 = 0; p0 < NP; p0 += GRP) {
                out_t e[GRP][EPV];
#pragma unroll
                for (int q = 0; q < GRP; q++) {
                    const u32x4_t v = patch_chunk(p0 + q);
                    __builtin_memcpy(e[q], &v, 16);
                }
                epilogue_apply_prepared_group<Out<OUT>::DT, EPV, GRP>(prepared, e);
#pragma unroll
                for (int q = 0; q < GRP; q++) {
                    u32x4_t v;
                    __builtin_memcpy(&v, e[q], 16);
                    store_chunk(p0 + q, v);
                }
            }
        }
    } else {
#pragma unroll
        for (int pass = 0; pass < TS / RPP; pass++) store_chunk(pass, patch_chunk(pass));
    }
    wave_lds_fence();  // the next band overwrites the patch
}
template <int OUT, int TN, bool EPI, class acc_t, int TS = 32>
__device__ __forceinline__ void store_band_via_lds(char *patch, typename Out<OUT>::T *Cb, const acc_t (&acc)[TN], int m_base,
                                                   int n_base, int lane, int M, int N, const DevEpilogue &epi) {
    const EpiPrepared<Out<OUT>::DT, 16 / (int)sizeof(typename Out<OUT>::T)> none{};
    store_band_via_lds<OUT, TN, EPI, acc_t, TS, false>(patch, Cb, acc, m_base, n_base, lane, M, N, epi, none);
}

// A product cut along K (grid.y ranges): every workgroup of a tile writes its accumulators, unrounded, to its own
// slab of the workspace -- in the accumulator layout, 16 bytes per lane and instruction, so a slab is written and
// read in whole 1 KB pieces -- and counts itself in on the tile's arrival counter; the one that arrives last adds all
// slabs in range order (its own included, from memory: the order, and therefore the rounding, does not depend on who
// was last) and goes on to store the tile.  One launch instead of two, and the other workgroups' compute units are
// free as soon as their slab is out.  Returns true in the workgroup that now holds the tile's sums.
template <int NW, int TM, int TN, class acc_t>
__device__ __forceinline__ bool splitk_exchange(acc_t (&acc)[TM][TN], void *partials, int *arrival, int *flag, int tid) {
    typedef decltype(acc_t{}[0]) elem_ref_t;
    typedef std::remove_cv_t<std::remove_reference_t<elem_ref_t>> elem_t;
    typedef elem_t quad_t __attribute__((ext_vector_type(4)));
    constexpr unsigned WAVE_BYTES = TM * TN * 4 * 1024, SLAB = NW * WAVE_BYTES;
    const int lane = tid & 63, wave = tid >> 6;
    const unsigned mine = wave * WAVE_BYTES + lane * 16;
    char *slab0 = (char *)partials + (size_t)blockIdx.x * SLAB;
    const size_t range_pitch = (size_t)gridDim.x * SLAB;
    {
        const __amdgpu_buffer_rsrc_t out = agent_buffer(slab0 + blockIdx.y * range_pitch, SLAB);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int q = 0; q < 4; q++)
                    store16_agent(out, mine + ((i * TN + j) * 4 + q) * 1024,
                                  quad_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]});
    }
    if (!arrive_and_check_last(&arrival[blockIdx.x], (int)gridDim.y, flag, tid)) return false;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;
    // The slabs come from memory (a round trip of a microsecond or more) and are added in range order; what hides the
    // latency is the number of loads in flight: a whole slab's share of this wavefront at a time where the registers
    // allow it (TM * TN * 4 loads of 16 bytes per lane), half of it otherwise.
    constexpr int PER = TM * TN * 4, CHUNK = PER <= 32 ? PER : PER / 2;
    for (unsigned r = 0; r < gridDim.y; r++) {
        const __amdgpu_buffer_rsrc_t in = agent_buffer(slab0 + r * range_pitch, SLAB);
#pragma unroll
        for (int c0 = 0; c0 < PER; c0 += CHUNK) {
            quad_t v[CHUNK];
#pragma unroll
            for (int c = 0; c < CHUNK; c++) v[c] = load16_agent<quad_t>(in, mine + (c0 + c) * 1024);
#pragma unroll
            for (int c = 0; c < CHUNK; c++) {
                const int t = (c0 + c) / 4, q = (c0 + c) % 4;
#pragma unroll
                for (int e = 0; e < 4; e++) acc[t / TN][t % TN][4 * q + e] += v[c][e];
            }
        }
    }
    arrival_reset(&arrival[blockIdx.x], tid);
    return true;
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                            typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                            int tiles_m, int tiles_n, int stages_per_split,
                                                            void *__restrict__ partials, int *__restrict__ arrival) {
    HODU_DYNAMIC_LDS(smem);
    typedef Compute32<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, ES = Cfg::ES, SB = Cfg::SB, PA = Cfg::PA, PB = Cfg::PB, PBS = Cfg::PBS,
                  P = Cfg::P;
    constexpr bool B_F8 = Cfg::B_F8, B_PAIR = Cfg::B_PAIR;
    typedef RowDenseGeom<ES, ES> GA;
    typedef RowDenseGeom<SB, ES> GB;

    HODU_STAMP(0);
    const int tid = threadIdx.x, lane = tid & 63;
    // the wavefront's index as a scalar: what a DMA instruction needs besides the lane's offset inside the tile --
    // the operand's base address, the LDS destination in M0 -- is then wave-uniform and stays in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int lr = lane & 31, lh = lane >> 5;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

    // LDS: NST stages of A, then NST buffers of B
    constexpr int NST = Cfg::NST;
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    constexpr int B_BASE = NST * Cfg::A_BYTES;

    // ---- DMA plan of this wavefront: PA + PB instructions, each one 1 KB of LDS ----
    // k-dense operand: 8 rows x 128 B; lane -> (row, slot), the slot holds chunk slot ^ ((row >> 1) & 7).
    // row-dense operand: KPI consecutive k-rows of ROWS elements; lane -> (k-row, slot), the slot holds chunk
    // slot ^ swz(k); a chunk that starts past the operand's last row is fetched from the last whole chunk
    // instead (its columns are never stored).
    // An address is the scalar base of the tile (its first row, or its first column of k-row 0; advanced by a
    // stage's worth per stage) plus the lane's 32-bit byte offset inside the tile, fixed for the whole launch: an
    // instruction then costs one M0 write and the load itself, no vector arithmetic.  pipe_offsets_fit() on the
    // host guarantees that the offsets stay below 4 GB.
    unsigned offa[PA], offb[PB];      // byte offset of this lane inside the tile, stage (buffer) 0
    unsigned lda[PA], ldb[PB];        // block offset inside a buffer (wave-uniform)
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = p * Cfg::NW + wave;
        if constexpr (Cfg::LA == LM_K) {
            const int trow = q * 8 + (lane >> 3), dchunk = kd_slot(trow, lane & 7);
            int row = m0 + trow;
            row = row < g.M ? row : g.M - 1;
            offa[p] = (unsigned)((long)(row - m0) * g.a_m * ES) + dchunk * 16;
        } else {
            constexpr int CPR = Cfg::BM / GA::EPC, KPI = 64 / CPR;  // chunks per k-row, k-rows per instruction
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ GA::swz(k);
            int col = m0 + c * GA::EPC;
            col = col <= g.M - GA::EPC ? col : g.M - GA::EPC;
            // (the clamped column may lie left of the tile's first one: the offset is taken from the clamped base)
            offa[p] = (unsigned)(((long)k * g.a_k + (col - (m0 <= g.M - GA::EPC ? m0 : g.M - GA::EPC))) * ES);
        }
        lda[p] = q * 1024;
    }
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int q = p * Cfg::NW + wave;
        if constexpr (Cfg::LB == LM_K) {
            const int trow = q * 8 + (lane >> 3), dchunk = kd_slot(trow, lane & 7);
            int row = n0 + trow;
            row = row < g.N ? row : g.N - 1;
            offb[p] = (unsigned)((long)(row - n0) * g.b_n * SB) + dchunk * 16;
        } else {
            constexpr int CPR = Cfg::BN / GB::EPC, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ GB::swz(k);
            int col = n0 + c * GB::EPC;
            col = col <= g.N - GB::EPC ? col : g.N - GB::EPC;
            offb[p] = (unsigned)(((long)k * g.b_k + (col - (n0 <= g.N - GB::EPC ? n0 : g.N - GB::EPC))) * SB);
        }
        ldb[p] = B_BASE + q * 1024;
    }
    // scalar bases: k-dense -> first row of the tile; row-dense -> first (clamped) column of the tile in k-row 0
    const char *base_a = Cfg::LA == LM_K ? A + (ao + (long)m0 * g.a_m) * ES
                                         : A + (ao + (m0 <= g.M - GA::EPC ? m0 : g.M - GA::EPC)) * ES;
    const char *base_b = Cfg::LB == LM_K ? B + (bo + (long)n0 * g.b_n) * SB
                                         : B + (bo + (n0 <= g.N - GB::EPC ? n0 : g.N - GB::EPC)) * SB;
    // bytes a stage advances an operand's source by: 128 bytes of k, or a stage's k-rows; a k-dense f8 buffer
    // is 128 bytes of k as well, but that is two stages
    const long a_adv = Cfg::LA == LM_K ? P_ROW_BYTES : (long)GA::STAGE_K * g.a_k * ES;
    const long b_adv = Cfg::LB == LM_K ? P_ROW_BYTES : (long)GB::STAGE_K * g.b_k * SB;

    // Split K: blockIdx.y owns stages [t0, t0 + T) and writes its accumulators, unrounded, to its own slab of
    // `partials`; a second kernel adds the slabs in a fixed order and rounds once.  (stages_per_split is even
    // when the right operand's buffers hold pairs of stages.)
    const int T_all = g.K * ES / P_ROW_BYTES;
    const int t0 = blockIdx.y * stages_per_split;
    const int T = T_all - t0 < stages_per_split ? T_all - t0 : stages_per_split;  // stages of this workgroup
    const int TB = B_PAIR ? (T + 1) / 2 : T;        // right-operand buffers' worth of k
    base_a = uniform_ptr(base_a + t0 * a_adv);
    base_b = uniform_ptr(base_b + (B_PAIR ? t0 >> 1 : t0) * b_adv);

    // What to fetch next, decided at a stage's barrier and carried to the slices that issue it.  Every stage
    // issues a full list -- PA instructions of A, PBS of B -- so that the number of instructions in flight at any
    // barrier is a compile-time constant (s_waitcnt takes an immediate): past the end of K the list re-fetches the
    // last stage into a buffer nobody reads any more.
    struct Fetch {
        int a_src;       // stage of A (already clamped to T - 1)
        unsigned a_dst;  // byte offset of its LDS buffer
        int b_src;       // buffer's worth of B (clamped to TB - 1)
        unsigned b_dst;
        int b_half;      // paired buffers go out in two halves
        bool b_on;       // paired buffers: the very first stage has no free buffer to refill
    };
    // element e of a stage's issue list; after unrolling, e is a constant and the chains fold to one instruction
    auto dma_element = [&](int e, const Fetch &f) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (e == p) dma16_sbase(base_a + f.a_src * a_adv, offa[p], lds0 + f.a_dst + lda[p]);
#pragma unroll
        for (int p = 0; p < PBS; p++)
            if (e == PA + p && f.b_on) {
                unsigned voff = offb[p], off = ldb[p];
                if constexpr (B_PAIR) {
                    voff = f.b_half ? offb[p + PBS] : offb[p];
                    off = f.b_half ? ldb[p + PBS] : ldb[p];
                }
                dma16_sbase(base_b + f.b_src * b_adv, voff, lds0 + f.b_dst + off);
            }
    };

    // ---- fragment addresses ----
    // k-dense: lane (lr, lh) reads chunk 2*s + lh of row lr of a 32-row tile; the chunk sits at slot
    // chunk ^ ((row >> 1) & 7) of its row.  f8 storage: the lane's 8 k are 8 bytes, half lh of chunk s (second
    // stage of the pair: s + 4) of the 128-byte row.
    // row-dense: lane (lr, lh) needs the (SLICE_K / 2) k that start at k = SLICE_K * s + (SLICE_K / 2) * lh, of
    // row lr.  One or two transpose reads of RPT k-rows each deliver them; for each the lane supplies the
    // address of its share of k-row (that start) + RPT * e + kq, columns of its 16-column half of the tile.
    // (k % RPT) == kq whatever s and e are, so the swizzle is a per-lane constant and the slice / half offsets
    // are immediates.
    constexpr int TILE_BYTES = 32 * P_ROW_BYTES;  // k-dense: 32 rows
    const int frag_row = lr * P_ROW_BYTES;
    const int s16 = lane & 15;
    int a_frag[P_SLICES], b_frag[P_SLICES];  // k-dense: one address per slice, tiles are immediates
    int a_mn[TM], b_mn[TN];                  // row-dense: one address per tile, slices are immediates
#pragma unroll
    for (int sl = 0; sl < P_SLICES; sl++) {
        a_frag[sl] = (wave_m * TM) * TILE_BYTES + frag_row + (kd_slot(lr, 2 * sl + lh) << 4);
        b_frag[sl] = B_BASE + (wave_n * TN) * TILE_BYTES + frag_row +
                     (B_F8 ? (kd_slot(lr, sl) << 4) + lh * 8 : (kd_slot(lr, 2 * sl + lh) << 4));
    }
    {
        const int kq = ES == 2 ? s16 >> 2 : s16 >> 1, sub = ES == 2 ? (s16 & 3) : (s16 & 1);
        const int col_bytes = ((lane >> 4) & 1) * 16 * ES + sub * 8;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int bytes = (wave_m * TM + i) * 32 * ES + col_bytes, c = bytes >> 4;
            a_mn[i] = (lh * (GA::SLICE_K / 2) + kq) * Cfg::BM * ES + ((c ^ GA::swz(kq)) << 4) + (bytes & 8);
        }
    }
    {
        const int kq = SB == 2 ? s16 >> 2 : s16 >> 1, sub = SB == 2 ? (s16 & 3) : (s16 & 1);
        const int col_bytes = ((lane >> 4) & 1) * 16 * SB + sub * 8;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int bytes = (wave_n * TN + j) * 32 * SB + col_bytes, c = bytes >> 4;
            b_mn[j] = B_BASE + (lh * (GB::SLICE_K / 2) + kq) * Cfg::BN * SB + ((c ^ GB::swz(kq)) << 4) + (bytes & 8);
        }
    }
    // fragment of the left operand: tile i, slice SL, from the stage buffer at byte offset `buf`
    auto read_a = [&](unsigned buf, auto sl_, int i) -> u32x4_t {
        constexpr int SL = decltype(sl_)::value;
        if constexpr (Cfg::LA == LM_K) {
            return lds_get(smem + buf, a_frag[SL] + i * TILE_BYTES);
        } else {
            const u32x2_t lo = lds_get_tr<ES>(smem + buf, a_mn[i] + (SL * GA::SLICE_K) * Cfg::BM * ES);
            const u32x2_t hi = lds_get_tr<ES>(smem + buf, a_mn[i] + (SL * GA::SLICE_K + GA::RPT) * Cfg::BM * ES);
            return u32x4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    // fragment of the right operand; f8 storage comes back as 8 raw bytes in .x/.y and is widened at its use.
    // `second`: the stage is the second of its pair (paired buffers only)
    auto read_b = [&](unsigned buf, int second, auto sl_, int j) -> u32x4_t {
        constexpr int SL = decltype(sl_)::value;
        if constexpr (Cfg::LB == LM_K && !B_F8) {
            return lds_get(smem + buf, b_frag[SL] + j * TILE_BYTES);
        } else if constexpr (Cfg::LB == LM_K) {
            // chunk s + 4 instead of s: bit 6 of the byte offset flipped (the swizzle is an XOR)
            const u32x2_t v = lds_get64(smem + buf, (b_frag[SL] ^ (second << 6)) + j * TILE_BYTES);
            return u32x4_t{v.x, v.y, 0u, 0u};
        } else if constexpr (B_F8) {
            const u32x2_t v = lds_get_tr<1>(smem + buf, b_mn[j] + (SL * GB::SLICE_K) * Cfg::BN * SB);
            return u32x4_t{v.x, v.y, 0u, 0u};
        } else {
            const u32x2_t lo = lds_get_tr<SB>(smem + buf, b_mn[j] + (SL * GB::SLICE_K) * Cfg::BN * SB);
            const u32x2_t hi = lds_get_tr<SB>(smem + buf, b_mn[j] + (SL * GB::SLICE_K + GB::RPT) * Cfg::BN * SB);
            return u32x4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    u32x4_t fa[2][TM], fb[2][TN];  // [register set][tile]: slice s lives in set s % 2
    u32x4_t bwide = u32x4_t{0u, 0u, 0u, 0u};  // f8e4m3 storage: the widened first right fragment of the next slice

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;

    // One k-slice of work, in an explicitly pinned order: the MFMAs of slice CUR (register set CUR % 2),
    // with the fragment reads of slice RD (from the buffers at rd_a / rd_b) and elements [D0, D0 + DN) of the
    // issue list `f` spread evenly between them.  Neither the reads nor the DMA then arrive in bursts: a burst of
    // DMA instructions fills the memory pipeline's issue queue and stalls the wavefront in front of its next MFMA.
    auto slice_step = [&](auto cur_, auto rd_, auto d0_, auto dn_, unsigned rd_a, unsigned rd_b, int rd_second,
                          const Fetch &f, bool do_dma) {
        constexpr int SET = decltype(cur_)::value & 1, RD = decltype(rd_)::value;
        constexpr int D0 = decltype(d0_)::value, DN = decltype(dn_)::value;
        constexpr int MF = TM * TN, RN = TM + TN;
        // f8e4m3 storage: a right fragment is widened to bf16 one group of TM MFMAs AHEAD of its use, right behind an
        // MFMA that has just been issued, so that the conversions run in that MFMA's shadow; widened in front of
        // its first use they hold the matrix core up for their own latency once per group, which a wavefront that has
        // its SIMD to itself cannot hide (measured on 128 x 128 tiles, M = 256: 0.60 -> 0.56 us per 64-k stage; the
        // four conversions per fragment are full-rate instructions, 16 cycles of issue against 32 per MFMA, so with
        // one or two MFMAs per fragment the wavefront's own instruction issue stays the limit: 0.45 us without any
        // conversion, 0.39 us with bf16 weights).  `bwide` carries the first fragment of the next slice across the call.
        u32x4_t bcur = B_F8 ? bwide : fb[SET][0], bnext = bcur;
#pragma unroll
        for (int idx = 0; idx < MF; idx++) {
#pragma unroll
            for (int r = 0; r < RN; r++) {
                if (r * MF / RN != idx) continue;
                typedef std::integral_constant<int, RD> RS;
                // (f8e4m3: the next slice's first right fragment is needed first, by the conversion at the end of this one)
                const bool b_turn = B_F8 ? (r == 0 || r > TM) : r >= TM;
                const int bi = B_F8 ? (r == 0 ? 0 : r - TM) : r - TM, ai = B_F8 ? r - 1 : r;
                if (!b_turn) fa[RD & 1][ai] = read_a(rd_a, RS{}, ai);
                else fb[RD & 1][bi] = read_b(rd_b, rd_second, RS{}, bi);
            }
            if (idx % TM == 0 && idx > 0) bcur = B_F8 ? bnext : fb[SET][idx / TM];
            // operands swapped: the accumulator then holds, per lane, runs of 4 consecutive n of one m
            Cmp::mma(bcur, fa[SET][idx % TM], acc[idx % TM][idx / TM]);
            if constexpr (B_F8) {
                if (idx % TM == 0 && idx / TM + 1 < TN) bnext = widen_f8x8(u32x2_t{fb[SET][idx / TM + 1].x, fb[SET][idx / TM + 1].y});
                if (idx == MF - 1) bwide = widen_f8x8(u32x2_t{fb[RD & 1][0].x, fb[RD & 1][0].y});
            }
#pragma unroll
            for (int d = 0; d < DN; d++) {
                // (in the gaps BETWEEN those that take a fragment read where the spacing allows it: a read and a DMA
                // instruction behind the same MFMA take longer to issue than the MFMA runs, and the next one starts late)
                constexpr int GAP = DN > 0 ? MF / DN : 1;
                if (d * MF / (DN > 0 ? DN : 1) + (GAP > 1 ? GAP / 2 : 0) != idx) continue;
                if (do_dma) dma_element(D0 + d, f);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    typedef std::integral_constant<int, 2> I2;
    typedef std::integral_constant<int, 3> I3;
    constexpr int PH = P / 2;  // elements of a stage's list issued during its slice 3; the rest during the next slice 0
    typedef std::integral_constant<int, PH> DH;
    typedef std::integral_constant<int, P - PH> DR;

    // ---- prologue: ring slot j gets stage j of A and buffer j of B (with paired buffers: stages 2j, 2j+1), clamped
    // to the last one so that every group has PA + PB instructions ----
#pragma unroll
    for (int j = 0; j < NST; j++) {
        const int ta = j < T ? j : T - 1, tb = j < TB ? j : TB - 1;
#pragma unroll
        for (int p = 0; p < PA; p++)
            dma16_sbase(base_a + ta * a_adv, offa[p], lds0 + (unsigned)j * Cfg::A_BYTES + lda[p]);
#pragma unroll
        for (int p = 0; p < PB; p++)
            dma16_sbase(base_b + tb * b_adv, offb[p], lds0 + (unsigned)j * Cfg::B_BYTES + ldb[p]);
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((NST - 1) * (PA + PB)));  // group 0 has landed
    __builtin_amdgcn_s_barrier();
    HODU_STAMP(1);
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < TM; i++) fa[0][i] = read_a(0u, I0{}, i);
#pragma unroll
    for (int j = 0; j < TN; j++) fb[0][j] = read_b(0u, 0, I0{}, j);
    if constexpr (B_F8) bwide = widen_f8x8(u32x2_t{fb[0][0].x, fb[0][0].y});

    // Instructions that may still be in flight at the barrier of stage t without touching what stage t+1 reads:
    // the NST - 2 youngest issue groups.  Groups, oldest first: the NST groups of the prologue (PA + PB each), then
    // one list per stage (P each; with paired buffers stage 0's list has no B part).  Loads return in issue order.
    auto list_size = [](int j) { return j < NST ? PA + PB : (j == NST && B_PAIR ? PA : P); };
    auto allowed_at = [&](int t) {
        int n = 0;
        for (int j = t + 2; j <= NST + t - 1; j++) n += list_size(j);
        return n;
    };
    auto wait_stage = [&](int t) {
        // t < NST: the window still overlaps the prologue; one immediate per case
        if constexpr (NST == 2) {
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        } else if constexpr (NST == 3) {
            constexpr int W0 = PA + PB, W1 = B_PAIR ? PA : P;
            if (t == 0) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(W0));
            else if (t == 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(W1));
            else __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(P));
        } else {
            constexpr int L0 = B_PAIR ? PA : P;
            constexpr int W0 = 2 * (PA + PB), W1 = PA + PB + L0, W2 = L0 + P;
            if (t == 0) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(W0));
            else if (t == 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(W1));
            else if (t == 2) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(W2));
            else __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(2 * P));
        }
        (void)allowed_at;
    };

    // Ring bookkeeping (byte offsets): where stage t and stage t+1 live, and which pair buffer was vacated last.
    unsigned a_cur = 0, b_cur = 0;          // buffers of stage t
    unsigned b_prev_pair = 0;               // paired buffers: the buffer of the pair before the current one
    int a_slot = 0, b_slot = 0;             // ring slots of stage t
    Fetch f{};                              // list decided at the previous stage's barrier (second half pending)
    bool f_on = false;

    // The loop body is branch-free apart from the DMA predicates: past the last stage the reads fetch
    // LDS bytes nobody uses and the barrier is one too many, both harmless and cheaper than a second
    // copy of the MFMA code.
    for (int t = 0; t < T; t++) {
        const int a_next_slot = a_slot + 1 == NST ? 0 : a_slot + 1;
        // B moves to its next buffer every stage, or every second stage when the buffers hold pairs
        const bool b_moves = !B_PAIR || (t & 1);
        const int b_next_slot = b_moves ? (b_slot + 1 == NST ? 0 : b_slot + 1) : b_slot;
        const unsigned a_next = (unsigned)a_next_slot * Cfg::A_BYTES, b_next = (unsigned)b_next_slot * Cfg::B_BYTES;

        // slice 0: multiply it, read slice 1, issue the second half of the list the previous stage started
        slice_step(I0{}, I1{}, DH{}, DR{}, a_cur, b_cur, t & 1, f, f_on);
        slice_step(I1{}, I2{}, I0{}, I0{}, a_cur, b_cur, t & 1, f, false);
        slice_step(I2{}, I3{}, I0{}, I0{}, a_cur, b_cur, t & 1, f, false);
        // stage t+1 has landed and every read of stage t has returned
        wait_stage(t);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // the list of this stage: A's stage t + NST into the buffer stage t just vacated; B likewise, or -- paired
        // buffers -- a half of the pair that goes where the last finished pair was: odd t finishes pair t/2 and
        // sends the first half of pair t/2 + NST there, the next even stage sends the second half
        f.a_src = t + NST < T ? t + NST : T - 1;
        f.a_dst = a_cur;
        if constexpr (B_PAIR) {
            const int pair = (t & 1) ? (t >> 1) + NST : ((t - 2) >> 1) + NST;
            f.b_src = pair < TB ? pair : TB - 1;
            f.b_dst = (t & 1) ? b_cur : b_prev_pair;
            f.b_half = (t & 1) ? 0 : 1;
            f.b_on = t >= 1;
            if (t & 1) b_prev_pair = b_cur;
        } else {
            f.b_src = t + NST < TB ? t + NST : TB - 1;
            f.b_dst = b_cur;
            f.b_half = 0;
            f.b_on = true;
        }
        f_on = true;
        // slice 3: multiply it, read slice 0 of stage t+1, issue the first half of the list
        slice_step(I3{}, I0{}, I0{}, DH{}, a_next, b_next, (t + 1) & 1, f, true);
        a_cur = a_next;
        b_cur = b_next;
        a_slot = a_next_slot;
        b_slot = b_next_slot;
    }

    // the clamped re-fetches of the last stages are still writing LDS: the workgroup must not end (and hand its
    // LDS to another) before they are done
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));

    out_t *Cb;
    // every wavefront's DMA has landed before any wavefront reuses LDS for its epilogue
    __syncthreads();
    HODU_STAMP(2);
    char *patch = smem + wave * (32 * (TN * 32 * 4 + 16));  // sized for 4-byte outputs, the largest
    if (gridDim.y > 1 && arrival != nullptr) {
        // cut along K, summed here: only the workgroup that arrives last stores the tile
        if (!splitk_exchange<Cfg::NW, TM, TN>(acc, partials, arrival, reinterpret_cast<int *>(smem + Cfg::LDS_BYTES - 16), tid)) {
            HODU_STAMP(3);
            return;
        }
        __syncthreads();  // (the flag word lies outside every wavefront's patch; the barrier orders LDS reuse all the same)
        HODU_STAMP(4);
    } else if (gridDim.y > 1) {
        constexpr int ACC = Cfg::CK == CK_I8 ? OUT_I32 : OUT_F32;
        typedef typename Out<ACC>::T part_t;
        part_t *Pb = (part_t *)partials + ((long)blockIdx.y * g.batches + batch) * (long)g.M * g.N;
#pragma unroll
        for (int i = 0; i < TM; i++)
            store_band_via_lds<ACC, TN, false>(patch, Pb, acc[i], m0 + wave_m * TM * 32 + i * 32, n0 + wave_n * TN * 32, lane, g.M, g.N, g.epi);
        return;
    }
    Cb = C + batch * (long)g.M * g.N;
    EpiPrepared<Out<Cfg::OUT>::DT, 16 / (int)sizeof(out_t)> steps{};
    if (g.epi.n != 0) steps = band_columns_prepare<Cfg::OUT, TN, 32>(g.epi, n0 + wave_n * TN * 32, lane, g.N);
#pragma unroll
    for (int i = 0; i < TM; i++)
        store_band_via_lds<Cfg::OUT, TN, true, acc_t, 32, true>(patch, Cb, acc[i], m0 + wave_m * TM * 32 + i * 32, n0 + wave_n * TN * 32, lane, g.M,
                                                                g.N, g.epi, steps);
    HODU_STAMP(5);
}

// splits > 1: K is cut into that many ranges of whole stages, each range a workgroup of its own (grid.y);
// the partial sums go through the context's workspace (splits x batches x M x N accumulators, which requires
// batches * M * N to be a multiple of 4 for the vectorised second pass -- the caller checks)
template <class Cfg> int launch_pipe(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g,
                                     int splits = 1) {
    auto kernel = mfma_pipe_kernel<Cfg>;
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    const int T = (int)((long)g.K * Cfg::ES / P_ROW_BYTES);
    int per = T;
    void *partials = nullptr;
    if (splits > 1) {
        per = (T + splits - 1) / splits;
        if (Cfg::B_PAIR && (per & 1)) per++;
        splits = (T + per - 1) / per;
    }
    const long elems = g.batches * (long)g.M * g.N;
    // the ranges of a tile meet inside the kernel (one arrival counter per tile) wherever there is a counter for every
    // tile; a product with more tiles than that -- it does not need cutting -- keeps the second kernel
    const bool in_kernel = splits > 1 && total <= kArrivalSlots;
    int *arrival = nullptr;
    if (splits > 1) {
        const size_t bytes = in_kernel ? (size_t)splits * total * Cfg::BM * Cfg::BN * 4 : (size_t)splits * elems * 4;
        int rc = ensure_workspace(ctx, bytes);
        if (rc == HODU_ROCM_OK && in_kernel) rc = ensure_arrival(ctx);
        if (rc != HODU_ROCM_OK) return rc;
        partials = ctx->workspace.ptr;
        if (in_kernel) arrival = ctx->arrival;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)total, (unsigned)(splits > 1 ? splits : 1)), dim3(Cfg::NT), Cfg::LDS_BYTES,
                       ctx->stream, (const char *)a, (const char *)b, (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n,
                       per, partials, arrival);
    HODU_HIP(hipGetLastError());
    if (splits > 1 && !in_kernel) {
        const unsigned blocks = (unsigned)((elems + 1023) / 1024);
        if (Cfg::CK == CK_I8)
            hipLaunchKernelGGL((splitk_reduce_kernel<Cfg::OUT, int32_t>), dim3(blocks), dim3(256), 0, ctx->stream,
                               (const int32_t *)partials, (typename Out<Cfg::OUT>::T *)c, elems, splits, g.N, g.epi);
        else
            hipLaunchKernelGGL((splitk_reduce_kernel<Cfg::OUT, float>), dim3(blocks), dim3(256), 0, ctx->stream,
                               (const float *)partials, (typename Out<Cfg::OUT>::T *)c, elems, splits, g.N, g.epi);
        HODU_HIP(hipGetLastError());
    }
    return HODU_ROCM_OK;
}

// How many ways to cut K for a product that fills `tiles` workgroups of the chosen shape on `cus` compute
// units: enough to occupy the machine, at most 8, and never fewer than 4 stages per range.  1 = do not split.
inline int pick_splits(long tiles, long cus, int stages, long elems, int forced) {
    if (elems % 4 != 0 || stages < 2) return 1;
    if (forced >= 1) return forced < stages ? forced : stages;
    if (tiles * 2 > cus) return 1;
    long s = cus / tiles;
    if (s > 8) s = 8;
    if (s > stages / 4) s = stages / 4;
    return s >= 2 ? (int)s : 1;
}

// K a whole number of 128-byte stages; the row-dense layouts exist for 8- and 16-bit types and fetch whole
// 16-byte chunks of a k-row; alignment is what pick_mode already established
// the DMA addresses are a scalar base plus a 32-bit byte offset per lane that spans up to 256 rows (k-dense) or 128
// k-rows (row-dense) of the operand: the stride that separates them must keep that below 4 GB
inline bool pipe_offsets_fit(long stride, int elem_bytes) {
    return stride >= 0 && stride <= ((1L << 32) - 8192) / (256L * elem_bytes);
}

template <int CK> bool pipe_eligible(int la, int lb, const DevProduct &g) {
    constexpr int ES = Compute<CK>::ES;
    if (g.K <= 0 || ((long)g.K * ES) % P_ROW_BYTES != 0) return false;
    if (!pipe_offsets_fit(la == LM_K ? g.a_m : g.a_k, ES) || !pipe_offsets_fit(lb == LM_K ? g.b_n : g.b_k, ES)) return false;
    if (la == LM_K && lb == LM_K) return true;
    if (ES > 2 || la == LM_SCALAR || lb == LM_SCALAR) return false;
    constexpr int EPC = 16 / ES;  // a row-dense operand is fetched in whole 16-byte chunks of a k-row
    return (la == LM_K || (g.M >= EPC && g.M % EPC == 0)) && (lb == LM_K || (g.N >= EPC && g.N % EPC == 0));
}

// bf16 left operand k-dense, f8e4m3 right operand k-dense or row-dense.  DMA moves 16-byte chunks, so the
// byte-sized operand needs 16-byte alignment of everything pick_mode only checked to 8; its k-dense form
// moves whole 128-byte lines of k, i.e. K is a multiple of 128.
inline bool pipe_f8_eligible(int la, int lb, const void *b, const DevProduct &g) {
    if (la != LM_K || lb == LM_SCALAR || g.K <= 0 || g.K % 64 != 0) return false;
    if (!pipe_offsets_fit(g.a_m, 2) || !pipe_offsets_fit(lb == LM_K ? g.b_n : g.b_k, 1)) return false;
    if (((uintptr_t)b + (uintptr_t)g.b_off) % 16 != 0) return false;
    for (int d = 0; d < g.nb; d++)
        if (g.b_bs[d] % 16 != 0) return false;
    if (lb == LM_K) return g.K % 128 == 0 && (g.N == 1 || g.b_n % 16 == 0);
    return g.N >= 16 && g.N % 16 == 0 && g.b_k % 16 == 0;
}

}  // namespace mfma
}  // namespace hodu
