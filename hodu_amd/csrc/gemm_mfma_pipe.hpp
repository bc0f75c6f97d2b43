// Software-pipelined MFMA tile kernel for products whose operands are BOTH k-dense in their
// compute type (bf16 x bf16, f16 x f16, i8 x i8, f32 x f32 with `stride_k == 1`, 16-byte aligned
// rows, K a multiple of 128 bytes).  Same tiles, same MFMA instructions and same results as the
// general kernel in gemm_mfma.hpp; what differs is how the K loop is fed:
//
//   * K advances 128 bytes per stage (64 bf16 / 128 i8 / 32 f32 = four MFMA k-slices).  Every DMA
//     request is one whole 128-byte cache line of one row: fetching rows in 64-byte halves feeds a
//     compute unit at 29 B/clk, whole lines at 47 B/clk (measured on the 4096 x 4096 x 14336 sweep);
//   * two stages of LDS, written by LDS-DMA only (global_load_lds_dwordx4: no staging registers, no
//     ds_write).  The DMA of stage t+2 is issued, into the buffer stage t just vacated, while the
//     last k-slice of stage t multiplies, so it has the whole of stage t+1 to land;
//   * a stage is an array of 1 KB blocks, one block = 8 rows x 128 B = exactly what one wavefront-wide
//     DMA instruction writes, 128 bytes apart; the eight 16-byte chunks of a row are XOR-swizzled by
//     row % 8 -- applied to the SOURCE address of the DMA -- so that an MFMA fragment read (16 lanes =
//     16 rows, one chunk) touches all 64 banks once (lds_swizzled in gemm_mfma.hpp);
//   * the MFMA fragments live in one register set that is refilled one k-slice ahead of its use, each
//     ds_read_b128 interleaved with the MFMAs of the previous slice, so that LDS and the matrix cores
//     run side by side instead of in alternating bursts;
//   * one bare s_barrier per stage, preceded by s_waitcnt vmcnt(0) lgkmcnt(0): at that point the only
//     DMA in flight is the next stage's, and every fragment read of the current stage has returned.
//
// Row-dense operands (stride 1 along m or n: a [K, N] row-major right operand, a transposed left
// operand) of the 16-bit types take the same path.  A stage of such an operand is 64 k-rows of the
// tile's ROWS contiguous elements, DMA'd as whole rows (1 KB = 1024 / (2 * ROWS) k-rows per
// instruction) into a plain [k][ROWS] array whose 16-byte chunks are XOR-swizzled by (k % 4) << 2.
// The MFMA fragment -- 8 consecutive k of ONE row per lane -- comes out of that k-major array
// through two ds_read_b64_tr_b16 (LDS transpose reads: each hands a lane 4 consecutive k of its own
// column from four rows that 16 lanes read together), so no register-level transpose and no second
// LDS layout is needed.
//
// f8e4m3 right operands (the fused to_dtype of a weight) are DMA'd as the bytes they are and widened
// to bf16 between the fragment read and the MFMA (v_cvt_scalef32_pk_bf16_fp8, exact): no widened
// copy ever exists in LDS or HBM.  k-dense f8 rows still move as whole 128-byte lines, which is 128 k
// = two stages of the bf16 left operand, so the right operand's two buffers each hold a PAIR of
// stages and are refilled one half per stage; row-dense f8 ([K, N] bytes) moves 64 k-rows per stage.
//
// Hazards.  The barrier in stage t is reached by a wavefront only after all its reads of stage t
// have RETURNED (lgkmcnt(0)) and its own share of stage t+1 has landed (vmcnt(0)); past it, stage t's
// buffer is dead for everybody and stage t+1 is complete for everybody.
#pragma once

#include <type_traits>

#include "gemm_mfma.hpp"

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

template <int CK_, int OUT_, int BM_, int BN_, int WM_, int WN_, int LA_ = LM_K, int LB_ = LM_K, int SKB_ = SK_SAME>
struct PipeConfig {
    static constexpr int CK = CK_, OUT = OUT_, BM = BM_, BN = BN_, WM = WM_, WN = WN_, LA = LA_, LB = LB_, SKB = SKB_;
    static constexpr int NT = WM * WN * 64, NW = WM * WN;
    static constexpr int ES = Compute<CK>::ES;
    static constexpr bool B_F8 = SKB == SK_F8;
    static constexpr int SB = B_F8 ? 1 : ES;               // bytes of a right-operand element in memory
    static constexpr bool B_PAIR = B_F8 && LB == LM_K;     // right-operand buffers hold two stages each
    static constexpr int BK = P_ROW_BYTES / ES;
    // k-dense: 8-row blocks of 1 KB, 128 bytes apart; row-dense: [k-rows of a stage][ROWS] with no gaps
    static constexpr int A_BYTES = (BM / 8) * (LA == LM_K ? SWZ_BLOCK : 1024);
    static constexpr int B_BYTES = LB == LM_K ? (BN / 8) * SWZ_BLOCK : (BK * BN * SB);
    static constexpr int LDS_BYTES = 2 * (A_BYTES + B_BYTES);
    static constexpr int PA = (BM / 8) / NW;                                    // DMA instructions per wavefront: a stage of A,
    static constexpr int PB = (LB == LM_K ? BN / 8 : BK * BN * SB / 1024) / NW;  // a buffer of B,
    static constexpr int PBS = B_PAIR ? PB / 2 : PB;                            // what of B goes out per stage
    static constexpr int P = PA + PBS;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;  // 32x32 MFMA tiles per wave
    static_assert(!B_F8 || CK == CK_BF16, "f8e4m3 storage widens to bf16");
    static_assert(P_ROW_BYTES == ROW_BYTES, "the pipelined kernel uses the swizzled 128-byte-row layout");
    static_assert((BM / 8) % NW == 0 && PB >= 1 && (!B_PAIR || PB % 2 == 0), "DMA split");
    static_assert((PA + PB) * 2 < 64, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
    static_assert((LA == LM_K || (ES <= 2 && BM >= 128)) && (LB == LM_K || (ES <= 2 && BN >= 128)),
                  "row-dense operands: 8- and 16-bit types, tiles of at least 128 rows");
};

// issued through inline assembly so that the compiler's own wait-count bookkeeping (which would put
// an s_waitcnt vmcnt(0) in front of the next LDS read) stays out of the way; completion is awaited
// explicitly before the barrier that publishes the stage
__device__ __forceinline__ void dma16_raw(const char *gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory");
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

// 8 f8e4m3 -> 8 bf16 (exact)
__device__ __forceinline__ u32x4_t widen_f8x8(const u32x2_t &v) {
    return u32x4_t{f8pair_to_bf16pair(v.x, false), f8pair_to_bf16pair(v.x, true), f8pair_to_bf16pair(v.y, false),
                   f8pair_to_bf16pair(v.y, true)};
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                            typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                            int tiles_m, int tiles_n) {
    extern __shared__ __align__(16) char smem[];
    typedef Compute32<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, ES = Cfg::ES, SB = Cfg::SB, PA = Cfg::PA, PB = Cfg::PB, PBS = Cfg::PBS,
                  P = Cfg::P;
    constexpr bool B_F8 = Cfg::B_F8, B_PAIR = Cfg::B_PAIR;
    typedef RowDenseGeom<ES, ES> GA;
    typedef RowDenseGeom<SB, ES> GB;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int lr = lane & 31, lh = lane >> 5;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

    // LDS: [A stage 0][A stage 1][B buffer 0][B buffer 1]
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    constexpr int B_BASE = 2 * Cfg::A_BYTES;

    // ---- DMA plan of this wavefront: PA + PB instructions, each one 1 KB of LDS ----
    // k-dense operand: a block of 8 rows x 128 B; lane -> (row in block, slot), the slot holds chunk slot ^ row.
    // row-dense operand: KPI consecutive k-rows of ROWS elements; lane -> (k-row, slot), the slot holds chunk
    // slot ^ swz(k); a chunk that starts past the operand's last row is fetched from the last whole chunk
    // instead (its columns are never stored).
    const char *gpa[PA], *gpb[PB];    // source address of this lane for stage (buffer) 0
    unsigned lda[PA], ldb[PB];        // block offset inside a buffer (wave-uniform)
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = p * Cfg::NW + wave;
        if constexpr (Cfg::LA == LM_K) {
            const int drow = lane >> 3, dchunk = (lane & 7) ^ drow;
            int row = m0 + q * 8 + drow;
            row = row < g.M ? row : g.M - 1;
            gpa[p] = A + (ao + (long)row * g.a_m) * ES + dchunk * 16;
            lda[p] = q * SWZ_BLOCK;
        } else {
            constexpr int CPR = Cfg::BM / GA::EPC, KPI = 64 / CPR;  // chunks per k-row, k-rows per instruction
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ GA::swz(k);
            int col = m0 + c * GA::EPC;
            col = col <= g.M - GA::EPC ? col : g.M - GA::EPC;
            gpa[p] = A + (ao + (long)k * g.a_k + col) * ES;
            lda[p] = q * 1024;
        }
    }
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int q = p * Cfg::NW + wave;
        if constexpr (Cfg::LB == LM_K) {
            const int drow = lane >> 3, dchunk = (lane & 7) ^ drow;
            int row = n0 + q * 8 + drow;
            row = row < g.N ? row : g.N - 1;
            gpb[p] = B + (bo + (long)row * g.b_n) * SB + dchunk * 16;
            ldb[p] = B_BASE + q * SWZ_BLOCK;
        } else {
            constexpr int CPR = Cfg::BN / GB::EPC, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ GB::swz(k);
            int col = n0 + c * GB::EPC;
            col = col <= g.N - GB::EPC ? col : g.N - GB::EPC;
            gpb[p] = B + (bo + (long)k * g.b_k + col) * SB;
            ldb[p] = B_BASE + q * 1024;
        }
    }
    // bytes a stage advances an operand's source by: 128 bytes of k, or a stage's k-rows; a k-dense f8 buffer
    // is 128 bytes of k as well, but that is two stages
    const long a_adv = Cfg::LA == LM_K ? P_ROW_BYTES : (long)GA::STAGE_K * g.a_k * ES;
    const long b_adv = Cfg::LB == LM_K ? P_ROW_BYTES : (long)GB::STAGE_K * g.b_k * SB;

    const int T = g.K * ES / P_ROW_BYTES;           // stages
    const int TB = B_PAIR ? (T + 1) / 2 : T;        // right-operand buffers' worth of k

    // element e of a stage's issue list: its PA instructions of A (stage t_a), then PBS of B (buffer tb; a paired
    // buffer goes out in two halves, and which half is a run-time fact: the issuing stage's parity).  After
    // unrolling, e is a constant and the chains below fold to one instruction.
    auto dma_element = [&](int e, int t_a, bool do_a, int tb, int half, bool do_b) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (e == p && do_a)
                dma16_raw(gpa[p] + t_a * a_adv, __builtin_amdgcn_readfirstlane(lds0 + (unsigned)(t_a & 1) * Cfg::A_BYTES + lda[p]));
#pragma unroll
        for (int p = 0; p < PBS; p++)
            if (e == PA + p && do_b) {
                const char *src = gpb[p];
                unsigned off = ldb[p];
                if constexpr (B_PAIR) {
                    src = half ? gpb[p + PBS] : gpb[p];
                    off = half ? ldb[p + PBS] : ldb[p];
                }
                dma16_raw(src + tb * b_adv, __builtin_amdgcn_readfirstlane(lds0 + (unsigned)(tb & 1) * Cfg::B_BYTES + off));
            }
    };

    // ---- fragment addresses ----
    // k-dense: lane (lr, lh) reads chunk 2*s + lh of row lr of a 32-row tile (four consecutive 8-row
    // blocks); the chunk sits at slot chunk ^ (row % 8) of its row.  f8 storage: the lane's 8 k are 8 bytes,
    // half lh of chunk s (second stage of the pair: s + 4) of the 128-byte row.
    // row-dense: lane (lr, lh) needs the (SLICE_K / 2) k that start at k = SLICE_K * s + (SLICE_K / 2) * lh, of
    // row lr.  One or two transpose reads of RPT k-rows each deliver them; for each the lane supplies the
    // address of its share of k-row (that start) + RPT * e + kq, columns of its 16-column half of the tile.
    // (k % RPT) == kq whatever s and e are, so the swizzle is a per-lane constant and the slice / half offsets
    // are immediates.
    const int frag_row = (lr >> 3) * SWZ_BLOCK + (lr & 7) * P_ROW_BYTES;
    const int s16 = lane & 15;
    int a_frag[P_SLICES], b_frag[P_SLICES];  // k-dense: one address per slice, tiles are immediates
    int a_mn[TM], b_mn[TN];                  // row-dense: one address per tile, slices are immediates
#pragma unroll
    for (int sl = 0; sl < P_SLICES; sl++) {
        a_frag[sl] = (wave_m * TM) * 4 * SWZ_BLOCK + frag_row + (((2 * sl + lh) ^ (lr & 7)) << 4);
        b_frag[sl] = B_BASE + (wave_n * TN) * 4 * SWZ_BLOCK + frag_row +
                     (B_F8 ? ((sl ^ (lr & 7)) << 4) + lh * 8 : (((2 * sl + lh) ^ (lr & 7)) << 4));
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
    // fragment of the left operand: tile i, slice SL of stage t
    auto read_a = [&](int t, auto sl_, int i) -> u32x4_t {
        constexpr int SL = decltype(sl_)::value;
        const char *buf = smem + (t & 1) * Cfg::A_BYTES;
        if constexpr (Cfg::LA == LM_K) {
            return lds_get(buf, a_frag[SL] + i * 4 * SWZ_BLOCK);
        } else {
            const u32x2_t lo = lds_get_tr<ES>(buf, a_mn[i] + (SL * GA::SLICE_K) * Cfg::BM * ES);
            const u32x2_t hi = lds_get_tr<ES>(buf, a_mn[i] + (SL * GA::SLICE_K + GA::RPT) * Cfg::BM * ES);
            return u32x4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    // fragment of the right operand; f8 storage comes back as 8 raw bytes in .x/.y and is widened at its use
    auto read_b = [&](int t, auto sl_, int j) -> u32x4_t {
        constexpr int SL = decltype(sl_)::value;
        const int tb = B_PAIR ? t >> 1 : t;
        const char *buf = smem + (tb & 1) * Cfg::B_BYTES;
        if constexpr (Cfg::LB == LM_K && !B_F8) {
            return lds_get(buf, b_frag[SL] + j * 4 * SWZ_BLOCK);
        } else if constexpr (Cfg::LB == LM_K) {
            // second stage of the pair: chunk s + 4, i.e. bit 6 of the byte offset flipped (the swizzle is an XOR)
            const u32x2_t v = lds_get64(buf, (b_frag[SL] ^ ((t & 1) << 6)) + j * 4 * SWZ_BLOCK);
            return u32x4_t{v.x, v.y, 0u, 0u};
        } else if constexpr (B_F8) {
            const u32x2_t v = lds_get_tr<1>(buf, b_mn[j] + (SL * GB::SLICE_K) * Cfg::BN * SB);
            return u32x4_t{v.x, v.y, 0u, 0u};
        } else {
            const u32x2_t lo = lds_get_tr<SB>(buf, b_mn[j] + (SL * GB::SLICE_K) * Cfg::BN * SB);
            const u32x2_t hi = lds_get_tr<SB>(buf, b_mn[j] + (SL * GB::SLICE_K + GB::RPT) * Cfg::BN * SB);
            return u32x4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    u32x4_t fa[2][TM], fb[2][TN];  // [register set][tile]: slice s lives in set s % 2

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;

    // One k-slice of work, in an explicitly pinned order: the MFMAs of slice CUR (register set CUR % 2),
    // with the fragment reads of slice RD of stage t_rd and DMA instructions [D0, D0 + DN) of the issue list
    // spread evenly between them.  The issue list of a stage is its PA instructions of A followed by PBS of B.
    // Neither the reads nor the DMA then arrive in bursts: a burst of DMA instructions fills the memory
    // pipeline's issue queue and stalls the wavefront in front of its next MFMA.
    //   t_a / do_a   stage of A to fetch, and whether it exists
    //   tb / half / do_b   buffer of B to fetch (a half of it when the buffers hold pairs), and whether it exists
    auto slice_step = [&](auto cur_, auto rd_, auto d0_, auto dn_, int t_rd, int t_a, bool do_a, int tb, int half,
                          bool do_b) {
        constexpr int SET = decltype(cur_)::value & 1, RD = decltype(rd_)::value;
        constexpr int D0 = decltype(d0_)::value, DN = decltype(dn_)::value;
        constexpr int MF = TM * TN, RN = TM + TN;
        u32x4_t bcur = fb[SET][0];
#pragma unroll
        for (int idx = 0; idx < MF; idx++) {
#pragma unroll
            for (int r = 0; r < RN; r++) {
                if (r * MF / RN != idx) continue;
                typedef std::integral_constant<int, RD> RS;
                if (r < TM) fa[RD & 1][r] = read_a(t_rd, RS{}, r);
                else fb[RD & 1][r - TM] = read_b(t_rd, RS{}, r - TM);
            }
            if (idx % TM == 0) bcur = B_F8 ? widen_f8x8(u32x2_t{fb[SET][idx / TM].x, fb[SET][idx / TM].y}) : fb[SET][idx / TM];
            // operands swapped: the accumulator then holds, per lane, runs of 4 consecutive n of one m
            Cmp::mma(bcur, fa[SET][idx % TM], acc[idx % TM][idx / TM]);
#pragma unroll
            for (int d = 0; d < DN; d++) {
                if (d * MF / (DN > 0 ? DN : 1) != idx) continue;
                dma_element(D0 + d, t_a, do_a, tb, half, do_b);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    typedef std::integral_constant<int, 2> I2;
    typedef std::integral_constant<int, 3> I3;
    constexpr int PH = P / 2;  // DMA instructions of a stage issued during slice 3; the rest during the next slice 0
    typedef std::integral_constant<int, PH> DH;
    typedef std::integral_constant<int, P - PH> DR;

    // prologue: stages 0 and 1 of A, buffers 0 and 1 of B (with paired buffers that is stages 0..3 of B)
    auto issue_all = [&](int t, bool do_a, bool do_b) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (do_a) dma16_raw(gpa[p] + t * a_adv, __builtin_amdgcn_readfirstlane(lds0 + (unsigned)(t & 1) * Cfg::A_BYTES + lda[p]));
#pragma unroll
        for (int p = 0; p < PB; p++)
            if (do_b) dma16_raw(gpb[p] + t * b_adv, __builtin_amdgcn_readfirstlane(lds0 + (unsigned)(t & 1) * Cfg::B_BYTES + ldb[p]));
    };
    issue_all(0, true, true);
    if (T > 1) {
        issue_all(1, true, TB > 1);
        // everything of stage 0 has landed once at most stage 1's instructions are outstanding
        if (TB > 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm(PA + PB));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(PA));
    } else {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < TM; i++) fa[0][i] = read_a(0, I0{}, i);
#pragma unroll
    for (int j = 0; j < TN; j++) fb[0][j] = read_b(0, I0{}, j);

    // What stage t issues behind its barrier (second half of the list: during slice 0 of stage t+1):
    //   A: stage t+2.
    //   B, one buffer per stage: buffer t+2.
    //   B, paired buffers: buffer b holds stages 2b, 2b+1 and is free once stage 2b+1 is done.  Odd t frees
    //      buffer (t-1)/2 and issues the first half of buffer (t+3)/2 into it; the following even stage issues
    //      the second half.  Both have two or more stages to land.
    auto b_target = [&](int t, int &tb, int &half, bool &ok) {
        if constexpr (B_PAIR) {
            tb = (t + 2 + (t & 1)) >> 1;
            half = (t & 1) ? 0 : 1;
            ok = t >= 1 && tb < TB;
        } else {
            tb = t + 2;
            half = 0;
            ok = tb < TB;
        }
    };

    // The loop body is branch-free apart from the DMA predicates: past the last stage the reads fetch
    // LDS bytes nobody uses and the barrier is one too many, both harmless and cheaper than a second
    // copy of the MFMA code.
    for (int t = 0; t < T; t++) {
        int tb, half;
        bool ok_b;
        // slice 0: multiply it, read slice 1, issue the second half of what stage t-1 started (stage 1 came whole)
        b_target(t - 1, tb, half, ok_b);
        slice_step(I0{}, I1{}, DH{}, DR{}, t, t + 1, t >= 1 && t + 1 < T, tb, half, t >= 1 && ok_b);
        slice_step(I1{}, I2{}, I0{}, I0{}, t, 0, false, 0, 0, false);
        slice_step(I2{}, I3{}, I0{}, I0{}, t, 0, false, 0, 0, false);
        // everything issued so far has landed (the youngest of it a whole stage ago) and every read of stage t
        // has returned
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // slice 3: multiply it, read slice 0 of stage t+1, issue the first half of this stage's list
        b_target(t, tb, half, ok_b);
        slice_step(I3{}, I0{}, I0{}, DH{}, t + 1, t + 2, t + 2 < T, tb, half, ok_b);
    }

    out_t *Cb = C + batch * (long)g.M * g.N;
    const bool vec_ok = (g.N & 3) == 0;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
            store_tile32<Cfg::OUT>(Cb, acc[i][j], m0 + wave_m * TM * 32 + i * 32 + lr, n0 + wave_n * TN * 32 + j * 32, lh,
                                   g.M, g.N, vec_ok);
}

template <class Cfg> int launch_pipe(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    static bool configured = false;  // benign race: the attribute call is idempotent
    auto kernel = mfma_pipe_kernel<Cfg>;
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

// K a whole number of 128-byte stages; the row-dense layouts exist for 8- and 16-bit types and fetch whole
// 16-byte chunks of a k-row; alignment is what pick_mode already established
template <int CK> bool pipe_eligible(int la, int lb, const DevProduct &g) {
    constexpr int ES = Compute<CK>::ES;
    if (g.K <= 0 || ((long)g.K * ES) % P_ROW_BYTES != 0) return false;
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
    if (((uintptr_t)b + (uintptr_t)g.b_off) % 16 != 0) return false;
    for (int d = 0; d < g.nb; d++)
        if (g.b_bs[d] % 16 != 0) return false;
    if (lb == LM_K) return g.K % 128 == 0 && (g.N == 1 || g.b_n % 16 == 0);
    return g.N >= 16 && g.N % 16 == 0 && g.b_k % 16 == 0;
}

}  // namespace mfma
}  // namespace hodu
