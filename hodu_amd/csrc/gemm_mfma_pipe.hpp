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
// Hazards.  The barrier in stage t is reached by a wavefront only after all its reads of stage t
// have RETURNED (lgkmcnt(0)) and its own share of stage t+1 has landed (vmcnt(0)); past it, stage t's
// buffer is dead for everybody and stage t+1 is complete for everybody.
#pragma once

#include <type_traits>

#include "gemm_mfma.hpp"

namespace hodu {
namespace mfma {

constexpr int P_ROW_BYTES = 128;   // == ROW_BYTES of the swizzled layout
constexpr int P_SLICES = 4;        // 32-byte k-slices per stage

// s_waitcnt immediate for gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
constexpr int waitcnt_vm(int n) { return (n & 15) | 0x70 | 0xF00 | ((n >> 4) << 14); }
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | 0x70 | ((n >> 4) << 14); }

template <int CK_, int OUT_, int BM_, int BN_, int WM_, int WN_, int LA_ = LM_K, int LB_ = LM_K> struct PipeConfig {
    static constexpr int CK = CK_, OUT = OUT_, BM = BM_, BN = BN_, WM = WM_, WN = WN_, LA = LA_, LB = LB_;
    static constexpr int NT = WM * WN * 64, NW = WM * WN;
    static constexpr int ES = Compute<CK>::ES;
    static constexpr int BK = P_ROW_BYTES / ES;
    // k-dense: 8-row blocks of 1 KB, 128 bytes apart; row-dense: [64 k][ROWS] with no gaps
    static constexpr int A_BYTES = (BM / 8) * (LA == LM_K ? SWZ_BLOCK : 1024);
    static constexpr int B_BYTES = (BN / 8) * (LB == LM_K ? SWZ_BLOCK : 1024);
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int BLOCKS = (BM + BN) / 8;     // DMA instructions per stage
    static constexpr int DMA_PER_WAVE = BLOCKS / NW;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;  // 32x32 MFMA tiles per wave
    static_assert(P_ROW_BYTES == ROW_BYTES, "the pipelined kernel uses the swizzled 128-byte-row layout");
    static_assert(BLOCKS % NW == 0 && (BM / 8) % NW == 0, "DMA split");
    static_assert((LA == LM_K || (ES <= 2 && BM >= 128)) && (LB == LM_K || (ES <= 2 && BN >= 128)),
                  "row-dense operands: 8- and 16-bit types, tiles of at least 128 rows");
    static_assert(DMA_PER_WAVE * 2 < 64, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
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
template <int ES> __device__ __forceinline__ u32x2_t lds_get_tr(const char *lds, int off) {
    if constexpr (ES == 2) {
        typedef short s16x4_t __attribute__((ext_vector_type(4)));
        typedef s16x4_t __attribute__((address_space(3))) * lds_ptr_t;
        return bitcast<u32x2_t>(__builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)(lds + off)));
    } else {
        typedef int i32x2_t __attribute__((ext_vector_type(2)));
        typedef i32x2_t __attribute__((address_space(3))) * lds_ptr_t;
        return bitcast<u32x2_t>(__builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr_t)(uintptr_t)(lds + off)));
    }
}

// Row-dense operand geometry for element size ES (1 or 2 bytes); a "chunk" is 16 bytes of one k-row.
//   swizzle   chunk c of k-row k sits at slot c ^ swz(k); one transpose read takes its 16 lanes through
//             RPT consecutive k-rows, 32 (ES = 2) or 16 (ES = 1) bytes of each, and the swizzle puts those rows
//             into different banks
template <int ES> struct RowDenseGeom {
    static constexpr int RPT = ES == 2 ? 4 : 8;          // k-rows one transpose read covers
    static constexpr int EPC = 16 / ES;                   // elements per chunk
    static constexpr int STAGE_K = 128 / ES;              // k-rows per stage
    static constexpr int SLICE_K = 32 / ES;               // k per MFMA slice
    static __device__ __forceinline__ int swz(int k) { return ES == 2 ? (k & 3) << 2 : (k & 7); }
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                            typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                            int tiles_m, int tiles_n) {
    extern __shared__ __align__(16) char smem[];
    typedef Compute32<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, ES = Cfg::ES, P = Cfg::DMA_PER_WAVE;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int lr = lane & 31, lh = lane >> 5;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

    // ---- DMA plan of this wavefront: P instructions per stage, each one 1 KB of LDS ----
    // k-dense operand: a block of 8 rows x 128 B; lane -> (row in block, slot), the slot holds chunk slot ^ row.
    // row-dense operand: KPI consecutive k-rows of ROWS elements; lane -> (k-row, slot), slot holds chunk
    // slot ^ ((k % 4) << 2); a chunk that starts past the operand's last row is fetched from the last
    // whole chunk instead (its columns are never stored).
    constexpr int PA = (Cfg::BM / 8) / Cfg::NW;  // the first PA instructions of a wavefront belong to A
    const char *gp[P];       // source address of this lane for stage 0
    unsigned lds_off[P];     // block offset inside a stage (wave-uniform)
#pragma unroll
    for (int p = 0; p < P; p++) {
        if (p < PA) {
            const int q = p * Cfg::NW + wave;
            if constexpr (Cfg::LA == LM_K) {
                const int drow = lane >> 3, dchunk = (lane & 7) ^ drow;
                int row = m0 + q * 8 + drow;
                row = row < g.M ? row : g.M - 1;
                gp[p] = A + (ao + (long)row * g.a_m) * ES + dchunk * 16;
                lds_off[p] = q * SWZ_BLOCK;
            } else {
                typedef RowDenseGeom<ES> RD;
                constexpr int CPR = Cfg::BM / RD::EPC, KPI = 64 / CPR;  // chunks per k-row, k-rows per instruction
                const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ RD::swz(k);
                int col = m0 + c * RD::EPC;
                col = col <= g.M - RD::EPC ? col : g.M - RD::EPC;
                gp[p] = A + (ao + (long)k * g.a_k + col) * ES;
                lds_off[p] = q * 1024;
            }
        } else {
            const int q = (p - PA) * Cfg::NW + wave;
            if constexpr (Cfg::LB == LM_K) {
                const int drow = lane >> 3, dchunk = (lane & 7) ^ drow;
                int row = n0 + q * 8 + drow;
                row = row < g.N ? row : g.N - 1;
                gp[p] = B + (bo + (long)row * g.b_n) * ES + dchunk * 16;
                lds_off[p] = Cfg::A_BYTES + q * SWZ_BLOCK;
            } else {
                typedef RowDenseGeom<ES> RD;
                constexpr int CPR = Cfg::BN / RD::EPC, KPI = 64 / CPR;
                const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ RD::swz(k);
                int col = n0 + c * RD::EPC;
                col = col <= g.N - RD::EPC ? col : g.N - RD::EPC;
                gp[p] = B + (bo + (long)k * g.b_k + col) * ES;
                lds_off[p] = Cfg::A_BYTES + q * 1024;
            }
        }
    }
    // bytes a stage advances each operand's source by: 128 bytes of k, or 64 k-rows
    const long a_adv = Cfg::LA == LM_K ? P_ROW_BYTES : P_ROW_BYTES * g.a_k;
    const long b_adv = Cfg::LB == LM_K ? P_ROW_BYTES : P_ROW_BYTES * g.b_k;
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    auto issue = [&](int t) {
        const unsigned stage = lds0 + (unsigned)(t & 1) * Cfg::STAGE_BYTES;
#pragma unroll
        for (int p = 0; p < P; p++)
            dma16_raw(gp[p] + t * (p < PA ? a_adv : b_adv), __builtin_amdgcn_readfirstlane(stage + lds_off[p]));
    };

    // ---- fragment addresses ----
    // k-dense: lane (lr, lh) reads chunk 2*s + lh of row lr of a 32-row tile (four consecutive 8-row
    // blocks); the chunk sits at slot chunk ^ (row % 8) of its row.
    // row-dense: lane (lr, lh) needs the 16 bytes of k that start at k = SLICE_K * s + (SLICE_K / 2) * lh, of
    // row lr.  Two transpose reads of RPT k-rows each deliver them; for both the lane supplies the
    // address of its share of k-row (that start) + RPT * e + kq, columns of its 16-column half of the tile.
    // (k % RPT) == kq whatever s and e are, so the swizzle is a per-lane constant and the slice / half offsets
    // are immediates.
    const int frag_row = (lr >> 3) * SWZ_BLOCK + (lr & 7) * P_ROW_BYTES;
    typedef RowDenseGeom<ES> RD;
    const int s16 = lane & 15;
    const int kq = ES == 2 ? s16 >> 2 : s16 >> 1;                         // k-row within a transpose read
    const int sub = ES == 2 ? (s16 & 3) : (s16 & 1);                      // 8-byte piece within the 16 columns
    const int col_bytes = ((lane >> 4) & 1) * 16 * ES + sub * 8;          // of this lane's address, inside the tile
    int a_frag[P_SLICES], b_frag[P_SLICES];  // k-dense: one address per slice, tiles are immediates
    int a_mn[TM], b_mn[TN];                  // row-dense: one address per tile, slices are immediates
#pragma unroll
    for (int sl = 0; sl < P_SLICES; sl++) {
        const int slot = ((2 * sl + lh) ^ (lr & 7)) << 4;
        a_frag[sl] = (wave_m * TM) * 4 * SWZ_BLOCK + frag_row + slot;
        b_frag[sl] = Cfg::A_BYTES + (wave_n * TN) * 4 * SWZ_BLOCK + frag_row + slot;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int bytes = (wave_m * TM + i) * 32 * ES + col_bytes, c = bytes >> 4;
        a_mn[i] = (lh * (RD::SLICE_K / 2) + kq) * Cfg::BM * ES + ((c ^ RD::swz(kq)) << 4) + (bytes & 8);
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int bytes = (wave_n * TN + j) * 32 * ES + col_bytes, c = bytes >> 4;
        b_mn[j] = Cfg::A_BYTES + (lh * (RD::SLICE_K / 2) + kq) * Cfg::BN * ES + ((c ^ RD::swz(kq)) << 4) + (bytes & 8);
    }
    auto read_a = [&](const char *stage, auto sl_, int i) -> u32x4_t {
        constexpr int SL = decltype(sl_)::value;
        if constexpr (Cfg::LA == LM_K) {
            return lds_get(stage, a_frag[SL] + i * 4 * SWZ_BLOCK);
        } else {
            const u32x2_t lo = lds_get_tr<ES>(stage, a_mn[i] + (SL * RD::SLICE_K) * Cfg::BM * ES);
            const u32x2_t hi = lds_get_tr<ES>(stage, a_mn[i] + (SL * RD::SLICE_K + RD::RPT) * Cfg::BM * ES);
            return u32x4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    auto read_b = [&](const char *stage, auto sl_, int j) -> u32x4_t {
        constexpr int SL = decltype(sl_)::value;
        if constexpr (Cfg::LB == LM_K) {
            return lds_get(stage, b_frag[SL] + j * 4 * SWZ_BLOCK);
        } else {
            const u32x2_t lo = lds_get_tr<ES>(stage, b_mn[j] + (SL * RD::SLICE_K) * Cfg::BN * ES);
            const u32x2_t hi = lds_get_tr<ES>(stage, b_mn[j] + (SL * RD::SLICE_K + RD::RPT) * Cfg::BN * ES);
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

    const int T = g.K * ES / P_ROW_BYTES;

    // One k-slice of work, in an explicitly pinned order: the MFMAs of slice CUR (register set CUR % 2),
    // with the fragment reads of slice RD of stage t_rd (RD < 0: none) and DMA instructions
    // [D0, D0 + DN) of stage t_dma spread evenly between them.  Neither the reads nor the DMA then
    // arrive in bursts: a burst of DMA instructions fills the memory pipeline's issue queue and
    // stalls the wavefront in front of its next MFMA.
    auto slice_step = [&](auto cur_, auto rd_, auto d0_, auto dn_, int t_rd, int t_dma, bool do_dma) {
        constexpr int SET = decltype(cur_)::value & 1, RD = decltype(rd_)::value;
        constexpr int D0 = decltype(d0_)::value, DN = decltype(dn_)::value;
        constexpr int MF = TM * TN, RN = RD >= 0 ? TM + TN : 0;
        const char *stage_rd = smem + (t_rd & 1) * Cfg::STAGE_BYTES;
        const unsigned stage_dma = lds0 + (unsigned)(t_dma & 1) * Cfg::STAGE_BYTES;
#pragma unroll
        for (int idx = 0; idx < MF; idx++) {
#pragma unroll
            for (int r = 0; r < RN; r++) {
                if (r * MF / (RN > 0 ? RN : 1) != idx) continue;
                typedef std::integral_constant<int, (RD >= 0 ? RD : 0)> RS;
                if (r < TM) fa[RS::value & 1][r] = read_a(stage_rd, RS{}, r);
                else fb[RS::value & 1][r - TM] = read_b(stage_rd, RS{}, r - TM);
            }
            // operands swapped: the accumulator then holds, per lane, runs of 4 consecutive n of one m
            Cmp::mma(fb[SET][idx / TM], fa[SET][idx % TM], acc[idx % TM][idx / TM]);
#pragma unroll
            for (int d = 0; d < DN; d++) {
                if (d * MF / (DN > 0 ? DN : 1) != idx) continue;
                if (do_dma)
                    dma16_raw(gp[D0 + d] + t_dma * (D0 + d < PA ? a_adv : b_adv),
                              __builtin_amdgcn_readfirstlane(stage_dma + lds_off[D0 + d]));
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

    issue(0);
    if (T > 1) {
        issue(1);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(P));
    } else {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < TM; i++) fa[0][i] = read_a(smem, I0{}, i);
#pragma unroll
    for (int j = 0; j < TN; j++) fb[0][j] = read_b(smem, I0{}, j);

    // The loop body is branch-free apart from the DMA predicates: past the last stage the reads fetch
    // LDS bytes nobody uses and the barrier is one too many, both harmless and cheaper than a second
    // copy of the MFMA code.
    for (int t = 0; t < T; t++) {
        // slice 0: multiply it, read slice 1, issue the second half of stage t+1's DMA (stage 1 came whole)
        slice_step(I0{}, I1{}, DH{}, DR{}, t, t + 1, t >= 1 && t + 1 < T);
        slice_step(I1{}, I2{}, I0{}, I0{}, t, 0, false);
        slice_step(I2{}, I3{}, I0{}, I0{}, t, 0, false);
        // stage t+1 (the only DMA in flight) has landed and every read of stage t has returned
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // slice 3: multiply it, read slice 0 of stage t+1, issue the first half of stage t+2's DMA
        slice_step(I3{}, I0{}, I0{}, DH{}, t + 1, t + 2, t + 2 < T);
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

}  // namespace mfma
}  // namespace hodu
