// The pipelined tile kernel of gemm_mfma_pipe.hpp on the 16 x 16 x 32 matrix instruction, for 16-bit operands, k-dense
// or row-dense.  Same feeding scheme -- whole 128-byte rows by LDS-DMA into a two-stage ring, source-side XOR swizzle,
// one barrier per 64-k stage, the tile leaving through LDS as whole rows -- and the same sums in the same order per
// output (k ascending in blocks of 32 instead of 16, which an f32 accumulator of exact products does not see; the
// bit-for-bit tests on exact-valued operands hold both variants to one result).
//
// Why a second instruction shape: the part is power-limited on large products, and from registers alone the
// 16 x 16 x 32 instruction sustains 1.89-1.95 PFLOP/s at 1.9-2.0 GHz on N(0,1) bf16 operands where the 32 x 32 x 16 one
// sustains 1.77-1.78 at 1.68 GHz (hodu_rocm_debug_mfma_clock, kinds 2 and 0): a quarter of the accumulator registers
// move per instruction, and the clock the power limit leaves is a fifth higher.
//
// What differs from the 32 x 32 kernel:
//   * a wavefront's 128 x 128 outputs are 8 x 8 accumulators of 4 registers; a fragment is 16 rows x 32 k, 16 bytes per
//     lane: lane (r = lane % 16, g = lane / 16) reads chunk 4 * slice + g of row r, one ds_read_b128 (k-dense), or
//     takes its 8 k of column r out of the k-major stage through two transpose reads of 4 k-rows each (row-dense);
//   * a stage is TWO slices of 32 k, 64 MFMAs of 16 cycles each.  Slice 0 multiplies while the 16 fragments of slice 1
//     are read (all issued in its first three quarters, so that they have returned at the barrier that follows it);
//     behind the barrier slice 1 multiplies while the next stage's slice 0 is read and the whole DMA list of the
//     stage after that goes out, one instruction every third to sixth MFMA, into the buffer the barrier has just
//     freed: it has more than a slice to land;
//   * the epilogue stages bands of 16 rows.
#pragma once

#include "gemm_mfma_pipe.hpp"

namespace hodu {
namespace mfma {

// f(integral_constant<int, 0>) .. f(integral_constant<int, N - 1>), in order: a loop whose index is a constant expression
template <int N, int I = 0, class F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

// (the instruction itself, with its accumulator tied: gfx950_insn.hpp)
template <int CK> struct Compute16;
template <> struct Compute16<CK_BF16> {
    typedef f32x4_acc_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        mfma16x16x32_bf16(a, b, c);
    }
};
template <> struct Compute16<CK_F16> {
    typedef f32x4_acc_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        mfma16x16x32_f16(a, b, c);
    }
};

// Row-dense stages: chunk c of k-row k sits at slot c ^ rd16_swz(k).  A transpose read is served 32 lanes at a time;
// the two groups of 16 among them read k-rows 8 apart, columns alike, so besides the (k % 4) << 2 that spreads the
// four k-rows of one group, bit 3 of k moves a row by two chunks (32 bytes): the 32 lanes then touch every bank once.
__device__ __forceinline__ int rd16_swz(int k) { return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1); }

// Cfg: a PipeConfig with operands stored in the compute type and a ring of two stages
template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe16_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                              typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                              int tiles_m, int tiles_n) {
    static_assert(!Cfg::B_F8 && Cfg::ES == 2 && Cfg::NST == 2, "16-bit operands stored in the compute type, two stages");
    typedef RowDenseGeom<Cfg::ES, Cfg::ES> G;
    HODU_DYNAMIC_LDS(smem);
    typedef Compute16<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int ES = Cfg::ES, PA = Cfg::PA, PB = Cfg::PB, P = PA + PB;
    constexpr int TM = Cfg::BM / Cfg::WM / 16, TN = Cfg::BN / Cfg::WN / 16;  // 16 x 16 accumulators per wavefront
    constexpr int MF = TM * TN, RN = TM + TN;
    static_assert(3 * RN + 1 <= MF, "a slice has a gap for every fragment read");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int r16 = lane & 15, g4 = lane >> 4;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

    // LDS: two stages of A, then two of B
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    constexpr int B_BASE = 2 * Cfg::A_BYTES;

    // DMA plan of this wavefront, as in mfma_pipe_kernel: an instruction writes 8 rows x 128 bytes; lane -> (row,
    // slot), the slot holds chunk slot ^ ((row >> 1) & 7); rows past the operand's last one re-fetch the last one
    // (their outputs are never stored).  Address = scalar base of the tile's first row, advanced 128 bytes per stage,
    // plus the lane's 32-bit byte offset inside the tile (the launcher checks that 256 rows stay below 4 GB).
    unsigned offa[PA], offb[PB];
    unsigned lda[PA], ldb[PB];
    // row-dense operand: an instruction writes KPI consecutive k-rows of the tile's ROWS contiguous elements; lane ->
    // (k-row, slot), the slot holds chunk slot ^ swz(k); a chunk that starts past the operand's last row is fetched
    // from the last whole chunk instead (its columns are never stored), and the scalar base is the tile's first
    // (clamped) column of k-row 0, advanced by a stage's k-rows per stage.
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = p * Cfg::NW + wave;
        if constexpr (Cfg::LA == LM_K) {
            const int trow = q * 8 + (lane >> 3), dchunk = kd_slot(trow, lane & 7);
            int row = m0 + trow;
            row = row < g.M ? row : g.M - 1;
            offa[p] = (unsigned)((long)(row - m0) * g.a_m * ES) + dchunk * 16;
        } else {
            constexpr int CPR = Cfg::BM / G::EPC, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ rd16_swz(k);
            int col = m0 + c * G::EPC;
            col = col <= g.M - G::EPC ? col : g.M - G::EPC;
            offa[p] = (unsigned)(((long)k * g.a_k + (col - (m0 <= g.M - G::EPC ? m0 : g.M - G::EPC))) * ES);
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
            offb[p] = (unsigned)((long)(row - n0) * g.b_n * ES) + dchunk * 16;
        } else {
            constexpr int CPR = Cfg::BN / G::EPC, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ rd16_swz(k);
            int col = n0 + c * G::EPC;
            col = col <= g.N - G::EPC ? col : g.N - G::EPC;
            offb[p] = (unsigned)(((long)k * g.b_k + (col - (n0 <= g.N - G::EPC ? n0 : g.N - G::EPC))) * ES);
        }
        ldb[p] = B_BASE + q * 1024;
    }
    const int T = g.K * ES / P_ROW_BYTES;  // stages
    const char *const base_a = uniform_ptr(Cfg::LA == LM_K ? A + (ao + (long)m0 * g.a_m) * ES
                                                           : A + (ao + (m0 <= g.M - G::EPC ? m0 : g.M - G::EPC)) * ES);
    const char *const base_b = uniform_ptr(Cfg::LB == LM_K ? B + (bo + (long)n0 * g.b_n) * ES
                                                           : B + (bo + (n0 <= g.N - G::EPC ? n0 : g.N - G::EPC)) * ES);
    // bytes a stage advances an operand's source by: 128 bytes of k, or a stage's k-rows
    const long a_adv = Cfg::LA == LM_K ? P_ROW_BYTES : (long)G::STAGE_K * g.a_k * ES;
    const long b_adv = Cfg::LB == LM_K ? P_ROW_BYTES : (long)G::STAGE_K * g.b_k * ES;

    // element e of the list that fetches stage `src` (already clamped to T - 1) into ring slot `slot`
    auto dma_element = [&](int e, int src, int slot) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (e == p) dma16_sbase(base_a + src * a_adv, offa[p], lds0 + (unsigned)slot * Cfg::A_BYTES + lda[p]);
#pragma unroll
        for (int p = 0; p < PB; p++)
            if (e == PA + p) dma16_sbase(base_b + src * b_adv, offb[p], lds0 + (unsigned)slot * Cfg::B_BYTES + ldb[p]);
    };

    // fragment addresses.  k-dense: lane (r16, g4) reads chunk 4 * slice + g4 of row r16 of a 16-row tile; every tile
    // starts on a multiple of 16 rows, so the swizzle term (row >> 1) & 7 is the lane's own, and the tiles are
    // immediates.  row-dense: the lane needs k = 32 * slice + 8 * g4 .. + 7 of column r16 of the tile; a transpose
    // read hands each of 16 lanes 4 consecutive k of its own column out of 4 k-rows, for which lane s of the 16
    // supplies the address of 4 columns (8 bytes) of k-row (that start) + s / 4.  k % 4 == s / 4 and bit 3 of k is
    // bit 0 of g4 whatever the slice and the half, so the swizzle is a per-lane constant and slices and halves are immediates; tiles are not (the
    // swizzle is an XOR on the chunk index), so there is an address per tile.
    constexpr int TILE_BYTES = 16 * P_ROW_BYTES;
    int a_frag[2], b_frag[2];
#pragma unroll
    for (int sl = 0; sl < 2; sl++) {
        const int at = r16 * P_ROW_BYTES + (kd_slot(r16, 4 * sl + g4) << 4);
        a_frag[sl] = (wave_m * TM) * TILE_BYTES + at;
        b_frag[sl] = B_BASE + (wave_n * TN) * TILE_BYTES + at;
    }
    int a_mn[TM], b_mn[TN];
    {
        const int kq = r16 >> 2, sub = r16 & 3;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int bytes = (wave_m * TM + i) * 16 * ES + sub * 8, c = bytes >> 4;
            a_mn[i] = (g4 * 8 + kq) * Cfg::BM * ES + ((c ^ rd16_swz(g4 * 8 + kq)) << 4) + (bytes & 8);
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int bytes = (wave_n * TN + j) * 16 * ES + sub * 8, c = bytes >> 4;
            b_mn[j] = B_BASE + (g4 * 8 + kq) * Cfg::BN * ES + ((c ^ rd16_swz(g4 * 8 + kq)) << 4) + (bytes & 8);
        }
    }
    u32x4_t fa[2][TM], fb[2][TN];  // [slice][tile]
    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = acc_t{0.f, 0.f, 0.f, 0.f};

    // the r-th fragment read of slice SL from ring slot `slot`, in the order of first use: the left operand's tiles,
    // then the right operand's
    auto read_fragment = [&](auto sl_, int r, int slot) {
        constexpr int SL = decltype(sl_)::value;
        if (r < TM) {
            const char *buf = smem + slot * Cfg::A_BYTES;
            if constexpr (Cfg::LA == LM_K) {
                fa[SL][r] = lds_get(buf, a_frag[SL] + r * TILE_BYTES);
            } else {
                const u32x2_t lo = lds_get_tr<ES>(buf, a_mn[r] + (SL * 32) * Cfg::BM * ES);
                const u32x2_t hi = lds_get_tr<ES>(buf, a_mn[r] + (SL * 32 + 4) * Cfg::BM * ES);
                fa[SL][r] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
            }
        } else {
            const char *buf = smem + slot * Cfg::B_BYTES;
            if constexpr (Cfg::LB == LM_K) {
                fb[SL][r - TM] = lds_get(buf, b_frag[SL] + (r - TM) * TILE_BYTES);
            } else {
                const u32x2_t lo = lds_get_tr<ES>(buf, b_mn[r - TM] + (SL * 32) * Cfg::BN * ES);
                const u32x2_t hi = lds_get_tr<ES>(buf, b_mn[r - TM] + (SL * 32 + 4) * Cfg::BN * ES);
                fb[SL][r - TM] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
            }
        }
    };
    // One slice of work in a pinned order: the MFMAs of slice CUR with the reads of slice 1 - CUR (from ring slot
    // rd_slot) and, in slice 1 -- behind the barrier --, the DMA list between them.  A read goes behind MFMAs 1, 4, 7, ..,
    // so that the last one is out a quarter of a slice before the slice ends (in slice 0 the barrier's wait for the
    // reads follows, in slice 1 the loop's back edge, where the compiler waits for every read in flight); a DMA
    // instruction goes behind one of the MFMAs 3, 6, 9, .., never into the gap that already took a read.
    auto slice_step = [&](auto cur_, int rd_slot, int dma_src, int dma_slot) {
        constexpr int CUR = decltype(cur_)::value;
        typedef std::integral_constant<int, 1 - CUR> RS;
        constexpr int DSLOTS = (MF - 4) / 3;
        static_assert(DSLOTS >= P, "a gap of its own for every DMA instruction");
#pragma unroll
        for (int idx = 0; idx < MF; idx++) {
            // operands swapped: a lane's accumulator then holds 4 consecutive n of one m
            Cmp::mma(fb[CUR][idx / TM], fa[CUR][idx % TM], acc[idx % TM][idx / TM]);
            if (idx % 3 == 1 && idx / 3 < RN) read_fragment(RS{}, idx / 3, rd_slot);
            if constexpr (CUR == 1) {
#pragma unroll
                for (int d = 0; d < P; d++)
                    if (3 * (1 + d * DSLOTS / P) == idx) dma_element(d, dma_src, dma_slot);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    // prologue: stage 0 into slot 0, stage 1 (or stage 0 again) into slot 1
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int src = j < T ? j : T - 1;
#pragma unroll
        for (int e = 0; e < P; e++) dma_element(e, src, j);
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(P));  // slot 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < RN; r++) read_fragment(I0{}, r, 0);

    // Past the last stage the reads fetch LDS bytes nobody uses and the list re-fetches the last stage into a buffer
    // nobody reads: both harmless, and the number of instructions in flight stays what the waits assume.
    int slot = 0;
    for (int t = 0; t < T; t++) {
        slice_step(I0{}, slot, 0, 0);
        // stage t + 1 has landed (its list went out a slice and a half ago) and every read of stage t has returned
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        slice_step(I1{}, slot ^ 1, t + 2 < T ? t + 2 : T - 1, slot);
        slot ^= 1;
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // the re-fetches of the last stages are still writing LDS
    mfma_results_settle();                      // the accumulators are read next
    __syncthreads();

    // epilogue: bands of 16 rows through a wavefront-private patch of LDS
    char *patch = smem + wave * (16 * (TN * 16 * 4 + 16));
    out_t *Cb = C + batch * (long)g.M * g.N;
    EpiPrepared<Out<Cfg::OUT>::DT, 16 / (int)sizeof(out_t)> steps{};
    if (g.epi.n != 0) steps = band_columns_prepare<Cfg::OUT, TN, 16>(g.epi, n0 + wave_n * TN * 16, lane, g.N);
#pragma unroll
    for (int i = 0; i < TM; i++)
        store_band_via_lds<Cfg::OUT, TN, true, acc_t, 16, true>(patch, Cb, acc[i], m0 + (wave_m * TM + i) * 16, n0 + wave_n * TN * 16, lane,
                                                                g.M, g.N, g.epi, steps);
}

// ---------------------------------------------------------------------------------------------------------------
// The same kernel with the loop's non-MFMA instructions spaced by issue slots.
//
// One wavefront per SIMD issues everything in order, one instruction per four cycles; a 16 x 16 x 32 MFMA occupies
// the matrix core for 16, so a gap between two MFMAs has room for three other instructions and every one beyond
// that idles the matrix core for four cycles.  What the first kernel spent there: each LDS-DMA instruction with its
// own M0 computation and write (s_add, s_mov m0, s_nop, load: four slots in one gap), and the compiler's address
// arithmetic for sixteen of them gathered in a single gap.  Here
//   * a wavefront's DMA instructions of an operand write 1 KB pieces that lie 1 KB apart in LDS, so the instruction's
//     immediate offset (added to the global AND the LDS address) steps through four of them under one M0 value: the
//     lane's global offset carries the opposite of that step, and base pointer and lane offsets are biased by 4 KB so
//     that no offset goes below zero.  Four M0 writes per stage instead of sixteen, each a single s_add_u32 of a
//     literal to a per-wavefront base, placed one gap ahead of the first load that needs it;
//   * the stage loop is unrolled by two with the ring slot a literal, so every LDS address of a fragment read is an
//     immediate on one of four registers and no M0 value needs arithmetic;
//   * the source pointers advance by one add per operand and stage; the last two stages, which fetch nothing, are
//     a copy of the loop body without the DMA list instead of re-fetching a clamped stage.
// Needs an even number of stages (K a multiple of 128 elements), at least two; anything else takes the first kernel.
// an even number of 128-byte stages, at least two
inline bool pipe16r_stages_ok(long K, int elem_bytes) { return K > 0 && (K * elem_bytes) % (2 * P_ROW_BYTES) == 0; }

// STEPS: the instantiation that applies fused element-wise steps where the rows leave (the plain product's carries
// none of their registers)
template <class Cfg, bool STEPS>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe16r_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                               typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                               int tiles_m, int tiles_n) {
    static_assert(!Cfg::B_F8 && Cfg::ES == 2 && Cfg::NST == 2, "16-bit operands stored in the compute type, two stages");
    typedef RowDenseGeom<Cfg::ES, Cfg::ES> G;
    HODU_DYNAMIC_LDS(smem);
    typedef Compute16<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int ES = Cfg::ES, PA = Cfg::PA, PB = Cfg::PB, P = PA + PB;
    constexpr int TM = Cfg::BM / Cfg::WM / 16, TN = Cfg::BN / Cfg::WN / 16;
    constexpr int MF = TM * TN, RN = TM + TN;
    constexpr int GRP = 4, BIAS = 4096;  // DMA instructions per M0 value; what keeps the lane offsets non-negative
    static_assert(PA % GRP == 0 && PB % GRP == 0 && 3 * RN + 1 <= MF, "DMA groups of four; a gap for every fragment read");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int r16 = lane & 15, g4 = lane >> 4;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

    // LDS: two stages of A, then two of B.  Piece q (1 KB: 8 rows of 128 bytes, or KPI k-rows of a row-dense tile) of
    // a stage is fetched by wavefront q / PA as its instruction q % PA.
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    constexpr int B_BASE = 2 * Cfg::A_BYTES;
    unsigned offa[PA], offb[PB];
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = wave * PA + p;
        unsigned off;
        if constexpr (Cfg::LA == LM_K) {
            const int trow = q * 8 + (lane >> 3), dchunk = kd_slot(trow, lane & 7);
            int row = m0 + trow;
            row = row < g.M ? row : g.M - 1;
            off = (unsigned)((long)(row - m0) * g.a_m * ES) + dchunk * 16;
        } else {
            constexpr int CPR = Cfg::BM / G::EPC, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ rd16_swz(k);
            int col = m0 + c * G::EPC;
            col = col <= g.M - G::EPC ? col : g.M - G::EPC;
            off = (unsigned)(((long)k * g.a_k + (col - (m0 <= g.M - G::EPC ? m0 : g.M - G::EPC))) * ES);
        }
        offa[p] = off + BIAS - (p % GRP) * 1024;
    }
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int q = wave * PB + p;
        unsigned off;
        if constexpr (Cfg::LB == LM_K) {
            const int trow = q * 8 + (lane >> 3), dchunk = kd_slot(trow, lane & 7);
            int row = n0 + trow;
            row = row < g.N ? row : g.N - 1;
            off = (unsigned)((long)(row - n0) * g.b_n * ES) + dchunk * 16;
        } else {
            constexpr int CPR = Cfg::BN / G::EPC, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ rd16_swz(k);
            int col = n0 + c * G::EPC;
            col = col <= g.N - G::EPC ? col : g.N - G::EPC;
            off = (unsigned)(((long)k * g.b_k + (col - (n0 <= g.N - G::EPC ? n0 : g.N - G::EPC))) * ES);
        }
        offb[p] = off + BIAS - (p % GRP) * 1024;
    }
    const unsigned wbase_a = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)wave * (PA * 1024));
    const unsigned wbase_b = __builtin_amdgcn_readfirstlane(lds0 + B_BASE + (unsigned)wave * (PB * 1024));
    const int T = g.K * ES / P_ROW_BYTES;  // stages: even, at least two (the launcher checks)
    const long a_adv = Cfg::LA == LM_K ? P_ROW_BYTES : (long)G::STAGE_K * g.a_k * ES;
    const long b_adv = Cfg::LB == LM_K ? P_ROW_BYTES : (long)G::STAGE_K * g.b_k * ES;
    // source of the stage the next DMA list fetches, less the bias the lane offsets carry
    const char *pa = uniform_ptr((Cfg::LA == LM_K ? A + (ao + (long)m0 * g.a_m) * ES
                                                  : A + (ao + (m0 <= g.M - G::EPC ? m0 : g.M - G::EPC)) * ES) - BIAS);
    const char *pb = uniform_ptr((Cfg::LB == LM_K ? B + (bo + (long)n0 * g.b_n) * ES
                                                  : B + (bo + (n0 <= g.N - G::EPC ? n0 : g.N - G::EPC)) * ES) - BIAS);

    // element d of the DMA list of a stage into ring slot SLOT: the left operand's pieces, then the right one's
    auto dma_element = [&](auto slot_, auto d_) {
        constexpr int SLOT = decltype(slot_)::value, D = decltype(d_)::value;
        if constexpr (D < PA) dma16_imm<(D % GRP) * 1024>(pa, offa[D]);
        else dma16_imm<((D - PA) % GRP) * 1024>(pb, offb[D - PA]);
        (void)SLOT;
    };
    // the M0 value the group of list element d needs
    auto dma_m0 = [&](auto slot_, auto d_) {
        constexpr int SLOT = decltype(slot_)::value, D = decltype(d_)::value;
        if constexpr (D < PA) m0_set<SLOT * Cfg::A_BYTES + (D / GRP) * GRP * 1024>(wbase_a);
        else m0_set<SLOT * Cfg::B_BYTES + ((D - PA) / GRP) * GRP * 1024>(wbase_b);
    };

    constexpr int TILE_BYTES = 16 * P_ROW_BYTES;
    int a_frag[2], b_frag[2];
#pragma unroll
    for (int sl = 0; sl < 2; sl++) {
        const int at = r16 * P_ROW_BYTES + (kd_slot(r16, 4 * sl + g4) << 4);
        a_frag[sl] = (wave_m * TM) * TILE_BYTES + at;
        b_frag[sl] = B_BASE + (wave_n * TN) * TILE_BYTES + at;
    }
    int a_mn[TM], b_mn[TN];
    {
        const int kq = r16 >> 2, sub = r16 & 3;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int bytes = (wave_m * TM + i) * 16 * ES + sub * 8, c = bytes >> 4;
            a_mn[i] = (g4 * 8 + kq) * Cfg::BM * ES + ((c ^ rd16_swz(g4 * 8 + kq)) << 4) + (bytes & 8);
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int bytes = (wave_n * TN + j) * 16 * ES + sub * 8, c = bytes >> 4;
            b_mn[j] = B_BASE + (g4 * 8 + kq) * Cfg::BN * ES + ((c ^ rd16_swz(g4 * 8 + kq)) << 4) + (bytes & 8);
        }
    }
    u32x4_t fa[2][TM], fb[2][TN];  // [slice][tile]
    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = acc_t{0.f, 0.f, 0.f, 0.f};

    // the r-th fragment read of slice SL from ring slot SLOT, in the order of first use
    auto read_fragment = [&](auto sl_, auto slot_, int r) {
        constexpr int SL = decltype(sl_)::value, SLOT = decltype(slot_)::value;
        if (r < TM) {
            const char *buf = smem + SLOT * Cfg::A_BYTES;
            if constexpr (Cfg::LA == LM_K) {
                fa[SL][r] = lds_get(buf, a_frag[SL] + r * TILE_BYTES);
            } else {
                const u32x2_t lo = lds_get_tr<ES>(buf, a_mn[r] + (SL * 32) * Cfg::BM * ES);
                const u32x2_t hi = lds_get_tr<ES>(buf, a_mn[r] + (SL * 32 + 4) * Cfg::BM * ES);
                fa[SL][r] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
            }
        } else {
            const char *buf = smem + SLOT * Cfg::B_BYTES;
            if constexpr (Cfg::LB == LM_K) {
                fb[SL][r - TM] = lds_get(buf, b_frag[SL] + (r - TM) * TILE_BYTES);
            } else {
                const u32x2_t lo = lds_get_tr<ES>(buf, b_mn[r - TM] + (SL * 32) * Cfg::BN * ES);
                const u32x2_t hi = lds_get_tr<ES>(buf, b_mn[r - TM] + (SL * 32 + 4) * Cfg::BN * ES);
                fb[SL][r - TM] = u32x4_t{lo.x, lo.y, hi.x, hi.y};
            }
        }
    };
    // One slice in a pinned order: the MFMAs of slice CUR; behind MFMAs 1, 4, 7, .. a read of slice 1 - CUR from ring
    // slot RSLOT (none when READ is off: the last slice of the tile); in slice 1 with DMA on, list element d behind MFMA
    // 3 * (1 + d * DSLOTS / P) -- a gap that holds nothing else -- and the M0 write of a group of four in the gap
    // before its first element.
    constexpr int DSLOTS = (MF - 4) / 3;
    static_assert(DSLOTS >= P, "a gap of its own for every DMA instruction");
    auto slice_step = [&](auto cur_, auto rslot_, auto read_, auto dma_, auto dslot_) {
        constexpr int CUR = decltype(cur_)::value;
        constexpr bool READ = decltype(read_)::value, DMA = decltype(dma_)::value;
        typedef std::integral_constant<int, 1 - CUR> RS;
        static_for<MF>([&](auto idx_) {
            constexpr int idx = decltype(idx_)::value;
            // operands swapped: a lane's accumulator then holds 4 consecutive n of one m
            Cmp::mma(fb[CUR][idx / TM], fa[CUR][idx % TM], acc[idx % TM][idx / TM]);
            if constexpr (READ && idx % 3 == 1 && idx / 3 < RN) read_fragment(RS{}, rslot_, idx / 3);
            if constexpr (DMA) {
                static_for<P>([&](auto d_) {
                    constexpr int d = decltype(d_)::value;
                    if constexpr (3 * (1 + d * DSLOTS / P) == idx) dma_element(dslot_, d_);
                    if constexpr (d % GRP == 0 && 3 * (1 + d * DSLOTS / P) - 1 == idx) dma_m0(dslot_, d_);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    typedef std::true_type Yes;
    typedef std::false_type No;

    // prologue: stage 0 into slot 0, stage 1 into slot 1
    static_for<2>([&](auto j_) {
        static_for<P>([&](auto d_) {
            constexpr int d = decltype(d_)::value;
            if constexpr (d % GRP == 0) {
                dma_m0(j_, d_);
                m0_wait_state();
            }
            dma_element(j_, d_);
        });
        pa += a_adv;
        pb += b_adv;
    });
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(P));  // slot 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < RN; r++) read_fragment(I0{}, I0{}, r);

    // stage t out of ring slot SLOT: slice 0 multiplies while slice 1's fragments are read; behind the barrier (stage
    // t + 1 has landed, every read of stage t has returned) slice 1 multiplies while the next stage's slice 0 is read
    // from the other slot and, with DMA on, stage t + 2 is sent for into the slot the barrier has just freed
    auto stage = [&](auto slot_, auto dma_, auto last_) {
        constexpr int SLOT = decltype(slot_)::value;
        typedef std::integral_constant<int, 1 - SLOT> Other;
        typedef std::integral_constant<bool, !decltype(last_)::value> ReadNext;
        slice_step(I0{}, slot_, Yes{}, No{}, slot_);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        slice_step(I1{}, Other{}, ReadNext{}, dma_, slot_);
        if constexpr (decltype(dma_)::value) {
            pa += a_adv;
            pb += b_adv;
        }
    };
    for (int t = 0; t + 2 < T; t += 2) {
        stage(I0{}, Yes{}, No{});
        stage(I1{}, Yes{}, No{});
    }
    stage(I0{}, No{}, No{});
    stage(I1{}, No{}, Yes{});
    mfma_results_settle();  // the accumulators are read next
    __syncthreads();

    // epilogue: bands of 16 rows through a wavefront-private patch of LDS
    char *patch = smem + wave * (16 * (TN * 16 * 4 + 16));
    out_t *Cb = C + batch * (long)g.M * g.N;
    if constexpr (STEPS) {
        const auto steps = band_columns_prepare<Cfg::OUT, TN, 16>(g.epi, n0 + wave_n * TN * 16, lane, g.N);
#pragma unroll
        for (int i = 0; i < TM; i++)
            store_band_via_lds<Cfg::OUT, TN, true, acc_t, 16, true>(patch, Cb, acc[i], m0 + (wave_m * TM + i) * 16,
                                                                    n0 + wave_n * TN * 16, lane, g.M, g.N, g.epi, steps);
    } else {
#pragma unroll
        for (int i = 0; i < TM; i++)
            store_band_via_lds<Cfg::OUT, TN, false, acc_t, 16>(patch, Cb, acc[i], m0 + (wave_m * TM + i) * 16,
                                                               n0 + wave_n * TN * 16, lane, g.M, g.N, g.epi);
    }
}

// The same tile with f8e4m3 weights (the fused to_dtype of the right operand): the weight's bytes move as they are and
// are widened to bf16 between the fragment read (8 bytes per lane) and the MFMA, one fragment ahead of its use, in the
// shadow of the MFMAs of the fragment before.
//   k-dense weights ([N, K] bytes): whole 128-byte lines, i.e. 128 k, the k of TWO stages of the bf16 left operand, so
//     a right-operand buffer holds a pair of stages and the ring two pairs.  A pair's buffer is free behind the barrier
//     of the pair's second stage and is needed four stages on, so its refill goes out in two halves, behind that
//     barrier and behind the next one: every stage issues 8 + 4 DMA instructions.
//   row-dense weights ([K, N] bytes): a stage is 64 k-rows of the tile's 256 bytes, in a ring of two like the left
//     operand's (8 + 4 instructions per stage as well); a fragment is one 8-bit transpose read of 8 k-rows.
template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe16_f8w_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                                  typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                                  int tiles_m, int tiles_n) {
    static_assert(Cfg::LA == LM_K && Cfg::B_F8 && Cfg::NST == 2, "bf16 x f8e4m3, the left operand k-dense, two stages");
    HODU_DYNAMIC_LDS(smem);
    typedef Compute16<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr bool PAIR = Cfg::B_PAIR;  // k-dense weights
    constexpr int ES = Cfg::ES, PA = Cfg::PA, PB = Cfg::PB, PBS = Cfg::PBS, P = PA + PBS;
    constexpr int TM = Cfg::BM / Cfg::WM / 16, TN = Cfg::BN / Cfg::WN / 16;
    constexpr int MF = TM * TN;
    static_assert(TM == 8 && TN == 8 && P <= 19, "the schedule below is written for 128 x 128 outputs per wavefront");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int r16 = lane & 15, g4 = lane >> 4;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

    // LDS: two stages of A (64 k of bf16 each), then two buffers of B (k-dense: 128 k each; row-dense: 64 k-rows each)
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    constexpr int B_BASE = 2 * Cfg::A_BYTES;

    // DMA plan.  k-dense: an instruction writes 8 rows x 128 bytes; lane -> (row, slot), the slot holds chunk
    // slot ^ ((row >> 1) & 7); rows past the operand's last one re-fetch the last one.  Address = scalar base of the
    // tile's first row (advanced 128 bytes per stage of A, per pair of B) + the lane's 32-bit offset inside the tile.
    // row-dense weights: an instruction writes 4 k-rows of 256 bytes; lane -> (k-row, slot), the slot holds chunk
    // slot ^ (k % 16) (a transpose read serves 32 lanes at a time, 16 k-rows of 16 bytes: the swizzle spreads them over
    // all banks); a chunk that starts past the last column is fetched from the last whole chunk instead.
    unsigned offa[PA], offb[PB];
    unsigned lda[PA], ldb[PB];
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = p * Cfg::NW + wave, trow = q * 8 + (lane >> 3);
        int row = m0 + trow;
        row = row < g.M ? row : g.M - 1;
        offa[p] = (unsigned)((long)(row - m0) * g.a_m * ES) + kd_slot(trow, lane & 7) * 16;
        lda[p] = q * 1024;
    }
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int q = p * Cfg::NW + wave;
        if constexpr (PAIR) {
            const int trow = q * 8 + (lane >> 3);
            int row = n0 + trow;
            row = row < g.N ? row : g.N - 1;
            offb[p] = (unsigned)((long)(row - n0) * g.b_n) + kd_slot(trow, lane & 7) * 16;
        } else {
            constexpr int CPR = Cfg::BN / 16, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ (k & 15);
            int col = n0 + c * 16;
            col = col <= g.N - 16 ? col : g.N - 16;
            offb[p] = (unsigned)((long)k * g.b_k + (col - (n0 <= g.N - 16 ? n0 : g.N - 16)));
        }
        ldb[p] = B_BASE + q * 1024;
    }
    const int T = g.K * ES / P_ROW_BYTES;  // stages (k-dense weights: even, K is a multiple of 128)
    const int TB = PAIR ? T / 2 : T;       // right-operand buffers' worth of k
    const char *const base_a = uniform_ptr(A + (ao + (long)m0 * g.a_m) * ES);
    const char *const base_b = uniform_ptr(PAIR ? B + bo + (long)n0 * g.b_n : B + bo + (n0 <= g.N - 16 ? n0 : g.N - 16));
    const long b_adv = PAIR ? P_ROW_BYTES : 64L * g.b_k;

    auto dma_a = [&](int e, int src, int slot) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (e == p) dma16_sbase(base_a + (long)src * P_ROW_BYTES, offa[p], lds0 + (unsigned)slot * Cfg::A_BYTES + lda[p]);
    };
    // element e of a stage's share of the list that fetches buffer's worth `src` of B into buffer `buf` (k-dense: half
    // `half` of the pair's rows)
    auto dma_b = [&](int e, int src, int buf, int half) {
#pragma unroll
        for (int p = 0; p < PBS; p++)
            if (e == p) {
                unsigned voff = offb[p], off = ldb[p];
                if constexpr (PAIR) {
                    voff = half ? offb[p + PBS] : offb[p];
                    off = half ? ldb[p + PBS] : ldb[p];
                }
                dma16_sbase(base_b + src * b_adv, voff, lds0 + (unsigned)buf * Cfg::B_BYTES + off);
            }
    };

    // fragment addresses.  A: lane (r16, g4) reads chunk 4 * slice + g4 of row r16 (16 bytes).  B k-dense: the lane's
    // 8 k are 8 bytes: half g4 % 2 of chunk 4 * (stage % 2) + 2 * slice + g4 / 2 of the row's 128-byte line; slice and
    // stage flip bits 5 and 6 of the byte offset (the swizzle is an XOR on the chunk index).  B row-dense: the 16 lanes
    // of group g4 take their 8 k of column r16 out of k-rows 32 * slice + 8 * g4 .. + 7 through one transpose read, for
    // which lane s of the 16 supplies the address of 8 columns of k-row (that start) + s / 2; k % 16 is
    // 8 * (g4 % 2) + s / 2 whatever the slice, so the swizzle is the lane's own and slices are immediates; tiles are not.
    constexpr int TILE_BYTES = 16 * P_ROW_BYTES;
    int a_frag[2];
#pragma unroll
    for (int sl = 0; sl < 2; sl++) a_frag[sl] = (wave_m * TM) * TILE_BYTES + r16 * P_ROW_BYTES + (kd_slot(r16, 4 * sl + g4) << 4);
    const int b_frag = B_BASE + (wave_n * TN) * TILE_BYTES + r16 * P_ROW_BYTES + (kd_slot(r16, g4 >> 1) << 4) + (g4 & 1) * 8;
    int b_mn[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int kq = r16 >> 1, bytes = (wave_n * TN + j) * 16 + (r16 & 1) * 8, c = bytes >> 4, k = 8 * g4 + kq;
        b_mn[j] = B_BASE + k * Cfg::BN + ((c ^ (k & 15)) << 4) + (bytes & 8);
    }

    u32x4_t fa[2][TM];
    u32x2_t fb[2][TN];  // raw bytes
    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = acc_t{0.f, 0.f, 0.f, 0.f};

    // the r-th fragment read of slice SL of stage `st` (ring slot st % 2): the left operand's tiles, then the right's
    auto read_fragment = [&](auto sl_, int r, int st) {
        constexpr int SL = decltype(sl_)::value;
        if (r < TM) {
            fa[SL][r] = lds_get(smem + (st & 1) * Cfg::A_BYTES, a_frag[SL] + r * TILE_BYTES);
        } else if constexpr (PAIR) {
            const int at = (b_frag ^ (SL << 5) ^ ((st & 1) << 6)) + (r - TM) * TILE_BYTES;
            fb[SL][r - TM] = lds_get64(smem + ((st >> 1) & 1) * Cfg::B_BYTES, at);
        } else {
            fb[SL][r - TM] = lds_get_tr<1>(smem + (st & 1) * Cfg::B_BYTES, b_mn[r - TM] + SL * 32 * Cfg::BN);
        }
    };
    u32x4_t bwide = u32x4_t{0u, 0u, 0u, 0u};  // the widened first right fragment of the next slice
    // One slice in a pinned order, as in mfma_pipe16_kernel: a read behind MFMAs 1, 4, 7, .., in slice 1 a DMA instruction
    // behind MFMAs 3, 6, 9, ..; the right fragment of the next group of TM MFMAs is widened behind the first four
    // MFMAs of the current group, the first fragment of the next slice behind this slice's last four.
    auto slice_step = [&](auto cur_, int rd_stage, int a_src, int a_slot, int b_src, int b_buf, int b_half) {
        constexpr int CUR = decltype(cur_)::value;
        typedef std::integral_constant<int, 1 - CUR> RS;
        constexpr int DSLOTS = (MF - 4) / 3;
        static_assert(DSLOTS >= P, "a gap of its own for every DMA instruction");
        u32x4_t bcur = bwide, bnext = bcur;
        // one conversion (two values) behind each of the first four MFMAs of a group: four in a row take longer to
        // issue than the MFMA in front of them runs
        auto widen_part = [&](u32x4_t &dst, const u32x2_t &raw, int part) {
            const uint32_t w = part < 2 ? raw.x : raw.y;
            const uint32_t v = bitcast<uint32_t>(part & 1 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)
                                                          : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
            if (part == 0) dst.x = v;
            else if (part == 1) dst.y = v;
            else if (part == 2) dst.z = v;
            else dst.w = v;
        };
#pragma unroll
        for (int idx = 0; idx < MF; idx++) {
            if (idx % TM == 0 && idx > 0) bcur = bnext;
            Cmp::mma(bcur, fa[CUR][idx % TM], acc[idx % TM][idx / TM]);
            if (idx % TM < 4 && idx / TM + 1 < TN) widen_part(bnext, fb[CUR][idx / TM + 1], idx % TM);
            if (idx >= MF - 4) widen_part(bwide, fb[1 - CUR][0], idx - (MF - 4));
            if (idx % 3 == 1 && idx / 3 < TM + TN) read_fragment(RS{}, idx / 3, rd_stage);
            if constexpr (CUR == 1) {
#pragma unroll
                for (int d = 0; d < P; d++)
                    if (3 * (1 + d * DSLOTS / P) == idx) {
                        if (d < PA) dma_a(d, a_src, a_slot);
                        else dma_b(d - PA, b_src, b_buf, b_half);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    // prologue: stage 0 of A and buffer 0 of B, then stage 1 of A and (k-dense: the first half of) buffer 1 of B (clamped)
#pragma unroll
    for (int e = 0; e < PA; e++) dma_a(e, 0, 0);
#pragma unroll
    for (int e = 0; e < PBS; e++) dma_b(e, 0, 0, 0);
    if constexpr (PAIR) {
#pragma unroll
        for (int e = 0; e < PBS; e++) dma_b(e, 0, 0, 1);
    }
#pragma unroll
    for (int e = 0; e < PA; e++) dma_a(e, 1 < T ? 1 : T - 1, 1);
#pragma unroll
    for (int e = 0; e < PBS; e++) dma_b(e, 1 < TB ? 1 : TB - 1, 1, 0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(PA + PBS));  // stage 0 and buffer 0 have landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < TM + TN; r++) read_fragment(I0{}, r, 0);
    bwide = widen_f8x8(fb[0][0]);

    // Past the last stage the reads fetch LDS bytes nobody uses and the lists re-fetch the last stage (pair) into
    // buffers nobody reads: harmless, and the number of instructions in flight stays what the waits assume.
    for (int t = 0; t < T; t++) {
        slice_step(I0{}, t, 0, 0, 0, 0, 0);
        // stage t + 1 (and its pair) has landed and every read of stage t has returned
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // A: stage t + 2 into the slot of stage t.  B row-dense: likewise.  B k-dense: odd t has just finished pair
        // t / 2 and sends the first half of pair t / 2 + 2 into its buffer; the next (even) stage sends the second half
        const int a_src = t + 2 < T ? t + 2 : T - 1;
        if constexpr (PAIR) {
            const int pair = (t & 1) ? (t + 3) >> 1 : (t + 2) >> 1;
            slice_step(I1{}, t + 1, a_src, t & 1, pair < TB ? pair : TB - 1, pair & 1, (t & 1) ? 0 : 1);
        } else {
            slice_step(I1{}, t + 1, a_src, t & 1, a_src, t & 1, 0);
        }
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // the re-fetches of the last stages are still writing LDS
    mfma_results_settle();                      // the accumulators are read next
    __syncthreads();

    char *patch = smem + wave * (16 * (TN * 16 * 4 + 16));
    out_t *Cb = C + batch * (long)g.M * g.N;
    EpiPrepared<Out<Cfg::OUT>::DT, 16 / (int)sizeof(out_t)> steps{};
    if (g.epi.n != 0) steps = band_columns_prepare<Cfg::OUT, TN, 16>(g.epi, n0 + wave_n * TN * 16, lane, g.N);
#pragma unroll
    for (int i = 0; i < TM; i++)
        store_band_via_lds<Cfg::OUT, TN, true, acc_t, 16, true>(patch, Cb, acc[i], m0 + (wave_m * TM + i) * 16, n0 + wave_n * TN * 16, lane,
                                                                g.M, g.N, g.epi, steps);
}

// mfma_pipe16_f8w_kernel with its LDS-DMA spaced by issue slots, as mfma_pipe16r_kernel does for 16-bit operands: a
// wavefront's pieces of an operand lie 1 KB apart in LDS and four of them share one M0 write (two groups for a stage of
// the left operand, one for a stage's share of the right one), each M0 write -- a single s_add_u32 of a literal to a
// base that depends on the ring slot -- in the gap before its group's first load and every load alone with the
// conversion or fragment read its gap already holds.  Everything else is that kernel: the weight's bytes move as they are and
// are widened to bf16 between the fragment read (8 bytes per lane) and the MFMA, one fragment ahead of its use, in the
// shadow of the MFMAs of the fragment before.
//   k-dense weights ([N, K] bytes): whole 128-byte lines, i.e. 128 k, the k of TWO stages of the bf16 left operand, so
//     a right-operand buffer holds a pair of stages and the ring two pairs.  A pair's buffer is free behind the barrier
//     of the pair's second stage and is needed four stages on, so its refill goes out in two halves, behind that
//     barrier and behind the next one: every stage issues 8 + 4 DMA instructions.
//   row-dense weights ([K, N] bytes): a stage is 64 k-rows of the tile's 256 bytes, in a ring of two like the left
//     operand's (8 + 4 instructions per stage as well); a fragment is one 8-bit transpose read of 8 k-rows.
template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe16r_f8w_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                                  typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                                  int tiles_m, int tiles_n) {
    static_assert(Cfg::LA == LM_K && Cfg::B_F8 && Cfg::NST == 2, "bf16 x f8e4m3, the left operand k-dense, two stages");
    HODU_DYNAMIC_LDS(smem);
    typedef Compute16<Cfg::CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr bool PAIR = Cfg::B_PAIR;  // k-dense weights
    constexpr int ES = Cfg::ES, PA = Cfg::PA, PB = Cfg::PB, PBS = Cfg::PBS, P = PA + PBS;
    constexpr int TM = Cfg::BM / Cfg::WM / 16, TN = Cfg::BN / Cfg::WN / 16;
    constexpr int MF = TM * TN;
    static_assert(TM == 8 && TN == 8 && P <= 19, "the schedule below is written for 128 x 128 outputs per wavefront");
    constexpr int GRP = 4, BIAS = 4096;  // DMA instructions per M0 value; what keeps the biased lane offsets non-negative
    static_assert(PA % GRP == 0 && PBS == GRP, "groups of four: two for a stage of A, one for a stage's share of B");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int r16 = lane & 15, g4 = lane >> 4;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

    // LDS: two stages of A (64 k of bf16 each), then two buffers of B (k-dense: 128 k each; row-dense: 64 k-rows each)
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    constexpr int B_BASE = 2 * Cfg::A_BYTES;

    // DMA plan.  k-dense: an instruction writes 8 rows x 128 bytes; lane -> (row, slot), the slot holds chunk
    // slot ^ ((row >> 1) & 7); rows past the operand's last one re-fetch the last one.  Address = scalar base of the
    // tile's first row (advanced 128 bytes per stage of A, per pair of B) + the lane's 32-bit offset inside the tile.
    // row-dense weights: an instruction writes 4 k-rows of 256 bytes; lane -> (k-row, slot), the slot holds chunk
    // slot ^ (k % 16) (a transpose read serves 32 lanes at a time, 16 k-rows of 16 bytes: the swizzle spreads them over
    // all banks); a chunk that starts past the last column is fetched from the last whole chunk instead.
    // (piece q of a buffer is instruction q % PA -- q % PB -- of wavefront q / PA -- q / PB --; a lane's offset carries the
    // bias and the opposite of the immediate offset its instruction adds back to the global and the LDS address)
    unsigned offa[PA], offb[PB];
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = wave * PA + p, trow = q * 8 + (lane >> 3);
        int row = m0 + trow;
        row = row < g.M ? row : g.M - 1;
        offa[p] = (unsigned)((long)(row - m0) * g.a_m * ES) + kd_slot(trow, lane & 7) * 16 + BIAS - (p % GRP) * 1024;
    }
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int q = wave * PB + p;
        if constexpr (PAIR) {
            const int trow = q * 8 + (lane >> 3);
            int row = n0 + trow;
            row = row < g.N ? row : g.N - 1;
            offb[p] = (unsigned)((long)(row - n0) * g.b_n) + kd_slot(trow, lane & 7) * 16 + BIAS - (p % GRP) * 1024;
        } else {
            constexpr int CPR = Cfg::BN / 16, KPI = 64 / CPR;
            const int k = q * KPI + lane / CPR, c = (lane % CPR) ^ (k & 15);
            int col = n0 + c * 16;
            col = col <= g.N - 16 ? col : g.N - 16;
            offb[p] = (unsigned)((long)k * g.b_k + (col - (n0 <= g.N - 16 ? n0 : g.N - 16))) + BIAS - (p % GRP) * 1024;
        }
    }
    const unsigned wbase_a = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)wave * (PA * 1024));
    const unsigned wbase_b = __builtin_amdgcn_readfirstlane(lds0 + B_BASE + (unsigned)wave * (PB * 1024));
    const int T = g.K * ES / P_ROW_BYTES;  // stages (k-dense weights: even, K is a multiple of 128)
    const int TB = PAIR ? T / 2 : T;       // right-operand buffers' worth of k
    const char *const base_a = uniform_ptr(A + (ao + (long)m0 * g.a_m) * ES - BIAS);
    const char *const base_b = uniform_ptr((PAIR ? B + bo + (long)n0 * g.b_n : B + bo + (n0 <= g.N - 16 ? n0 : g.N - 16)) - BIAS);
    const long b_adv = PAIR ? P_ROW_BYTES : 64L * g.b_k;

    // list element e of a stage: the left operand's PA pieces of stage `src` (M0 of its group set beforehand from the
    // ring slot), then the stage's PBS pieces of the right operand (k-dense: half `half` of the pair's rows)
    auto dma_a = [&](auto e_, int src) {
        constexpr int E = decltype(e_)::value;
        dma16_imm<(E % GRP) * 1024>(base_a + (long)src * P_ROW_BYTES, offa[E]);
    };
    auto dma_b = [&](auto e_, int src, int half) {
        constexpr int E = decltype(e_)::value;
        unsigned voff = offb[E];
        if constexpr (PAIR) voff = half ? offb[E + PBS] : offb[E];
        dma16_imm<(E % GRP) * 1024>(base_b + src * b_adv, voff);
    };
    // M0 for group `grp` of the left operand's pieces into ring slot `slot`, and for the right operand's share
    auto m0_a = [&](auto grp_, int slot) {
        m0_set<decltype(grp_)::value * GRP * 1024>(wbase_a + (unsigned)slot * Cfg::A_BYTES);
    };
    auto m0_b = [&](int buf, int half) {
        m0_set<0>(wbase_b + (unsigned)buf * Cfg::B_BYTES + (PAIR ? (unsigned)half * (PBS * 1024) : 0u));
    };

    // fragment addresses.  A: lane (r16, g4) reads chunk 4 * slice + g4 of row r16 (16 bytes).  B k-dense: the lane's
    // 8 k are 8 bytes: half g4 % 2 of chunk 4 * (stage % 2) + 2 * slice + g4 / 2 of the row's 128-byte line; slice and
    // stage flip bits 5 and 6 of the byte offset (the swizzle is an XOR on the chunk index).  B row-dense: the 16 lanes
    // of group g4 take their 8 k of column r16 out of k-rows 32 * slice + 8 * g4 .. + 7 through one transpose read, for
    // which lane s of the 16 supplies the address of 8 columns of k-row (that start) + s / 2; k % 16 is
    // 8 * (g4 % 2) + s / 2 whatever the slice, so the swizzle is the lane's own and slices are immediates; tiles are not.
    constexpr int TILE_BYTES = 16 * P_ROW_BYTES;
    int a_frag[2];
#pragma unroll
    for (int sl = 0; sl < 2; sl++) a_frag[sl] = (wave_m * TM) * TILE_BYTES + r16 * P_ROW_BYTES + (kd_slot(r16, 4 * sl + g4) << 4);
    const int b_frag = B_BASE + (wave_n * TN) * TILE_BYTES + r16 * P_ROW_BYTES + (kd_slot(r16, g4 >> 1) << 4) + (g4 & 1) * 8;
    int b_mn[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int kq = r16 >> 1, bytes = (wave_n * TN + j) * 16 + (r16 & 1) * 8, c = bytes >> 4, k = 8 * g4 + kq;
        b_mn[j] = B_BASE + k * Cfg::BN + ((c ^ (k & 15)) << 4) + (bytes & 8);
    }

    u32x4_t fa[2][TM];
    u32x2_t fb[2][TN];  // raw bytes
    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = acc_t{0.f, 0.f, 0.f, 0.f};

    // the r-th fragment read of slice SL of stage `st` (ring slot st % 2): the left operand's tiles, then the right's
    auto read_fragment = [&](auto sl_, int r, int st) {
        constexpr int SL = decltype(sl_)::value;
        if (r < TM) {
            fa[SL][r] = lds_get(smem + (st & 1) * Cfg::A_BYTES, a_frag[SL] + r * TILE_BYTES);
        } else if constexpr (PAIR) {
            const int at = (b_frag ^ (SL << 5) ^ ((st & 1) << 6)) + (r - TM) * TILE_BYTES;
            fb[SL][r - TM] = lds_get64(smem + ((st >> 1) & 1) * Cfg::B_BYTES, at);
        } else {
            fb[SL][r - TM] = lds_get_tr<1>(smem + (st & 1) * Cfg::B_BYTES, b_mn[r - TM] + SL * 32 * Cfg::BN);
        }
    };
    u32x4_t bwide = u32x4_t{0u, 0u, 0u, 0u};  // the widened first right fragment of the next slice
    // One slice in a pinned order, as in mfma_pipe16_kernel: a read behind MFMAs 1, 4, 7, .., in slice 1 a DMA instruction
    // behind MFMAs 3, 6, 9, ..; the right fragment of the next group of TM MFMAs is widened behind the first four
    // MFMAs of the current group, the first fragment of the next slice behind this slice's last four.
    auto slice_step = [&](auto cur_, int rd_stage, int a_src, int a_slot, int b_src, int b_buf, int b_half) {
        constexpr int CUR = decltype(cur_)::value;
        typedef std::integral_constant<int, 1 - CUR> RS;
        constexpr int DSLOTS = (MF - 4) / 3;
        static_assert(DSLOTS >= P, "a gap of its own for every DMA instruction");
        u32x4_t bcur = bwide, bnext = bcur;
        // one conversion (two values) behind each of the first four MFMAs of a group: four in a row take longer to
        // issue than the MFMA in front of them runs
        auto widen_part = [&](u32x4_t &dst, const u32x2_t &raw, int part) {
            const uint32_t w = part < 2 ? raw.x : raw.y;
            const uint32_t v = bitcast<uint32_t>(part & 1 ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)
                                                          : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
            if (part == 0) dst.x = v;
            else if (part == 1) dst.y = v;
            else if (part == 2) dst.z = v;
            else dst.w = v;
        };
#pragma unroll
        for (int idx = 0; idx < MF; idx++) {
            if (idx % TM == 0 && idx > 0) bcur = bnext;
            Cmp::mma(bcur, fa[CUR][idx % TM], acc[idx % TM][idx / TM]);
            if (idx % TM < 4 && idx / TM + 1 < TN) widen_part(bnext, fb[CUR][idx / TM + 1], idx % TM);
            if (idx >= MF - 4) widen_part(bwide, fb[1 - CUR][0], idx - (MF - 4));
            if (idx % 3 == 1 && idx / 3 < TM + TN) read_fragment(RS{}, idx / 3, rd_stage);
            if constexpr (CUR == 1) {
                static_for<P>([&](auto d_) {
                    constexpr int d = decltype(d_)::value;
                    if (3 * (1 + d * DSLOTS / P) == idx) {
                        if constexpr (d < PA) dma_a(d_, a_src);
                        else dma_b(std::integral_constant<int, (d < PA ? 0 : d - PA)>{}, b_src, b_half);
                    }
                    // the group's M0 one gap ahead of its first load
                    if (d % GRP == 0 && 3 * (1 + d * DSLOTS / P) - 1 == idx) {
                        if constexpr (d < PA) m0_a(std::integral_constant<int, d / GRP>{}, a_slot);
                        else m0_b(b_buf, b_half);
                    }
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    // prologue: stage 0 of A and buffer 0 of B, then stage 1 of A and (k-dense: the first half of) buffer 1 of B (clamped)
    auto fetch_a = [&](int src, int slot) {
        static_for<PA>([&](auto e_) {
            constexpr int E = decltype(e_)::value;
            if constexpr (E % GRP == 0) {
                m0_a(std::integral_constant<int, E / GRP>{}, slot);
                m0_wait_state();
            }
            dma_a(e_, src);
        });
    };
    auto fetch_b = [&](int src, int buf, int half) {
        m0_b(buf, half);
        m0_wait_state();
        static_for<PBS>([&](auto e_) { dma_b(e_, src, half); });
    };
    fetch_a(0, 0);
    fetch_b(0, 0, 0);
    if constexpr (PAIR) fetch_b(0, 0, 1);
    fetch_a(1 < T ? 1 : T - 1, 1);
    fetch_b(1 < TB ? 1 : TB - 1, 1, 0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(PA + PBS));  // stage 0 and buffer 0 have landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < TM + TN; r++) read_fragment(I0{}, r, 0);
    bwide = widen_f8x8(fb[0][0]);

    // Past the last stage the reads fetch LDS bytes nobody uses and the lists re-fetch the last stage (pair) into
    // buffers nobody reads: harmless, and the number of instructions in flight stays what the waits assume.
    for (int t = 0; t < T; t++) {
        slice_step(I0{}, t, 0, 0, 0, 0, 0);
        // stage t + 1 (and its pair) has landed and every read of stage t has returned
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // A: stage t + 2 into the slot of stage t.  B row-dense: likewise.  B k-dense: odd t has just finished pair
        // t / 2 and sends the first half of pair t / 2 + 2 into its buffer; the next (even) stage sends the second half
        const int a_src = t + 2 < T ? t + 2 : T - 1;
        if constexpr (PAIR) {
            const int pair = (t & 1) ? (t + 3) >> 1 : (t + 2) >> 1;
            slice_step(I1{}, t + 1, a_src, t & 1, pair < TB ? pair : TB - 1, pair & 1, (t & 1) ? 0 : 1);
        } else {
            slice_step(I1{}, t + 1, a_src, t & 1, a_src, t & 1, 0);
        }
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // the re-fetches of the last stages are still writing LDS
    mfma_results_settle();                      // the accumulators are read next
    __syncthreads();

    char *patch = smem + wave * (16 * (TN * 16 * 4 + 16));
    out_t *Cb = C + batch * (long)g.M * g.N;
    EpiPrepared<Out<Cfg::OUT>::DT, 16 / (int)sizeof(out_t)> steps{};
    if (g.epi.n != 0) steps = band_columns_prepare<Cfg::OUT, TN, 16>(g.epi, n0 + wave_n * TN * 16, lane, g.N);
#pragma unroll
    for (int i = 0; i < TM; i++)
        store_band_via_lds<Cfg::OUT, TN, true, acc_t, 16, true>(patch, Cb, acc[i], m0 + (wave_m * TM + i) * 16, n0 + wave_n * TN * 16, lane,
                                                                g.M, g.N, g.epi, steps);
}

template <class Cfg> int launch_pipe16_f8w(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    auto kernel = mfma_pipe16_f8w_kernel<Cfg>;
    static_assert(Cfg::NW * 16 * ((Cfg::BN / Cfg::WN) * 4 + 16) <= Cfg::LDS_BYTES, "the epilogue's patches fit the ring");
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    if (g.K <= 0 || g.K % (Cfg::B_PAIR ? 128 : 64) != 0) return fail(HODU_ROCM_UNSUPPORTED, "K is not a whole number of stages");
    hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream, (const char *)a, (const char *)b,
                       (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <class Cfg> int launch_pipe16r_f8w(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    auto kernel = mfma_pipe16r_f8w_kernel<Cfg>;
    static_assert(Cfg::NW * 16 * ((Cfg::BN / Cfg::WN) * 4 + 16) <= Cfg::LDS_BYTES, "the epilogue's patches fit the ring");
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    if (g.K <= 0 || g.K % (Cfg::B_PAIR ? 128 : 64) != 0) return fail(HODU_ROCM_UNSUPPORTED, "K is not a whole number of stages");
    hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream, (const char *)a, (const char *)b,
                       (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <class Cfg> int launch_pipe16r(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    auto kernel = g.epi.n != 0 ? mfma_pipe16r_kernel<Cfg, true> : mfma_pipe16r_kernel<Cfg, false>;
    static_assert(Cfg::NW * 16 * ((Cfg::BN / Cfg::WN) * 4 + 16) <= Cfg::LDS_BYTES, "the epilogue's patches fit the ring");
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    if (!pipe16r_stages_ok(g.K, Cfg::ES)) return fail(HODU_ROCM_UNSUPPORTED, "K is not an even number of stages");
    hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream, (const char *)a, (const char *)b,
                       (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <class Cfg> int launch_pipe16(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    auto kernel = mfma_pipe16_kernel<Cfg>;
    static_assert(Cfg::NW * 16 * ((Cfg::BN / Cfg::WN) * 4 + 16) <= Cfg::LDS_BYTES, "the epilogue's patches fit the ring");
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    if (g.K <= 0 || ((long)g.K * Cfg::ES) % P_ROW_BYTES != 0) return fail(HODU_ROCM_UNSUPPORTED, "K is not a whole number of stages");
    hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream, (const char *)a, (const char *)b,
                       (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace mfma
}  // namespace hodu
