// The pipelined tile kernel of gemm_mfma_pipe.hpp on the 16 x 16 x 32 matrix instruction, for 16-bit operands that are
// both k-dense.  Same feeding scheme -- whole 128-byte rows by LDS-DMA into a two-stage ring, source-side XOR swizzle,
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
//     lane: lane (r = lane % 16, g = lane / 16) reads chunk 4 * slice + g of row r, one ds_read_b128;
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

typedef float f32x4_acc_t __attribute__((ext_vector_type(4)));

template <int CK> struct Compute16;
template <> struct Compute16<CK_BF16> {
    typedef f32x4_acc_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<bf16x8_t>(a), bitcast<bf16x8_t>(b), c, 0, 0, 0);
    }
};
template <> struct Compute16<CK_F16> {
    typedef f32x4_acc_t acc_t;
    static __device__ __forceinline__ void mma(const u32x4_t &a, const u32x4_t &b, acc_t &c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<f16x8_t>(a), bitcast<f16x8_t>(b), c, 0, 0, 0);
    }
};

// Cfg: a PipeConfig with both operands k-dense, stored in the compute type, and a ring of two stages
template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe16_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                              typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                              int tiles_m, int tiles_n) {
    static_assert(Cfg::LA == LM_K && Cfg::LB == LM_K && !Cfg::B_F8 && Cfg::ES == 2 && Cfg::NST == 2, "k-dense 16-bit operands, two stages");
    extern __shared__ __align__(16) char smem[];
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
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = p * Cfg::NW + wave, trow = q * 8 + (lane >> 3), dchunk = kd_slot(trow, lane & 7);
        int row = m0 + trow;
        row = row < g.M ? row : g.M - 1;
        offa[p] = (unsigned)((long)(row - m0) * g.a_m * ES) + dchunk * 16;
        lda[p] = q * 1024;
    }
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int q = p * Cfg::NW + wave, trow = q * 8 + (lane >> 3), dchunk = kd_slot(trow, lane & 7);
        int row = n0 + trow;
        row = row < g.N ? row : g.N - 1;
        offb[p] = (unsigned)((long)(row - n0) * g.b_n * ES) + dchunk * 16;
        ldb[p] = B_BASE + q * 1024;
    }
    const int T = g.K * ES / P_ROW_BYTES;  // stages
    const char *const base_a = uniform_ptr(A + (ao + (long)m0 * g.a_m) * ES);
    const char *const base_b = uniform_ptr(B + (bo + (long)n0 * g.b_n) * ES);

    // element e of the list that fetches stage `src` (already clamped to T - 1) into ring slot `slot`
    auto dma_element = [&](int e, int src, int slot) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (e == p) dma16_sbase(base_a + (long)src * P_ROW_BYTES, offa[p], lds0 + (unsigned)slot * Cfg::A_BYTES + lda[p]);
#pragma unroll
        for (int p = 0; p < PB; p++)
            if (e == PA + p) dma16_sbase(base_b + (long)src * P_ROW_BYTES, offb[p], lds0 + (unsigned)slot * Cfg::B_BYTES + ldb[p]);
    };

    // fragment addresses: lane (r16, g4) reads chunk 4 * slice + g4 of row r16 of a 16-row tile; every tile starts on
    // a multiple of 16 rows, so the swizzle term (row >> 1) & 7 is the lane's own
    constexpr int TILE_BYTES = 16 * P_ROW_BYTES;
    int a_frag[2], b_frag[2];
#pragma unroll
    for (int sl = 0; sl < 2; sl++) {
        const int at = r16 * P_ROW_BYTES + (kd_slot(r16, 4 * sl + g4) << 4);
        a_frag[sl] = (wave_m * TM) * TILE_BYTES + at;
        b_frag[sl] = B_BASE + (wave_n * TN) * TILE_BYTES + at;
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
        if (r < TM) fa[SL][r] = lds_get(smem + slot * Cfg::A_BYTES, a_frag[SL] + r * TILE_BYTES);
        else fb[SL][r - TM] = lds_get(smem + slot * Cfg::B_BYTES, b_frag[SL] + (r - TM) * TILE_BYTES);
    };
    // One slice of work in a pinned order: the MFMAs of slice CUR with the reads of slice 1 - CUR (from ring slot
    // rd_slot) and, in slice 1 -- behind the barrier --, the DMA list between them.  A read goes behind MFMAs 1, 4, 7, ..,
    // so that the last one is out a quarter of a slice before the slice ends (in slice 0 the barrier's wait for the
    // reads follows, in slice 1 the loop's back edge, where the compiler waits for every read in flight); a DMA
    // instruction goes behind one of the MFMAs 4, 7, 10, .. (the compiler moves a read in front of the MFMA it is
    // grouped with, so the reads sit in the gaps behind MFMAs 0, 3, 6, .. and the DMA instructions in gaps of their own).
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
                    if (3 * (1 + d * DSLOTS / P) + 1 == idx) dma_element(d, dma_src, dma_slot);
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
    __syncthreads();

    // epilogue: bands of 16 rows through a wavefront-private patch of LDS
    char *patch = smem + wave * (16 * (TN * 16 * 4 + 16));
    out_t *Cb = C + batch * (long)g.M * g.N;
#pragma unroll
    for (int i = 0; i < TM; i++)
        store_band_via_lds<Cfg::OUT, TN, true, acc_t, 16>(patch, Cb, acc[i], m0 + (wave_m * TM + i) * 16, n0 + wave_n * TN * 16, lane,
                                                          g.M, g.N, g.epi);
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
