// f8e4m3 x f8e4m3 and f8e5m2 x f8e5m2 products on the 16 x 16 x 128 form of the gfx950 8-bit matrix instruction
// (v_mfma_scale_f32_16x16x128_f8f6f4 with unit scales): the 256 x 256 tile of gemm_mfma_pipe_f8.hpp on four
// wavefronts, each owning 128 x 128 outputs as 8 x 8 accumulators of 4 registers.  Same operands, same feeding
// scheme (whole 128-byte rows by LDS-DMA into a two-stage ring, source-side XOR swizzle, one barrier per 128-k stage,
// the tile leaving through LDS as whole rows), same sums: f32 accumulation over k in blocks of 128 instead of 64,
// narrowed once.
//
// Why: from registers alone this form sustains 4.4 PFLOP/s on N(0,1) f8e4m3 operands where the 32 x 32 x 64 form
// sustains 4.0 (hodu_rocm_debug_mfma_clock, kinds 3 and 1) -- the part is power-limited and the small accumulator tile
// leaves it a higher clock -- and four wavefronts read a third fewer fragment bytes out of LDS than eight.
//
// A stage is ONE instruction deep in k, so what alternates between register sets are the two halves of a
// wavefront's rows; both halves run column by column (b_j against four rows), so b_j is due at the half's (4j)-th MFMA.
// Per stage t (ring slot t % 2):
//   first half    MFMAs of rows a0..a3; reads of this stage's b2..b7, just ahead of their use, and of a4..a7;
//   barrier       stage t + 1 has landed, every read of stage t has returned;
//   second half   MFMAs of rows a4..a7; reads of stage t + 1's a0..a3, b0, b1 (b0, b1 into the other of two register
//                 sets); the whole DMA list of stage t + 2 into the slot the barrier has just freed, in gaps of its
//                 own -- 20 fragment reads in the first half, 12 reads and 16 DMA instructions in the second.
#pragma once

#include "gemm_mfma_pipe_f8.hpp"

namespace hodu {
namespace mfma {

typedef float f32x4_f8acc_t __attribute__((ext_vector_type(4)));

// FMT: the instruction's operand format code, 0 = e4m3, 1 = e5m2 (both operands alike).  The instruction itself,
// written out with its accumulator tied: mfma16x16x128_f8 of gfx950_insn.hpp.
template <int FMT> __device__ __forceinline__ void mma_f8_16(const i32x8_t &a, const i32x8_t &b, f32x4_f8acc_t &c) {
    mfma16x16x128_f8<FMT>(a, b, c);
}

template <int OUT_, int BM_, int BN_> struct PipeF8x16Config {
    static constexpr int OUT = OUT_, BM = BM_, BN = BN_, WM = 2, WN = 2, NT = WM * WN * 64, NW = WM * WN;
    static constexpr int A_BYTES = BM * P_ROW_BYTES, B_BYTES = BN * P_ROW_BYTES;
    static constexpr int LDS_BYTES = 2 * (A_BYTES + B_BYTES);
    static constexpr int PA = (BM / 8) / NW, PB = (BN / 8) / NW, P = PA + PB;
    static constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
    static_assert(TM == 8 && TN == 8 && P == 16, "the schedule below is written for 128 x 128 outputs per wavefront");
    static_assert(LDS_BYTES <= 160 * 1024 && NW * 16 * (TN * 16 * 4 + 16) <= LDS_BYTES, "LDS budget");
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe_f8x16_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                                  typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                                  int tiles_m, int tiles_n) {
    HODU_DYNAMIC_LDS(smem);
    typedef typename Out<Cfg::OUT>::T out_t;
    typedef f32x4_f8acc_t acc_t;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, PA = Cfg::PA, PB = Cfg::PB, P = Cfg::P, HALF = TM / 2;
    constexpr int FMT = Cfg::OUT == OUT_F8E5M2 ? 1 : 0;
    constexpr int TILE_BYTES = 16 * P_ROW_BYTES, B_BASE = 2 * Cfg::A_BYTES;

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
    const unsigned lds0 = (unsigned)(uintptr_t)smem;

    // DMA plan, as in mfma_pipe_f8_kernel: one instruction = 8 rows x 128 bytes; the slot of a lane holds chunk
    // slot ^ ((row >> 1) & 7); rows past the operand's last one re-fetch the last one (their outputs are never stored).
    // Address = scalar base of the tile's first row (advanced 128 bytes per stage) + the lane's 32-bit offset inside
    // the tile (the launcher checks that 256 rows stay below 4 GB).
    unsigned offa[PA], offb[PB];
    unsigned lda[PA], ldb[PB];
#pragma unroll
    for (int p = 0; p < PA; p++) {
        const int q = p * Cfg::NW + wave, trow = q * 8 + (lane >> 3);
        int row = m0 + trow;
        row = row < g.M ? row : g.M - 1;
        offa[p] = (unsigned)((long)(row - m0) * g.a_m) + kd_slot(trow, lane & 7) * 16;
        lda[p] = q * 1024;
    }
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int q = p * Cfg::NW + wave, trow = q * 8 + (lane >> 3);
        int row = n0 + trow;
        row = row < g.N ? row : g.N - 1;
        offb[p] = (unsigned)((long)(row - n0) * g.b_n) + kd_slot(trow, lane & 7) * 16;
        ldb[p] = B_BASE + q * 1024;
    }
    const int T = g.K / P_ROW_BYTES;
    const char *const base_a = uniform_ptr(A + ao + (long)m0 * g.a_m);
    const char *const base_b = uniform_ptr(B + bo + (long)n0 * g.b_n);

    // element e of stage `src`'s list (PA of A, then PB of B; src already clamped to T - 1) into ring slot `slot`
    auto dma_element = [&](int e, int src, int slot) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (e == p) dma16_sbase(base_a + (long)src * P_ROW_BYTES, offa[p], lds0 + (unsigned)slot * Cfg::A_BYTES + lda[p]);
#pragma unroll
        for (int p = 0; p < PB; p++)
            if (e == PA + p) dma16_sbase(base_b + (long)src * P_ROW_BYTES, offb[p], lds0 + (unsigned)slot * Cfg::B_BYTES + ldb[p]);
    };

    // fragment addresses: the instruction wants 32 k per lane, the same 32 in both operands -- which 32 is free, the
    // sum runs over all 128 either way.  Lane (r16, g4) takes chunks g4 and g4 + 4 of row r16 of a 16-row tile: each of
    // the two reads then has the four lane groups on four neighbouring chunks, the pattern of the 16-bit kernel's
    // reads (with chunks 2 * g4 and 2 * g4 + 1 the counters showed every read conflicting two ways).  Tiles start on
    // multiples of 16 rows, so the swizzle term is the lane's own and tiles are immediates.
    int a_fr[2], b_fr[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int at = r16 * P_ROW_BYTES + (kd_slot(r16, g4 + 4 * h) << 4);
        a_fr[h] = (wave_m * TM) * TILE_BYTES + at;
        b_fr[h] = B_BASE + (wave_n * TN) * TILE_BYTES + at;
    }
    auto fragment = [&](const char *buf, const int (&fr)[2], int tile) -> i32x8_t {
        const i32x4_t lo = bitcast<i32x4_t>(lds_get(buf, fr[0] + tile * TILE_BYTES));
        const i32x4_t hi = bitcast<i32x4_t>(lds_get(buf, fr[1] + tile * TILE_BYTES));
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    i32x8_t fa[TM], fb[2][TN];
    auto read_a = [&](int slot, int i) { fa[i] = fragment(smem + slot * Cfg::A_BYTES, a_fr, i); };

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = acc_t{0.f, 0.f, 0.f, 0.f};

    // prologue: stages 0 and 1 (clamped), wait for stage 0
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int src = j < T ? j : T - 1;
#pragma unroll
        for (int e = 0; e < P; e++) dma_element(e, src, j);
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(P));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < HALF; i++) read_a(0, i);
    fb[0][0] = fragment(smem, b_fr, 0);
    fb[0][1] = fragment(smem, b_fr, 1);

    // One stage with the right fragments in set SET.  Both halves run column by column (b_j against four rows), so a
    // half needs its four left fragments and b0 at once and b_j from its (4j)-th MFMA on.  Past the last stage the
    // reads fetch LDS bytes nobody uses and the list re-fetches the last stage into a slot nobody reads: harmless,
    // and the in-flight count stays what the waits assume.
    auto stage = [&](auto set_, int slot, int dma_src) {
        constexpr int SET = decltype(set_)::value;
        // first half: rows a0 .. a3; b2 .. b7 of this stage behind MFMAs 0, 2, .., 10 (b_j is due at MFMA 4j), a4 .. a7
        // behind 12, 15, 18, 21
#pragma unroll
        for (int idx = 0; idx < HALF * TN; idx++) {
            mma_f8_16<FMT>(fb[SET][idx / HALF], fa[idx % HALF], acc[idx % HALF][idx / HALF]);
            if (idx % 2 == 0 && idx / 2 + 2 < TN) fb[SET][idx / 2 + 2] = fragment(smem + slot * Cfg::B_BYTES, b_fr, idx / 2 + 2);
            if (idx >= 12 && (idx - 12) % 3 == 0 && (idx - 12) / 3 < HALF) read_a(slot, HALF + (idx - 12) / 3);
            __builtin_amdgcn_sched_barrier(0);
        }
        // stage t + 1 has landed (its list went out a stage ago) and every read of stage t has returned
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // second half: rows a4 .. a7; the next stage's a0 .. a3 behind MFMAs 0, 3, 6, 9, its b0 and b1 behind 12 and 15,
        // the DMA list of the stage after that behind the other MFMAs up to the 23rd
#pragma unroll
        for (int idx = 0; idx < HALF * TN; idx++) {
            mma_f8_16<FMT>(fb[SET][idx / HALF], fa[HALF + idx % HALF], acc[HALF + idx % HALF][idx / HALF]);
            if (idx % 3 == 0 && idx / 3 < HALF) read_a(slot ^ 1, idx / 3);
            if (idx == 12 || idx == 15) fb[SET ^ 1][(idx - 12) / 3] = fragment(smem + (slot ^ 1) * Cfg::B_BYTES, b_fr, (idx - 12) / 3);
            if (idx % 3 != 0 && idx - 1 - idx / 3 < P) dma_element(idx - 1 - idx / 3, dma_src, slot);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, 0> S0;
    typedef std::integral_constant<int, 1> S1;
    // two stages per trip, so that the right-fragment set is a compile-time constant
    int t = 0;
    for (; t + 1 < T; t += 2) {
        stage(S0{}, 0, t + 2 < T ? t + 2 : T - 1);
        stage(S1{}, 1, t + 3 < T ? t + 3 : T - 1);
    }
    if (t < T) stage(S0{}, 0, T - 1);
    // the re-fetches of the last stages still write LDS: wait for them, then for everybody's, before LDS is reused
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    mfma_results_settle();  // the accumulators are read next
    __syncthreads();

    char *patch = smem + wave * (16 * (TN * 16 * 4 + 16));
    out_t *Cb = C + batch * (long)g.M * g.N;
#pragma unroll
    for (int i = 0; i < TM; i++)
        store_band_via_lds<Cfg::OUT, TN, false, acc_t, 16>(patch, Cb, acc[i], m0 + (wave_m * TM + i) * 16, n0 + wave_n * TN * 16, lane,
                                                           g.M, g.N, g.epi);
}

template <class Cfg> int launch_pipe_f8x16(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    auto kernel = mfma_pipe_f8x16_kernel<Cfg>;
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    if (g.K <= 0 || g.K % P_ROW_BYTES != 0) return fail(HODU_ROCM_UNSUPPORTED, "K is not a whole number of stages");
    hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(Cfg::NT), Cfg::LDS_BYTES, ctx->stream, (const char *)a, (const char *)b,
                       (typename Out<Cfg::OUT>::T *)c, g, tiles_m, tiles_n);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace mfma
}  // namespace hodu
