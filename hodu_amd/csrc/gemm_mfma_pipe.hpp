// Software-pipelined MFMA tile kernel for products whose operands are BOTH k-dense in their
// compute type (bf16 x bf16, f16 x f16, i8 x i8, f32 x f32 with `stride_k == 1`, 16-byte aligned
// rows, K a multiple of 64 bytes).  Same tiles, same MFMA instructions and same results as the
// general kernel in gemm_mfma.hpp; what differs is how the K loop is fed:
//
//   * K advances 64 bytes per stage (32 bf16 / 64 i8 / 16 f32: one MFMA k-slice), four stages of
//     LDS; each stage is written by LDS-DMA only (global_load_lds_dwordx4: no staging registers,
//     no ds_write), three stages ahead of the stage being multiplied;
//   * a stage is an array of 1 KB blocks, one block = 16 rows x 64 B = exactly what one wavefront-wide
//     DMA instruction writes.  The four 16-byte chunks of a row are XOR-swizzled by (row / 4) % 4 --
//     applied to the SOURCE address of the DMA -- so that the MFMA fragment read (16 lanes = 16
//     rows, one chunk) touches all 64 banks once;
//   * the MFMA fragments live in one register set that is refilled half a step ahead of its use, each
//     ds_read_b128 interleaved with the MFMAs of the other k-slice, so that LDS (128 B/clk, about as
//     busy as the matrix cores at this tile shape) and the matrix cores run side by side instead of
//     in alternating bursts;
//   * the barrier is a bare s_barrier preceded by an s_waitcnt vmcnt(n) that leaves the DMA of the
//     two newest stages in flight (a __syncthreads() would drain them).
//
// Hazards.  DMA of stage t+3 is issued right after the barrier of step t into the buffer that held
// stage t-1.  Every wavefront reaches that barrier only after issuing the slice-0 MFMAs of stage t,
// which follow its last reads of stage t-1 and the MFMAs that consumed them.
#pragma once

#include <type_traits>

#include "gemm_mfma.hpp"

namespace hodu {
namespace mfma {

constexpr int P_ROW_BYTES = 64;
constexpr int P_STAGES = 4;
constexpr int P_AHEAD = 3;

// s_waitcnt immediate for gfx9: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
constexpr int waitcnt_vm(int n) { return (n & 15) | 0x70 | 0xF00 | ((n >> 4) << 14); }

template <int CK_, int OUT_, int BM_, int BN_, int WM_, int WN_> struct PipeConfig {
    static constexpr int CK = CK_, OUT = OUT_, BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    static constexpr int NT = WM * WN * 64, NW = WM * WN;
    static constexpr int ES = Compute<CK>::ES;
    static constexpr int BK = P_ROW_BYTES / ES;
    static constexpr int A_BYTES = BM * P_ROW_BYTES, B_BYTES = BN * P_ROW_BYTES;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = P_STAGES * STAGE_BYTES;
    static constexpr int BLOCKS = (BM + BN) / 16;    // DMA instructions per stage
    static constexpr int DMA_PER_WAVE = BLOCKS / NW;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;  // 32x32 MFMA tiles per wave
    static_assert(BLOCKS % NW == 0, "DMA split");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU");
};

// issued through inline assembly so that the compiler's own wait-count bookkeeping (which would put
// an s_waitcnt vmcnt(0) in front of the next LDS read) stays out of the way; completion is awaited
// explicitly with waitcnt_vm() before the barrier that publishes the stage
__device__ __forceinline__ void dma16_raw(const char *gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory");
}

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

    // ---- DMA plan of this wavefront: P instructions per stage, each one 1 KB block (16 rows) ----
    // lane -> (row in block, slot); the slot holds global chunk slot ^ ((row / 4) % 4)
    const int drow = lane >> 2, dchunk = (lane & 3) ^ ((lane >> 4) & 3);
    const char *gp[P];       // source address of this lane for stage 0
    unsigned lds_off[P];     // block offset inside a stage (wave-uniform)
#pragma unroll
    for (int p = 0; p < P; p++) {
        const int q = wave * P + p;
        if (q < Cfg::BM / 16) {
            int row = m0 + q * 16 + drow;
            row = row < g.M ? row : g.M - 1;
            gp[p] = A + (ao + (long)row * g.a_m) * ES + dchunk * 16;
            lds_off[p] = q * 1024;
        } else {
            const int qb = q - Cfg::BM / 16;
            int row = n0 + qb * 16 + drow;
            row = row < g.N ? row : g.N - 1;
            gp[p] = B + (bo + (long)row * g.b_n) * ES + dchunk * 16;
            lds_off[p] = Cfg::A_BYTES + qb * 1024;
        }
    }
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    auto issue = [&](int t) {
        const unsigned stage = lds0 + (unsigned)(t % P_STAGES) * Cfg::STAGE_BYTES;
        const long koff = (long)t * P_ROW_BYTES;
#pragma unroll
        for (int p = 0; p < P; p++)
            dma16_raw(gp[p] + koff, __builtin_amdgcn_readfirstlane(stage + lds_off[p]));
    };

    // ---- fragment addresses: lane (lr, lh) reads chunk 2*s + lh of row lr of a 32-row tile, which is
    // two consecutive 16-row blocks; the chunk sits at slot chunk ^ ((row / 4) % 4) of its row ----
    const int row16 = lr & 15, swz = (row16 >> 2) & 3;
    const int frag_row = (lr >> 4) * 1024 + row16 * P_ROW_BYTES;
    int a_frag[2], b_frag[2];
#pragma unroll
    for (int sl = 0; sl < 2; sl++) {
        const int slot = ((2 * sl + lh) ^ swz) << 4;
        a_frag[sl] = (wave_m * TM) * 2048 + frag_row + slot;
        b_frag[sl] = Cfg::A_BYTES + (wave_n * TN) * 2048 + frag_row + slot;
    }
    u32x4_t fa[2][TM], fb[2][TN];  // [k slice][tile]: ONE register set, refilled slice by slice
    auto read_slice = [&](int t, auto slice) {
        constexpr int SL = decltype(slice)::value;
        const char *stage = smem + (t % P_STAGES) * Cfg::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < TM; i++) fa[SL][i] = lds_get(stage, a_frag[SL] + i * 2048);
#pragma unroll
        for (int j = 0; j < TN; j++) fb[SL][j] = lds_get(stage, b_frag[SL] + j * 2048);
    };

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;

    const int T = g.K * ES / P_ROW_BYTES;
    // publish a stage: wait until at most `newer` younger stages' DMA are still in flight, then meet
    auto publish = [&](int newer) {
        if (newer >= 2) __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * P));
        else if (newer == 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm(P));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    auto multiply = [&](auto slice) {
        constexpr int SL = decltype(slice)::value;
        // operands swapped: the accumulator then holds, per lane, runs of 4 consecutive n of one m
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int i = 0; i < TM; i++) Cmp::mma(fb[SL][j], fa[SL][i], acc[i][j]);
    };
    // asks the scheduler to put one fragment read behind every PER-th MFMA of the block just written
    auto interleave = [&]() {
        constexpr int READS = TM + TN, MFMAS = TM * TN, PER = MFMAS / READS > 0 ? MFMAS / READS : 1;
#pragma unroll
        for (int r = 0; r < READS; r++) {
            __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // DS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, MFMAS > PER * READS ? MFMAS - PER * READS : 0, 0);
    };
    typedef std::integral_constant<int, 0> S0;
    typedef std::integral_constant<int, 1> S1;

    for (int t = 0; t < P_AHEAD && t < T; t++) issue(t);
    publish((T - 1 < P_AHEAD - 1 ? T - 1 : P_AHEAD - 1));
    read_slice(0, S0{});

    // One register set of fragments, refilled half a step ahead of its use: while slice 0 of stage t
    // multiplies, slice 1 of stage t is read; then the barrier that publishes stage t+1; while slice 1
    // multiplies, slice 0 of stage t+1 is read.  Each read goes into registers whose last consumer
    // has already been issued, and LDS (128 B/clk -- a step's fragment reads take about as long as
    // its MFMAs at this tile shape) runs beside the matrix cores instead of in bursts.
    for (int t = 0; t < T; t++) {
        read_slice(t, S1{});
        multiply(S0{});
        interleave();
        if (t + 1 < T) {
            publish(t + 2 < T ? 1 : 0);
            if (t + P_AHEAD < T) issue(t + P_AHEAD);
            read_slice(t + 1, S0{});
        }
        multiply(S1{});
        interleave();
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

// both operands k-dense, 16-byte aligned, K a whole number of 64-byte stages
template <int CK> bool pipe_eligible(int la, int lb, const DevProduct &g) {
    return la == LM_K && lb == LM_K && g.K > 0 && ((long)g.K * Compute<CK>::ES) % P_ROW_BYTES == 0;
}

}  // namespace mfma
}  // namespace hodu
