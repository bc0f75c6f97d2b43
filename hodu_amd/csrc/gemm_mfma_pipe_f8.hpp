// f8e4m3 x f8e4m3 and f8e5m2 x f8e5m2 products on the native gfx950 8-bit MFMA (v_mfma_scale_f32_32x32x64_f8f6f4
// with unit scales: 64 k per instruction, twice the arithmetic of the bf16 instruction for the same
// operand bytes; the instruction's format fields select e4m3 or e5m2).  hodu's own f8 matmul / dot (lhs, rhs and
// result all of one f8 type; crates/hodu_cpu_kernels/kernels/ops_matrix.c:351-352, :713-714) lands here when both operands are k-dense
// and K is a multiple of 128; products accumulate in f32 and are narrowed once, round-to-nearest-even
// and saturating at +-448 (e5m2: +-57344) like every other f8 product of this library (the reference re-rounds
// its f8 accumulator after every k, ops_matrix.c:572-573).
//
// Same feeding scheme as gemm_mfma_pipe.hpp -- whole 128-byte rows by LDS-DMA into a two-stage ring,
// XOR-swizzled so that fragment reads are conflict-free, one barrier per stage, epilogue through LDS
// -- with one difference forced by the instruction: a lane's operand is 32 bytes (8 VGPRs), so a
// double-buffered set of all fragments would not fit beside the accumulators.  The k loop therefore
// advances in WINDOWS of 64 k (two per stage); within a window the right operand's fragments are all
// resident (double-buffered across windows), the left operand's are streamed through two registers
// sets, each prefetched while the previous one feeds TN MFMAs (256 cycles, more than an LDS round trip).
#pragma once

#include "device_types.hpp"
#include "gemm_mfma_pipe.hpp"

namespace hodu {
namespace mfma {

enum { OUT_F8E4M3 = 4, OUT_F8E5M2 = 5 };

template <> struct Out<OUT_F8E4M3> {
    static constexpr int DT = HODU_F8E4M3;
    typedef uint8_t T;
    // same narrowing as the generic kernel's f8e4m3 products: round to nearest even, saturating at +-448
    static __device__ __forceinline__ T cvt(float v) { return f32_to_f8e4m3_sat(v); }
    static __device__ __forceinline__ uint32_t cvt4(float a, float b, float c, float d) { return f32x4_to_f8e4m3_sat(a, b, c, d); }
};

template <> struct Out<OUT_F8E5M2> {
    static constexpr int DT = HODU_F8E5M2;
    typedef uint8_t T;
    static __device__ __forceinline__ T cvt(float v) { return f32_to_f8e5m2_sat(v); }
    static __device__ __forceinline__ uint32_t cvt4(float a, float b, float c, float d) { return f32x4_to_f8e5m2_sat(a, b, c, d); }
};

struct FragF8 {
    u32x4_t lo, hi;  // 32 consecutive bytes of k
};
typedef int i32x8_t __attribute__((ext_vector_type(8)));
// FMT: the instruction's operand format code, 0 = e4m3, 1 = e5m2 (both operands alike)
template <int FMT> __device__ __forceinline__ void mma_f8(const FragF8 &a, const FragF8 &b, f32x16_t &c) {
    const i32x8_t av = {(int)a.lo.x, (int)a.lo.y, (int)a.lo.z, (int)a.lo.w, (int)a.hi.x, (int)a.hi.y, (int)a.hi.z, (int)a.hi.w};
    const i32x8_t bv = {(int)b.lo.x, (int)b.lo.y, (int)b.lo.z, (int)b.lo.w, (int)b.hi.x, (int)b.hi.y, (int)b.hi.z, (int)b.hi.w};
    // cbsz = blgp = FMT; scale bytes 0x7F = 2^0
    c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
}

// WN_: wavefronts along n (2 along m).  The 256 x 256 tile runs with 2 x 4: two wavefronts share a SIMD, and one's
// LDS reads and DMA issue overlap the other's MFMAs (measured 2410 against 2540 cycles per 128-k stage with 2 x 2, where
// a wavefront owns 128 x 128 outputs and has its SIMD to itself; 2048 is the matrix core's own time).
template <int OUT_, int BM_, int BN_, int PH_ = 50, bool PROBE_ = false, int WN_ = 2> struct PipeF8Config {
    static constexpr int OUT = OUT_, BM = BM_, BN = BN_, WM = 2, WN = WN_, NT = WM * WN * 64, NW = WM * WN, NST = 2;
    // share of a stage's DMA list issued right behind the stage's barrier, in the last quarter of the stage, where the
    // next stage's first fragment reads crowd as well; the rest goes out during the next stage's first half.  Measured
    // cycles per stage of the 2 x 2 tile: 3409 with 100 %, 2755 with 50 %, 2552 with 25 %, 2594 with none.
    static constexpr int PH_PERCENT = PH_;
    static constexpr bool PROBE = PROBE_;    // measurement builds only: per-wavefront cycle stamps around the waits
    static constexpr int A_BYTES = BM * P_ROW_BYTES, B_BYTES = BN * P_ROW_BYTES;
    static constexpr int LDS_BYTES = NST * (A_BYTES + B_BYTES);
    static constexpr int PA = (BM / 8) / NW, PB = (BN / 8) / NW, P = PA + PB;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    static_assert(TM % 2 == 0 && TN % TM == 0 || TM % TN == 0, "window schedule");
    static_assert(TM % 2 == 0, "the streamed left fragments alternate between two register sets");
    static_assert(LDS_BYTES <= 160 * 1024 && NW * 32 * (TN * 128 + 16) <= LDS_BYTES, "LDS budget");
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void mfma_pipe_f8_kernel(const char *__restrict__ A, const char *__restrict__ B,
                                                               typename Out<Cfg::OUT>::T *__restrict__ C, DevProduct g,
                                                               int tiles_m, int tiles_n, int stages_per_split,
                                                               void *__restrict__ partials, int *__restrict__ arrival) {
    HODU_DYNAMIC_LDS(smem);
    typedef typename Out<Cfg::OUT>::T out_t;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, PA = Cfg::PA, PB = Cfg::PB, P = Cfg::P;
    constexpr int TILE_BYTES = 32 * P_ROW_BYTES, B_BASE = 2 * Cfg::A_BYTES;

    const int tid = threadIdx.x, lane = tid & 63;
    // the wavefront's index as a scalar: everything a DMA instruction needs besides the lane's row offset -- the
    // operand's base address, the LDS destination in M0 -- is then wave-uniform and stays in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const int lr = lane & 31, lh = lane >> 5;

    long batch;
    int tm, tn;
    tile_of(blockIdx.x, (long)gridDim.x, tiles_m, tiles_n, batch, tm, tn);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    const unsigned lds0 = (unsigned)(uintptr_t)smem;

    // DMA plan: one instruction = 8 rows x 128 bytes; the slot of a lane holds chunk slot ^ ((row >> 1) & 7).
    // Address = scalar base of the tile's first row (advanced 128 bytes per stage) + the lane's 32-bit offset of
    // its (clamped) row and chunk inside the tile, fixed for the whole launch: a DMA instruction costs one M0
    // write and the load itself, no vector arithmetic.  (The launcher checks that 256 rows stay below 4 GB.)
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
    const int T_all = g.K / P_ROW_BYTES;
    const int t0 = blockIdx.y * stages_per_split;
    const int T = T_all - t0 < stages_per_split ? T_all - t0 : stages_per_split;
    const char *const base_a = uniform_ptr(A + ao + (long)m0 * g.a_m + (long)t0 * P_ROW_BYTES);
    const char *const base_b = uniform_ptr(B + bo + (long)n0 * g.b_n + (long)t0 * P_ROW_BYTES);

    // element e of stage `src`'s issue list (PA of A, then PB of B) into ring slot `slot`
    auto dma_element = [&](int e, int src, int slot) {
#pragma unroll
        for (int p = 0; p < PA; p++)
            if (e == p) dma16_sbase(base_a + (long)src * P_ROW_BYTES, offa[p], lds0 + (unsigned)slot * Cfg::A_BYTES + lda[p]);
#pragma unroll
        for (int p = 0; p < PB; p++)
            if (e == PA + p) dma16_sbase(base_b + (long)src * P_ROW_BYTES, offb[p], lds0 + (unsigned)slot * Cfg::B_BYTES + ldb[p]);
    };

    // fragment addresses: window w, lane (lr, lh) reads bytes 64*w + 32*lh .. +31 of row lr = chunks 4w + 2lh, +1
    int a_fr[2][2], b_fr[2][2];
#pragma unroll
    for (int w = 0; w < 2; w++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int slot = kd_slot(lr, 4 * w + 2 * lh + h) << 4;
            a_fr[w][h] = (wave_m * TM) * TILE_BYTES + lr * P_ROW_BYTES + slot;
            b_fr[w][h] = B_BASE + (wave_n * TN) * TILE_BYTES + lr * P_ROW_BYTES + slot;
        }
    auto read_a = [&](int slot, auto w_, int i) -> FragF8 {
        constexpr int W = decltype(w_)::value;
        const char *buf = smem + slot * Cfg::A_BYTES;
        return FragF8{lds_get(buf, a_fr[W][0] + i * TILE_BYTES), lds_get(buf, a_fr[W][1] + i * TILE_BYTES)};
    };
    auto read_b = [&](int slot, auto w_, int j) -> FragF8 {
        constexpr int W = decltype(w_)::value;
        const char *buf = smem + slot * Cfg::B_BYTES;
        return FragF8{lds_get(buf, b_fr[W][0] + j * TILE_BYTES), lds_get(buf, b_fr[W][1] + j * TILE_BYTES)};
    };

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;

    unsigned long long probe_wait = 0, probe_barrier = 0;
    const unsigned long long probe_start = Cfg::PROBE ? __builtin_amdgcn_s_memtime() : 0;
    FragF8 fbw[2][TN];  // right fragments of the current window and of the next
    FragF8 fa[2];       // left fragments: the one multiplying and the one arriving
    typedef std::integral_constant<int, 0> W0;
    typedef std::integral_constant<int, 1> W1;

    // One window (64 k) of MFMAs.  CUR: this window (its right fragments are in fbw[CUR], left fragment 0 in fa[0]).
    // The next window NXT lives in ring slot `slot_nxt`.  LATE = false: its fragments are prefetched throughout
    // (it is the second window of the same stage).  LATE = true: it belongs to the NEXT stage, which becomes
    // readable only behind this stage's barrier, placed in front of the last left fragment's MFMAs -- everything
    // of this stage has been read by then; the next window's right fragments and first left fragment, and elements
    // [D0, D0 + DN) of the issue list, all go into that last quarter.
    auto window = [&](auto cur_, auto late_, auto d0_, auto dn_, int slot_cur, int slot_nxt, int dma_src, int dma_slot,
                      bool do_dma) {
        constexpr int CUR = decltype(cur_)::value, NXT = CUR ^ 1;
        constexpr bool LATE = decltype(late_)::value;
        constexpr int D0 = decltype(d0_)::value, DN = decltype(dn_)::value;
        typedef std::integral_constant<int, CUR> WC;
        typedef std::integral_constant<int, NXT> WN_;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const bool last = i == TM - 1;
            if (LATE && last) {
                // stage t+1 has landed, every read of stage t has returned
                if constexpr (Cfg::PROBE) {
                    const unsigned long long c0 = __builtin_amdgcn_s_memtime();
                    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
                    const unsigned long long c1 = __builtin_amdgcn_s_memtime();
                    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
                    __builtin_amdgcn_s_barrier();
                    const unsigned long long c2 = __builtin_amdgcn_s_memtime();
                    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
                    probe_wait += c1 - c0;
                    probe_barrier += c2 - c1;
                } else {
                    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
                    __builtin_amdgcn_s_barrier();
                }
                asm volatile("" ::: "memory");
            }
            if (!last) fa[(i + 1) & 1] = read_a(slot_cur, WC{}, i + 1);
            else fa[(i + 1) & 1] = read_a(slot_nxt, WN_{}, 0);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                // the next window's right fragments: spread over the window, or bunched behind the barrier
                const bool due = LATE ? last : (j * TM / TN == i);
                if (due) fbw[NXT][j] = read_b(slot_nxt, WN_{}, j);
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                mma_f8<Cfg::OUT == OUT_F8E5M2 ? 1 : 0>(fbw[CUR][j], fa[i & 1], acc[i][j]);
                // DMA: in a LATE window only behind the barrier; otherwise spread over all MFMAs
                constexpr int SLOTS = LATE ? TN : TM * TN;
                const int pos = LATE ? j : i * TN + j;
                if (!LATE || last) {
#pragma unroll
                    for (int d = 0; d < DN; d++)
                        if (d * SLOTS / (DN > 0 ? DN : 1) == pos && do_dma) dma_element(D0 + d, dma_src, dma_slot);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    constexpr int PH = P * Cfg::PH_PERCENT / 100;  // issued behind the barrier of the stage; the rest during the next stage's first window
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, PH> DH;
    typedef std::integral_constant<int, P - PH> DR;
    typedef std::integral_constant<bool, false> EARLY;
    typedef std::integral_constant<bool, true> LATE;

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
    fa[0] = read_a(0, W0{}, 0);
#pragma unroll
    for (int j = 0; j < TN; j++) fbw[0][j] = read_b(0, W0{}, j);

    int slot = 0;
    int pend_src = 0, pend_slot = 0;
    bool pend = false;
    for (int t = 0; t < T; t++) {
        // window 0: the rest of the previous stage's issue list goes out here
        window(W0{}, EARLY{}, DH{}, DR{}, slot, slot, pend_src, pend_slot, pend);
        // window 1: behind its barrier, stage t + 2 (clamped: the in-flight count stays constant) goes into this slot
        pend_src = t + 2 < T ? t + 2 : T - 1;
        pend_slot = slot;
        pend = true;
        window(W1{}, LATE{}, I0{}, DH{}, slot, slot ^ 1, pend_src, pend_slot, true);
        slot ^= 1;
    }
    // the clamped re-fetches still write LDS: wait for them, then for everybody's, before LDS is reused
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
    if constexpr (Cfg::PROBE) {
        // measurement builds: `partials` is the stamp buffer, four words per wavefront
        if (lane == 0) {
            unsigned long long *w = (unsigned long long *)partials + ((long)blockIdx.x * Cfg::NW + wave) * 4;
            w[0] = __builtin_amdgcn_s_memtime() - probe_start;
            w[1] = probe_wait;
            w[2] = probe_barrier;
            w[3] = (unsigned long long)T;
        }
    }

    char *patch = smem + wave * (32 * (TN * 32 * 4 + 16));
    if (!Cfg::PROBE && gridDim.y > 1 && arrival != nullptr) {
        // cut along K, summed here: only the workgroup that arrives last stores the tile
        if (!splitk_exchange<Cfg::NW, TM, TN>(acc, partials, arrival, reinterpret_cast<int *>(smem + Cfg::LDS_BYTES - 16), tid)) return;
        __syncthreads();
    } else if (!Cfg::PROBE && gridDim.y > 1) {
        float *Pb = (float *)partials + ((long)blockIdx.y * g.batches + batch) * (long)g.M * g.N;
#pragma unroll
        for (int i = 0; i < TM; i++)
            store_band_via_lds<OUT_F32, TN, false>(patch, Pb, acc[i], m0 + wave_m * TM * 32 + i * 32, n0 + wave_n * TN * 32, lane, g.M, g.N, g.epi);
        return;
    }
    out_t *Cb = C + batch * (long)g.M * g.N;
#pragma unroll
    for (int i = 0; i < TM; i++)
        store_band_via_lds<Cfg::OUT, TN, false>(patch, Cb, acc[i], m0 + wave_m * TM * 32 + i * 32, n0 + wave_n * TN * 32, lane, g.M, g.N, g.epi);
}

template <class Cfg>
int launch_pipe_f8(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g, int splits) {
    auto kernel = mfma_pipe_f8_kernel<Cfg>;
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES)) return rc;
    const int tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    const long total = g.batches * tiles_m * tiles_n;
    if (total > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", total);
    const int T = (int)(g.K / P_ROW_BYTES);
    int per = T;
    void *partials = nullptr;
    if (splits > 1) {
        per = (T + splits - 1) / splits;
        splits = (T + per - 1) / per;
    }
    const long elems = g.batches * (long)g.M * g.N;
    const bool in_kernel = splits > 1 && total <= kArrivalSlots;  // as in launch_pipe
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
        hipLaunchKernelGGL((splitk_reduce_kernel<Cfg::OUT, float>), dim3(blocks), dim3(256), 0, ctx->stream,
                           (const float *)partials, (typename Out<Cfg::OUT>::T *)c, elems, splits, g.N, g.epi);
        HODU_HIP(hipGetLastError());
    }
    return HODU_ROCM_OK;
}

}  // namespace mfma
}  // namespace hodu
