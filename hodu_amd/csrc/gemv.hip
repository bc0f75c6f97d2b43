// Decode-shape products with 1..4 rows on the left: y[m, n] = sum_k x[m, k] * W[n, k], W k-dense
// (`input.matmul(weight.transpose(-2, -1))`, crates/hodu_nn/src/modules/linear.rs:38-47), bf16
// activations against bf16 or f8e4m3 weights.  Replaces the single-thread M < 512 path of
// hodu_cpu_dot_bf16 (kernels/ops_matrix.c:486-548) for the shape where only the weight bytes matter.
//
// Pure streaming: a wavefront owns R whole weight rows and reads each one as consecutive 1 KB
// pieces (64 lanes x 16 bytes: every request is whole cache lines of one row).  All loads of a
// wavefront -- R rows x up to 4 KB -- are issued before the first is consumed, so with a few
// wavefronts per SIMD a compute unit keeps tens of KB in flight and the kernel is one memory
// latency plus the transfer.  The arithmetic rides on the vector ALU: f8e4m3 pairs widen to bf16
// pairs (v_cvt_scalef32_pk_bf16_fp8, exact) and v_dot2_f32_bf16 accumulates in f32; the 64 partial
// sums of an output meet through DPP row operations, and the sum is rounded once to bf16.
//
// Measured alternatives that did not pay on 4096 x 4096 f8e4m3 weights (4.9 us as built): staging the
// activations in LDS (+0.7 us: a barrier in front of the first multiply), renumbering workgroups so
// that one XCD writes whole output lines (+0.1 us), four rows per wavefront (+0.3 us).  Non-temporal
// weight loads did pay (5.1 -> 4.9 us).  A kernel that only reads the same 16.8 MB, in any of five
// shapes of grid and loads in flight, takes 3.9-4.3 us, an empty kernel launches every 1.3-2.4 us
// (it varies from machine to machine), and about 0.3 us is the acknowledged output store.
#include "common.hpp"
#include "device_types.hpp"
#include "gemm_mfma.hpp"

namespace hodu {
namespace {

using mfma::bitcast;
using mfma::SK_F8;
using mfma::SK_SAME;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int GEMV_NCH = 4;    // 1 KB pieces of a row in flight per row

template <int SKB> struct WeightVec {
    static constexpr int EPL = SKB == SK_F8 ? 16 : 8;  // elements in one 16-byte lane load
    static constexpr int XV = EPL / 8;                  // 16-byte vectors of bf16 activations matching it
};

// acc += dot(w (EPL elements), x (EPL bf16))
template <int SKB>
__device__ __forceinline__ float dot16(const u32x4_t &w, const u32x4_t *x, float acc) {
    if constexpr (SKB == SK_F8) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const bf16x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[q], 1.0f, false);
            const bf16x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[q], 1.0f, true);
            // 16 bytes of f8 = elements 4q..4q+3 in word q; x[0] holds bf16 0..7, x[1] holds 8..15
            acc = __builtin_amdgcn_fdot2_f32_bf16(lo, bitcast<bf16x2_t>(x[q >> 1][(2 * q) & 3]), acc, false);
            acc = __builtin_amdgcn_fdot2_f32_bf16(hi, bitcast<bf16x2_t>(x[q >> 1][(2 * q + 1) & 3]), acc, false);
        }
    } else {
#pragma unroll
        for (int q = 0; q < 4; q++)
            acc = __builtin_amdgcn_fdot2_f32_bf16(bitcast<bf16x2_t>(w[q]), bitcast<bf16x2_t>(x[0][q]), acc, false);
    }
    return acc;
}

// sum over the 64 lanes of a wavefront, result in every lane: four DPP steps inside each row of 16
// lanes (a few cycles each, no LDS round trips), then the four row sums through scalar registers
__device__ __forceinline__ float wave_sum(float v) {
    int x = bitcast<int>(v);
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    x = bitcast<int>(v);
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    x = bitcast<int>(v);
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, x, 0x141, 0xF, 0xF, true));  // row_half_mirror
    x = bitcast<int>(v);
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, x, 0x140, 0xF, 0xF, true));  // row_mirror
    x = bitcast<int>(v);
    return bitcast<float>(__builtin_amdgcn_readlane(x, 0)) + bitcast<float>(__builtin_amdgcn_readlane(x, 16)) +
           bitcast<float>(__builtin_amdgcn_readlane(x, 32)) + bitcast<float>(__builtin_amdgcn_readlane(x, 48));
}

// second launch bound: wavefronts per SIMD to leave room for (caps the register budget at 128 for M <= 2)
template <int SKB, int M, int R, int NW>
__global__ __launch_bounds__(NW * 64, (M <= 2 ? 4 : 2)) void gemv_rowstream_kernel(const char *__restrict__ X,
                                                                                  const char *__restrict__ W,
                                                                                  uint16_t *__restrict__ Y, int N, int K,
                                                                                  long x_row_bytes, long w_row_bytes,
                                                                                  DevEpilogue epi) {
    constexpr int EPL = WeightVec<SKB>::EPL, XV = WeightVec<SKB>::XV, SB = SKB == SK_F8 ? 1 : 2;
    constexpr int STEP = GEMV_NCH * 64 * EPL;  // k covered by one pass of a wavefront
    const int tid = threadIdx.x, lane = tid & 63;
    const int n0 = (blockIdx.x * NW + (tid >> 6)) * R;

    float acc[M][R];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[m][r] = 0.f;

    const char *wrow[R];  // rows past N repeat the last one; their results are not stored
#pragma unroll
    for (int r = 0; r < R; r++) wrow[r] = W + (long)(n0 + r < N ? n0 + r : N - 1) * w_row_bytes;

    auto load_weights = [&](int kc, u32x4_t (&wv)[R][GEMV_NCH]) {
#pragma unroll
        for (int c = 0; c < GEMV_NCH; c++) {
            const int k = kc + (c * 64 + lane) * EPL;
#pragma unroll
            for (int r = 0; r < R; r++) {
                wv[r][c] = u32x4_t{0u, 0u, 0u, 0u};
                // (read once, by this wavefront alone: the non-temporal hint keeps the weight stream from evicting the
                // activations every wavefront re-reads out of L2)
                if (k < K) wv[r][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(wrow[r] + (long)k * SB));
            }
        }
    };
    auto multiply = [&](const u32x4_t (&wv)[R][GEMV_NCH], const u32x4_t (&xv)[M][GEMV_NCH][XV]) {
#pragma unroll
        for (int c = 0; c < GEMV_NCH; c++)
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int m = 0; m < M; m++) acc[m][r] = dot16<SKB>(wv[r][c], xv[m][c], acc[m][r]);
    };

    for (int kc = 0; kc < K; kc += STEP) {
        u32x4_t wv[R][GEMV_NCH], xv[M][GEMV_NCH][XV];
        // activations first (issue order is return order), then the weights
#pragma unroll
        for (int c = 0; c < GEMV_NCH; c++) {
            const int k = kc + (c * 64 + lane) * EPL;
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int v = 0; v < XV; v++) {
                    xv[m][c][v] = u32x4_t{0u, 0u, 0u, 0u};
                    if (k < K) xv[m][c][v] = *reinterpret_cast<const u32x4_t *>(X + m * x_row_bytes + (long)k * 2 + v * 16);
                }
        }
        load_weights(kc, wv);
        multiply(wv, xv);
    }

    // the R results of a row of x leave in one store instruction: lane r writes column n0 + r
#pragma unroll
    for (int m = 0; m < M; m++) {
        float mine = 0.f;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float v = wave_sum(acc[m][r]);
            mine = lane == r ? v : mine;
        }
        if (lane < R && n0 + lane < N) Y[(long)m * N + n0 + lane] = mfma::finish<mfma::OUT_BF16>(epi, mine, n0 + lane);
    }
}

// The same product for weights with many rows (N >= 16 per compute unit): one wavefront per SIMD walks groups of R
// rows, group g, g + (wavefronts in the grid), ... -- the wavefronts together sweep a contiguous window of rows
// through the weight matrix -- with the next group's weight loads issued before the current group is multiplied and
// reduced, so the memory pipe does not drain between groups, and (K within one pass) the activations loaded once per
// wavefront instead of once per row group: with one-shot wavefronts x crosses the L2 -> CU path as often as there
// are row groups, as many bytes as the weights themselves.  No load sits behind a branch.
// Measured on f8e4m3 weights, M = 1: 14336 x 4096 11.0 -> 10.7 us (a kernel that only reads those bytes: 10.0),
// 4096 x 4096 4.9 -> 4.8 us (3.9); two to four wavefronts per SIMD with fewer groups each measured the same.
//   MULTI: K takes several passes of NCH KB per lane-row; the items are (group, pass) pairs, a group's passes back to
//   back, the activations of a pass travel with its weights.
template <int SKB, int M, int R, int NCH, bool MULTI, int NW>
__global__ __launch_bounds__(NW * 64, 1) void gemv_walk_kernel(const char *__restrict__ X, const char *__restrict__ W,
                                                                uint16_t *__restrict__ Y, int N, int K, long x_row_bytes,
                                                                long w_row_bytes, int groups, int passes, DevEpilogue epi) {
    constexpr int EPL = WeightVec<SKB>::EPL, XV = WeightVec<SKB>::XV, SB = SKB == SK_F8 ? 1 : 2;
    constexpr int STEP = NCH * 64 * EPL;  // k covered by one pass of a wavefront
    const int tid = threadIdx.x, lane = tid & 63;
    const int total = gridDim.x * NW;
    int g = blockIdx.x * NW + (tid >> 6), p = 0;
    if (g >= groups) return;

    typedef u32x4_t wbuf_t[R][NCH];
    typedef u32x4_t xbuf_t[M][NCH][XV];
    wbuf_t wa, wb;
    xbuf_t xa, xb;
    float acc[M][R];

    // Every load is unconditional -- a lane whose k lies past K reads the row's last vector instead and the weights
    // it fetched are replaced by zeros afterwards (selects, no branches: a branch around each load makes the compiler
    // wait for one load before it issues the next, which serialises the whole stream)
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    auto load_x = [&](int pass, xbuf_t &xv) {
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const int k = pass * STEP + (c * 64 + lane) * EPL, kk = k < K ? k : K - EPL;
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int v = 0; v < XV; v++)
                    xv[m][c][v] = *reinterpret_cast<const u32x4_t *>(X + m * x_row_bytes + (long)kk * 2 + v * 16);
        }
    };
    auto load_w = [&](int group, int pass, wbuf_t &wv) {
        const char *wrow[R];  // rows past N repeat the last one; their results are not stored
#pragma unroll
        for (int r = 0; r < R; r++) wrow[r] = W + (long)(group * R + r < N ? group * R + r : N - 1) * w_row_bytes;
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const int k = pass * STEP + (c * 64 + lane) * EPL, kk = k < K ? k : K - EPL;
#pragma unroll
            for (int r = 0; r < R; r++)
                wv[r][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(wrow[r] + (long)kk * SB));
        }
    };
    auto work = [&](int group, int pass, const wbuf_t &wv, const xbuf_t &xv) {
        if (pass == 0) {
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int r = 0; r < R; r++) acc[m][r] = 0.f;
        }
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const bool live = pass * STEP + (c * 64 + lane) * EPL < K;
#pragma unroll
            for (int r = 0; r < R; r++) {
                const u32x4_t wlive = live ? wv[r][c] : zero;
#pragma unroll
                for (int m = 0; m < M; m++) acc[m][r] = dot16<SKB>(wlive, xv[m][c], acc[m][r]);
            }
        }
        if (pass + 1 < passes) return;
        const int n0 = group * R;
#pragma unroll
        for (int m = 0; m < M; m++) {
            float mine = 0.f;
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float v = wave_sum(acc[m][r]);
                mine = lane == r ? v : mine;
            }
            if (lane < R && n0 + lane < N) Y[(long)m * N + n0 + lane] = mfma::finish<mfma::OUT_BF16>(epi, mine, n0 + lane);
        }
    };
    auto advance = [&](int &group, int &pass) {
        if (MULTI && pass + 1 < passes) pass++;
        else { pass = 0; group += total; }
    };

    // items of this wavefront: its row groups g, g + total, ... times the passes of each.  The steady-state loop
    // handles two items per trip with both prefetches unconditional (so nothing in it branches around a load and the
    // pending loads at its head are the same on entry and on the back edge); the last one or two items follow it.
    const int items = ((groups - g + total - 1) / total) * (MULTI ? passes : 1);
    int g1 = g, p1 = p;  // the item whose loads are issued next
    auto fetch = [&](wbuf_t &wv, xbuf_t &xv) {
        advance(g1, p1);
        if constexpr (MULTI) load_x(p1, xv);
        load_w(g1, p1, wv);
    };
    auto step = [&](const wbuf_t &wv, const xbuf_t &xv) {
        // (the loads just issued stay in front of the multiply: the scheduler would otherwise pull the multiply's
        // first instructions, and with them the wait for the current item's data, ahead of them)
        __builtin_amdgcn_sched_barrier(0);
        work(g, p, wv, xv);
        advance(g, p);
        __builtin_amdgcn_sched_barrier(0);
    };
    load_x(0, xa);
    load_w(g, 0, wa);
    int i = 0;
    for (; i + 2 < items; i += 2) {
        fetch(wb, xb);
        step(wa, xa);
        fetch(wa, xa);
        step(wb, MULTI ? xb : xa);
    }
    if (items - i == 2) {
        fetch(wb, xb);
        step(wa, xa);
        step(wb, MULTI ? xb : xa);
    } else {
        step(wa, xa);
    }
}

template <int SKB, int M, int NCH, bool MULTI>
int launch_walk(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g) {
    constexpr int ES = 2, SB = SKB == SK_F8 ? 1 : 2, R = 2, NW = 4;
    constexpr int STEP = NCH * 64 * WeightVec<SKB>::EPL;
    const char *X = (const char *)x + g.a_off * ES;
    const char *Wp = (const char *)w + g.b_off * SB;
    const long groups = (g.N + R - 1) / R;
    const long simds = 4L * ctx->props.multiProcessorCount;
    const long waves = groups < simds ? groups : simds;
    const unsigned blocks = (unsigned)((waves + NW - 1) / NW);
    const int passes = (int)((g.K + STEP - 1) / STEP);
    hipLaunchKernelGGL((gemv_walk_kernel<SKB, M, R, NCH, MULTI, NW>), dim3(blocks), dim3(NW * 64), 0, ctx->stream, X, Wp,
                       (uint16_t *)y, g.N, g.K, g.a_m * (long)ES, g.b_n * (long)SB, (int)groups, passes, g.epi);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

// one pass where K fits 4 or 8 chunks of 64 lanes x 16 bytes, several passes of 4 chunks beyond that
template <int SKB, int M>
int launch_walk_for(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g) {
    constexpr int STEP4 = 4 * 64 * WeightVec<SKB>::EPL;
    if (g.K <= STEP4) return launch_walk<SKB, M, 4, false>(ctx, x, w, y, g);
    if (g.K <= 2 * STEP4) return launch_walk<SKB, M, 8, false>(ctx, x, w, y, g);
    return launch_walk<SKB, M, 4, true>(ctx, x, w, y, g);
}

template <int SKB, int M, int R, int NW>
int launch_one(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g) {
    constexpr int ES = 2, SB = SKB == SK_F8 ? 1 : 2;
    const char *X = (const char *)x + g.a_off * ES;
    const char *Wp = (const char *)w + g.b_off * SB;
    const long waves = (g.N + R - 1) / R;
    const unsigned blocks = (unsigned)((waves + NW - 1) / NW);
    hipLaunchKernelGGL((gemv_rowstream_kernel<SKB, M, R, NW>), dim3(blocks), dim3(NW * 64), 0, ctx->stream, X, Wp,
                       (uint16_t *)y, g.N, g.K, g.a_m * (long)ES, g.b_n * (long)SB, g.epi);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

// shape: 0 = 4 wavefronts x 1 row each, 1 = 4 x 2, 2 = 8 x 2
template <int SKB, int M>
int launch_rows(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g, int shape) {
    if (shape == 0) return launch_one<SKB, M, 1, 4>(ctx, x, w, y, g);
    if (shape == 1) return launch_one<SKB, M, 2, 4>(ctx, x, w, y, g);
    return launch_one<SKB, M, 2, 8>(ctx, x, w, y, g);
}

template <int SKB>
int run_gemv(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g, const char *name) {
    constexpr int ES = 2, SB = SKB == SK_F8 ? 1 : 2, EPL = WeightVec<SKB>::EPL;
    // applicability: one product, both operands k-dense, every 16-byte vector load aligned and inside its row
    auto al = [](long elems, int bytes) { return (elems * bytes) % 16 == 0; };
    if (g.M < 1 || g.M > 4 || g.batches != 1 || g.K % EPL != 0) return HODU_ROCM_UNSUPPORTED;
    if (g.a_k != 1 || g.b_k != 1) return HODU_ROCM_UNSUPPORTED;
    if (!(g.M == 1 || al(g.a_m, ES)) || !(g.N == 1 || al(g.b_n, SB))) return HODU_ROCM_UNSUPPORTED;
    if (((uintptr_t)x + (uintptr_t)g.a_off * ES) % 16 || ((uintptr_t)w + (uintptr_t)g.b_off * SB) % 16)
        return HODU_ROCM_UNSUPPORTED;
    // two rows per wavefront (activation registers shared by both) once that still leaves every compute
    // unit two workgroups; measured on 4096 x 4096 f8 weights, 4 x 1, 4 x 2 and 8 x 2 are within 3 %
    const long cus = ctx->props.multiProcessorCount;
    int shape = g.N >= 16 * cus ? 1 : 0;
    if (ctx->force_tile == 31) shape = 0;
    if (ctx->force_tile == 32) shape = 1;
    if (ctx->force_tile == 34) shape = 2;
    ctx->last_kernel = name;
    // many rows: the walking kernel (one wavefront per SIMD, weights of the next row group in flight)
    const bool walk = ctx->force_tile == 33 || (ctx->force_tile < 0 && g.N >= 16 * cus && g.N < (1L << 30));
    if (walk) {
        ctx->last_kernel = SKB == SK_F8 ? "gemv_bf16_f8w_walk" : "gemv_bf16_walk";
        switch (g.M) {
        case 1: return launch_walk_for<SKB, 1>(ctx, x, w, y, g);
        case 2: return launch_walk_for<SKB, 2>(ctx, x, w, y, g);
        case 3: return launch_walk_for<SKB, 3>(ctx, x, w, y, g);
        default: return launch_walk_for<SKB, 4>(ctx, x, w, y, g);
        }
    }
    switch (g.M) {
    case 1: return launch_rows<SKB, 1>(ctx, x, w, y, g, shape);
    case 2: return launch_rows<SKB, 2>(ctx, x, w, y, g, shape);
    case 3: return launch_rows<SKB, 3>(ctx, x, w, y, g, shape);
    default: return launch_rows<SKB, 4>(ctx, x, w, y, g, shape);
    }
}

}  // namespace

int launch_gemv(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    if (g.M > 4 || g.K == 0) return HODU_ROCM_UNSUPPORTED;
    if (kind == PK_BF16_F8W) return run_gemv<SK_F8>(ctx, a, b, c, g, "gemv_bf16_f8w");
    if (kind == PK_SAME && dtype == HODU_BF16) return run_gemv<SK_SAME>(ctx, a, b, c, g, "gemv_bf16");
    return HODU_ROCM_UNSUPPORTED;
}

}  // namespace hodu
