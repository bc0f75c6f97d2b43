// f64 products on the matrix cores (v_mfma_f64_16x16x4_f64): the reference multiplies f64 in f64
// (hodu_cpu_matmul_f64 / hodu_cpu_dot_f64, kernels/ops_matrix.c:486-548, plain sequential accumulation), and so does
// the MFMA's FMA chain -- only the order of the k differs.
//
// The instruction takes ONE double per lane and operand (lane l: row l % 16, k = l / 16) and runs for 64 cycles, so a
// wavefront needs 16 bytes of operands per lane every 64 cycles: far below what the vector memory pipeline delivers,
// and nothing has to be transposed.  Operands therefore go from memory straight into the MFMA's registers -- no LDS, no
// barriers:
//   * a workgroup is 2 x 2 wavefronts, a wavefront owns TM x TN tiles of 16 x 16 outputs (64 x 64 for large products,
//     32 x 32 and 16 x 16 for smaller ones, so that every compute unit gets a workgroup; neighbouring wavefronts share
//     operand rows through the caches);
//   * k is fed in chunks of 8: lane (r, q) takes k0 + 2 q and k0 + 2 q + 1 of row r -- one 16-byte load where the
//     operand is k-dense, two 8-byte loads (16 lanes = one 128-byte line) where it is row-dense; both operands use
//     the same order, which is all the sum needs;
//   * the fragments of the next chunks are in flight while this one multiplies (a ring of DEPTH chunks);
//   * lane (r, q) ends with column n0 + r, rows m0 + 4 e + q of each tile (register e): the fused element-wise steps,
//     then stores of which sixteen lanes fill 128 consecutive bytes of a row.
#include "common.hpp"
#include "device_types.hpp"
#include "epilogue.hpp"

namespace hodu {
namespace {

typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef f64x2 f64x2_any __attribute__((aligned(8)));  // 16-byte load from an 8-byte-aligned address

// Two consecutive k of one row (or column) of an operand: `p` points at element (row, k), ks is the k stride
template <bool KDENSE> __device__ __forceinline__ f64x2 load_k2(const double *p, long ks) {
    if constexpr (KDENSE) return *reinterpret_cast<const f64x2_any *>(p);
    return f64x2{p[0], p[ks]};
}

template <int TM, int TN, int DEPTH, bool A_KDENSE, bool B_KDENSE>
__global__ __launch_bounds__(256) void gemm_f64_kernel(const double *__restrict__ A, const double *__restrict__ B,
                                                       double *__restrict__ C, DevProduct g, int tiles_m, int tiles_n) {
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 15, lq = lane >> 4;
    // consecutive workgroups walk down a column of tiles: they share the right operand's rows
    const long per_batch = (long)tiles_m * tiles_n;
    const long batch = blockIdx.x / per_batch;
    const int t = (int)(blockIdx.x % per_batch);
    const int m0 = (t % tiles_m) * BM + (wave >> 1) * (TM * 16), n0 = (t / tiles_m) * BN + (wave & 1) * (TN * 16);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    // rows past the edge are clamped: they are multiplied like the others and not stored
    const double *ap[TM], *bp[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + 16 * i + lr;
        ap[i] = A + ao + (long)(m < g.M ? m : g.M - 1) * g.a_m + 2 * lq * g.a_k;
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + 16 * j + lr;
        bp[j] = B + bo + (long)(n < g.N ? n : g.N - 1) * g.b_n + 2 * lq * g.b_k;
    }

    f64x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = f64x4{0., 0., 0., 0.};

    const int chunks = g.K / 8;  // whole chunks; the rest of K follows with guarded loads
    f64x2 af[DEPTH][TM], bf[DEPTH][TN];
    auto fetch = [&](int slot, int c) {  // chunk c (clamped to the last whole one: a harmless re-read)
        const long k = (long)(c < chunks ? c : chunks - 1) * 8;
#pragma unroll
        for (int i = 0; i < TM; i++) af[slot][i] = load_k2<A_KDENSE>(ap[i] + k * g.a_k, g.a_k);
#pragma unroll
        for (int j = 0; j < TN; j++) bf[slot][j] = load_k2<B_KDENSE>(bp[j] + k * g.b_k, g.b_k);
    };
    auto multiply = [&](const f64x2 (&a2)[TM], const f64x2 (&b2)[TN]) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a2[i][h], b2[j][h], acc[i][j], 0, 0, 0);
    };
    if (chunks > 0) {
#pragma unroll
        for (int s = 0; s < DEPTH; s++) fetch(s, s);
        int c = 0;
        for (; c + DEPTH <= chunks; c += DEPTH) {
            if (c + DEPTH < chunks) {
#pragma unroll
                for (int s = 0; s < DEPTH; s++) {
                    multiply(af[s], bf[s]);
                    fetch(s, c + DEPTH + s);
                }
            } else {  // nothing left to fetch
#pragma unroll
                for (int s = 0; s < DEPTH; s++) multiply(af[s], bf[s]);
            }
        }
        const int rest = chunks - c;
#pragma unroll
        for (int s = 0; s < DEPTH; s++)
            if (s < rest) multiply(af[s], bf[s]);
    }
    if (chunks * 8 < g.K) {  // the last k, fewer than 8: element loads, zeros past the end
        f64x2 a2[TM], b2[TN];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int k = chunks * 8 + 2 * lq + h;
            const long rel = (long)chunks * 8 + h;  // (the pointers already stand at 2 q)
#pragma unroll
            for (int i = 0; i < TM; i++) a2[i][h] = k < g.K ? ap[i][rel * g.a_k] : 0.;
#pragma unroll
            for (int j = 0; j < TN; j++) b2[j][h] = k < g.K ? bp[j][rel * g.b_k] : 0.;
        }
        multiply(a2, b2);
    }

    // ---- lane (r, q) holds, of tile (i, j), rows m0 + 16 i + 4 e + q (e = 0..3) of column n0 + 16 j + r: sixteen lanes
    // store 128 consecutive bytes of a row ----
    double *Cb = C + batch * (long)g.M * g.N;
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int col = n0 + 16 * j + lr;
        if (col >= g.N) continue;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int row = m0 + 16 * i + 4 * e + lq;
                if (row >= g.M) continue;
                double v = acc[i][j][e];
                if (g.epi.n != 0) v = epilogue_apply<HODU_F64>(g.epi, v, col);
                Cb[(long)row * g.N + col] = v;
            }
    }
}

template <int TM, int TN, int DEPTH>
int run_f64(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g, const char *const (&names)[4]) {
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    const long tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN, tiles = g.batches * tiles_m * tiles_n;
    if (tiles > 0x7fffffffL) return HODU_ROCM_UNSUPPORTED;
    const bool ak = g.a_k == 1, bk = g.b_k == 1;
    auto go = [&](auto kernel, const char *name) {
        ctx->last_kernel = name;
        hipLaunchKernelGGL(kernel, dim3((unsigned)tiles), dim3(256), 0, ctx->stream, (const double *)a, (const double *)b,
                           (double *)c, g, (int)tiles_m, (int)tiles_n);
    };
    if (ak && bk) go(gemm_f64_kernel<TM, TN, DEPTH, true, true>, names[0]);
    else if (ak) go(gemm_f64_kernel<TM, TN, DEPTH, true, false>, names[1]);
    else if (bk) go(gemm_f64_kernel<TM, TN, DEPTH, false, true>, names[2]);
    else go(gemm_f64_kernel<TM, TN, DEPTH, false, false>, names[3]);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace

// Every f64 product: thin ones (a few rows or columns, a matrix times a vector) included -- their tiles are mostly
// padding, but the operands still arrive as whole cache lines, [1, 4096] x [4096, 4096] in 58 us where the generic
// kernel takes 664.
int launch_gemm_f64(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    if (kind != PK_SAME || dtype != HODU_F64 || g.M < 1 || g.N < 1 || g.K < 1 || g.batches < 1) return HODU_ROCM_UNSUPPORTED;
    if (ctx->force_tile >= 0 && (ctx->force_tile < 41 || ctx->force_tile > 43)) return HODU_ROCM_UNSUPPORTED;
    static const char *const big[4] = {"mfma_f64_128x128_KK", "mfma_f64_128x128_KM", "mfma_f64_128x128_MK", "mfma_f64_128x128_MM"};
    static const char *const small[4] = {"mfma_f64_64x64_KK", "mfma_f64_64x64_KM", "mfma_f64_64x64_MK", "mfma_f64_64x64_MM"};
    static const char *const tiny[4] = {"mfma_f64_32x32_KK", "mfma_f64_32x32_KM", "mfma_f64_32x32_MK", "mfma_f64_32x32_MM"};
    const int cus = ctx->props.multiProcessorCount;
    auto tiles = [&](long bm) { return g.batches * ((g.M + bm - 1) / bm) * ((g.N + bm - 1) / bm); };
    // the largest tile that still gives every compute unit a workgroup
    const int size = ctx->force_tile >= 0 ? ctx->force_tile - 41 : tiles(128) >= cus ? 0 : tiles(64) >= cus ? 1 : 2;
    if (size == 0) return run_f64<4, 4, 2>(ctx, a, b, c, g, big);
    if (size == 1) return run_f64<2, 2, 4>(ctx, a, b, c, g, small);
    return run_f64<1, 1, 8>(ctx, a, b, c, g, tiny);
}

}  // namespace hodu
