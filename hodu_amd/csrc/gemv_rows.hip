// Products with at most 16 rows on the left against a ROW-dense right operand: y[m, n] = sum_k x[m, k] * W[k, n],
// W stored [K, N] with N contiguous (`x.matmul(w)` with the weight as it lies in memory; Tensor::dot_2d passes both
// layouts through unchanged, crates/hodu_core/src/tensor/ops/matrix.rs:323-324, :350-354).  The reference walks this
// case with one thread for M < 512 (kernels/ops_matrix.c:486-548).  Only the weight bytes matter, so the kernel is
// a weighted sum of W's rows:
//   * a lane owns V neighbouring output columns (16 bytes of a weight row: whole cache lines per wavefront);
//   * K is cut into chunks; a workgroup is one (64 * V columns, chunk) pair and its four wavefronts take every
//     fourth k-row of the chunk, a few rows in flight each; the chunk's x values sit in LDS as f32 (one broadcast
//     read per k and row of x);
//   * the four wavefronts meet in LDS, the chunk's partial sums (f32) go to the context's workspace, and a second
//     kernel adds the chunks in a fixed order, applies the fused element-wise steps and rounds once.
// bf16, f16 and f32; f32 accumulation of exact products, as everywhere.
#include "common.hpp"
#include "device_types.hpp"
#include "gemm_mfma.hpp"

namespace hodu {
namespace {

using mfma::finish;
using mfma::Out;

// one product kind: how x and W are stored, what they accumulate in
struct RowsBf16 {
    typedef uint16_t XS; typedef uint16_t WS; typedef float A;
    static constexpr int OUT = mfma::OUT_BF16;
    static __device__ __forceinline__ float x(XS v) { return bf16_bits_to_f32(v); }
    static __device__ __forceinline__ float w(WS v) { return bf16_bits_to_f32(v); }
};
struct RowsF16 {
    typedef uint16_t XS; typedef uint16_t WS; typedef float A;
    static constexpr int OUT = mfma::OUT_F16;
    static __device__ __forceinline__ float x(XS v) { return f16_bits_to_f32(v); }
    static __device__ __forceinline__ float w(WS v) { return f16_bits_to_f32(v); }
};
struct RowsF32 {
    typedef float XS; typedef float WS; typedef float A;
    static constexpr int OUT = mfma::OUT_F32;
    static __device__ __forceinline__ float x(XS v) { return v; }
    static __device__ __forceinline__ float w(WS v) { return v; }
};
// MT: rows of x handled (M rounded up; the rows past M multiply by zero); V: columns per lane
template <class T, int MT, int V>
__global__ __launch_bounds__(256) void gemv_rows_kernel(const typename T::XS *__restrict__ x, const typename T::WS *__restrict__ w,
                                                       typename T::A *__restrict__ partial, int M, int N, int K, long a_m,
                                                       long a_k, long b_k, int per_chunk) {
    typedef typename T::A A;
    typedef typename T::WS WS;
    struct alignas(sizeof(WS) * V) Vec { WS e[V]; };
    HODU_DYNAMIC_LDS(smem);
    A *xs = reinterpret_cast<A *>(smem);  // [per_chunk][MT]; later [3][64][MT * V] for the wavefronts to meet
    // weight rows a wavefront has loads out for at a time: deep where the accumulators leave the registers for it
    constexpr int RIF = MT * V <= 32 ? 8 : 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int begin = blockIdx.y * per_chunk;
    const int rows = K - begin < per_chunk ? K - begin : per_chunk;
    for (int i = tid; i < rows * MT; i += 256) {
        const int r = i / MT, m = i % MT;
        xs[i] = m < M ? T::x(x[(long)m * a_m + (long)(begin + r) * a_k]) : (A)0;
    }
    __syncthreads();
    const long n0 = ((long)blockIdx.x * 64 + lane) * V;
    A acc[MT][V];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int v = 0; v < V; v++) acc[m][v] = (A)0;
    if (n0 < N) {
        const WS *col = w + n0 + (long)begin * b_k;
        for (int r0 = wave; r0 < rows; r0 += 4 * RIF) {
            Vec raw[RIF];
#pragma unroll
            for (int u = 0; u < RIF; u++) {
                const int r = r0 + 4 * u;
                if (r < rows) raw[u] = *reinterpret_cast<const Vec *>(col + (long)r * b_k);
            }
#pragma unroll
            for (int u = 0; u < RIF; u++) {
                const int r = r0 + 4 * u;
                if (r < rows) {
                    A wv[V];
#pragma unroll
                    for (int v = 0; v < V; v++) wv[v] = T::w(raw[u].e[v]);
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const A xv = xs[r * MT + m];
#pragma unroll
                        for (int v = 0; v < V; v++) acc[m][v] += xv * wv[v];
                    }
                }
            }
        }
    }
    __syncthreads();  // the x values are no longer needed: the same LDS carries the wavefronts' sums
    A *meet = reinterpret_cast<A *>(smem);
    if (wave > 0) {
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int v = 0; v < V; v++) meet[((wave - 1) * (MT * V) + m * V + v) * 64 + lane] = acc[m][v];
    }
    __syncthreads();
    if (wave == 0 && n0 < N) {
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (m < M) {  // (no early exit: the loop must unroll for the accumulators to stay in registers)
#pragma unroll
                for (int v = 0; v < V; v++) {
                    A s = acc[m][v];
#pragma unroll
                    for (int k = 0; k < 3; k++) s += meet[(k * (MT * V) + m * V + v) * 64 + lane];
                    partial[((long)blockIdx.y * M + m) * N + n0 + v] = s;
                }
            }
        }
    }
}

// out[j] = steps(round(sum over chunks of partial[chunk][j])): a workgroup owns 64 outputs, its four wavefronts take
// every fourth chunk and meet in LDS; the order of the additions is fixed
template <int OUT, class A>
__global__ __launch_bounds__(256) void gemv_rows_finish_kernel(const A *__restrict__ partial, typename Out<OUT>::T *__restrict__ out,
                                                              long elems, int chunks, int N, DevEpilogue epi) {
    __shared__ A meet[3][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long j = (long)blockIdx.x * 64 + lane;
    A acc = (A)0;
    if (j < elems) {
#pragma unroll 8
        for (int c = wave; c < chunks; c += 4) acc += partial[(long)c * elems + j];
    }
    if (wave > 0) meet[wave - 1][lane] = acc;
    __syncthreads();
    if (wave == 0 && j < elems) out[j] = finish<OUT>(epi, (A)(acc + meet[0][lane] + meet[1][lane] + meet[2][lane]), j % N);
}

template <class T, int MT, int V>
int launch_rows(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g, const char *name) {
    typedef typename T::A A;
    const long cus = ctx->props.multiProcessorCount;
    const long xblocks = ((long)g.N / V + 63) / 64;
    // enough workgroups to fill the chip; fewer chunks as M grows (each adds M * N partial sums to write and read)
    long chunks = ((g.M <= 4 ? 4 : 2) * cus + xblocks - 1) / xblocks;
    if (chunks > g.K / 16) chunks = g.K / 16;  // at least 16 k-rows per chunk
    if (chunks < 1) chunks = 1;
    int per_chunk = (int)((g.K + chunks - 1) / chunks);
    const size_t x_bytes = (size_t)per_chunk * MT * sizeof(A), meet_bytes = (size_t)3 * 64 * MT * V * sizeof(A);
    if (x_bytes > 48 * 1024) return HODU_ROCM_UNSUPPORTED;
    chunks = (g.K + per_chunk - 1) / per_chunk;
    if (chunks > 65535 || xblocks > 0x7FFFFFFFL) return HODU_ROCM_UNSUPPORTED;
    const size_t lds = x_bytes > meet_bytes ? x_bytes : meet_bytes;
    int rc = ensure_workspace(ctx, (size_t)chunks * g.M * g.N * sizeof(A));
    if (rc != HODU_ROCM_OK) return rc;
    auto kernel = gemv_rows_kernel<T, MT, V>;
    constexpr int LDS_MAX = 104 * 1024;  // 3 x 64 x (16 x 8) accumulators to meet at MT = 16
    if (lds > (size_t)LDS_MAX) return HODU_ROCM_UNSUPPORTED;
    rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), LDS_MAX);
    if (rc != HODU_ROCM_OK) return rc;
    A *partial = (A *)ctx->workspace.ptr;
    ctx->last_kernel = name;
    hipLaunchKernelGGL(kernel, dim3((unsigned)xblocks, (unsigned)chunks), dim3(256), lds, ctx->stream,
                       (const typename T::XS *)x + g.a_off, (const typename T::WS *)w + g.b_off, partial, g.M, g.N, g.K, g.a_m,
                       g.a_k, g.b_k, per_chunk);
    HODU_HIP(hipGetLastError());
    const long elems = (long)g.M * g.N;
    hipLaunchKernelGGL((gemv_rows_finish_kernel<T::OUT, A>), dim3((unsigned)((elems + 63) / 64)), dim3(256), 0, ctx->stream,
                       (const A *)partial, (typename Out<T::OUT>::T *)y, elems, (int)chunks, g.N, g.epi);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <class T> int run_rows(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g, const char *name) {
    typedef typename T::WS WS;
    // 16 bytes of a weight row per lane up to 4 rows of x, 8 bytes beyond (the accumulators are MT x V registers)
    constexpr int V16 = 16 / (int)sizeof(WS), V8 = 8 / (int)sizeof(WS);
    const uintptr_t base = (uintptr_t)w + (uintptr_t)g.b_off * sizeof(WS);
    auto fits = [&](int v) { return g.N % v == 0 && base % (v * sizeof(WS)) == 0 && (g.b_k * (long)sizeof(WS)) % (v * (long)sizeof(WS)) == 0; };
    if (g.M <= 4 && fits(V16)) {
        if (g.M == 1) return launch_rows<T, 1, V16>(ctx, x, w, y, g, name);
        if (g.M == 2) return launch_rows<T, 2, V16>(ctx, x, w, y, g, name);
        return launch_rows<T, 4, V16>(ctx, x, w, y, g, name);
    }
    if (!fits(V8)) return HODU_ROCM_UNSUPPORTED;
    if (g.M <= 4) return launch_rows<T, 4, V8>(ctx, x, w, y, g, name);
    if (g.M <= 8) return launch_rows<T, 8, V8>(ctx, x, w, y, g, name);
    return launch_rows<T, 16, V8>(ctx, x, w, y, g, name);
}

}  // namespace

// returns HODU_ROCM_UNSUPPORTED (no error text) when the shape is not this kernel's
int launch_gemv_rows(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    if (kind != PK_SAME || g.M > 16 || g.batches != 1 || g.b_n != 1 || g.K < 64 || g.N < 64) return HODU_ROCM_UNSUPPORTED;
    // Where it pays, measured on [M, 4096] x [4096, 4096] against the tile kernels: f32 for every M <= 16 (16.8-27.7 us
    // against 283 us: the f32 tile kernel is not cut along K), bf16 / f16 up to M = 4 (12.9-15.8 us against 16-17 us
    // for the pipelined kernel cut along K, which wins from M = 8 on).  f8e4m3 weights and the i8 product stay with
    // the pipelined kernels (13.7 us against 15.6 us here at M = 1).
    switch (dtype) {
    case HODU_BF16: return g.M <= 4 ? run_rows<RowsBf16>(ctx, a, b, c, g, "gemv_rows_bf16") : HODU_ROCM_UNSUPPORTED;
    case HODU_F16: return g.M <= 4 ? run_rows<RowsF16>(ctx, a, b, c, g, "gemv_rows_f16") : HODU_ROCM_UNSUPPORTED;
    case HODU_F32: return run_rows<RowsF32>(ctx, a, b, c, g, "gemv_rows_f32");
    default: return HODU_ROCM_UNSUPPORTED;
    }
}

}  // namespace hodu
