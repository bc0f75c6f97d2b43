// Generic strided product kernel: every dtype hodu multiplies, any strides / offsets / stride-0
// broadcasts, any extents.  It is the correctness floor under the MFMA and skinny kernels: they
// take the layouts and dtypes they are built for and everything else lands here.
//
// Replaces the general path of the reference (crates/hodu_cpu_kernels/kernels/ops_matrix.c:144-192
// and the strided dot path :527-548): one thread per output element there, a 64x64 output tile per
// 256-thread workgroup here, operands staged through LDS in the accumulate type.
//
// Arithmetic: narrow floats (f8, bf16, f16) and f32 accumulate in f32 and round once on store
// (RNE; f8 saturates); f64 in f64; integers wrap in their own width, as the reference's do.
#include "common.hpp"
#include "device_types.hpp"
#include "elem.hpp"
#include "epilogue.hpp"

namespace hodu {
namespace {

constexpr int TILE = 64;  // output tile edge
constexpr int TK = 16;    // k-slice staged per step

// EA / EB: element traits of the operands as stored; EC: of the output.  EA::acc == EB::acc == EC::acc.
// EPI: the instantiation that applies fused element-wise steps (behind a call: the plain product should not pay for
// the stack that costs)
template <class EA, class EB, class EC, bool EPI>
__global__ __launch_bounds__(256) void generic_product_kernel(const typename EA::storage *__restrict__ A,
                                                             const typename EB::storage *__restrict__ B,
                                                             typename EC::storage *__restrict__ C, DevProduct g,
                                                             int tiles_m, int tiles_n) {
    typedef typename EC::acc acc_t;
    __shared__ acc_t As[TK][TILE + 1];
    __shared__ acc_t Bs[TK][TILE + 1];

    const long tile = blockIdx.x;
    const long per_batch = (long)tiles_m * tiles_n;
    const long batch = tile / per_batch;
    const int tm = (int)((tile % per_batch) / tiles_n), tn = (int)((tile % per_batch) % tiles_n);
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    const int m0 = tm * TILE, n0 = tn * TILE;
    const int t = threadIdx.x, tx = t & 15, ty = t >> 4;

    // let neighbouring threads walk whichever operand dim is dense in memory
    const bool a_kfast = g.a_k == 1 || (g.a_m != 1 && g.a_k < g.a_m);
    const bool b_nfast = g.b_n == 1 || (g.b_k != 1 && g.b_n < g.b_k);

    acc_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (acc_t)0;

    for (int k0 = 0; k0 < g.K; k0 += TK) {
#pragma unroll
        for (int r = 0; r < (TILE * TK) / 256; r++) {
            const int idx = t + r * 256;
            int mm, kk;
            if (a_kfast) { kk = idx % TK; mm = idx / TK; } else { mm = idx % TILE; kk = idx / TILE; }
            const int m = m0 + mm, k = k0 + kk;
            acc_t v = (acc_t)0;
            if (m < g.M && k < g.K) v = EA::load(A[ao + (long)m * g.a_m + (long)k * g.a_k]);
            As[kk][mm] = v;
            int nn, kb;
            if (b_nfast) { nn = idx % TILE; kb = idx / TILE; } else { kb = idx % TK; nn = idx / TK; }
            const int n = n0 + nn, k2 = k0 + kb;
            acc_t w = (acc_t)0;
            if (n < g.N && k2 < g.K) w = EB::load(B[bo + (long)k2 * g.b_k + (long)n * g.b_n]);
            Bs[kb][nn] = w;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; kk++) {
            acc_t a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = As[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = Bs[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }

    typename EC::storage *Cb = C + batch * (long)g.M * g.N;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int m = m0 + ty + 16 * i;
        if (m >= g.M) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int n = n0 + tx + 16 * j;
            if (n < g.N) {
                typename EC::storage v = EC::store(acc[i][j]);
                if constexpr (EPI) v = epilogue_apply_call<EC::id>(g.epi, v, n);
                Cb[(long)m * g.N + n] = v;
            }
        }
    }
}

template <class EA, class EB, class EC>
int run(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    const int tiles_m = (g.M + TILE - 1) / TILE, tiles_n = (g.N + TILE - 1) / TILE;
    const long blocks = g.batches * tiles_m * tiles_n;
    if (blocks <= 0) return HODU_ROCM_OK;
    if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "product needs %ld workgroups", blocks);
    auto kernel = g.epi.n != 0 ? generic_product_kernel<EA, EB, EC, true> : generic_product_kernel<EA, EB, EC, false>;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const typename EA::storage *)a,
                       (const typename EB::storage *)b, (typename EC::storage *)c, g, tiles_m, tiles_n);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace

int launch_generic(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c,
                       const DevProduct &g) {
    if (kind == PK_BF16_F8W) return run<Elem<HODU_BF16>, Elem<HODU_F8E4M3>, Elem<HODU_BF16>>(ctx, a, b, c, g);
    if (kind == PK_I32_I8I8) return run<Elem<HODU_I8>, Elem<HODU_I8>, Elem<HODU_I32>>(ctx, a, b, c, g);
    switch (dtype) {
#define CASE(ID) case ID: return run<Elem<ID>, Elem<ID>, Elem<ID>>(ctx, a, b, c, g);
        CASE(HODU_F8E4M3) CASE(HODU_F8E5M2) CASE(HODU_BF16) CASE(HODU_F16) CASE(HODU_F32) CASE(HODU_F64)
        CASE(HODU_U8) CASE(HODU_U16) CASE(HODU_U32) CASE(HODU_U64) CASE(HODU_I8) CASE(HODU_I16) CASE(HODU_I32)
        CASE(HODU_I64)
#undef CASE
    default: return fail(HODU_ROCM_UNSUPPORTED, "matmul/dot: dtype id %d is not a product dtype", dtype);
    }
}

}  // namespace hodu
