// Small f32 products: too few output tiles to fill the chip with LDS-tiled workgroups, and so little K per tile that
// a load -> LDS -> barrier -> multiply loop spends its time waiting (hodu's own CPU-sized case, dot of two
// [512, 512] f32 matrices, is one: crates/hodu_core/src/tensor/ops/matrix.rs:323-354 hands it to the backend as one
// 2-D product).  Here a workgroup owns ONE 32 x 32 output tile and its four wavefronts a quarter of K each:
//   * operands go from memory straight into the MFMA's registers -- v_mfma_f32_32x32x2_f32 wants one float per lane
//     and operand, so nothing has to be transposed through LDS.  The order in which k is fed is free as long as both
//     operands agree: a lane of half h takes k0 + 4 h .. + 3 of every 8-wide chunk, one 16-byte load where the
//     operand is k-dense, four dword loads (32 lanes = one 128-byte line each) where it is row-dense;
//   * a ring of four chunks of both operands is in flight per wavefront (no barrier in the loop; deeper rings and
//     eight wavefronts per tile measured no better);
//   * the four partial tiles meet in LDS and are added in a fixed order (wavefront 0, 1, 2, 3), the fused
//     element-wise steps run on the rounded sum, 16-byte stores.
// The MFMA is fed with swapped operands, so lane (r, h) ends with row m0 + r, columns n0 + 8 q + 4 h + e.
// f32 products, f32 accumulation (the matrix core's f32 FMA chain), as everywhere.
#include "common.hpp"
#include "device_types.hpp"
#include "epilogue.hpp"

namespace hodu {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef f32x4 f32x4_any __attribute__((aligned(4)));  // 16-byte load from a 4-byte-aligned address

constexpr int SF_DEPTH = 4;  // chunks (of 8 k) a wavefront has loads out for
constexpr int SF_WAVES = 4;  // wavefronts that share a tile's K

// Four consecutive k of one row (or column) of an operand: `p` points at element (row, k), ks is the k stride
template <bool KDENSE> __device__ __forceinline__ f32x4 load_k4(const float *p, long ks) {
    if constexpr (KDENSE) return *reinterpret_cast<const f32x4_any *>(p);
    return f32x4{p[0], p[ks], p[2 * ks], p[3 * ks]};
}

template <bool A_KDENSE, bool B_KDENSE>
__global__ __launch_bounds__(64 * SF_WAVES) void small_f32_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                        float *__restrict__ C, DevProduct g, int tiles_m, int tiles_n,
                                                        int vec_store) {
    __shared__ float part[SF_WAVES][16][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 31, lh = lane >> 5;
    const long per_batch = (long)tiles_m * tiles_n;
    const long batch = blockIdx.x / per_batch;
    const int t = (int)(blockIdx.x % per_batch);
    const int m0 = (t / tiles_n) * 32, n0 = (t % tiles_n) * 32;
    long ao, bo;
    batch_offsets(g, batch, ao, bo);
    // rows past the edge are clamped: they are multiplied like the others and not stored
    const int m = m0 + lr < g.M ? m0 + lr : g.M - 1, n = n0 + lr < g.N ? n0 + lr : g.N - 1;
    const float *ap = A + ao + (long)m * g.a_m, *bp = B + bo + (long)n * g.b_n;

    // this wavefront's whole chunks of 8 k: [c0, c1); the ragged rest of K, if any, goes to the last wavefront
    const int whole = g.K / 8, per_wave = (whole + SF_WAVES - 1) / SF_WAVES;
    const int c0 = wave * per_wave < whole ? wave * per_wave : whole;
    const int c1 = c0 + per_wave < whole ? c0 + per_wave : whole;
    const int count = c1 - c0;

    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    f32x4 ar[SF_DEPTH], br[SF_DEPTH];
    auto fetch = [&](int slot, int c) {  // chunk c (clamped to the wavefront's last one: a harmless re-read)
        c = c < c1 ? c : c1 - 1;
        const long k = (long)c * 8 + 4 * lh;
        ar[slot] = load_k4<A_KDENSE>(ap + k * g.a_k, g.a_k);
        br[slot] = load_k4<B_KDENSE>(bp + k * g.b_k, g.b_k);
    };
    auto multiply = [&](int slot) {
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(br[slot][j], ar[slot][j], acc, 0, 0, 0);
    };
    if (count > 0) {
#pragma unroll
        for (int s = 0; s < SF_DEPTH; s++) fetch(s, c0 + s);
        int c = c0;
        for (; c + SF_DEPTH <= c1; c += SF_DEPTH) {
            if (c + SF_DEPTH < c1) {
#pragma unroll
                for (int s = 0; s < SF_DEPTH; s++) {
                    multiply(s);
                    fetch(s, c + SF_DEPTH + s);
                }
            } else {  // nothing left to fetch
#pragma unroll
                for (int s = 0; s < SF_DEPTH; s++) multiply(s);
            }
        }
        const int rest = c1 - c;
#pragma unroll
        for (int s = 0; s < SF_DEPTH; s++)
            if (s < rest) multiply(s);
    }
    if (wave == SF_WAVES - 1 && whole * 8 < g.K) {  // the last k, fewer than 8: element loads, zeros past the end
        f32x4 a4, b4;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int k = whole * 8 + 4 * lh + j;
            a4[j] = k < g.K ? ap[(long)k * g.a_k] : 0.f;
            b4[j] = k < g.K ? bp[(long)k * g.b_k] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b4[j], a4[j], acc, 0, 0, 0);
    }

    // ---- the four quarters of K meet: wavefront q adds registers 4 q .. 4 q + 3 of all four, in a fixed order ----
#pragma unroll
    for (int e = 0; e < 16; e++) part[wave][e][lane] = acc[e];
    __syncthreads();
    static_assert(SF_WAVES == 4, "wavefront q stores registers 4 q .. 4 q + 3");
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        v[e] = part[0][4 * wave + e][lane];
#pragma unroll
        for (int p = 1; p < SF_WAVES; p++) v[e] += part[p][4 * wave + e][lane];
    }
    const int row = m0 + lr, col = n0 + 8 * wave + 4 * lh;
    if (row >= g.M || col >= g.N) return;
    if (g.epi.n != 0) {
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = epilogue_apply<HODU_F32>(g.epi, v[e], col + e < g.N ? col + e : g.N - 1);
    }
    float *dst = C + (batch * g.M + row) * (long)g.N + col;
    if (vec_store && col + 4 <= g.N) {
        *reinterpret_cast<f32x4 *>(dst) = f32x4{v[0], v[1], v[2], v[3]};
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (col + e < g.N) dst[e] = v[e];
    }
}

}  // namespace

// Takes f32 products that would otherwise leave most of the chip idle: fewer 128 x 128 tiles than compute units,
// and few enough 32 x 32 tiles that reading both operands once per tile (no sharing through LDS) stays cheap.
int launch_small_f32(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    if (kind != PK_SAME || dtype != HODU_F32 || g.M < 1 || g.N < 1 || g.K < 1 || g.batches < 1) return HODU_ROCM_UNSUPPORTED;
    const long tiles_m = (g.M + 31) / 32, tiles_n = (g.N + 31) / 32, tiles = g.batches * tiles_m * tiles_n;
    const long big_tiles = g.batches * ((g.M + 127) / 128) * ((g.N + 127) / 128);
    const int cus = ctx->props.multiProcessorCount;
    if (ctx->force_tile != 40) {
        if (ctx->force_tile >= 0 || big_tiles >= cus) return HODU_ROCM_UNSUPPORTED;
        // Measured against the tiled kernels (which cut K across workgroups when tiles are few): ahead up to about
        // two tiles per compute unit (512^3 6.5 against 11.9 us, 768^3 19.8 / 25.2, 1024^3 35.0 / 35.1), and, where
        // the tiles leave most of the chip idle, only while K is short (64 tiles: K = 1024 9.3 / 11.7, K = 4096 30 / 22)
        if (tiles * 4 > 9L * cus || (tiles * 2 < cus && g.K > 2048)) return HODU_ROCM_UNSUPPORTED;
        if (g.M < 17) return HODU_ROCM_UNSUPPORTED;  // the few-rows kernels' ground
    }
    if (tiles > 0x7fffffffL) return HODU_ROCM_UNSUPPORTED;
    const int vec_store = (uintptr_t)c % 16 == 0 && g.N % 4 == 0;
    const bool ak = g.a_k == 1, bk = g.b_k == 1;
    auto go = [&](auto kernel, const char *name) {
        ctx->last_kernel = name;
        hipLaunchKernelGGL(kernel, dim3((unsigned)tiles), dim3(64 * SF_WAVES), 0, ctx->stream, (const float *)a, (const float *)b, (float *)c, g,
                           (int)tiles_m, (int)tiles_n, vec_store);
    };
    if (ak && bk) go(small_f32_kernel<true, true>, "small_f32_KK");
    else if (ak) go(small_f32_kernel<true, false>, "small_f32_KM");
    else if (bk) go(small_f32_kernel<false, true>, "small_f32_MK");
    else go(small_f32_kernel<false, false>, "small_f32_MM");
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace hodu
