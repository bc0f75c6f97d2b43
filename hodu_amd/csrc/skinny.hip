// Bandwidth-bound products with at most 16 rows on the left (decode-shape GEMV / skinny GEMM):
// y[m, n] = sum_k x[m, k] * W[n, k]  with the weight's k dense in memory -- the layout a Linear
// layer hands over (`input.matmul(weight.transpose(-2, -1))`, crates/hodu_nn/src/modules/linear.rs:38-47).
// Replaces the M < 512 single-thread paths of hodu_cpu_dot_<dt> (kernels/ops_matrix.c:486-548).
//
// The weight is the only operand that matters: every byte of it is read from HBM exactly once with
// 128-bit loads, 16 consecutive k of one row per lane, four neighbouring lanes covering 64
// contiguous bytes of that row.  Those 16 bytes ARE a lane's MFMA operand (k-packed), so the loaded
// registers feed the matrix core directly (f8e4m3 weights pass through v_cvt_scalef32_pk_bf16_fp8
// first) -- no LDS staging, no shuffles.  The left operand's rows occupy the MFMA's 16 m slots;
// slots beyond M are zero, which costs nothing on a memory-bound kernel and makes M = 1..16 one
// code path.
//
// Work split: a workgroup owns 16 weight rows (one MFMA column block); its 8 wavefronts split K, so
// a 4096-wide row keeps 8 KB per wavefront in flight; partial sums meet in LDS (a wavefront-level
// reduction per output element), are rounded once and stored.
#include "common.hpp"
#include "device_types.hpp"
#include "gemm_mfma.hpp"
#include "agent_scope.hpp"

namespace hodu {
namespace {

using mfma::bitcast;
using mfma::CK_BF16;
using mfma::CK_F16;
using mfma::CK_F32;
using mfma::CK_I8;
using mfma::Compute;
using mfma::Out;
using mfma::SK_F8;
using mfma::SK_SAME;

constexpr int CHUNK = 8;                 // weight vectors in flight per lane (8 KB per wavefront)
constexpr int X_LDS_LIMIT = 144 * 1024;  // bytes of LDS the staged left operand may take

__device__ __forceinline__ u32x4_t ldg16(const char *p) { return *reinterpret_cast<const u32x4_t *>(p); }
// a weight vector: read once by one wavefront, so with the non-temporal hint (the stream then does not push the
// activations, which every workgroup re-reads, out of L2)
__device__ __forceinline__ u32x4_t ldg16_stream(const char *p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p)); }

// 16 f8e4m3 -> two chunks of 8 bf16 (exact)
__device__ __forceinline__ void widen_f8x16(const u32x4_t &w, u32x4_t &lo, u32x4_t &hi) {
    lo.x = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.x, 1.0f, false));
    lo.y = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.x, 1.0f, true));
    lo.z = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.y, 1.0f, false));
    lo.w = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.y, 1.0f, true));
    hi.x = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.z, 1.0f, false));
    hi.y = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.z, 1.0f, true));
    hi.z = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.w, 1.0f, false));
    hi.w = bitcast<uint32_t>(__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.w, 1.0f, true));
}

// CK: type fed to the matrix core; SKB: weight storage (CK itself, or f8e4m3 widened to bf16).
// STAGE: the left operand (M x K, a few KB) is first copied to LDS, rows x_pitch bytes apart,
// so that the MFMA's left fragments come from LDS instead of nearly-empty global loads (for M = 1
// only 4 of 64 lanes carry a left-operand row).  !STAGE: a wavefront's left fragments come straight from memory
// (cache hits), issued together with the weight loads they meet in the MFMA -- for a left operand that does not
// fit in LDS, and where copying all of it into every workgroup costs more than reading it in place.
// NBLK blocks of 16 weight rows per workgroup, KW wavefronts splitting K for each: the staged copy of x is shared
// by all of them, so a larger NBLK means proportionally fewer copies of x through the memory pipeline
template <int CK, int SKB, int OUT, int NBLK, int KW, bool STAGE = true>
__global__ __launch_bounds__(NBLK * KW * 64) void skinny_kdense_kernel(const char *__restrict__ X,
                                                                  const char *__restrict__ W,
                                                                  typename Out<OUT>::T *__restrict__ Y, DevProduct g,
                                                                  int tiles_n, int k_per_wave, int x_pitch) {
    typedef Compute<CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef typename Out<OUT>::T out_t;
    constexpr int ES = Cmp::ES;                         // bytes per element of x (and of W unless f8)
    constexpr int SB = SKB == SK_F8 ? 1 : ES;           // bytes per stored weight element
    constexpr int EPL = 16 / SB;                        // weight elements per lane per load
    HODU_DYNAMIC_LDS(xs);
    constexpr int NT = NBLK * KW * 64;
    __shared__ acc_t red[NBLK * KW][64];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const long batch = blockIdx.x / tiles_n;
    const int blk = wave / KW, kw = wave % KW;
    const int n0 = ((int)(blockIdx.x % tiles_n) * NBLK + blk) * 16;
    long ao, bo;
    batch_offsets(g, batch, ao, bo);

    int n = n0 + lr;
    n = n < g.N ? n : g.N - 1;
    const char *wrow = W + (bo + (long)n * g.b_n) * SB;
    const bool has_x = lr < g.M;
    const char *xrow = X + (ao + (long)(has_x ? lr : 0) * g.a_m) * ES;

    const int kbeg = kw * k_per_wave;
    int kend = kbeg + k_per_wave;
    kend = kend < g.K ? kend : g.K;

    // Loads return in issue order.  The copy of x into LDS therefore starts FIRST: its loads (cache hits) are all
    // in flight together, the first chunk of weight loads (HBM) goes out right behind them, and the copy
    // finishes while the weights are still on their way.  (Issued after the weights, every load of the copy
    // loop waited for all of them, and the loop made one cache round trip per iteration.)
    constexpr int XB = 16;  // vectors of x a thread keeps in flight
    const int vec_per_row = g.K * ES / 16, x_vecs = STAGE ? g.M * vec_per_row : 0;
    u32x4_t xr[XB];
#pragma unroll
    for (int i = 0; i < XB; i++) {
        const int v = tid + i * NT;
        xr[i] = mfma::zero4();
        if (v < x_vecs) {
            const int row = v / vec_per_row, col = v - row * vec_per_row;
            xr[i] = ldg16(X + (ao + (long)row * g.a_m) * ES + col * 16);
        }
    }
    u32x4_t wv[CHUNK];
    // !STAGE: the left fragments of a block of CHUNK weight vectors (two per vector of 16 f8 weights)
    u32x4_t xa[STAGE ? 1 : CHUNK], xb[STAGE || SKB != SK_F8 ? 1 : CHUNK];
    auto load_block = [&](int kb) {
#pragma unroll
        for (int u = 0; u < CHUNK; u++) {
            const int k = kb + (u * 4 + lg) * EPL;
            wv[u] = k < kend ? ldg16_stream(wrow + (long)k * SB) : mfma::zero4();
        }
        if constexpr (!STAGE) {
#pragma unroll
            for (int u = 0; u < CHUNK; u++) {
                const int k = kb + (u * 4 + lg) * EPL;
                const bool ok = k < kend && has_x;
                xa[u] = ok ? ldg16(xrow + (long)k * ES) : mfma::zero4();
                if constexpr (SKB == SK_F8) xb[u] = ok ? ldg16(xrow + (long)(k + 8) * ES) : mfma::zero4();
            }
        }
    };
    load_block(kbeg);
    if constexpr (STAGE) {
#pragma unroll
        for (int i = 0; i < XB; i++) {
            const int v = tid + i * NT;
            if (v < x_vecs) {
                const int row = v / vec_per_row, col = v - row * vec_per_row;
                *reinterpret_cast<u32x4_t *>(xs + row * x_pitch + col * 16) = xr[i];
            }
        }
        for (int v = tid + XB * NT; v < x_vecs; v += NT) {  // a left operand larger than XB vectors per thread
            const int row = v / vec_per_row, col = v - row * vec_per_row;
            *reinterpret_cast<u32x4_t *>(xs + row * x_pitch + col * 16) = ldg16(X + (ao + (long)row * g.a_m) * ES + col * 16);
        }
        __syncthreads();
    }
    const char *xl = xs + lr * x_pitch;

    acc_t acc = acc_t{0, 0, 0, 0};
    for (int kb = kbeg; kb < kend; kb += CHUNK * 4 * EPL) {
        if (kb != kbeg) load_block(kb);
#pragma unroll
        for (int u = 0; u < CHUNK; u++) {
            const int k = kb + (u * 4 + lg) * EPL;
            u32x4_t fa = mfma::zero4(), fb = mfma::zero4();
            if constexpr (STAGE) {
                if (k < kend && has_x) {
                    fa = *reinterpret_cast<const u32x4_t *>(xl + k * ES);
                    if (SKB == SK_F8) fb = *reinterpret_cast<const u32x4_t *>(xl + (k + 8) * ES);
                }
            } else {
                fa = xa[u];
                if constexpr (SKB == SK_F8) fb = xb[u];
            }
            if (SKB == SK_F8) {
                u32x4_t lo, hi;
                widen_f8x16(wv[u], lo, hi);
                Cmp::mma(fa, lo, acc);
                Cmp::mma(fb, hi, acc);
            } else {
                Cmp::mma(fa, wv[u], acc);
            }
        }
    }

    // lane holds y[m = 4*lg + e][n = n0 + lr] for e = 0..3 over this wavefront's k range
    red[wave][lane] = acc;
    __syncthreads();
    if (tid < 64 * NBLK) {  // wavefront b adds up row block b; (lr, lg) are the same in every wavefront
        acc_t s = red[wave * KW][lane];
#pragma unroll
        for (int w = 1; w < KW; w++) {
            const acc_t t = red[wave * KW + w][lane];
            s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
        }
        out_t *Yb = Y + batch * (long)g.M * g.N;
        const int col = ((int)(blockIdx.x % tiles_n) * NBLK + wave) * 16 + lr;
        if (col < g.N) {
            // the lane's four outputs share a column: what the fused steps need for it is fetched once
            EpiPrepared<Out<OUT>::DT, 1> prepared;
            if (g.epi.n != 0) prepared = epilogue_prepare<Out<OUT>::DT, 1>(g.epi, col, g.N);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int m = 4 * lg + e;
                out_t v = Out<OUT>::cvt(s[e]);
                if (g.epi.n != 0) epilogue_apply_prepared<Out<OUT>::DT, 1>(prepared, &v);
                if (m < g.M) Yb[(long)m * g.N + col] = v;
            }
        }
    }
}

// ---- the same product cut along K across workgroups -------------------------------------------------
// For M near 16 the left operand (M x K) is twice the bytes of the weight rows one workgroup streams, and in the
// kernel above every workgroup stages all of it: measured on M = 16, N = K = 4096 (f8 weights), 4.1 of 11.4 us.
// Here a workgroup takes 128 weight rows (8 wavefronts x 16) and ONE slice of K, stages only that slice of x (a
// few KB; x crosses the memory pipeline N/128 times in total instead of N/16 times), and there are still as many
// workgroups as compute units.  Each writes its 16 x 128 partial sums (laid out [slice][n][16]: a lane's four
// values are one 16-byte store) and bumps its column block's arrival counter; the workgroup that arrives last
// adds the slices in slice order -- so the result does not depend on who was last --, rounds once, stores, and
// zeroes the counter for the next launch.
// How the partial sums cross from one workgroup to another: agent_scope.hpp.
constexpr int SK_ROWS = 128;  // weight rows per workgroup
constexpr int SK_XVEC = 8;    // 16-byte vectors of x per thread: 512 threads x 8 x 16 B = 64 KB covers M = 16 x 2048 k of bf16
constexpr int SK_XBYTES = SK_XVEC * 512 * 16;

template <int CK, int SKB, int OUT>
__global__ __launch_bounds__(512) void skinny_splitk_kernel(const char *__restrict__ X, const char *__restrict__ W,
                                                           typename Out<OUT>::T *__restrict__ Y,
                                                           typename Compute<CK>::acc_t *__restrict__ partials,
                                                           int *__restrict__ arrival, DevProduct g, int n_blocks,
                                                           int slices, int k_per_slice, int x_pitch) {
    typedef Compute<CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef decltype(acc_t{}.x) part_t;
    constexpr int ES = Cmp::ES, SB = SKB == SK_F8 ? 1 : ES, EPL = 16 / SB;
    HODU_DYNAMIC_LDS(xs);
    __shared__ int last_flag;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int nb = blockIdx.x % n_blocks, ks = blockIdx.x / n_blocks;
    const int kbeg = ks * k_per_slice;
    int kend = kbeg + k_per_slice;
    kend = kend < g.K ? kend : g.K;

    int n = nb * SK_ROWS + wave * 16 + lr;
    const bool n_ok = n < g.N;
    n = n_ok ? n : g.N - 1;
    const char *wrow = W + (g.b_off + (long)n * g.b_n) * SB;

    // loads return in issue order: the slice of x (cache hits) first, the weights (HBM) right behind
    constexpr int XB = SK_XVEC;
    const int vec_per_row = (kend - kbeg) * ES / 16, x_vecs = g.M * vec_per_row;
    u32x4_t xr[XB];
#pragma unroll
    for (int i = 0; i < XB; i++) {
        const int v = tid + i * 512;
        xr[i] = mfma::zero4();
        if (v < x_vecs) {
            const int row = v / vec_per_row, col = v - row * vec_per_row;
            xr[i] = ldg16(X + (g.a_off + (long)row * g.a_m + kbeg) * ES + col * 16);
        }
    }
    u32x4_t wv[CHUNK];
#pragma unroll
    for (int u = 0; u < CHUNK; u++) {
        const int k = kbeg + (u * 4 + lg) * EPL;
        wv[u] = k < kend ? ldg16_stream(wrow + (long)k * SB) : mfma::zero4();
    }
#pragma unroll
    for (int i = 0; i < XB; i++) {
        const int v = tid + i * 512;
        if (v < x_vecs) {
            const int row = v / vec_per_row, col = v - row * vec_per_row;
            *reinterpret_cast<u32x4_t *>(xs + row * x_pitch + col * 16) = xr[i];
        }
    }
    __syncthreads();
    const char *xl = xs + lr * x_pitch;
    const bool has_x = lr < g.M;

    acc_t acc = acc_t{0, 0, 0, 0};
    for (int kb = kbeg; kb < kend; kb += CHUNK * 4 * EPL) {
        if (kb != kbeg) {
#pragma unroll
            for (int u = 0; u < CHUNK; u++) {
                const int k = kb + (u * 4 + lg) * EPL;
                wv[u] = k < kend ? ldg16_stream(wrow + (long)k * SB) : mfma::zero4();
            }
        }
#pragma unroll
        for (int u = 0; u < CHUNK; u++) {
            const int k = kb + (u * 4 + lg) * EPL;
            const bool ok = k < kend && has_x;
            u32x4_t xa = mfma::zero4(), xb = mfma::zero4();
            if (ok) {
                xa = *reinterpret_cast<const u32x4_t *>(xl + (k - kbeg) * ES);
                if (SKB == SK_F8) xb = *reinterpret_cast<const u32x4_t *>(xl + (k - kbeg + 8) * ES);
            }
            if (SKB == SK_F8) {
                u32x4_t lo, hi;
                widen_f8x16(wv[u], lo, hi);
                Cmp::mma(xa, lo, acc);
                Cmp::mma(xb, hi, acc);
            } else {
                Cmp::mma(xa, wv[u], acc);
            }
        }
    }
    // lane holds y[m = 4*lg + e][n] for e = 0..3: 16 consecutive bytes of [slice][n][16], written through at agent
    // scope and waited for before the barrier
    const __amdgpu_buffer_rsrc_t part = agent_buffer(partials, (unsigned)slices * (unsigned)g.N * 64u);
    if (n_ok) store16_agent(part, (((unsigned)ks * g.N + n) * 4 + lg) * 16u, acc);
    // every thread's sums have landed before thread 0 counts this workgroup in; whoever finds slices - 1 is last
    if (!arrive_and_check_last(&arrival[nb], slices, &last_flag, tid)) return;
    // 128 columns x 4 quads of m: thread -> (column, quad); the other workgroups' sums are read at agent scope
    // (a plain load could be served from a line this XCD cached during an earlier launch)
    const int col = nb * SK_ROWS + (tid >> 2), quad = tid & 3;
    if (col < g.N) {
        acc_t s = acc_t{0, 0, 0, 0};
        for (int k0 = 0; k0 < slices; k0 += 8) {  // eight slices' loads in flight, added in slice order
            acc_t v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                // past the last slice: the last slice again (a valid address), its value unused
                const int ksl = k0 + j < slices ? k0 + j : slices - 1;
                v[j] = load16_agent<acc_t>(part, (((unsigned)ksl * g.N + col) * 4 + quad) * 16u);
            }
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (k0 + j < slices) s += v[j];
        }
        EpiPrepared<Out<OUT>::DT, 1> prepared;  // the lane's four outputs share a column
        if (g.epi.n != 0) prepared = epilogue_prepare<Out<OUT>::DT, 1>(g.epi, col, g.N);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int m = quad * 4 + e;
            typename Out<OUT>::T v = Out<OUT>::cvt(s[e]);
            if (g.epi.n != 0) epilogue_apply_prepared<Out<OUT>::DT, 1>(prepared, &v);
            if (m < g.M) Y[(long)m * g.N + col] = v;
        }
    }
    arrival_reset(&arrival[nb], tid);
}

// applicable when one product (no batch) is wide and deep enough to be cut; returns UNSUPPORTED otherwise
template <int CK, int SKB, int OUT>
int launch_splitk(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g) {
    typedef typename Compute<CK>::acc_t acc_t;
    constexpr int ES = Compute<CK>::ES, SB = SKB == SK_F8 ? 1 : ES, EPL = 16 / SB, STEP = CHUNK * 4 * EPL;
    if (g.batches != 1 || g.M <= 4 || g.N < 8 * SK_ROWS || g.K < 4 * STEP) return HODU_ROCM_UNSUPPORTED;
    const int n_blocks = (g.N + SK_ROWS - 1) / SK_ROWS;
    if (n_blocks > kArrivalSlots || (long)g.N * 64 * 64 > 0xFFFFFFFFL) return HODU_ROCM_UNSUPPORTED;  // 32-bit buffer offsets
    // Measured against the one-pass kernel (f8 and bf16 weights, M = 5..16): the arrival counter and the last
    // workgroup's second look at the sums cost about 2 us, which pays off once the weights take 16 MB and x is
    // half as large as a workgroup's share of them, or 32 MB whatever M is, or when N is too small to give the
    // one-pass kernel a workgroup per compute unit.
    const long cus = ctx->props.multiProcessorCount;
    const long w_bytes = (long)g.N * g.K * SB;
    const bool pays = w_bytes >= (32L << 20) || (w_bytes >= (16L << 20) && g.M >= 8) ||
                      (g.N / 16 < cus / 2 && g.K >= 4096 && g.M >= 12);
    if (!pays && ctx->force_tile != 38) return HODU_ROCM_UNSUPPORTED;
    // as many slices as fill the machine, each a whole number of passes (STEP k) of a wavefront and small enough
    // that the slice of x fits the staging registers of one workgroup
    const int passes = (g.K + STEP - 1) / STEP;
    int slices = (int)((cus + n_blocks - 1) / n_blocks);
    slices = slices < passes ? slices : passes;
    int pass_per_slice = (passes + slices - 1) / slices;
    const int fit = SK_XBYTES / (g.M * ES) / STEP;
    if (fit < 1) return HODU_ROCM_UNSUPPORTED;
    pass_per_slice = pass_per_slice < fit ? pass_per_slice : fit;
    const int k_per_slice = pass_per_slice * STEP;
    slices = (g.K + k_per_slice - 1) / k_per_slice;
    if (slices < 2 || slices > 64) return HODU_ROCM_UNSUPPORTED;
    const int x_pitch = k_per_slice * ES + 16;
    const size_t lds = (size_t)g.M * x_pitch;
    int rc = ensure_workspace(ctx, (size_t)slices * g.N * 16 * sizeof(float));
    if (rc == HODU_ROCM_OK) rc = ensure_arrival(ctx);
    if (rc != HODU_ROCM_OK) return rc;
    auto kernel = skinny_splitk_kernel<CK, SKB, OUT>;
    rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), SK_XBYTES + 16 * 16);
    if (rc != HODU_ROCM_OK) return rc;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(n_blocks * slices)), dim3(512), lds, ctx->stream, (const char *)x, (const char *)w,
                       (typename Out<OUT>::T *)y, (acc_t *)ctx->workspace.ptr, ctx->arrival, g, n_blocks, slices, k_per_slice,
                       x_pitch);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

// the one-pass kernel with the left operand read in place: one block of 16 weight rows per workgroup
template <int CK, int SKB, int OUT>
int launch_unstaged(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g) {
    constexpr int ES = Compute<CK>::ES, SB = SKB == SK_F8 ? 1 : ES, EPL = 16 / SB, KW = 8;
    (void)ES;
    const int tiles_n = (g.N + 15) / 16;
    const long blocks = g.batches * tiles_n;
    if (blocks > 0x7FFFFFFFL) return HODU_ROCM_UNSUPPORTED;
    const int step = 4 * EPL;
    const int k_per_wave = ((g.K + KW - 1) / KW + step - 1) / step * step;
    hipLaunchKernelGGL((skinny_kdense_kernel<CK, SKB, OUT, 1, KW, false>), dim3((unsigned)blocks), dim3(KW * 64), 0, ctx->stream,
                       (const char *)x, (const char *)w, (typename Out<OUT>::T *)y, g, tiles_n, k_per_wave, 0);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <int CK, int SKB, int OUT, int NBLK, int KW>
int launch_shape(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g) {
    constexpr int ES = Compute<CK>::ES, SB = SKB == SK_F8 ? 1 : ES, EPL = 16 / SB;
    const int tiles_n = (g.N + 16 * NBLK - 1) / (16 * NBLK);
    const long blocks = g.batches * tiles_n;
    if (blocks > 0x7FFFFFFFL) return HODU_ROCM_UNSUPPORTED;
    const int step = 4 * EPL;  // k covered by one wavefront-wide load
    const int k_per_wave = ((g.K + KW - 1) / KW + step - 1) / step * step;
    // rows of the staged left operand are padded by 16 bytes so that the 16 row slots of a fragment
    // read hit different LDS banks
    const long pitch = (long)g.K * ES + 16;
    if (g.M * pitch > X_LDS_LIMIT) return launch_unstaged<CK, SKB, OUT>(ctx, x, w, y, g);  // it does not fit
    const int x_pitch = (int)pitch;
    const size_t lds = (size_t)g.M * x_pitch;
    auto kernel = skinny_kdense_kernel<CK, SKB, OUT, NBLK, KW>;
    if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), X_LDS_LIMIT)) return rc;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(NBLK * KW * 64), lds, ctx->stream, (const char *)x,
                       (const char *)w, (typename Out<OUT>::T *)y, g, tiles_n, k_per_wave, x_pitch);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <int CK, int SKB, int OUT>
int run_kdense(hodu_rocm_ctx *ctx, const void *x, const void *w, void *y, const DevProduct &g, const char *name) {
    constexpr int ES = Compute<CK>::ES, SB = SKB == SK_F8 ? 1 : ES, EPL = 16 / SB;
    // applicability: both operands k-dense and every vector load 16-byte aligned
    auto al = [](long elems, int bytes) { return (elems * bytes) % 16 == 0; };
    if (g.M > 16 || g.K % EPL != 0 || g.K < 4 * EPL) return HODU_ROCM_UNSUPPORTED;
    if (!(g.a_k == 1) || !(g.b_k == 1)) return HODU_ROCM_UNSUPPORTED;
    if (!(g.M == 1 || al(g.a_m, ES)) || !(g.N == 1 || al(g.b_n, SB))) return HODU_ROCM_UNSUPPORTED;
    if (((uintptr_t)x + (uintptr_t)g.a_off * ES) % 16 || ((uintptr_t)w + (uintptr_t)g.b_off * SB) % 16)
        return HODU_ROCM_UNSUPPORTED;
    for (int d = 0; d < g.nb; d++)
        if (!al(g.a_bs[d], ES) || !al(g.b_bs[d], SB)) return HODU_ROCM_UNSUPPORTED;

    // workgroup shape: (row blocks, wavefronts per block).  Every workgroup stages its own copy of x, so when x is
    // as large as the weights a workgroup streams (M near 16), fewer and fatter workgroups move fewer bytes.
    int shape = g.M > 8 && g.N >= 32 * 128 ? 1 : 0;  // measured at M = 16, N = K = 4096 (f8 weights): 11.6, 11.1, 14.5 us
    if (ctx->force_tile == 35) shape = 0;
    if (ctx->force_tile == 36) shape = 1;
    if (ctx->force_tile == 37) shape = 2;
    ctx->last_kernel = name;
    if (ctx->force_tile == 39) return launch_unstaged<CK, SKB, OUT>(ctx, x, w, y, g);
    if (ctx->force_tile < 35 || ctx->force_tile > 37) {  // the hook values 35..37 pin the one-pass kernel's shape, 38 this one
        const int rc = launch_splitk<CK, SKB, OUT>(ctx, x, w, y, g);
        if (rc != HODU_ROCM_UNSUPPORTED) {
            snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s_splitk", name);
            ctx->last_kernel = ctx->kernel_name;
            return rc;
        }
    }
    if (shape == 1) return launch_shape<CK, SKB, OUT, 2, 8>(ctx, x, w, y, g);
    if (shape == 2) return launch_shape<CK, SKB, OUT, 4, 4>(ctx, x, w, y, g);
    return launch_shape<CK, SKB, OUT, 1, 8>(ctx, x, w, y, g);
}

}  // namespace

int launch_skinny(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c,
                  const DevProduct &g) {
    if (g.M > 16 || g.K == 0) return HODU_ROCM_UNSUPPORTED;
    if (kind == PK_BF16_F8W) return run_kdense<CK_BF16, SK_F8, mfma::OUT_BF16>(ctx, a, b, c, g, "skinny_bf16_f8w");
    if (kind == PK_I32_I8I8) return run_kdense<CK_I8, SK_SAME, mfma::OUT_I32>(ctx, a, b, c, g, "skinny_i32_i8i8");
    switch (dtype) {
    case HODU_BF16: return run_kdense<CK_BF16, SK_SAME, mfma::OUT_BF16>(ctx, a, b, c, g, "skinny_bf16");
    case HODU_F16: return run_kdense<CK_F16, SK_SAME, mfma::OUT_F16>(ctx, a, b, c, g, "skinny_f16");
    case HODU_F32: return run_kdense<CK_F32, SK_SAME, mfma::OUT_F32>(ctx, a, b, c, g, "skinny_f32");
    default: return HODU_ROCM_UNSUPPORTED;
    }
}

}  // namespace hodu
