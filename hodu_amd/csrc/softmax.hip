// Softmax along one dim, as one kernel.  Tensor::softmax (crates/hodu_core/src/tensor/ops/normalization.rs:4-21) is
// five launches in the reference -- max(keep_dim), sub, exp, sum(keep_dim), div -- each a full pass over the tensor
// with a rounding to the storage type in between; scaled_dot_product_attention (crates/hodu_nn/src/modules/
// attention.rs:25-70) runs it on the [.., Sq, Sk] scores between its two batched products, after an optional causal
// masked_fill(-inf) (:40-48, mask[i][j] = j > i, :73-86).
//
// Here a row is read once: a wavefront owns a row whose dim is dense and at most 4096 long and keeps it in
// registers (max, exp, sum, scale without touching memory again); a longer dense row belongs to a workgroup, which
// reads it twice (an online maximum / sum pass, then the pass that writes); strided rows take three passes from
// memory with a thread per row; a dim other than the last one gets a thread per position of the other dims.  Arithmetic: elements widened exactly to f32 (f64 stays f64), exp and the sum in that
// type, one rounding (RNE) on store.  With `causal` the entries j > i of each [Sq, Sk] matrix count as -inf: they
// come out as exact zeros, and the mask tensor is never built.
#include "common.hpp"
#include "device_types.hpp"
#include "elem.hpp"

namespace hodu {
namespace {

struct DevSoftmax {
    long rows;         // kept positions
    long len;          // extent of the softmax dim
    long stride;       // its element stride in the input
    long offset;
    int kept_n;
    long kept_shape[16], kept_stride[16];
    int causal;        // 1: mask j > i, i = the row's index along the innermost kept dim (extent sq)
    long sq;
    long inner;        // product of the extents after the softmax dim (1: it is the last dim)
};

__device__ __forceinline__ long row_offset(const DevSoftmax &s, long row) {
    long off = 0;
    for (int d = s.kept_n - 1; d >= 0; d--) {
        off += (row % s.kept_shape[d]) * s.kept_stride[d];
        row /= s.kept_shape[d];
    }
    return off;
}

template <class W> __device__ __forceinline__ W wexp(W x);
template <> __device__ __forceinline__ float wexp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double wexp<double>(double x) { return exp(x); }

// over groups of LANES neighbouring lanes (a power of two)
template <class W, int LANES = 64> __device__ __forceinline__ W lanes_max(W v) {
#pragma unroll
    for (int m = LANES / 2; m >= 1; m >>= 1) {
        const W o = __shfl_xor(v, m, 64);
        v = o > v ? o : v;
    }
    return v;
}
template <class W, int LANES = 64> __device__ __forceinline__ W lanes_add(W v) {
#pragma unroll
    for (int m = LANES / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// one wavefront per row, the row (dense, len <= 64 * NPL) held in registers
template <class E, int NPL>
__global__ __launch_bounds__(256) void softmax_row_kernel(const typename E::storage *__restrict__ in,
                                                         typename E::storage *__restrict__ out, DevSoftmax s) {
    typedef typename E::acc W;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= s.rows) return;
    const typename E::storage *x = in + s.offset + row_offset(s, row);
    const long limit = s.causal ? (row % s.sq) + 1 : s.len;  // entries at or beyond `limit` are masked
    const W ninf = -(W)INFINITY;
    W v[NPL];
    W m = ninf;
#pragma unroll
    for (int i = 0; i < NPL; i++) {
        const long j = lane + 64L * i;
        v[i] = (j < s.len && j < limit) ? (W)E::load(x[j]) : ninf;
        m = v[i] > m ? v[i] : m;
    }
    m = lanes_max(m);
    W sum = (W)0;
#pragma unroll
    for (int i = 0; i < NPL; i++) {
        v[i] = v[i] == ninf ? (W)0 : wexp<W>(v[i] - m);
        sum += v[i];
    }
    sum = lanes_add(sum);
    typename E::storage *y = out + row * s.len;
#pragma unroll
    for (int i = 0; i < NPL; i++) {
        const long j = lane + 64L * i;
        if (j < s.len) y[j] = E::store(v[i] / sum);
    }
}

// the same with 16-byte accesses: a lane holds NV vectors of V neighbouring entries (len a multiple of V, rows and
// bases 16-byte aligned)
// LPR lanes per row: short rows share a wavefront (64 / LPR of them) instead of leaving most of its lanes idle
template <class E, int NV, int V, int LPR = 64>
__global__ __launch_bounds__(256) void softmax_row_vec_kernel(const typename E::storage *__restrict__ in,
                                                             typename E::storage *__restrict__ out, DevSoftmax s) {
    typedef typename E::acc W;
    typedef typename E::storage S;
    struct alignas(16) Vec { S e[V]; };
    const long row = (long)blockIdx.x * (256 / LPR) + (threadIdx.x / LPR);
    const int lane = threadIdx.x % LPR;
    if (row >= s.rows) return;  // (whole groups of LPR lanes leave together; the shuffles stay inside a group)
    const S *x = in + s.offset + row_offset(s, row);
    const long limit = s.causal ? (row % s.sq) + 1 : s.len;
    const W ninf = -(W)INFINITY;
    W v[NV][V];
    W m = ninf;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const long j0 = (lane + (long)LPR * i) * V;
        Vec raw;
        if (j0 < s.len && j0 < limit) raw = *reinterpret_cast<const Vec *>(x + j0);
#pragma unroll
        for (int e = 0; e < V; e++) {
            v[i][e] = (j0 + e < s.len && j0 + e < limit) ? (W)E::load(raw.e[e]) : ninf;
            m = v[i][e] > m ? v[i][e] : m;
        }
    }
    m = lanes_max<W, LPR>(m);
    W sum = (W)0;
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
        for (int e = 0; e < V; e++) {
            v[i][e] = v[i][e] == ninf ? (W)0 : wexp<W>(v[i][e] - m);
            sum += v[i][e];
        }
    sum = lanes_add<W, LPR>(sum);
    S *y = out + row * s.len;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const long j0 = (lane + (long)LPR * i) * V;
        if (j0 >= s.len) continue;
        Vec o;
#pragma unroll
        for (int e = 0; e < V; e++) o.e[e] = E::store(v[i][e] / sum);
        *reinterpret_cast<Vec *>(y + j0) = o;
    }
}

// a dense row of any length: a workgroup per row, two passes.  Pass 1 keeps, per thread, a running maximum m and the
// sum l of exp(x - m) over its entries (rescaled when m moves), then the 256 pairs meet: (m, l) + (m', l') =
// (M = max(m, m'), l exp(m - M) + l' exp(m' - M)).  Pass 2 reads the row again (from L2 for all but very long rows)
// and writes exp(x - M) / L.  V > 1: 16 bytes per lane (len a multiple of V, rows and bases 16-byte aligned).
template <class W> __device__ __forceinline__ void meet(W &m, W &l, W m2, W l2) {
    const W big = m2 > m ? m2 : m;
    if (big == -(W)INFINITY) return;  // both empty: l stays 0
    l = l * wexp<W>(m - big) + l2 * wexp<W>(m2 - big);
    m = big;
}

template <class E, int V>
__global__ __launch_bounds__(256) void softmax_long_kernel(const typename E::storage *__restrict__ in,
                                                          typename E::storage *__restrict__ out, DevSoftmax s) {
    typedef typename E::acc W;
    typedef typename E::storage S;
    struct alignas(sizeof(S) * V) Vec { S e[V]; };
    __shared__ W wave_m[4], wave_l[4];
    const long row = blockIdx.x;
    const int tid = threadIdx.x;
    const S *x = in + s.offset + row_offset(s, row);
    long limit = s.causal ? (row % s.sq) + 1 : s.len;
    limit = limit < s.len ? limit : s.len;
    const W ninf = -(W)INFINITY;
    W m = ninf, l = (W)0;
    for (long j0 = (long)tid * V; j0 < limit; j0 += 256L * V) {
        W v[V];
        if constexpr (V == 1) {
            v[0] = (W)E::load(x[j0]);
        } else {
            const Vec raw = *reinterpret_cast<const Vec *>(x + j0);
#pragma unroll
            for (int e = 0; e < V; e++) v[e] = j0 + e < limit ? (W)E::load(raw.e[e]) : ninf;
        }
        W vm = v[0];
#pragma unroll
        for (int e = 1; e < V; e++) vm = v[e] > vm ? v[e] : vm;
        if (vm > m) {
            l *= wexp<W>(m - vm);  // exp(-inf) = 0 on the first entries
            m = vm;
        }
        if (m != ninf) {
#pragma unroll
            for (int e = 0; e < V; e++) l += wexp<W>(v[e] - m);
        }
    }
#pragma unroll
    for (int k = 32; k >= 1; k >>= 1) meet(m, l, (W)__shfl_xor(m, k, 64), (W)__shfl_xor(l, k, 64));
    if ((tid & 63) == 0) { wave_m[tid >> 6] = m; wave_l[tid >> 6] = l; }
    __syncthreads();
    m = wave_m[0]; l = wave_l[0];
#pragma unroll
    for (int w = 1; w < 4; w++) meet(m, l, wave_m[w], wave_l[w]);
    const W inv = (W)1 / l;
    S *y = out + row * s.len;
    for (long j0 = (long)tid * V; j0 < s.len; j0 += 256L * V) {
        if constexpr (V == 1) {
            y[j0] = E::store(j0 < limit ? wexp<W>((W)E::load(x[j0]) - m) * inv : (W)0);
        } else {
            Vec o;
            if (j0 < limit) {
                const Vec raw = *reinterpret_cast<const Vec *>(x + j0);
#pragma unroll
                for (int e = 0; e < V; e++) o.e[e] = E::store(j0 + e < limit ? wexp<W>((W)E::load(raw.e[e]) - m) * inv : (W)0);
            } else {
#pragma unroll
                for (int e = 0; e < V; e++) o.e[e] = E::store((W)0);
            }
            *reinterpret_cast<Vec *>(y + j0) = o;
        }
    }
}

// softmax along a dim that is not the last one: a thread per kept position (neighbouring threads are neighbouring
// positions of the dims after the softmax dim, so their loads and stores are neighbours in memory), two passes: an
// online maximum / sum over the dim, then the pass that writes.  The output is contiguous in the input's shape:
// position (outer, j, inner) at (outer * len + j) * inner_extent + inner.
template <class E>
__global__ __launch_bounds__(256) void softmax_cols_kernel(const typename E::storage *__restrict__ in,
                                                          typename E::storage *__restrict__ out, DevSoftmax s) {
    typedef typename E::acc W;
    const long row = (long)blockIdx.x * 256 + threadIdx.x;
    if (row >= s.rows) return;
    const typename E::storage *x = in + s.offset + row_offset(s, row);
    W m = -(W)INFINITY, l = (W)0;
    for (long j = 0; j < s.len; j++) {
        const W v = (W)E::load(x[j * s.stride]);
        if (v > m) {
            l *= wexp<W>(m - v);  // exp(-inf) = 0 on the first entry
            m = v;
        }
        if (m != -(W)INFINITY) l += wexp<W>(v - m);
    }
    const W inv = (W)1 / l;
    typename E::storage *y = out + (row / s.inner) * s.len * s.inner + row % s.inner;
    for (long j = 0; j < s.len; j++) y[j * s.inner] = E::store(wexp<W>((W)E::load(x[j * s.stride]) - m) * inv);
}

// any stride, any length: a thread per row, three passes from memory
template <class E>
__global__ __launch_bounds__(256) void softmax_strided_kernel(const typename E::storage *__restrict__ in,
                                                             typename E::storage *__restrict__ out, DevSoftmax s) {
    typedef typename E::acc W;
    const long row = (long)blockIdx.x * 256 + threadIdx.x;
    if (row >= s.rows) return;
    const typename E::storage *x = in + s.offset + row_offset(s, row);
    const long limit = s.causal ? ((row % s.sq) + 1 < s.len ? (row % s.sq) + 1 : s.len) : s.len;
    W m = -(W)INFINITY;
    for (long j = 0; j < limit; j++) {
        const W v = (W)E::load(x[j * s.stride]);
        m = v > m ? v : m;
    }
    W sum = (W)0;
    for (long j = 0; j < limit; j++) sum += wexp<W>((W)E::load(x[j * s.stride]) - m);
    typename E::storage *y = out + row * s.len;
    for (long j = 0; j < s.len; j++) y[j] = E::store(j < limit ? wexp<W>((W)E::load(x[j * s.stride]) - m) / sum : (W)0);
}

// Softmax along the last dim with scaled_dot_product_attention's attn_mask (crates/hodu_nn/src/modules/attention.rs:
// 50-56) and, optionally, its causal mask folded in.  The reference fills masked scores with get_neg_inf(dtype)
// (:88-96) through masked_fill and then runs the softmax over ALL entries: -inf in f32 / f64, a finite stand-in in the
// 16-bit types (-65504 converted to the dtype).  This kernel substitutes the same fill for a masked entry and computes
// the same function, so a masked entry of a row with an open one is an exact zero, a row masked entirely is uniform
// in bf16 / f16 and NaN in f32 / f64.  The mask (one byte per element, 0 = masked) keeps its own strides over the
// input's shape -- 0 where it is broadcast -- and is never expanded.  One wavefront per row, three passes over it
// (maximum, sum, write): the second and third read what the first brought into L2.
struct DevMaskedSoftmax {
    long rows, len;
    long in_stride, in_off;         // element stride of the softmax dim in the input, offset of the input layout
    long mask_stride, mask_off;     // the same for the mask
    int lead_n;                     // dims in front of the softmax dim
    long lead_shape[16], in_lead[16], mask_lead[16];
    int causal;
    long sq;
    double fill;                    // what a masked score counts as
};

template <class E>
__global__ __launch_bounds__(256) void softmax_masked_kernel(const typename E::storage *__restrict__ in,
                                                            typename E::storage *__restrict__ out,
                                                            const unsigned char *__restrict__ mask, DevMaskedSoftmax s) {
    typedef typename E::acc W;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= s.rows) return;  // (whole wavefronts leave together: the shuffles below stay complete)
    long xo = s.in_off, mo = s.mask_off, rem = row;
    for (int d = s.lead_n - 1; d >= 0; d--) {
        const long i = rem % s.lead_shape[d];
        rem /= s.lead_shape[d];
        xo += i * s.in_lead[d];
        mo += i * s.mask_lead[d];
    }
    const typename E::storage *x = in + xo;
    const unsigned char *mk = mask + mo;
    long limit = s.causal ? (row % s.sq) + 1 : s.len;
    limit = limit < s.len ? limit : s.len;
    const W fill = (W)s.fill;
    auto value = [&](long j) -> W { return (j < limit && mk[j * s.mask_stride] != 0) ? (W)E::load(x[j * s.in_stride]) : fill; };
    W m = -(W)INFINITY;
    for (long j = lane; j < s.len; j += 64) {
        const W v = value(j);
        m = v > m ? v : m;
    }
    m = lanes_max(m);
    W sum = (W)0;
    for (long j = lane; j < s.len; j += 64) sum += wexp<W>(value(j) - m);
    sum = lanes_add(sum);
    typename E::storage *y = out + row * s.len;
    for (long j = lane; j < s.len; j += 64) y[j] = E::store(wexp<W>(value(j) - m) / sum);
}

template <class E> int run_masked(hodu_rocm_ctx *ctx, const void *in, void *out, const void *mask, const DevMaskedSoftmax &s) {
    typedef typename E::storage S;
    if (s.rows == 0 || s.len == 0) return HODU_ROCM_OK;
    const long blocks = (s.rows + 3) / 4;
    if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "softmax needs %ld workgroups", blocks);
    ctx->last_kernel = "softmax_masked";
    hipLaunchKernelGGL(softmax_masked_kernel<E>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out,
                       (const unsigned char *)mask, s);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <class E> int run(hodu_rocm_ctx *ctx, const void *in, void *out, const DevSoftmax &s, bool dim_is_last) {
    typedef typename E::storage S;
    if (s.rows == 0 || s.len == 0) return HODU_ROCM_OK;
    // the row kernel writes row `r` at out + r * len: the softmax dim must be the output's last dim
    if (dim_is_last && s.stride == 1 && s.len <= 4096) {
        const long blocks = (s.rows + 3) / 4;
        if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "softmax needs %ld workgroups", blocks);
        constexpr int V = 16 / (int)sizeof(S);
        bool vec = s.len % V == 0 && s.offset % V == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0;
        for (int d = 0; d < s.kept_n; d++) vec = vec && s.kept_stride[d] % V == 0;
        if (vec) {
            ctx->last_kernel = "softmax_row_vec";
            const long vecs = s.len / V;
#define LAUNCHV(NV) hipLaunchKernelGGL((softmax_row_vec_kernel<E, NV, V>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, s)
#define LAUNCHS(LPR) hipLaunchKernelGGL((softmax_row_vec_kernel<E, 1, V, LPR>), dim3((unsigned)((s.rows + 256 / LPR - 1) / (256 / LPR))), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, s)
            if (vecs <= 16) LAUNCHS(16);
            else if (vecs <= 32) LAUNCHS(32);
            else if (vecs <= 64) LAUNCHV(1);
            else if (vecs <= 128) LAUNCHV(2);
            else if (vecs <= 256) LAUNCHV(4);
            else if (vecs <= 512) LAUNCHV(8);
            else LAUNCHV(64 / V);  // up to 4096 entries
#undef LAUNCHS
#undef LAUNCHV
            HODU_HIP(hipGetLastError());
            return HODU_ROCM_OK;
        }
        ctx->last_kernel = "softmax_row";
#define LAUNCH(NPL) hipLaunchKernelGGL((softmax_row_kernel<E, NPL>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, s)
        if (s.len <= 64 * 2) LAUNCH(2);
        else if (s.len <= 64 * 8) LAUNCH(8);
        else if (s.len <= 64 * 16) LAUNCH(16);
        else if (s.len <= 64 * 32) LAUNCH(32);
        else LAUNCH(64);
#undef LAUNCH
        HODU_HIP(hipGetLastError());
        return HODU_ROCM_OK;
    }
    if (!dim_is_last) {
        const long blocks = (s.rows + 255) / 256;
        if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "softmax needs %ld workgroups", blocks);
        ctx->last_kernel = "softmax_cols";
        hipLaunchKernelGGL(softmax_cols_kernel<E>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, s);
        HODU_HIP(hipGetLastError());
        return HODU_ROCM_OK;
    }
    if (s.stride == 1 && s.rows <= 0x7FFFFFFFL) {
        constexpr int V = 16 / (int)sizeof(S);
        bool vec = s.len % V == 0 && s.offset % V == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0;
        for (int d = 0; d < s.kept_n; d++) vec = vec && s.kept_stride[d] % V == 0;
        if (vec) {
            ctx->last_kernel = "softmax_long_vec";
            hipLaunchKernelGGL((softmax_long_kernel<E, V>), dim3((unsigned)s.rows), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, s);
        } else {
            ctx->last_kernel = "softmax_long";
            hipLaunchKernelGGL((softmax_long_kernel<E, 1>), dim3((unsigned)s.rows), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, s);
        }
        HODU_HIP(hipGetLastError());
        return HODU_ROCM_OK;
    }
    const long blocks = (s.rows + 255) / 256;
    if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "softmax needs %ld workgroups", blocks);
    ctx->last_kernel = "softmax_strided";
    hipLaunchKernelGGL(softmax_strided_kernel<E>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, s);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace

// r: the reduction over the softmax dim as parsed from reduce_metadata (one reduced dim); inner: product of the
// extents after that dim (1: it is the tensor's last); sq: extent of the dim before it (for the causal mask)
int launch_softmax(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const Reduction &r, long inner,
                   int causal, long sq) {
    const bool dim_is_last = inner == 1;
    DevSoftmax s{};
    s.inner = inner;
    s.rows = r.n_out;
    s.len = r.reduce_size;
    s.stride = r.red_n > 0 ? r.red_stride[0] : 1;
    s.offset = r.offset;
    s.kept_n = r.kept_n;
    for (int d = 0; d < 16; d++) {
        s.kept_shape[d] = d < r.kept_n ? r.kept_shape[d] : 1;
        s.kept_stride[d] = d < r.kept_n ? r.kept_stride[d] : 0;
    }
    s.causal = causal;
    s.sq = sq > 0 ? sq : 1;
    switch (dtype) {
    case HODU_BF16: return run<Elem<HODU_BF16>>(ctx, in, out, s, dim_is_last);
    case HODU_F16: return run<Elem<HODU_F16>>(ctx, in, out, s, dim_is_last);
    case HODU_F32: return run<Elem<HODU_F32>>(ctx, in, out, s, dim_is_last);
    case HODU_F64: return run<Elem<HODU_F64>>(ctx, in, out, s, dim_is_last);
    default: return fail(HODU_ROCM_UNSUPPORTED, "softmax: dtype id %d is not bf16 / f16 / f32 / f64", dtype);
    }
}

// shape / in_strides / mask_strides: the input's nd extents and the two layouts' element strides over them (softmax dim
// last, nd >= 1); the output is contiguous in that shape
int launch_softmax_masked(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const void *mask, int nd,
                          const long *shape, const long *in_strides, long in_off, const long *mask_strides, long mask_off,
                          int causal) {
    DevMaskedSoftmax s{};
    s.len = shape[nd - 1];
    s.in_stride = in_strides[nd - 1];
    s.mask_stride = mask_strides[nd - 1];
    s.in_off = in_off;
    s.mask_off = mask_off;
    s.lead_n = nd - 1;
    s.rows = 1;
    for (int d = 0; d < 16; d++) {
        s.lead_shape[d] = d < nd - 1 ? shape[d] : 1;
        s.in_lead[d] = d < nd - 1 ? in_strides[d] : 0;
        s.mask_lead[d] = d < nd - 1 ? mask_strides[d] : 0;
        s.rows *= s.lead_shape[d];
    }
    s.causal = causal;
    s.sq = nd >= 2 ? shape[nd - 2] : 1;
    if (s.sq <= 0) s.sq = 1;
    switch (dtype) {
    case HODU_BF16: s.fill = -65536.0; return run_masked<Elem<HODU_BF16>>(ctx, in, out, mask, s);
    case HODU_F16: s.fill = -65504.0; return run_masked<Elem<HODU_F16>>(ctx, in, out, mask, s);
    case HODU_F32: s.fill = -(double)INFINITY; return run_masked<Elem<HODU_F32>>(ctx, in, out, mask, s);
    case HODU_F64: s.fill = -(double)INFINITY; return run_masked<Elem<HODU_F64>>(ctx, in, out, mask, s);
    default: return fail(HODU_ROCM_UNSUPPORTED, "softmax: dtype id %d is not bf16 / f16 / f32 / f64", dtype);
    }
}

}  // namespace hodu
