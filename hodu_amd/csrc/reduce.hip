// Sum over some dims of a strided tensor: what Tensor::sum_to_shape launches, one dim at a time, on the gradients of a
// matmul whose operand was broadcast (crates/hodu_core/src/tensor/gradient/vjp_matrix.rs:41-43,
// tensor/ops/reduce.rs:19-50).  Replaces hodu_cpu_sum_<dt> (crates/hodu_cpu_kernels/kernels/ops_reduce.c:47-118,
// :127-130, :133-237, :345-352): one thread per output element there, walking the reduced dims innermost first.
//
// Arithmetic as for the products: narrow floats and f32 accumulate in f32 and round once on store (the reference
// re-rounds its bf16 / f16 / f8 accumulator after every add), f64 in f64, integers wrap.
//
// Kernels, chosen by where the unit stride is and by how many outputs there are:
//   * the outputs' last dim is dense (leading dims are summed: the sum_to_shape case): a thread owns V neighbouring
//     outputs and walks the reduced dims; neighbouring threads read neighbouring addresses, 16 bytes per lane when
//     alignment allows.  HBM-bound, every input element is read once;
//   * the same with few outputs and a long reduction (the gradient of a bias: [batch * rows, features] summed to
//     [features]): one thread per output vector would leave most of the chip idle, so the reduced index space is cut
//     into chunks, one workgroup per (64 output vectors, chunk), its four wavefronts taking every fourth row; the
//     chunks' partial sums (in the accumulate type) go through the context's workspace and a second kernel adds
//     them in chunk order and rounds once.  Few outputs with a long reduction take this form whatever their layout (a
//     strided tensor summed to a scalar): uncoalesced reads across a whole chip beat one lane walking the tensor alone;
//   * the innermost reduced dim is dense (a row sum): a wavefront owns an output, its lanes stride over that dim
//     (16 bytes per lane when alignment allows), and the lane sums meet in a butterfly; few long rows (sum_all of a
//     large tensor is one) are cut into chunks across workgroups in the same two-kernel way.
// The same file holds the product of two long vectors (Tensor::matmul of two 1-D tensors is mul + sum_all in the
// reference): chunks of sum_k a[k] b[k] across workgroups, then the same second kernel.
#include "common.hpp"
#include "device_types.hpp"
#include "elem.hpp"

namespace hodu {
namespace {

// Reduction without the host-only parts, small enough to pass by value
struct DevReduction {
    long n_out, reduce_size, offset;
    int kept_n, red_n;
    long kept_shape[16], kept_stride[16];
    long red_shape[16], red_stride[16];
};

// element offset of output index `o` (row-major over the kept dims)
__device__ __forceinline__ long kept_offset(const DevReduction &r, long o) {
    long off = 0;
    for (int d = r.kept_n - 1; d >= 0; d--) {
        off += (o % r.kept_shape[d]) * r.kept_stride[d];
        o /= r.kept_shape[d];
    }
    return off;
}

// element offset of index `i` over all reduced dims but the innermost
__device__ __forceinline__ long outer_red_offset(const DevReduction &r, long i) {
    long off = 0;
    for (int d = r.red_n - 2; d >= 0; d--) {
        off += (i % r.red_shape[d]) * r.red_stride[d];
        i /= r.red_shape[d];
    }
    return off;
}

template <class E, int V>
__global__ __launch_bounds__(256) void sum_by_output_kernel(const typename E::storage *__restrict__ in,
                                                           typename E::storage *__restrict__ out, DevReduction r) {
    typedef typename E::storage S;
    typedef typename E::acc A;
    const long o = ((long)blockIdx.x * 256 + threadIdx.x) * V;
    if (o >= r.n_out) return;
    const S *base = in + r.offset + kept_offset(r, o);
    A acc[V];
#pragma unroll
    for (int v = 0; v < V; v++) acc[v] = (A)0;
    const long inner = r.red_n > 0 ? r.red_shape[r.red_n - 1] : 1, inner_stride = r.red_n > 0 ? r.red_stride[r.red_n - 1] : 0;
    const long outer = r.reduce_size / (inner > 0 ? inner : 1);
    for (long i = 0; i < outer; i++) {
        const S *p = base + outer_red_offset(r, i);
        for (long j = 0; j < inner; j++, p += inner_stride) {
            if constexpr (V == 1) {
                acc[0] += E::load(p[0]);
            } else {
                struct alignas(sizeof(S) * V) Vec { S e[V]; };
                const Vec x = *reinterpret_cast<const Vec *>(p);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] += E::load(x.e[v]);
            }
        }
    }
    if constexpr (V == 1) {
        out[o] = E::store(acc[0]);
    } else {
        struct alignas(sizeof(S) * V) Vec { S e[V]; };
        Vec y;
#pragma unroll
        for (int v = 0; v < V; v++) y.e[v] = E::store(acc[v]);
        *reinterpret_cast<Vec *>(out + o) = y;
    }
}

template <class A> __device__ __forceinline__ A lanes_sum(A v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// flattened index over ALL reduced dims -> element offset
__device__ __forceinline__ long red_offset(const DevReduction &r, long i) {
    long off = 0;
    for (int d = r.red_n - 1; d >= 0; d--) {
        off += (i % r.red_shape[d]) * r.red_stride[d];
        i /= r.red_shape[d];
    }
    return off;
}

// few outputs, long reduction: workgroup (x, y) sums chunk y of the reduced index space for output vectors
// 64 x .. 64 x + 63; wavefront w takes indices chunk_begin + w, + 4, ..; partial[y][output] in the accumulate type
template <class E, int V>
__global__ __launch_bounds__(256) void sum_chunks_kernel(const typename E::storage *__restrict__ in,
                                                        typename E::acc *__restrict__ partial, DevReduction r,
                                                        long per_chunk) {
    typedef typename E::storage S;
    typedef typename E::acc A;
    __shared__ A meet[3][64][V];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long o = ((long)blockIdx.x * 64 + lane) * V;
    const long begin = (long)blockIdx.y * per_chunk;
    const long end = begin + per_chunk < r.reduce_size ? begin + per_chunk : r.reduce_size;
    A acc[V];
#pragma unroll
    for (int v = 0; v < V; v++) acc[v] = (A)0;
    if (o < r.n_out) {
        const S *base = in + r.offset + kept_offset(r, o);
        struct alignas(sizeof(S) * V) Vec { S e[V]; };
        constexpr int IF = 4;  // loads in flight per lane: the additions keep their order (index by index)
        long i = begin + wave;
        for (; i + 4 * (IF - 1) < end; i += 4 * IF) {
            Vec x[IF];
#pragma unroll
            for (int u = 0; u < IF; u++) x[u] = *reinterpret_cast<const Vec *>(base + red_offset(r, i + 4 * u));
#pragma unroll
            for (int u = 0; u < IF; u++)
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] += E::load(x[u].e[v]);
        }
        for (; i < end; i += 4) {
            const Vec x = *reinterpret_cast<const Vec *>(base + red_offset(r, i));
#pragma unroll
            for (int v = 0; v < V; v++) acc[v] += E::load(x.e[v]);
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int v = 0; v < V; v++) meet[wave - 1][lane][v] = acc[v];
    }
    __syncthreads();
    if (wave == 0 && o < r.n_out) {
#pragma unroll
        for (int v = 0; v < V; v++)
            partial[(long)blockIdx.y * r.n_out + o + v] = acc[v] + meet[0][lane][v] + meet[1][lane][v] + meet[2][lane][v];
    }
}

// out[o] = round(sum over chunks of partial[chunk][o]): a workgroup owns 64 outputs, its four wavefronts take every
// fourth chunk (several loads in flight each) and meet in LDS; the order of the additions is fixed
template <class E>
__global__ __launch_bounds__(256) void sum_finish_kernel(const typename E::acc *__restrict__ partial,
                                                        typename E::storage *__restrict__ out, long n_out, int chunks) {
    typedef typename E::acc A;
    __shared__ A meet[3][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long o = (long)blockIdx.x * 64 + lane;
    A acc = (A)0;
    if (o < n_out) {
#pragma unroll 8
        for (int c = wave; c < chunks; c += 4) acc += partial[(long)c * n_out + o];
    }
    if (wave > 0) meet[wave - 1][lane] = acc;
    __syncthreads();
    if (wave == 0 && o < n_out) out[o] = E::store(acc + meet[0][lane] + meet[1][lane] + meet[2][lane]);
}


// one wavefront per output; the innermost reduced dim has stride 1
// V > 1: every row start is a multiple of V elements and 16 bytes (the launcher checks), a lane reads V at a time
template <class E, int V>
__global__ __launch_bounds__(256) void sum_by_row_kernel(const typename E::storage *__restrict__ in,
                                                        typename E::storage *__restrict__ out, DevReduction r) {
    typedef typename E::storage S;
    typedef typename E::acc A;
    const long o = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (o >= r.n_out) return;
    const S *base = in + r.offset + kept_offset(r, o);
    const long inner = r.red_shape[r.red_n - 1], outer = r.reduce_size / inner;
    A acc = (A)0;
    for (long i = 0; i < outer; i++) {
        const S *p = base + outer_red_offset(r, i);
        if constexpr (V == 1) {
            for (long j = lane; j < inner; j += 64) acc += E::load(p[j]);
        } else {
            struct alignas(sizeof(S) * V) Vec { S e[V]; };
            const long whole = inner / V;
            for (long j = lane; j < whole; j += 64) {
                const Vec x = reinterpret_cast<const Vec *>(p)[j];
#pragma unroll
                for (int v = 0; v < V; v++) acc += E::load(x.e[v]);
            }
            for (long j = whole * V + lane; j < inner; j += 64) acc += E::load(p[j]);
        }
    }
    acc = lanes_sum(acc);
    if (lane == 0) out[o] = E::store(acc);
}

// sum of the 256 threads' values, in thread 0 (fixed order: butterfly inside a wavefront, then the four wavefronts)
template <class A> __device__ __forceinline__ A block_sum(A v, A *meet4) {
    v = lanes_sum(v);
    if ((threadIdx.x & 63) == 0) meet4[threadIdx.x >> 6] = v;
    __syncthreads();
    return meet4[0] + meet4[1] + meet4[2] + meet4[3];
}

// few outputs, each a long dense row (sum_all of a large tensor is one such row): a workgroup sums chunk y of row x,
// 16 bytes per lane when V > 1 (rows start on vector boundaries), and leaves partial[y][x] for sum_finish_kernel
template <class E, int V>
__global__ __launch_bounds__(256) void sum_row_chunks_kernel(const typename E::storage *__restrict__ in,
                                                            typename E::acc *__restrict__ partial, DevReduction r,
                                                            long per_chunk) {
    typedef typename E::storage S;
    typedef typename E::acc A;
    __shared__ A meet4[4];
    const long o = blockIdx.x;
    const long inner = r.red_shape[r.red_n - 1], outer = r.reduce_size / inner;
    const long begin = (long)blockIdx.y * per_chunk;  // a multiple of V
    const long end = begin + per_chunk < inner ? begin + per_chunk : inner;
    const S *base = in + r.offset + kept_offset(r, o);
    A acc = (A)0;
    for (long i = 0; i < outer; i++) {
        const S *p = base + outer_red_offset(r, i);
        if constexpr (V == 1) {
            for (long j = begin + threadIdx.x; j < end; j += 256) acc += E::load(p[j]);
        } else {
            struct alignas(sizeof(S) * V) Vec { S e[V]; };
            const long whole = begin + (end - begin) / V * V;
            for (long j = begin + (long)threadIdx.x * V; j < whole; j += 256L * V) {
                const Vec x = *reinterpret_cast<const Vec *>(p + j);
#pragma unroll
                for (int v = 0; v < V; v++) acc += E::load(x.e[v]);
            }
            for (long j = whole + threadIdx.x; j < end; j += 256) acc += E::load(p[j]);
        }
    }
    acc = block_sum(acc, meet4);
    if (threadIdx.x == 0) partial[(long)blockIdx.y * r.n_out + o] = acc;
}

// the product of two vectors (Tensor::matmul of two 1-D tensors: mul, then sum_all in the reference,
// crates/hodu_core/src/tensor/ops/matrix.rs:38-47): chunk y of sum_k a[k] b[k], as above
template <class E, int V>
__global__ __launch_bounds__(256) void inner_product_kernel(const typename E::storage *__restrict__ a,
                                                           const typename E::storage *__restrict__ b,
                                                           typename E::acc *__restrict__ partial, long K, long a_k, long b_k,
                                                           long per_chunk) {
    typedef typename E::storage S;
    typedef typename E::acc A;
    __shared__ A meet4[4];
    const long begin = (long)blockIdx.x * per_chunk;
    const long end = begin + per_chunk < K ? begin + per_chunk : K;
    A acc = (A)0;
    if constexpr (V == 1) {
        for (long k = begin + threadIdx.x; k < end; k += 256) acc += E::load(a[k * a_k]) * E::load(b[k * b_k]);
    } else {  // both dense and aligned
        struct alignas(sizeof(S) * V) Vec { S e[V]; };
        const long whole = begin + (end - begin) / V * V;
        for (long k = begin + (long)threadIdx.x * V; k < whole; k += 256L * V) {
            const Vec x = *reinterpret_cast<const Vec *>(a + k), y = *reinterpret_cast<const Vec *>(b + k);
#pragma unroll
            for (int v = 0; v < V; v++) acc += E::load(x.e[v]) * E::load(y.e[v]);
        }
        for (long k = whole + threadIdx.x; k < end; k += 256) acc += E::load(a[k]) * E::load(b[k]);
    }
    acc = block_sum(acc, meet4);
    if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}

template <class S> __global__ __launch_bounds__(256) void zero_kernel(S *out, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = (S)0;
}

template <class E> int run(hodu_rocm_ctx *ctx, const void *in, void *out, const Reduction &red) {
    typedef typename E::storage S;
    DevReduction r{};
    r.n_out = red.n_out; r.reduce_size = red.reduce_size; r.offset = red.offset;
    r.kept_n = red.kept_n; r.red_n = red.red_n;
    for (int d = 0; d < 16; d++) {
        r.kept_shape[d] = d < red.kept_n ? red.kept_shape[d] : 1;
        r.kept_stride[d] = d < red.kept_n ? red.kept_stride[d] : 0;
        r.red_shape[d] = d < red.red_n ? red.red_shape[d] : 1;
        r.red_stride[d] = d < red.red_n ? red.red_stride[d] : 0;
    }
    if (r.n_out == 0) return HODU_ROCM_OK;
    if (r.reduce_size == 0) {  // an empty sum is zero (INIT_VAL of the reference's macro)
        const long blocks = (r.n_out + 255) / 256;
        if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "sum needs %ld workgroups", blocks);
        hipLaunchKernelGGL(zero_kernel<S>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (S *)out, r.n_out);
        HODU_HIP(hipGetLastError());
        ctx->last_kernel = "sum_empty";
        return HODU_ROCM_OK;
    }
    const bool row_dense = r.red_n > 0 && r.red_stride[r.red_n - 1] == 1 && r.red_shape[r.red_n - 1] >= 128;
    const bool out_dense = r.kept_n > 0 && r.kept_stride[r.kept_n - 1] == 1;
    constexpr int V = 16 / (int)sizeof(S);
    if (row_dense && !out_dense) {
        const long blocks = (r.n_out + 3) / 4;
        if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "sum needs %ld workgroups", blocks);
        // 16 bytes per lane: every row must start on a vector boundary
        bool vec = V > 1 && r.offset % V == 0 && (uintptr_t)in % 16 == 0;
        for (int d = 0; d < r.kept_n; d++) vec = vec && r.kept_stride[d] % V == 0;
        for (int d = 0; d + 1 < r.red_n; d++) vec = vec && r.red_stride[d] % V == 0;
        // few long rows (sum_all of a large tensor is one row): a wavefront per row would leave the chip idle
        const long cus = ctx->props.multiProcessorCount;
        const long inner = r.red_shape[r.red_n - 1];
        if (r.n_out < 2 * cus && inner >= 16384 && r.n_out <= 0x7FFFFFFFL) {
            typedef typename E::acc A;
            long chunks = (4 * cus + r.n_out - 1) / r.n_out;
            if (chunks > inner / 4096) chunks = inner / 4096;  // at least 4096 entries per chunk
            if (chunks > 65535) chunks = 65535;
            if (chunks >= 2) {
                long per_chunk = (inner + chunks - 1) / chunks;
                per_chunk = (per_chunk + 63) / 64 * 64;  // chunks start on vector boundaries
                chunks = (inner + per_chunk - 1) / per_chunk;
                int rc = ensure_workspace(ctx, (size_t)chunks * r.n_out * sizeof(A));
                if (rc != HODU_ROCM_OK) return rc;
                A *partial = (A *)ctx->workspace.ptr;
                if (vec) {
                    ctx->last_kernel = "sum_row_chunks_vec";
                    hipLaunchKernelGGL((sum_row_chunks_kernel<E, V>), dim3((unsigned)r.n_out, (unsigned)chunks), dim3(256), 0,
                                       ctx->stream, (const S *)in, partial, r, per_chunk);
                } else {
                    ctx->last_kernel = "sum_row_chunks";
                    hipLaunchKernelGGL((sum_row_chunks_kernel<E, 1>), dim3((unsigned)r.n_out, (unsigned)chunks), dim3(256), 0,
                                       ctx->stream, (const S *)in, partial, r, per_chunk);
                }
                HODU_HIP(hipGetLastError());
                hipLaunchKernelGGL(sum_finish_kernel<E>, dim3((unsigned)((r.n_out + 63) / 64)), dim3(256), 0, ctx->stream,
                                   (const A *)partial, (S *)out, r.n_out, (int)chunks);
                HODU_HIP(hipGetLastError());
                return HODU_ROCM_OK;
            }
        }
        if (vec) {
            ctx->last_kernel = "sum_by_row_vec";
            hipLaunchKernelGGL((sum_by_row_kernel<E, V>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, r);
        } else {
            ctx->last_kernel = "sum_by_row";
            hipLaunchKernelGGL((sum_by_row_kernel<E, 1>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, r);
        }
        HODU_HIP(hipGetLastError());
        return HODU_ROCM_OK;
    }
    // V outputs per thread as one 16-byte load: the outputs' last dim must be dense, a whole number of vectors
    // long, and every other stride, the offset and both bases must keep a vector aligned
    bool vec = V > 1 && out_dense && r.kept_shape[r.kept_n - 1] % V == 0 && r.offset % V == 0 &&
               (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0;
    for (int d = 0; d + 1 < r.kept_n; d++) vec = vec && r.kept_stride[d] % V == 0;
    for (int d = 0; d < r.red_n; d++) vec = vec && r.red_stride[d] % V == 0;
    const long threads = vec ? r.n_out / V : r.n_out;
    // few outputs and a long reduction: cut the reduced index space into chunks (see the top of the file)
    const long cus = ctx->props.multiProcessorCount;
    // (whatever the outputs' layout: a lane per output walking a long reduction alone is the slowest choice there is)
    if (threads < cus * 256 && r.reduce_size >= 64) {
        typedef typename E::acc A;
        const long xblocks = (threads + 63) / 64;
        long chunks = (4 * cus + xblocks - 1) / xblocks;           // about four workgroups per CU
        if (chunks > r.reduce_size / 8) chunks = r.reduce_size / 8;  // at least 8 indices per chunk
        if (chunks > 65535) chunks = 65535;
        if (chunks >= 2 && xblocks <= 0x7FFFFFFFL) {
            const long per_chunk = (r.reduce_size + chunks - 1) / chunks;
            chunks = (r.reduce_size + per_chunk - 1) / per_chunk;
            int rc = ensure_workspace(ctx, (size_t)chunks * r.n_out * sizeof(A));
            if (rc != HODU_ROCM_OK) return rc;
            A *partial = (A *)ctx->workspace.ptr;
            if (vec) {
                ctx->last_kernel = "sum_chunks_vec";
                hipLaunchKernelGGL((sum_chunks_kernel<E, V>), dim3((unsigned)xblocks, (unsigned)chunks), dim3(256), 0, ctx->stream,
                                   (const S *)in, partial, r, per_chunk);
            } else {
                ctx->last_kernel = "sum_chunks";
                hipLaunchKernelGGL((sum_chunks_kernel<E, 1>), dim3((unsigned)xblocks, (unsigned)chunks), dim3(256), 0, ctx->stream,
                                   (const S *)in, partial, r, per_chunk);
            }
            HODU_HIP(hipGetLastError());
            hipLaunchKernelGGL(sum_finish_kernel<E>, dim3((unsigned)((r.n_out + 63) / 64)), dim3(256), 0, ctx->stream,
                               (const A *)partial, (S *)out, r.n_out, (int)chunks);
            HODU_HIP(hipGetLastError());
            return HODU_ROCM_OK;
        }
    }
    const long blocks = (threads + 255) / 256;
    if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "sum needs %ld workgroups", blocks);
    if (vec) {
        ctx->last_kernel = "sum_by_output_vec";
        hipLaunchKernelGGL((sum_by_output_kernel<E, V>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, r);
    } else {
        ctx->last_kernel = "sum_by_output";
        hipLaunchKernelGGL((sum_by_output_kernel<E, 1>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, r);
    }
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace

namespace {
template <class E> int run_inner(hodu_rocm_ctx *ctx, const void *a_v, const void *b_v, void *out, long K, long a_k, long b_k,
                                 long a_off, long b_off) {
    typedef typename E::storage S;
    typedef typename E::acc A;
    const S *a = (const S *)a_v + a_off, *b = (const S *)b_v + b_off;
    const long cus = ctx->props.multiProcessorCount;
    long chunks = 4 * cus;
    if (chunks > K / 4096) chunks = K / 4096;
    if (chunks < 1) chunks = 1;
    long per_chunk = (K + chunks - 1) / chunks;
    per_chunk = (per_chunk + 63) / 64 * 64;
    chunks = (K + per_chunk - 1) / per_chunk;
    int rc = ensure_workspace(ctx, (size_t)chunks * sizeof(A));
    if (rc != HODU_ROCM_OK) return rc;
    A *partial = (A *)ctx->workspace.ptr;
    constexpr int V = 16 / (int)sizeof(S);
    const bool vec = V > 1 && a_k == 1 && b_k == 1 && (uintptr_t)a % 16 == 0 && (uintptr_t)b % 16 == 0;
    if (vec) {
        ctx->last_kernel = "inner_product_vec";
        hipLaunchKernelGGL((inner_product_kernel<E, V>), dim3((unsigned)chunks), dim3(256), 0, ctx->stream, a, b, partial, K, a_k, b_k, per_chunk);
    } else {
        ctx->last_kernel = "inner_product";
        hipLaunchKernelGGL((inner_product_kernel<E, 1>), dim3((unsigned)chunks), dim3(256), 0, ctx->stream, a, b, partial, K, a_k, b_k, per_chunk);
    }
    HODU_HIP(hipGetLastError());
    hipLaunchKernelGGL(sum_finish_kernel<E>, dim3(1), dim3(256), 0, ctx->stream, (const A *)partial, (S *)out, 1L, (int)chunks);
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}
}  // namespace

// [1, K] x [K, 1] with a long K: returns HODU_ROCM_UNSUPPORTED (no error text) for anything else
int launch_inner_product(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    if (kind != PK_SAME || g.M != 1 || g.N != 1 || g.batches != 1 || g.K < 16384 || g.epi.n != 0) return HODU_ROCM_UNSUPPORTED;
    switch (dtype) {
#define CASE(ID) case ID: return run_inner<Elem<ID>>(ctx, a, b, c, g.K, g.a_k, g.b_k, g.a_off, g.b_off);
        CASE(HODU_F8E4M3) CASE(HODU_F8E5M2) CASE(HODU_BF16) CASE(HODU_F16) CASE(HODU_F32) CASE(HODU_F64)
        CASE(HODU_U8) CASE(HODU_U16) CASE(HODU_U32) CASE(HODU_U64) CASE(HODU_I8) CASE(HODU_I16) CASE(HODU_I32)
        CASE(HODU_I64)
#undef CASE
    default: return HODU_ROCM_UNSUPPORTED;
    }
}

int launch_sum(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const Reduction &r) {
    switch (dtype) {
#define CASE(ID) case ID: return run<Elem<ID>>(ctx, in, out, r);
        CASE(HODU_F8E4M3) CASE(HODU_F8E5M2) CASE(HODU_BF16) CASE(HODU_F16) CASE(HODU_F32) CASE(HODU_F64)
        CASE(HODU_U8) CASE(HODU_U16) CASE(HODU_U32) CASE(HODU_U64) CASE(HODU_I8) CASE(HODU_I16) CASE(HODU_I32)
        CASE(HODU_I64)
#undef CASE
    default: return fail(HODU_ROCM_UNSUPPORTED, "sum: dtype id %d has no sum kernel", dtype);
    }
}

}  // namespace hodu
