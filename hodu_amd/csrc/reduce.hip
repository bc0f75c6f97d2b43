// Sum over some dims of a strided tensor: what Tensor::sum_to_shape launches, one dim at a time, on the gradients of a
// matmul whose operand was broadcast (crates/hodu_core/src/tensor/gradient/vjp_matrix.rs:41-43,
// tensor/ops/reduce.rs:19-50).  Replaces hodu_cpu_sum_<dt> (crates/hodu_cpu_kernels/kernels/ops_reduce.c:47-118,
// :127-130, :133-237, :345-352): one thread per output element there, walking the reduced dims innermost first.
//
// Arithmetic as for the products: narrow floats and f32 accumulate in f32 and round once on store (the reference
// re-rounds its bf16 / f16 / f8 accumulator after every add), f64 in f64, integers wrap.
//
// Two kernels, chosen by where the unit stride is:
//   * the outputs' last dim is dense (leading dims are summed: the sum_to_shape case): a thread owns V neighbouring
//     outputs and walks the reduced dims; neighbouring threads read neighbouring addresses, 16 bytes per lane when
//     alignment allows.  HBM-bound, every input element is read once;
//   * the innermost reduced dim is dense (a row sum): a wavefront owns an output, its lanes stride over that dim,
//     and the lane sums meet in a butterfly.
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

// one wavefront per output; the innermost reduced dim has stride 1
template <class E>
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
        for (long j = lane; j < inner; j += 64) acc += E::load(p[j]);
    }
    acc = lanes_sum(acc);
    if (lane == 0) out[o] = E::store(acc);
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
    if (row_dense && !out_dense) {
        const long blocks = (r.n_out + 3) / 4;
        if (blocks > 0x7FFFFFFFL) return fail(HODU_ROCM_UNSUPPORTED, "sum needs %ld workgroups", blocks);
        ctx->last_kernel = "sum_by_row";
        hipLaunchKernelGGL(sum_by_row_kernel<E>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const S *)in, (S *)out, r);
        HODU_HIP(hipGetLastError());
        return HODU_ROCM_OK;
    }
    // V outputs per thread as one 16-byte load: the outputs' last dim must be dense, a whole number of vectors
    // long, and every other stride, the offset and both bases must keep a vector aligned
    constexpr int V = 16 / (int)sizeof(S);
    bool vec = V > 1 && out_dense && r.kept_shape[r.kept_n - 1] % V == 0 && r.offset % V == 0 &&
               (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0;
    for (int d = 0; d + 1 < r.kept_n; d++) vec = vec && r.kept_stride[d] % V == 0;
    for (int d = 0; d < r.red_n; d++) vec = vec && r.red_stride[d] % V == 0;
    const long threads = vec ? r.n_out / V : r.n_out;
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
