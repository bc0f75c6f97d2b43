// to_dtype casts and the strided gather (contiguous) for all 15 hodu dtypes.
//
// Replaces hodu_cpu_cast_<src>_to_<dst> (crates/hodu_cpu_kernels/kernels/ops_cast.c:34-103, table
// :108-388) and hodu_cpu_contiguous_<dt> (kernels/ops_memory.c:19-84).  These are HBM-bound byte
// movers: the dense path moves 8 elements per lane with wide loads/stores, the strided path walks
// the merged dims per output element.
//
// Conversion semantics follow the reference element for element so the bytes match its CPU path:
// the intermediate is chosen by the SOURCE type (narrow floats and f32 go through f32, f64 stays
// f64, integers convert directly, bool normalises to 0/1 first); f32 -> bf16 TRUNCATES
// (t_bf16.h:35-39); f32 -> f16 / f8 use the reference's own round-half-up-and-clamp routines
// (t_f16.h:50-84, t_f8e4m3.h:52-85, t_f8e5m2.h:52-84) rather than the hardware's RNE converts.
// One deliberate difference: f8e4m3 is DECODED as OCP E4M3FN (exponent 15 is finite up to 448),
// which is what hodu's Rust F8E4M3 type and the gfx950 matrix cores implement; the reference's C
// decoder (t_f8e4m3.h:34-38) reads those 14 codes as inf/NaN.
#include <utility>

#include "common.hpp"
#include "device_types.hpp"
#include "epilogue.hpp"  // ref_f32_to_f16

namespace hodu {
namespace {

#pragma clang fp contract(off)

// ---- the reference's narrowing routines, restated for the device -------------------------------
__device__ __forceinline__ uint8_t ref_f32_to_f8e4m3(float val) {
    if (val == 0.0f) return 0;
    if (val != val) return 0x7F;
    const uint32_t sign = val < 0 ? 1u : 0u;
    val = fabsf(val);
    if (isinf(val) || val > 448.0f) return (uint8_t)((sign << 7) | 0x7Fu);
    if (val < 0.001953125f) return (uint8_t)(sign << 7);
    int e;
    float m = frexpf(val, &e);
    e += 6;
    if (e <= 0) { m = ldexpf(m, e); e = 0; }
    else if (e >= 15) return (uint8_t)((sign << 7) | 0x7Fu);
    int mb = (int)((m * 2.0f - 1.0f) * 8.0f + 0.5f);
    if (mb > 7) mb = 7;
    return (uint8_t)((sign << 7) | (uint32_t)(e << 3) | (uint32_t)mb);
}

__device__ __forceinline__ uint8_t ref_f32_to_f8e5m2(float val) {
    if (val == 0.0f) return 0;
    if (val != val) return 0x7F;
    const uint32_t sign = val < 0 ? 1u : 0u;
    val = fabsf(val);
    if (isinf(val) || val > 57344.0f) return (uint8_t)((sign << 7) | 0x7Fu);
    if (val < 0.0000152587890625f) return (uint8_t)(sign << 7);
    int e;
    float m = frexpf(val, &e);
    e += 14;
    if (e <= 0) { m = ldexpf(m, e); e = 0; }
    else if (e >= 31) return (uint8_t)((sign << 7) | 0x7Fu);
    int mb = (int)((m * 2.0f - 1.0f) * 4.0f + 0.5f);
    if (mb > 3) mb = 3;
    return (uint8_t)((sign << 7) | (uint32_t)(e << 2) | (uint32_t)mb);
}

// the reference's f16 decoder (t_f16.h:27-48) agrees with IEEE binary16 on every code
__device__ __forceinline__ float ref_f16_to_f32(uint16_t h) { return f16_bits_to_f32(h); }

// ---- per-dtype load (to the reference's intermediate) and store ---------------------------------
// intermediates: float, double, int64_t (signed sources), uint64_t (unsigned sources and bool)
template <int DT> struct Src;
template <> struct Src<HODU_BOOL> { typedef uint8_t T; static __device__ __forceinline__ uint64_t get(T v) { return v != 0; } };
template <> struct Src<HODU_F8E4M3> { typedef uint8_t T; static __device__ __forceinline__ float get(T v) { return f8e4m3_to_f32(v); } };
template <> struct Src<HODU_F8E5M2> { typedef uint8_t T; static __device__ __forceinline__ float get(T v) { return f8e5m2_to_f32(v); } };
template <> struct Src<HODU_BF16> { typedef uint16_t T; static __device__ __forceinline__ float get(T v) { return bf16_bits_to_f32(v); } };
template <> struct Src<HODU_F16> { typedef uint16_t T; static __device__ __forceinline__ float get(T v) { return ref_f16_to_f32(v); } };
template <> struct Src<HODU_F32> { typedef float T; static __device__ __forceinline__ float get(T v) { return v; } };
template <> struct Src<HODU_F64> { typedef double T; static __device__ __forceinline__ double get(T v) { return v; } };
template <> struct Src<HODU_U8> { typedef uint8_t T; static __device__ __forceinline__ uint64_t get(T v) { return v; } };
template <> struct Src<HODU_U16> { typedef uint16_t T; static __device__ __forceinline__ uint64_t get(T v) { return v; } };
template <> struct Src<HODU_U32> { typedef uint32_t T; static __device__ __forceinline__ uint64_t get(T v) { return v; } };
template <> struct Src<HODU_U64> { typedef uint64_t T; static __device__ __forceinline__ uint64_t get(T v) { return v; } };
template <> struct Src<HODU_I8> { typedef int8_t T; static __device__ __forceinline__ int64_t get(T v) { return v; } };
template <> struct Src<HODU_I16> { typedef int16_t T; static __device__ __forceinline__ int64_t get(T v) { return v; } };
template <> struct Src<HODU_I32> { typedef int32_t T; static __device__ __forceinline__ int64_t get(T v) { return v; } };
template <> struct Src<HODU_I64> { typedef int64_t T; static __device__ __forceinline__ int64_t get(T v) { return v; } };

// float -> integer: C's (T)x truncates toward zero.  Going through a 64-bit integer reproduces
// what the reference's x86-64 build does for every value that fits 64 bits (a negative float to
// an unsigned type wraps there); beyond that the reference is undefined behaviour.
template <class I, class F> __device__ __forceinline__ I trunc_to(F v) { return (I)(int64_t)v; }

template <int DT> struct Dst;
template <> struct Dst<HODU_BOOL> {
    typedef uint8_t T;
    template <class W> static __device__ __forceinline__ T put(W w) { return w != (W)0; }
};
#define NARROW_DST(ID, TT, FN)                                                                 \
    template <> struct Dst<ID> {                                                               \
        typedef TT T;                                                                          \
        template <class W> static __device__ __forceinline__ T put(W w) { return FN((float)w); } \
    };
__device__ __forceinline__ uint16_t trunc_bf16(float f) { return (uint16_t)(__float_as_uint(f) >> 16); }
NARROW_DST(HODU_F8E4M3, uint8_t, ref_f32_to_f8e4m3)
NARROW_DST(HODU_F8E5M2, uint8_t, ref_f32_to_f8e5m2)
NARROW_DST(HODU_BF16, uint16_t, trunc_bf16)
NARROW_DST(HODU_F16, uint16_t, ref_f32_to_f16)
#undef NARROW_DST
template <> struct Dst<HODU_F32> {
    typedef float T;
    template <class W> static __device__ __forceinline__ T put(W w) { return (float)w; }
};
template <> struct Dst<HODU_F64> {
    typedef double T;
    template <class W> static __device__ __forceinline__ T put(W w) { return (double)w; }
};
#define INT_DST(ID, TT)                                                                        \
    template <> struct Dst<ID> {                                                               \
        typedef TT T;                                                                          \
        static __device__ __forceinline__ T put(float w) { return trunc_to<TT>(w); }           \
        static __device__ __forceinline__ T put(double w) { return trunc_to<TT>(w); }          \
        static __device__ __forceinline__ T put(int64_t w) { return (TT)w; }                   \
        static __device__ __forceinline__ T put(uint64_t w) { return (TT)w; }                  \
    };
INT_DST(HODU_U8, uint8_t)
INT_DST(HODU_U16, uint16_t)
INT_DST(HODU_U32, uint32_t)
INT_DST(HODU_I8, int8_t)
INT_DST(HODU_I16, int16_t)
INT_DST(HODU_I32, int32_t)
INT_DST(HODU_I64, int64_t)
#undef INT_DST
template <> struct Dst<HODU_U64> {
    typedef uint64_t T;
    // negative inputs wrap through the signed conversion, as the reference's x86-64 build does
    static __device__ __forceinline__ T put(float w) { return w < 0.0f ? (uint64_t)(int64_t)w : (uint64_t)w; }
    static __device__ __forceinline__ T put(double w) { return w < 0.0 ? (uint64_t)(int64_t)w : (uint64_t)w; }
    static __device__ __forceinline__ T put(int64_t w) { return (uint64_t)w; }
    static __device__ __forceinline__ T put(uint64_t w) { return w; }
};

// same-type casts copy the element unchanged, except bool -> bool which normalises
template <int S, int D> struct Convert {
    static __device__ __forceinline__ typename Dst<D>::T run(typename Src<S>::T v) { return Dst<D>::put(Src<S>::get(v)); }
};
#define IDENTITY(ID)                                                                           \
    template <> struct Convert<ID, ID> {                                                       \
        static __device__ __forceinline__ typename Dst<ID>::T run(typename Src<ID>::T v) { return v; } \
    };
IDENTITY(HODU_F8E4M3) IDENTITY(HODU_F8E5M2) IDENTITY(HODU_BF16) IDENTITY(HODU_F16) IDENTITY(HODU_F32)
IDENTITY(HODU_F64) IDENTITY(HODU_U8) IDENTITY(HODU_U16) IDENTITY(HODU_U32) IDENTITY(HODU_U64) IDENTITY(HODU_I8)
IDENTITY(HODU_I16) IDENTITY(HODU_I32) IDENTITY(HODU_I64)
#undef IDENTITY

// ---- kernels ------------------------------------------------------------------------------------
constexpr int VEC = 8;  // elements per lane on the dense path

template <class T, int N> struct alignas(sizeof(T) * N) Pack { T v[N]; };

// dense source (offset already applied), 8 elements per lane; `in` and `out` aligned to 8 elements
template <int S, int D>
__global__ __launch_bounds__(256) void cast_dense_kernel(const typename Src<S>::T *__restrict__ in,
                                                        typename Dst<D>::T *__restrict__ out, long n) {
    typedef typename Src<S>::T TS;
    typedef typename Dst<D>::T TD;
    const long packs = n / VEC;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long p = (long)blockIdx.x * blockDim.x + threadIdx.x; p < packs; p += stride) {
        const Pack<TS, VEC> x = reinterpret_cast<const Pack<TS, VEC> *>(in)[p];
        Pack<TD, VEC> y;
#pragma unroll
        for (int i = 0; i < VEC; i++) y.v[i] = Convert<S, D>::run(x.v[i]);
        reinterpret_cast<Pack<TD, VEC> *>(out)[p] = y;
    }
    // tail (< 8 elements)
    const long done = packs * VEC;
    if (blockIdx.x == 0 && threadIdx.x < n - done) out[done + threadIdx.x] = Convert<S, D>::run(in[done + threadIdx.x]);
}

// dense but not 8-element aligned: one element per lane, still coalesced
template <int S, int D>
__global__ __launch_bounds__(256) void cast_flat_kernel(const typename Src<S>::T *__restrict__ in,
                                                       typename Dst<D>::T *__restrict__ out, long n) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = Convert<S, D>::run(in[i]);
}

struct DevStrided {
    int nd;
    long shape[16];
    long strides[16];
};

// strided source: row-major unravel of the output index over the merged dims
template <int S, int D>
__global__ __launch_bounds__(256) void cast_strided_kernel(const typename Src<S>::T *__restrict__ in,
                                                          typename Dst<D>::T *__restrict__ out, long n,
                                                          DevStrided s) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        long rem = i, pos = 0;
        for (int d = s.nd - 1; d >= 0; d--) {
            pos += (rem % s.shape[d]) * s.strides[d];
            rem /= s.shape[d];
        }
        out[i] = Convert<S, D>::run(in[pos]);
    }
}

// strided source whose unit stride sits on a dim J other than the last one (a transposed view): 64 x 64 tiles over
// (J, last dim L) go through LDS, read along J and written along L, so that both sides move whole cache lines.
// What contiguous() of a transposed operand costs in the reference is this gather (ops_memory.c:78-83, one thread).
struct DevTranspose {
    int n_outer;                                       // the remaining dims, walked by the tile index
    long outer_shape[16], outer_in[16], outer_out[16];
    long n_j, n_l, in_l, out_j;                        // extents; source stride of L, destination stride of J
    long tiles_j, tiles_l;
};
constexpr int TT = 64;

template <int S, int D>
__global__ __launch_bounds__(256) void cast_transpose_kernel(const typename Src<S>::T *__restrict__ in,
                                                            typename Dst<D>::T *__restrict__ out, DevTranspose t) {
    typedef typename Dst<D>::T TD;
    // a row of 64 elements plus padding of one 4-byte bank (at least one element): the column reads of the second
    // phase then fall into different banks
    constexpr int PAD = sizeof(TD) >= 4 ? 1 : 4 / (int)sizeof(TD);
    __shared__ TD tile[TT][TT + PAD];
    long b = blockIdx.x;
    const long tl = b % t.tiles_l; b /= t.tiles_l;
    const long tj = b % t.tiles_j; b /= t.tiles_j;
    long in_off = 0, out_off = 0;
    for (int d = t.n_outer - 1; d >= 0; d--) {
        const long i = b % t.outer_shape[d];
        b /= t.outer_shape[d];
        in_off += i * t.outer_in[d];
        out_off += i * t.outer_out[d];
    }
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const long j0 = tj * TT, l0 = tl * TT;
    {   // lanes along J (source stride 1)
        const long j = j0 + tx;
        typename Src<S>::T x[TT / 4];  // all 16 loads in flight before the first conversion
#pragma unroll
        for (int i = 0; i < TT / 4; i++) {
            const long l = l0 + ty + 4 * i;
            if (j < t.n_j && l < t.n_l) x[i] = in[in_off + j + l * t.in_l];
        }
#pragma unroll
        for (int i = 0; i < TT / 4; i++) {
            const long l = l0 + ty + 4 * i;
            if (j < t.n_j && l < t.n_l) tile[ty + 4 * i][tx] = Convert<S, D>::run(x[i]);
        }
    }
    __syncthreads();
    {   // lanes along L (destination stride 1)
        const long l = l0 + tx;
#pragma unroll
        for (int r = ty; r < TT; r += 4) {
            const long j = j0 + r;
            if (j < t.n_j && l < t.n_l) out[out_off + j * t.out_j + l] = tile[tx][r];
        }
    }
}

// the same with V elements per lane on both sides (8 bytes of the wider type): a wavefront reads 64 * V elements of
// one source row and writes 64 / V lanes * V elements of each destination row; tiles are (64 * V) x 64.  The launcher
// checks that every address involved is a multiple of V elements.
template <int S, int D, int V>
__global__ __launch_bounds__(256) void cast_transpose_vec_kernel(const typename Src<S>::T *__restrict__ in,
                                                                typename Dst<D>::T *__restrict__ out, DevTranspose t) {
    typedef typename Src<S>::T TS;
    typedef typename Dst<D>::T TD;
    constexpr int TJ = TT * V;
    constexpr int PAD = sizeof(TD) >= 4 ? 1 : 4 / (int)sizeof(TD);  // row pitch = an odd number of 4-byte banks
    __shared__ TD tile[TT][TJ + PAD];
    long b = blockIdx.x;
    const long tl = b % t.tiles_l; b /= t.tiles_l;
    const long tj = b % t.tiles_j; b /= t.tiles_j;
    long in_off = 0, out_off = 0;
    for (int d = t.n_outer - 1; d >= 0; d--) {
        const long i = b % t.outer_shape[d];
        b /= t.outer_shape[d];
        in_off += i * t.outer_in[d];
        out_off += i * t.outer_out[d];
    }
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const long j0 = tj * TJ, l0 = tl * TT;
    {
        const long j = j0 + tx * V;
        Pack<TS, V> x[TT / 4];  // all loads in flight before the first conversion
#pragma unroll
        for (int i = 0; i < TT / 4; i++) {
            const long l = l0 + ty + 4 * i;
            if (j < t.n_j && l < t.n_l) x[i] = *reinterpret_cast<const Pack<TS, V> *>(in + in_off + j + l * t.in_l);
        }
#pragma unroll
        for (int i = 0; i < TT / 4; i++) {
            const long l = l0 + ty + 4 * i;
            if (j < t.n_j && l < t.n_l) {
#pragma unroll
                for (int v = 0; v < V; v++) tile[ty + 4 * i][tx * V + v] = Convert<S, D>::run(x[i].v[v]);
            }
        }
    }
    __syncthreads();
    {
        constexpr int LPR = TT / V;  // lanes per destination row
        const int lx = threadIdx.x % LPR, jy = threadIdx.x / LPR;
        const long l = l0 + lx * V;
#pragma unroll 4
        for (int r = jy; r < TJ; r += 256 / LPR) {
            const long j = j0 + r;
            if (j < t.n_j && l < t.n_l) {
                Pack<TD, V> y;
#pragma unroll
                for (int v = 0; v < V; v++) y.v[v] = tile[lx * V + v][r];
                *reinterpret_cast<Pack<TD, V> *>(out + out_off + j * t.out_j + l) = y;
            }
        }
    }
}

inline unsigned grid_for(long work_items, const hodu_rocm_ctx *ctx) {
    long blocks = (work_items + 255) / 256;
    const long cap = (long)ctx->props.multiProcessorCount * 16;  // grid-stride beyond this
    if (blocks > cap) blocks = cap;
    return (unsigned)(blocks < 1 ? 1 : blocks);
}

template <int S, int D>
int run_cast(hodu_rocm_ctx *ctx, const void *in_v, void *out_v, const Strided &s) {
    typedef typename Src<S>::T TS;
    typedef typename Dst<D>::T TD;
    if (s.n == 0) return HODU_ROCM_OK;
    const TS *in = (const TS *)in_v + s.offset;
    TD *out = (TD *)out_v;
    if (s.contiguous) {
        const bool aligned = ((uintptr_t)in % (sizeof(TS) * VEC) == 0) && ((uintptr_t)out % (sizeof(TD) * VEC) == 0);
        ctx->last_kernel = aligned ? "cast_dense_vec" : "cast_dense";
        if (aligned) {
            hipLaunchKernelGGL((cast_dense_kernel<S, D>), dim3(grid_for((s.n + VEC - 1) / VEC, ctx)), dim3(256), 0,
                               ctx->stream, in, out, s.n);
        } else {
            hipLaunchKernelGGL((cast_flat_kernel<S, D>), dim3(grid_for(s.n, ctx)), dim3(256), 0, ctx->stream, in, out,
                               s.n);
        }
    } else {
        // merge neighbouring dims that nest, drop extent-1 dims
        DevStrided d{};
        int nd = 0;
        for (int i = 0; i < s.nd; i++) {
            if (s.shape[i] == 1) continue;
            if (nd > 0 && d.strides[nd - 1] == s.strides[i] * s.shape[i]) {
                d.shape[nd - 1] *= s.shape[i];
                d.strides[nd - 1] = s.strides[i];
            } else {
                d.shape[nd] = s.shape[i];
                d.strides[nd] = s.strides[i];
                nd++;
            }
        }
        d.nd = nd;
        // a transposed view: the last dim is strided and some other dim has the unit stride
        int dj = -1;
        if (nd >= 2 && d.strides[nd - 1] != 1 && d.shape[nd - 1] >= 16)
            for (int i = 0; i < nd - 1; i++)
                if (d.strides[i] == 1 && d.shape[i] >= 16) dj = i;
        if (dj >= 0) {
            DevTranspose t{};
            long out_stride = 1, outer = 1;
            for (int i = nd - 1; i >= 0; i--) {  // destination strides: row-major over the merged dims
                if (i == dj) {
                    t.out_j = out_stride;
                } else if (i != nd - 1) {
                    // collected innermost first; the kernel walks them in the same order
                    t.outer_shape[t.n_outer] = d.shape[i];
                    t.outer_in[t.n_outer] = d.strides[i];
                    t.outer_out[t.n_outer] = out_stride;
                    t.n_outer++;
                    outer *= d.shape[i];
                }
                out_stride *= d.shape[i];
            }
            // the kernel peels outer dims from index n_outer - 1 down as the fastest-varying first: reverse so that
            // the innermost outer dim varies fastest
            for (int a = 0, b = t.n_outer - 1; a < b; a++, b--) {
                std::swap(t.outer_shape[a], t.outer_shape[b]);
                std::swap(t.outer_in[a], t.outer_in[b]);
                std::swap(t.outer_out[a], t.outer_out[b]);
            }
            t.n_j = d.shape[dj];
            t.n_l = d.shape[nd - 1];
            t.in_l = d.strides[nd - 1];
            t.tiles_l = (t.n_l + TT - 1) / TT;
            // V elements per lane: 8 bytes of the wider type, if every address stays a multiple of V elements
            constexpr int V = 8 / (int)(sizeof(TS) > sizeof(TD) ? sizeof(TS) : sizeof(TD));
            bool vec = V >= 2 && t.n_j % V == 0 && t.n_l % V == 0 && t.in_l % V == 0 &&
                       (uintptr_t)in % (V * sizeof(TS)) == 0 && (uintptr_t)out % (V * sizeof(TD)) == 0;
            for (int i = 0; i < t.n_outer; i++) vec = vec && t.outer_in[i] % V == 0;
            t.tiles_j = (t.n_j + (vec ? TT * V : TT) - 1) / (vec ? TT * V : TT);
            const long blocks = outer * t.tiles_j * t.tiles_l;
            if (blocks <= 0x7FFFFFFFL) {
                if constexpr (V >= 2) {
                    if (vec) {
                        ctx->last_kernel = "cast_transpose_vec";
                        hipLaunchKernelGGL((cast_transpose_vec_kernel<S, D, V>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, in, out, t);
                        HODU_HIP(hipGetLastError());
                        return HODU_ROCM_OK;
                    }
                }
                ctx->last_kernel = "cast_transpose";
                hipLaunchKernelGGL((cast_transpose_kernel<S, D>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, in, out, t);
                HODU_HIP(hipGetLastError());
                return HODU_ROCM_OK;
            }
        }
        ctx->last_kernel = "cast_strided";
        hipLaunchKernelGGL((cast_strided_kernel<S, D>), dim3(grid_for(s.n, ctx)), dim3(256), 0, ctx->stream, in, out,
                           s.n, d);
    }
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

template <int S>
int run_cast_from(hodu_rocm_ctx *ctx, int dst, const void *in, void *out, const Strided &s) {
    switch (dst) {
#define CASE(ID) case ID: return run_cast<S, ID>(ctx, in, out, s);
        CASE(HODU_BOOL) CASE(HODU_F8E4M3) CASE(HODU_F8E5M2) CASE(HODU_BF16) CASE(HODU_F16) CASE(HODU_F32)
        CASE(HODU_F64) CASE(HODU_U8) CASE(HODU_U16) CASE(HODU_U32) CASE(HODU_U64) CASE(HODU_I8) CASE(HODU_I16)
        CASE(HODU_I32) CASE(HODU_I64)
#undef CASE
    default: return fail(HODU_ROCM_UNSUPPORTED, "cast: unknown destination dtype id %d", dst);
    }
}

}  // namespace

int launch_cast(hodu_rocm_ctx *ctx, int src, int dst, const void *in, void *out, const Strided &s) {
    switch (src) {
#define CASE(ID) case ID: return run_cast_from<ID>(ctx, dst, in, out, s);
        CASE(HODU_BOOL) CASE(HODU_F8E4M3) CASE(HODU_F8E5M2) CASE(HODU_BF16) CASE(HODU_F16) CASE(HODU_F32)
        CASE(HODU_F64) CASE(HODU_U8) CASE(HODU_U16) CASE(HODU_U32) CASE(HODU_U64) CASE(HODU_I8) CASE(HODU_I16)
        CASE(HODU_I32) CASE(HODU_I64)
#undef CASE
    default: return fail(HODU_ROCM_UNSUPPORTED, "cast: unknown source dtype id %d", src);
    }
}

// contiguous(): a same-width copy; routed through the unsigned type of the element's size
int launch_gather(hodu_rocm_ctx *ctx, int dtype, const void *in, void *out, const Strided &s) {
    switch (dtype_size(dtype)) {
    case 1: return run_cast<HODU_U8, HODU_U8>(ctx, in, out, s);
    case 2: return run_cast<HODU_U16, HODU_U16>(ctx, in, out, s);
    case 4: return run_cast<HODU_U32, HODU_U32>(ctx, in, out, s);
    case 8: return run_cast<HODU_U64, HODU_U64>(ctx, in, out, s);
    default: return fail(HODU_ROCM_UNSUPPORTED, "contiguous: unknown dtype id %d", dtype);
    }
}

}  // namespace hodu
