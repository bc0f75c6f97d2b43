// Flat C interface over the host-side Tensor mirror, for bindings (ctypes) and tests.
// Every function returns 0 on success or 1 + ErrorKind on failure; hodu_host_last_error() returns the
// calling thread's message.  Handles are owned by the caller and released with hodu_host_tensor_free.
#include "tensor.hpp"

using namespace hodu_host;

namespace {
thread_local std::string g_error;

template <class F>
int guarded(F &&f) {
    try {
        f();
        return 0;
    } catch (const Error &e) {
        g_error = e.what();
        return 1 + (int)e.kind;
    } catch (const std::exception &e) {
        g_error = e.what();
        return 1 + (int)ErrorKind::InternalError;
    }
}

Dims dims_of(const size_t *p, size_t n) { return Dims(p, p + n); }
Tensor *box(Tensor t) { return new Tensor(std::move(t)); }
DType dtype_of(int id) {
    if (id < 0 || id > 14) throw Error(ErrorKind::InvalidArgument, "unknown dtype id " + std::to_string(id));
    return (DType)id;
}
}  // namespace

extern "C" {

typedef struct hodu_host_tensor hodu_host_tensor;
#define T(p) reinterpret_cast<const Tensor *>(p)
#define H(p) reinterpret_cast<hodu_host_tensor *>(p)

const char *hodu_host_last_error(void) { return g_error.c_str(); }

int hodu_host_tensor_from_bytes(int device, int dtype, const size_t *shape, size_t nd, const void *bytes, size_t nbytes,
                                hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(Tensor::from_bytes(device, dtype_of(dtype), dims_of(shape, nd), bytes, nbytes))); });
}
void hodu_host_tensor_free(hodu_host_tensor *t) { delete reinterpret_cast<Tensor *>(t); }

int hodu_host_tensor_ndim(const hodu_host_tensor *t) { return (int)T(t)->layout().ndim(); }
int hodu_host_tensor_dtype(const hodu_host_tensor *t) { return (int)T(t)->dtype(); }
int hodu_host_tensor_physical_dtype(const hodu_host_tensor *t) { return (int)T(t)->physical_dtype(); }
int hodu_host_tensor_shares_storage(const hodu_host_tensor *a, const hodu_host_tensor *b) {
    return T(a)->shares_storage_with(*T(b)) ? 1 : 0;
}
void hodu_host_tensor_layout(const hodu_host_tensor *t, size_t *shape, size_t *strides, size_t *offset) {
    const Layout &l = T(t)->layout();
    for (size_t i = 0; i < l.ndim(); i++) {
        shape[i] = l.shape()[i];
        strides[i] = l.strides()[i];
    }
    *offset = l.offset();
}
int hodu_host_tensor_to_bytes(const hodu_host_tensor *t, void *out, size_t nbytes) {
    return guarded([&] {
        if (nbytes != T(t)->size() * dtype_size(T(t)->dtype()))
            throw Error(ErrorKind::InvalidArgument, "to_bytes: byte count does not match the tensor");
        T(t)->to_bytes(out);
    });
}

int hodu_host_matmul(const hodu_host_tensor *a, const hodu_host_tensor *b, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->matmul(*T(b)))); });
}
// steps: n_steps entries of {op, operand tensor (add) or null, scalar bits (mul_scalar)}
typedef struct hodu_host_then {
    int op;
    const hodu_host_tensor *operand;
    unsigned char scalar[8];
} hodu_host_then;
int hodu_host_matmul_then(const hodu_host_tensor *a, const hodu_host_tensor *b, const hodu_host_then *steps, size_t n_steps,
                          hodu_host_tensor **out) {
    return guarded([&] {
        std::vector<Tensor::Then> then(n_steps);
        for (size_t i = 0; i < n_steps; i++) {
            then[i].op = steps[i].op;
            then[i].operand = T(steps[i].operand);
            std::memcpy(then[i].scalar, steps[i].scalar, 8);
        }
        *out = H(box(T(a)->matmul_then(*T(b), then)));
    });
}
int hodu_host_linear(const hodu_host_tensor *input, const hodu_host_tensor *weight, const hodu_host_tensor *bias, int relu,
                     hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(Tensor::linear(*T(input), *T(weight), bias ? T(bias) : nullptr, relu != 0))); });
}
long hodu_host_stats_fused_steps(void) { return stats().fused_steps; }
long hodu_host_stats_sum_kernels(void) { return stats().sum_kernels; }
long hodu_host_stats_softmax_kernels(void) { return stats().softmax_kernels; }
long hodu_host_stats_attention_kernels(void) { return stats().attention_kernels; }
int hodu_host_softmax(const hodu_host_tensor *t, int dim, int causal, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(t)->softmax(dim, causal != 0))); });
}
int hodu_host_softmax_masked(const hodu_host_tensor *t, const hodu_host_tensor *mask, int causal, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(t)->softmax_masked(*T(mask), causal != 0))); });
}
int hodu_host_attention_masked(const hodu_host_tensor *q, const hodu_host_tensor *k, const hodu_host_tensor *v,
                               const hodu_host_tensor *mask, int is_causal, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(Tensor::scaled_dot_product_attention(*T(q), *T(k), *T(v), is_causal != 0, T(mask)))); });
}
int hodu_host_attention(const hodu_host_tensor *q, const hodu_host_tensor *k, const hodu_host_tensor *v, int is_causal,
                        hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(Tensor::scaled_dot_product_attention(*T(q), *T(k), *T(v), is_causal != 0))); });
}
// the scalar `value` in dtype's storage (round-to-nearest-even), for mul_scalar steps; returns the byte count
int hodu_host_scalar_bits(int dtype, double value, unsigned char out[8], size_t *n) {
    return guarded([&] { *n = Tensor::scalar_bits(dtype_of(dtype), value, out); });
}
int hodu_host_sum(const hodu_host_tensor *t, const int *dims, size_t n_dims, int keep_dim, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(t)->sum(std::vector<int>(dims, dims + n_dims), keep_dim != 0))); });
}
int hodu_host_sum_to_shape(const hodu_host_tensor *t, const size_t *shape, size_t nd, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(t)->sum_to_shape(dims_of(shape, nd)))); });
}
// gradients of matmul / dot with respect to both operands (vjp_matrix.rs:17-67)
int hodu_host_matmul_vjp(const hodu_host_tensor *a, const hodu_host_tensor *b, const hodu_host_tensor *grad,
                         hodu_host_tensor **da, hodu_host_tensor **db) {
    return guarded([&] {
        Tensor::Grads g = Tensor::matmul_vjp(*T(a), *T(b), *T(grad));
        *da = H(box(g.first));
        *db = H(box(g.second));
    });
}
int hodu_host_dot_vjp(const hodu_host_tensor *a, const hodu_host_tensor *b, const hodu_host_tensor *grad,
                      hodu_host_tensor **da, hodu_host_tensor **db) {
    return guarded([&] {
        Tensor::Grads g = Tensor::dot_vjp(*T(a), *T(b), *T(grad));
        *da = H(box(g.first));
        *db = H(box(g.second));
    });
}
int hodu_host_dot(const hodu_host_tensor *a, const hodu_host_tensor *b, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->dot(*T(b)))); });
}
int hodu_host_to_dtype(const hodu_host_tensor *a, int dtype, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->to_dtype(dtype_of(dtype)))); });
}
int hodu_host_contiguous(const hodu_host_tensor *a, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->contiguous())); });
}
int hodu_host_transpose(const hodu_host_tensor *a, int d1, int d2, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->transpose(d1, d2))); });
}
int hodu_host_broadcast(const hodu_host_tensor *a, const size_t *shape, size_t nd, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->broadcast(dims_of(shape, nd)))); });
}
int hodu_host_reshape(const hodu_host_tensor *a, const size_t *shape, size_t nd, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->reshape(dims_of(shape, nd)))); });
}
int hodu_host_squeeze(const hodu_host_tensor *a, const int *dims, size_t n, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->squeeze(std::vector<int>(dims, dims + n)))); });
}
int hodu_host_unsqueeze(const hodu_host_tensor *a, int dim, hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->unsqueeze(dim))); });
}
int hodu_host_slice(const hodu_host_tensor *a, int dim, int start, int has_end, int end, int step,
                    hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->slice(dim, start, has_end != 0, end, step))); });
}
/* an arbitrary (shape, strides, offset) view over the same storage */
int hodu_host_view(const hodu_host_tensor *a, const size_t *shape, const size_t *strides, size_t nd, size_t offset,
                   hodu_host_tensor **out) {
    return guarded([&] { *out = H(box(T(a)->view(Layout(dims_of(shape, nd), dims_of(strides, nd), offset)))); });
}

/* 0 = reproduce the reference's forced copies, 1 = strided views go to the kernel as they are */
void hodu_host_set_matmul_mode(int mode) { matmul_mode() = mode == 0 ? MatmulMode::Reference : MatmulMode::NoCopy; }
int hodu_host_set_reference_sums(int device, int on) {
    return guarded([&] { RocmDevice::get(device)->set_reference_sums(on != 0); });
}
void hodu_host_stats(long *cast_kernels, long *contiguous_kernels, long *product_kernels, long *fused_products,
                     long long *bytes_copied) {
    Stats &s = stats();
    *cast_kernels = s.cast_kernels;
    *contiguous_kernels = s.contiguous_kernels;
    *product_kernels = s.product_kernels;
    *fused_products = s.fused_products;
    *bytes_copied = s.bytes_copied;
}
void hodu_host_stats_reset(void) { stats().reset(); }

}  // extern "C"
