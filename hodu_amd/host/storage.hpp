// Host-side mirror of hodu's backend storage for a ROCm device: what `be_rocm` would be in hodu_core.
//   RocmDevice  ~ be_cuda/device.rs:20-65   (one lazily created context per device id)
//   RocmStorage ~ be/storage.rs:13-176 (BackendStorageT), be_cpu/storage/ops_matrix.rs:24-321,
//                 be_cpu/storage.rs:697-772 (to_dtype, contiguous)
// Everything below talks to the GPU only through the C ABI of include/hodu_rocm_kernels.h.
#pragma once

#include <atomic>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>

#include "hodu_rocm_kernels.h"
#include "metadata.hpp"

namespace hodu_host {

// crates/hodu_core/src/types/dtype.rs:6-28 (repr(u8) discriminants; the C ABI uses the same ids)
enum class DType : int {
    BOOL = 0, F8E4M3 = 1, F8E5M2 = 2, BF16 = 3, F16 = 4, F32 = 5, F64 = 6, U8 = 7,
    U16 = 8, U32 = 9, U64 = 10, I8 = 11, I16 = 12, I32 = 13, I64 = 14,
};

inline size_t dtype_size(DType d) {
    static const size_t sz[15] = {1, 1, 1, 2, 2, 4, 8, 1, 2, 4, 8, 1, 2, 4, 8};
    return sz[(int)d];
}

inline const char *dtype_name(DType d) {
    static const char *nm[15] = {"bool", "f8e4m3", "f8e5m2", "bf16", "f16", "f32", "f64", "u8",
                                 "u16",  "u32",    "u64",    "i8",   "i16", "i32", "i64"};
    return nm[(int)d];
}

// Counters that let a caller (and the tests) see which device passes a Tensor-level call cost.
struct Stats {
    std::atomic<long> cast_kernels{0}, contiguous_kernels{0}, product_kernels{0}, fused_products{0};
    std::atomic<long> fused_steps{0};        // element-wise kernels that ran inside a product's store instead
    std::atomic<long> sum_kernels{0}, softmax_kernels{0}, attention_kernels{0};
    std::atomic<long long> bytes_copied{0};  // written by cast/contiguous passes
    void reset() { cast_kernels = contiguous_kernels = product_kernels = fused_products = fused_steps = sum_kernels = softmax_kernels = attention_kernels = 0; bytes_copied = 0; }
};
inline Stats &stats() {
    static Stats s;
    return s;
}

class RocmDevice {
public:
    // global registry filled on first use, like be_cuda/device.rs:20-65
    static std::shared_ptr<RocmDevice> get(int id) {
        static std::mutex mu;
        static std::map<int, std::shared_ptr<RocmDevice>> devices;
        std::lock_guard<std::mutex> lock(mu);
        auto it = devices.find(id);
        if (it != devices.end()) return it->second;
        hodu_rocm_ctx *ctx = nullptr;
        if (hodu_rocm_ctx_create(id, &ctx) != HODU_ROCM_OK)
            throw Error(ErrorKind::RocmKernelError, std::string("ctx_create: ") + hodu_rocm_last_error(nullptr));
        auto dev = std::shared_ptr<RocmDevice>(new RocmDevice(id, ctx));
        devices[id] = dev;
        return dev;
    }
    ~RocmDevice() { hodu_rocm_ctx_destroy(ctx_); }
    int id() const { return id_; }
    hodu_rocm_ctx *ctx() const { return ctx_; }
    void check(int rc, const char *what) const {
        if (rc != HODU_ROCM_OK)
            throw Error(ErrorKind::RocmKernelError, std::string(what) + ": " + hodu_rocm_last_error(ctx_));
    }
    // products of f8e4m3 / f8e5m2 / bf16 / f16 on this device in the CPU backend's arithmetic -- the running sum
    // re-rounded to the dtype after every multiply and add (crates/hodu_cpu_kernels/kernels/ops_matrix.c:196-240,
    // :351-354) -- for comparing devices byte for byte; off by default
    void set_reference_sums(bool on) const { check(hodu_rocm_ctx_set_reference_sums(ctx_, on ? 1 : 0), "set_reference_sums"); }

private:
    RocmDevice(int id, hodu_rocm_ctx *ctx) : id_(id), ctx_(ctx) {}
    int id_;
    hodu_rocm_ctx *ctx_;
};

// One device allocation, freed when the last storage that shares it goes away.
class DeviceBuf {
public:
    DeviceBuf(std::shared_ptr<RocmDevice> dev, size_t bytes) : dev_(std::move(dev)), bytes_(bytes) {
        // a zero-element tensor still owns a valid pointer
        dev_->check(hodu_rocm_alloc(dev_->ctx(), bytes ? bytes : 1, &ptr_), "alloc");
    }
    ~DeviceBuf() { hodu_rocm_free(dev_->ctx(), ptr_); }
    DeviceBuf(const DeviceBuf &) = delete;
    DeviceBuf &operator=(const DeviceBuf &) = delete;
    void *ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }

private:
    std::shared_ptr<RocmDevice> dev_;
    void *ptr_ = nullptr;
    size_t bytes_;
};

// Storage = device buffer + LOGICAL dtype (what hodu sees) + PHYSICAL dtype (what the bytes are).
// physical != dtype marks a deferred to_dtype: the cast has not run, and a following matmul/dot
// reads the narrow elements directly (fused entry points of the C ABI).  Every other consumer
// materialises first.  Deferred pairs: f8e4m3 -> bf16 and i8 -> i32.
class RocmStorage;

// An element-wise kernel the caller would launch on the product's output next, handed to the product instead
// (hodu_nn/src/modules/linear.rs:40-46: add(bias); attention.rs:37: mul_scalar; activation.rs:8-17: relu).
struct FusedStep {
    int op = 0;                         // HODU_ROCM_EPI_*
    const RocmStorage *vector = nullptr;  // ADD_ROW: storage of the operand, output dtype
    size_t stride = 0, offset = 0;      // ADD_ROW: the operand's layout along the output's last axis
    unsigned char scalar[8] = {0};      // MUL_SCALAR: the scalar in the output dtype
};
using FusedSteps = std::vector<FusedStep>;

class RocmStorage {
public:
    RocmStorage(std::shared_ptr<RocmDevice> dev, std::shared_ptr<DeviceBuf> buf, DType dtype, DType physical)
        : dev_(std::move(dev)), buf_(std::move(buf)), dtype_(dtype), physical_(physical) {}

    static RocmStorage from_host(const std::shared_ptr<RocmDevice> &dev, DType dt, const void *bytes, size_t n_elems) {
        auto buf = std::make_shared<DeviceBuf>(dev, n_elems * dtype_size(dt));
        if (n_elems) dev->check(hodu_rocm_memcpy_h2d(dev->ctx(), buf->ptr(), bytes, n_elems * dtype_size(dt)), "h2d");
        return RocmStorage(dev, buf, dt, dt);
    }

    DType dtype() const { return dtype_; }
    DType physical_dtype() const { return physical_; }
    bool deferred() const { return physical_ != dtype_; }
    const std::shared_ptr<RocmDevice> &device() const { return dev_; }
    const void *ptr() const { return buf_->ptr(); }
    size_t elems() const { return buf_->bytes() / dtype_size(physical_); }

    // BackendStorageT::to_cpu_storage: the elements of `layout`, row-major, in the LOGICAL dtype
    void to_host(const Layout &layout, void *out) const {
        check_span(layout, "to_host");
        RocmStorage dense = (deferred() || !layout.is_contiguous() || layout.offset() != 0) ? gather(layout) : *this;
        if (layout.size())
            dev_->check(hodu_rocm_memcpy_d2h(dev_->ctx(), out, dense.ptr(), layout.size() * dtype_size(dtype_)), "d2h");
    }

    // be_cpu/storage.rs:697-719.  Same dtype -> contiguous().  f8e4m3 -> bf16 and i8 -> i32 of a dense
    // layout are deferred (no kernel, buffer shared); everything else runs the cast kernel once.
    RocmStorage to_dtype(const Layout &layout, DType target, bool allow_defer = true) const {
        check_span(layout, "to_dtype");
        if (target == dtype_) return contiguous(layout);
        const bool dense = layout.is_contiguous() && layout.offset() == 0;
        const bool pair = (physical_ == DType::F8E4M3 && target == DType::BF16) ||
                          (physical_ == DType::I8 && target == DType::I32);
        if (allow_defer && !deferred() && dense && pair) return RocmStorage(dev_, buf_, target, physical_);
        if (deferred()) return gather(layout).to_dtype(Layout::from_shape(layout.shape()), target, allow_defer);
        return cast_kernel(layout, target);
    }

    // be_cpu/storage.rs:721-772: already dense with offset 0 -> share the buffer, else one gather pass
    RocmStorage contiguous(const Layout &layout) const {
        check_span(layout, "contiguous");
        if (layout.is_contiguous() && layout.offset() == 0 && !deferred()) return *this;
        return gather(layout);
    }

    // be_cpu/storage/ops_matrix.rs:24-185.  Output: fresh contiguous [batch.., M, N] in the logical dtype.
    RocmStorage call_ops_matmul(const RocmStorage &rhs, const Layout &ll, const Layout &rl,
                                const FusedSteps &fused = {}) const {
        check_pair(rhs, "matmul");
        check_span(ll, "matmul lhs");
        rhs.check_span(rl, "matmul rhs");
        Dims out_shape = matmul_out_shape(ll, rl);
        const Layout out_layout = Layout::from_shape(out_shape);
        const Metadata md = matmul_metadata(ll, rl, out_layout);
        return product(rhs, ll, rl, md, out_layout.size(), true, fused);
    }

    // be_cpu/storage/ops_matrix.rs:201-321.  Output: fresh contiguous [M, N].
    RocmStorage call_ops_dot(const RocmStorage &rhs, const Layout &ll, const Layout &rl, const FusedSteps &fused = {}) const {
        check_pair(rhs, "dot");
        check_span(ll, "dot lhs");
        rhs.check_span(rl, "dot rhs");
        const Metadata md = dot_metadata(ll, rl);
        return product(rhs, ll, rl, md, md[0] * md[2], false, fused);
    }

    // be_cpu/storage/ops_reduce.rs (call_ops_reduce, ReduceOp::Sum): output fresh and contiguous in the reduced shape
    RocmStorage call_ops_reduce_sum(const Layout &layout, const std::vector<size_t> &dims, bool keep_dim) const {
        check_span(layout, "sum");
        if (dtype_ == DType::BOOL) throw Error(ErrorKind::UnsupportedDTypeForOp, "sum: bool is not supported");
        if (deferred()) return gather(layout).call_ops_reduce_sum(Layout::from_shape(layout.shape()), dims, keep_dim);
        const Metadata md = reduce_metadata(layout, dims, keep_dim);
        size_t n_out = 1;
        const size_t nd = md[0], out_nd = md[2 + 2 * nd];
        for (size_t i = 0; i < out_nd; i++) n_out *= md[3 + 2 * nd + i];
        RocmStorage out = fresh(dtype_, n_out);
        if (n_out == 0) return out;
        dev_->check(hodu_rocm_sum(dev_->ctx(), (int)dtype_, ptr(), (void *)out.ptr(), md.data(), md.size()), "sum");
        stats().sum_kernels++;
        return out;
    }

    // Tensor::softmax (tensor/ops/normalization.rs:4-21) as one launch; output fresh and contiguous in the input's shape
    RocmStorage call_ops_softmax(const Layout &layout, size_t dim, bool causal) const {
        check_span(layout, "softmax");
        if (deferred()) return gather(layout).call_ops_softmax(Layout::from_shape(layout.shape()), dim, causal);
        const Metadata md = reduce_metadata(layout, {dim}, true);
        RocmStorage out = fresh(dtype_, layout.size());
        if (layout.size() == 0) return out;
        dev_->check(hodu_rocm_softmax(dev_->ctx(), (int)dtype_, ptr(), (void *)out.ptr(), md.data(), md.size(), causal ? 1 : 0),
                    "softmax");
        stats().softmax_kernels++;
        return out;
    }

    // softmax(-1) with attention's attn_mask folded in (crates/hodu_nn/src/modules/attention.rs:50-56): the mask's
    // storage is read through `mask_layout` -- already broadcast to the scores' shape, stride 0 where it repeats -- and
    // is never expanded.  One byte per element (bool / u8 / i8), 0 = masked out.
    RocmStorage call_ops_softmax_masked(const Layout &layout, bool causal, const RocmStorage &mask, const Layout &mask_layout) const {
        check_span(layout, "softmax");
        mask.check_span(mask_layout, "softmax mask");
        if (deferred()) return gather(layout).call_ops_softmax_masked(Layout::from_shape(layout.shape()), causal, mask, mask_layout);
        if (mask.deferred() || dtype_size(mask.dtype()) != 1)
            throw Error(ErrorKind::UnsupportedDTypeForOp, "softmax: the mask is a bool / u8 / i8 tensor (cast it with to_dtype first)");
        if (dev_->id() != mask.dev_->id()) throw Error(ErrorKind::DeviceMismatch, "softmax: the mask lives on another device");
        if (layout.ndim() == 0 || mask_layout.shape() != layout.shape())
            throw Error(ErrorKind::InvalidArgument, "softmax: the mask layout is not broadcast to the input's shape");
        const Metadata md = reduce_metadata(layout, {layout.ndim() - 1}, true);
        Metadata ml{layout.ndim()};
        ml.insert(ml.end(), mask_layout.strides().begin(), mask_layout.strides().end());
        ml.push_back(mask_layout.offset());
        RocmStorage out = fresh(dtype_, layout.size());
        if (layout.size() == 0) return out;
        dev_->check(hodu_rocm_softmax_masked(dev_->ctx(), (int)dtype_, ptr(), (void *)out.ptr(), md.data(), md.size(), causal ? 1 : 0,
                                             mask.ptr(), (int)mask.dtype(), ml.data(), ml.size()),
                    "softmax (masked)");
        stats().softmax_kernels++;
        return out;
    }

    // the whole of scaled_dot_product_attention as one launch, where the fused kernel takes the call (bf16 / f16,
    // head dim 64 or 128, dense aligned rows): *taken says whether it did.  md: hodu_rocm_attention's metadata.
    // mask, mask_layout: the attn_mask (attention.rs:50-56) read in place, its layout already broadcast to the scores'
    // shape [batch.., Sq, Sk] (stride 0 where it repeats); one byte per element, 0 = masked out.
    RocmStorage call_ops_attention(const RocmStorage &k, const RocmStorage &v, const Layout &ql, const Layout &kl, const Layout &vl,
                                   const Metadata &md, size_t out_elems, const unsigned char scale[8], bool causal,
                                   bool *taken, const RocmStorage *mask = nullptr, const Layout *mask_layout = nullptr) const {
        check_span(ql, "attention q");
        k.check_span(kl, "attention k");
        v.check_span(vl, "attention v");
        *taken = false;
        RocmStorage out = fresh(dtype_, out_elems);
        if (deferred() || k.deferred() || v.deferred() || k.dtype_ != dtype_ || v.dtype_ != dtype_ ||
            k.dev_->id() != dev_->id() || v.dev_->id() != dev_->id() || out_elems == 0)
            return out;
        int rc;
        if (mask) {
            mask->check_span(*mask_layout, "attention mask");
            if (mask->deferred() || dtype_size(mask->dtype()) != 1 || mask->dev_->id() != dev_->id()) return out;
            Metadata ml{mask_layout->ndim()};
            ml.insert(ml.end(), mask_layout->strides().begin(), mask_layout->strides().end());
            ml.push_back(mask_layout->offset());
            rc = hodu_rocm_attention_masked(dev_->ctx(), (int)dtype_, ptr(), k.ptr(), v.ptr(), (void *)out.ptr(), md.data(), md.size(),
                                            scale, causal ? 1 : 0, mask->ptr(), (int)mask->dtype(), ml.data(), ml.size());
        } else
            rc = hodu_rocm_attention(dev_->ctx(), (int)dtype_, ptr(), k.ptr(), v.ptr(), (void *)out.ptr(), md.data(),
                                     md.size(), scale, causal ? 1 : 0);
        if (rc == HODU_ROCM_UNSUPPORTED) return out;
        dev_->check(rc, "attention");
        stats().attention_kernels++;
        *taken = true;
        return out;
    }

    // be_cpu/storage/ops_matrix.rs:63-100: right-aligned broadcast of the batch dims, then [M, N]
    static Dims matmul_out_shape(const Layout &ll, const Layout &rl) {
        const size_t ln = ll.ndim(), rn = rl.ndim();
        if (ln < 2 || rn < 2) throw Error(ErrorKind::InvalidArgument, "matmul requires at least 2D tensors");
        const size_t lb = ln - 2, rb = rn - 2, bn = std::max(lb, rb);
        Dims out;
        for (size_t i = 0; i < bn; i++) {
            const size_t ld = i + lb >= bn ? ll.shape()[i + lb - bn] : 1;
            const size_t rd = i + rb >= bn ? rl.shape()[i + rb - bn] : 1;
            out.push_back(std::max(ld, rd));
        }
        out.push_back(ll.shape()[ln - 2]);
        out.push_back(rl.shape()[rn - 1]);
        return out;
    }

private:
    void check_span(const Layout &l, const char *what) const {
        if (l.span() > elems())
            throw Error(ErrorKind::InvalidLayout, std::string(what) + ": layout reaches element " +
                                                      std::to_string(l.span()) + " of a storage holding " +
                                                      std::to_string(elems()));
    }

    // validate_same_device / validate_same_dtype / validate_dtype_for_op (utils/valid.rs:50-76, :260-264)
    void check_pair(const RocmStorage &rhs, const char *op) const {
        if (dev_->id() != rhs.dev_->id())
            throw Error(ErrorKind::DeviceMismatch, std::string(op) + ": operands live on different devices");
        if (dtype_ != rhs.dtype_)
            throw Error(ErrorKind::DTypeMismatch, std::string(op) + ": " + dtype_name(dtype_) + " vs " + dtype_name(rhs.dtype_));
        if (dtype_ == DType::BOOL)
            throw Error(ErrorKind::UnsupportedDTypeForOp, std::string(op) + ": bool is not supported");
    }

    RocmStorage fresh(DType dt, size_t n) const {
        return RocmStorage(dev_, std::make_shared<DeviceBuf>(dev_, n * dtype_size(dt)), dt, dt);
    }

    // one pass: strided gather, fused with the pending cast when the storage is deferred
    RocmStorage gather(const Layout &layout) const {
        if (deferred()) return RocmStorage(dev_, buf_, physical_, physical_).cast_kernel(layout, dtype_);
        RocmStorage out = fresh(dtype_, layout.size());
        if (layout.size() == 0) return out;
        const Metadata md = contiguous_metadata(layout);
        dev_->check(hodu_rocm_contiguous(dev_->ctx(), (int)dtype_, ptr(), (void *)out.ptr(), md.data(), md.size()),
                    "contiguous");
        stats().contiguous_kernels++;
        stats().bytes_copied += (long long)(layout.size() * dtype_size(dtype_));
        return out;
    }

    RocmStorage cast_kernel(const Layout &layout, DType target) const {
        RocmStorage out = fresh(target, layout.size());
        if (layout.size() == 0) return out;
        const Metadata md = cast_metadata(layout);
        dev_->check(hodu_rocm_cast(dev_->ctx(), (int)physical_, (int)target, ptr(), (void *)out.ptr(), md.data(), md.size()),
                    "cast");
        stats().cast_kernels++;
        stats().bytes_copied += (long long)(layout.size() * dtype_size(target));
        return out;
    }

    using ProductFn = int (*)(hodu_rocm_ctx *, const void *, const void *, void *, const size_t *, size_t);

    static ProductFn plain_entry(DType dt, bool matmul) {
#define HODU_HOST_ENTRY(DT, name) \
    case DType::DT: return matmul ? hodu_rocm_matmul_##name : hodu_rocm_dot_##name;
        switch (dt) {
            HODU_HOST_ENTRY(F8E4M3, f8e4m3) HODU_HOST_ENTRY(F8E5M2, f8e5m2) HODU_HOST_ENTRY(BF16, bf16)
            HODU_HOST_ENTRY(F16, f16) HODU_HOST_ENTRY(F32, f32) HODU_HOST_ENTRY(F64, f64) HODU_HOST_ENTRY(U8, u8)
            HODU_HOST_ENTRY(U16, u16) HODU_HOST_ENTRY(U32, u32) HODU_HOST_ENTRY(U64, u64) HODU_HOST_ENTRY(I8, i8)
            HODU_HOST_ENTRY(I16, i16) HODU_HOST_ENTRY(I32, i32) HODU_HOST_ENTRY(I64, i64)
            default: throw Error(ErrorKind::UnsupportedDTypeForOp, "no product kernel for this dtype");
        }
#undef HODU_HOST_ENTRY
    }

    using ProductFnEx = int (*)(hodu_rocm_ctx *, const void *, const void *, void *, const size_t *, size_t,
                                const hodu_rocm_epilogue_step *, size_t);

    static ProductFnEx fused_entry(DType dt, bool matmul) {
#define HODU_HOST_ENTRY(DT, name) \
    case DType::DT: return matmul ? hodu_rocm_matmul_##name##_ex : hodu_rocm_dot_##name##_ex;
        switch (dt) {
            HODU_HOST_ENTRY(BF16, bf16) HODU_HOST_ENTRY(F16, f16) HODU_HOST_ENTRY(F32, f32) HODU_HOST_ENTRY(F64, f64)
            HODU_HOST_ENTRY(U8, u8) HODU_HOST_ENTRY(U16, u16) HODU_HOST_ENTRY(U32, u32) HODU_HOST_ENTRY(U64, u64)
            HODU_HOST_ENTRY(I8, i8) HODU_HOST_ENTRY(I16, i16) HODU_HOST_ENTRY(I32, i32) HODU_HOST_ENTRY(I64, i64)
            default: throw Error(ErrorKind::UnsupportedDTypeForOp, "products of this dtype take no fused steps");
        }
#undef HODU_HOST_ENTRY
    }

    RocmStorage product(const RocmStorage &rhs, const Layout &ll, const Layout &rl, const Metadata &md, size_t out_elems,
                        bool matmul, const FusedSteps &fused) const {
        RocmStorage out = fresh(dtype_, out_elems);
        if (out_elems == 0) return out;
        if (!fused.empty()) return product_fused(rhs, md, matmul, fused, out);
        ProductFn fn = nullptr;
        const RocmStorage *l = this, *r = &rhs;
        RocmStorage lm = *this, rm = rhs;  // materialised copies, used only when a deferred operand cannot be fused
        Metadata md_used = md;
        if (!deferred() && dtype_ == DType::BF16 && rhs.deferred() && rhs.physical_ == DType::F8E4M3) {
            fn = matmul ? hodu_rocm_matmul_bf16_f8e4m3w : hodu_rocm_dot_bf16_f8e4m3w;
        } else if (deferred() && rhs.deferred() && physical_ == DType::I8 && rhs.physical_ == DType::I8) {
            fn = matmul ? hodu_rocm_matmul_i32_i8i8 : hodu_rocm_dot_i32_i8i8;
        } else {
            // the views stay as they are: a materialised operand keeps its layout because the cast
            // writes the whole underlying buffer densely in storage order
            if (deferred()) { lm = RocmStorage(dev_, buf_, physical_, physical_).cast_kernel(Layout::from_shape({elems()}), dtype_); l = &lm; }
            if (rhs.deferred()) { rm = RocmStorage(rhs.dev_, rhs.buf_, rhs.physical_, rhs.physical_).cast_kernel(Layout::from_shape({rhs.elems()}), rhs.dtype_); r = &rm; }
            fn = plain_entry(dtype_, matmul);
        }
        (void)ll;
        (void)rl;
        dev_->check(fn(dev_->ctx(), l->ptr(), r->ptr(), (void *)out.ptr(), md_used.data(), md_used.size()),
                    matmul ? "matmul" : "dot");
        stats().product_kernels++;
        if (fn == hodu_rocm_matmul_bf16_f8e4m3w || fn == hodu_rocm_dot_bf16_f8e4m3w || fn == hodu_rocm_matmul_i32_i8i8 ||
            fn == hodu_rocm_dot_i32_i8i8)
            stats().fused_products++;
        return out;
    }

    // the product with the caller's next element-wise kernels applied in its store; deferred casts fuse as well
    RocmStorage product_fused(const RocmStorage &rhs, const Metadata &md, bool matmul, const FusedSteps &fused,
                              RocmStorage out) const {
        std::vector<hodu_rocm_epilogue_step> steps(fused.size());
        std::vector<RocmStorage> keep;  // operands whose pending cast had to be run first
        keep.reserve(fused.size());
        for (size_t i = 0; i < fused.size(); i++) {
            steps[i] = hodu_rocm_epilogue_step{};
            steps[i].op = fused[i].op;
            if (fused[i].op == HODU_ROCM_EPI_ADD_ROW) {
                const RocmStorage *v = fused[i].vector;
                if (!v) throw Error(ErrorKind::InvalidArgument, "fused add: no operand");
                if (v->dev_->id() != dev_->id()) throw Error(ErrorKind::DeviceMismatch, "fused add: operand on another device");
                if (v->dtype_ != dtype_)
                    throw Error(ErrorKind::DTypeMismatch, std::string("fused add: ") + dtype_name(dtype_) + " vs " + dtype_name(v->dtype_));
                if (v->deferred()) {
                    keep.push_back(RocmStorage(v->dev_, v->buf_, v->physical_, v->physical_).cast_kernel(Layout::from_shape({v->elems()}), v->dtype_));
                    v = &keep.back();
                }
                steps[i].vector = v->ptr();
                steps[i].stride = fused[i].stride;
                steps[i].offset = fused[i].offset;
            }
            std::memcpy(steps[i].scalar, fused[i].scalar, 8);
        }
        ProductFnEx fn = nullptr;
        const RocmStorage *l = this, *r = &rhs;
        RocmStorage lm = *this, rm = rhs;
        bool fused_cast = true;
        if (!deferred() && dtype_ == DType::BF16 && rhs.deferred() && rhs.physical_ == DType::F8E4M3) {
            fn = matmul ? hodu_rocm_matmul_bf16_f8e4m3w_ex : hodu_rocm_dot_bf16_f8e4m3w_ex;
        } else if (deferred() && rhs.deferred() && physical_ == DType::I8 && rhs.physical_ == DType::I8) {
            fn = matmul ? hodu_rocm_matmul_i32_i8i8_ex : hodu_rocm_dot_i32_i8i8_ex;
        } else {
            fused_cast = false;
            if (deferred()) { lm = RocmStorage(dev_, buf_, physical_, physical_).cast_kernel(Layout::from_shape({elems()}), dtype_); l = &lm; }
            if (rhs.deferred()) { rm = RocmStorage(rhs.dev_, rhs.buf_, rhs.physical_, rhs.physical_).cast_kernel(Layout::from_shape({rhs.elems()}), rhs.dtype_); r = &rm; }
            fn = fused_entry(dtype_, matmul);
        }
        dev_->check(fn(dev_->ctx(), l->ptr(), r->ptr(), (void *)out.ptr(), md.data(), md.size(), steps.data(), steps.size()),
                    matmul ? "matmul" : "dot");
        stats().product_kernels++;
        stats().fused_steps += (long)fused.size();
        if (fused_cast) stats().fused_products++;
        return out;
    }

    std::shared_ptr<RocmDevice> dev_;
    std::shared_ptr<DeviceBuf> buf_;
    DType dtype_, physical_;
};

}  // namespace hodu_host
