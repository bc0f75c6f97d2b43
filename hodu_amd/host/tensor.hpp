// Host-side mirror of the hodu Tensor methods on the matmul / dot / to_dtype path
// (crates/hodu_core/src/tensor/ops/matrix.rs, cast_memory.rs, shape.rs).  A Tensor is an immutable
// (storage, layout) pair; views share the storage (tensor/internal.rs:50-79).
#pragma once

#include <cmath>

#include "storage.hpp"

namespace hodu_host {

// How matmul_batched treats a non-contiguous operand:
//   Reference  exactly hodu today: Tensor::broadcast / transpose / reshape / squeeze first force
//              contiguity (shape.rs:232-237, :296-299), so a transposed weight is copied per call
//   NoCopy     the patched path: the broadcast layout is built straight on the existing layout
//              (Layout::broadcast_to) and the strided view goes to the kernel as is
enum class MatmulMode { Reference = 0, NoCopy = 1 };

inline MatmulMode &matmul_mode() {
    static MatmulMode mode = MatmulMode::NoCopy;
    return mode;
}

class Tensor {
public:
    Tensor(std::shared_ptr<const RocmStorage> storage, Layout layout)
        : storage_(std::move(storage)), layout_(std::move(layout)) {}

    // Tensor::from_bytes-like constructor: row-major elements of `dtype`, given as raw bits
    static Tensor from_bytes(int device, DType dtype, const Dims &shape, const void *bytes, size_t nbytes) {
        const size_t n = product(shape);
        if (nbytes != n * dtype_size(dtype))
            throw Error(ErrorKind::InvalidArgument, "from_bytes: byte count does not match the shape");
        auto dev = RocmDevice::get(device);
        return Tensor(std::make_shared<RocmStorage>(RocmStorage::from_host(dev, dtype, bytes, n)), Layout::from_shape(shape));
    }

    const Layout &layout() const { return layout_; }
    const Dims &shape() const { return layout_.shape(); }
    DType dtype() const { return storage_->dtype(); }
    DType physical_dtype() const { return storage_->physical_dtype(); }
    bool is_contiguous() const { return layout_.is_contiguous(); }  // tensor/core.rs:222-224
    size_t size() const { return layout_.size(); }
    bool shares_storage_with(const Tensor &o) const { return storage_->ptr() == o.storage_->ptr(); }

    void to_bytes(void *out) const { storage_->to_host(layout_, out); }

    // cast_memory.rs:11-38: result is contiguous in the tensor's shape
    Tensor to_dtype(DType target) const {
        return Tensor(std::make_shared<RocmStorage>(storage_->to_dtype(layout_, target)), Layout::from_shape(shape()));
    }

    // cast_memory.rs:56-83: an already contiguous tensor is returned as is (offset included)
    Tensor contiguous() const {
        if (is_contiguous()) return *this;
        return Tensor(std::make_shared<RocmStorage>(storage_->contiguous(layout_)), Layout::from_shape(shape()));
    }

    // shape.rs:13-60, :125-170, :232-279, :295-346: each forces contiguity first, then is a pure view
    Tensor reshape(const Dims &s) const { return is_contiguous() ? view(layout_.reshape(s)) : contiguous().reshape(s); }
    Tensor squeeze(const std::vector<int> &d) const { return is_contiguous() ? view(layout_.squeeze(d)) : contiguous().squeeze(d); }
    Tensor unsqueeze(int d) const { return is_contiguous() ? view(layout_.unsqueeze(d)) : contiguous().unsqueeze(d); }
    Tensor broadcast(const Dims &s) const { return is_contiguous() ? view(layout_.broadcast_to(s)) : contiguous().broadcast(s); }
    Tensor transpose(int a, int b) const { return is_contiguous() ? view(layout_.transpose(a, b)) : contiguous().transpose(a, b); }
    Tensor t() const { return transpose(-2, -1); }
    Tensor slice(int dim, int start, bool has_end, int end, int step) const {
        return view(layout_.slice(dim, start, has_end, end, step));
    }
    // a view with an arbitrary layout over the same storage (bounds are checked when it is used)
    Tensor view(const Layout &l) const { return Tensor(storage_, l); }

    // matrix.rs:13-92
    Tensor matmul(const Tensor &other) const {
        const size_t ln = layout_.ndim(), rn = other.layout_.ndim();
        if (ln < 1 || rn < 1) throw incompatible(other, "matmul");
        if (ln == 1 && rn == 1) return inner(other, "matmul");
        if (ln == 2 && rn == 1) {
            if (shape()[1] != other.shape()[0]) throw incompatible(other, "matmul");
            return dot_2d(other.reshape({other.shape()[0], 1})).squeeze({-1});
        }
        if (ln == 1 && rn == 2) {
            if (shape()[0] != other.shape()[0]) throw incompatible(other, "matmul");
            return reshape({1, shape()[0]}).dot_2d(other).squeeze({0});
        }
        if (ln == 2 && rn == 2) return dot_2d(other);
        return matmul_batched(other);
    }

    // matrix.rs:226-299: 1-D and 2-D only
    Tensor dot(const Tensor &other) const {
        const size_t ln = layout_.ndim(), rn = other.layout_.ndim();
        if (ln == 1 && rn == 1) return inner(other, "dot");
        if (ln == 2 && rn == 1) {
            if (shape()[1] != other.shape()[0]) throw incompatible(other, "dot");
            return dot_2d(other.reshape({other.shape()[0], 1})).squeeze({-1});
        }
        if (ln == 1 && rn == 2) {
            if (shape()[0] != other.shape()[0]) throw incompatible(other, "dot");
            return reshape({1, shape()[0]}).dot_2d(other).squeeze({0});
        }
        if (ln == 2 && rn == 2) return dot_2d(other);
        throw Error(ErrorKind::InternalError, "dot - only supports 1D and 2D tensors. Use matmul() for batched operations");
    }

    // ---- the product with its caller's next element-wise kernels fused in --------------------------------
    // What follows the product in hodu_nn: Linear::forward adds the bias (linear.rs:40-46), attention scales
    // the scores (attention.rs:37), ReLU follows a Linear (activation.rs:8-17).  Each Then is one such kernel,
    // applied in order inside the product's store; the result equals matmul(..) followed by Tensor::add /
    // mul_scalar / relu bit for bit.  Both operands must have at least two dimensions.
    struct Then {
        int op = 0;                    // HODU_ROCM_EPI_*
        const Tensor *operand = nullptr;  // add: a tensor that broadcasts to the output along its last axis only
        unsigned char scalar[8] = {0};    // mul_scalar: the scalar's bits in the output dtype (Scalar::to_dtype)
        static Then add(const Tensor &bias) { Then t; t.op = HODU_ROCM_EPI_ADD_ROW; t.operand = &bias; return t; }
        static Then mul_scalar(const void *bits, size_t n) {
            Then t; t.op = HODU_ROCM_EPI_MUL_SCALAR;
            std::memcpy(t.scalar, bits, n < 8 ? n : 8);
            return t;
        }
        static Then relu() { Then t; t.op = HODU_ROCM_EPI_RELU; return t; }
    };

    Tensor matmul_then(const Tensor &other, const std::vector<Then> &then) const {
        const size_t ln = layout_.ndim(), rn = other.layout_.ndim();
        if (ln < 2 || rn < 2)
            throw Error(ErrorKind::InvalidArgument, "matmul with fused steps needs operands of at least two dimensions");
        if (ln == 2 && rn == 2) return dot_2d(other, &then);
        return matmul_batched(other, &then);
    }

    // Linear::forward (hodu_nn/src/modules/linear.rs:40-46): input @ weight.T (+ bias); weight is [out, in]
    static Tensor linear(const Tensor &input, const Tensor &weight, const Tensor *bias, bool relu = false) {
        std::vector<Then> then;
        if (bias) then.push_back(Then::add(*bias));
        if (relu) then.push_back(Then::relu());
        const Tensor wt = weight.transpose(-2, -1);
        if (then.empty() || input.layout().ndim() < 2) {
            if (!then.empty()) throw Error(ErrorKind::InvalidArgument, "linear: a 1-D input takes no fused steps");
            return input.matmul(wt);
        }
        return input.matmul_then(wt, then);
    }

    // ---- backward through the path ------------------------------------------------------------------------
    // tensor/ops/reduce.rs:11-13, :135-175: negative dims count from the end; no dims = all of them
    Tensor sum(const std::vector<int> &dims, bool keep_dim) const {
        const size_t nd = layout_.ndim();
        std::vector<size_t> red;
        if (dims.empty()) for (size_t i = 0; i < nd; i++) red.push_back(i);
        for (int d : dims) red.push_back(layout_.axis(d));
        Dims out_shape;
        for (size_t i = 0; i < nd; i++) {
            const bool reduced = std::find(red.begin(), red.end(), i) != red.end();
            if (!reduced) out_shape.push_back(shape()[i]);
            else if (keep_dim) out_shape.push_back(1);
        }
        auto out = std::make_shared<RocmStorage>(storage_->call_ops_reduce_sum(layout_, red, keep_dim));
        return Tensor(out, Layout::from_shape(out_shape));
    }

    // tensor/ops/reduce.rs:19-50: leading extra dims first (innermost of them first), then every dim the target
    // holds at extent 1, one launch each
    Tensor sum_to_shape(const Dims &target) const {
        if (shape() == target) return *this;
        Tensor result = *this;
        if (shape().size() > target.size())
            for (size_t d = shape().size() - target.size(); d-- > 0;) result = result.sum({(int)d}, false);
        for (size_t i = 0; i < target.size() && i < result.shape().size(); i++)
            if (target[i] == 1 && result.shape()[i] > 1) result = result.sum({(int)i}, true);
        return result;
    }

    using Grads = std::pair<Tensor, Tensor>;  // (dA, dB)

    // tensor/gradient/vjp_matrix.rs:17-45: dA = grad @ B^T, dB = A^T @ grad, each summed down to its operand's
    // shape where matmul had broadcast it.  With a weight that has no batch dims (the Linear case) and dense a and
    // grad, NoCopy mode folds the batch into the contraction instead: dB = [B*M, K]^T @ [B*M, N] is one product
    // whose f32 accumulator runs over the batch as well -- no [B, K, N] intermediate, no sum launches, and one
    // rounding instead of B + 1.
    static Grads matmul_vjp(const Tensor &a, const Tensor &b, const Tensor &grad) {
        const Tensor da = grad.matmul(b.transpose(-2, -1)).sum_to_shape(a.shape());
        const size_t an = a.layout().ndim();
        if (matmul_mode() == MatmulMode::NoCopy && b.layout().ndim() == 2 && an > 2 && a.is_contiguous() && grad.is_contiguous()) {
            size_t rows = 1;
            for (size_t i = 0; i + 1 < an; i++) rows *= a.shape()[i];
            const Tensor a2 = a.view(Layout({rows, a.shape()[an - 1]}, {a.shape()[an - 1], 1}, a.layout().offset()));
            const Tensor g2 = grad.view(Layout({rows, grad.shape().back()}, {grad.shape().back(), 1}, grad.layout().offset()));
            return {da, a2.view(a2.layout().transpose(0, 1)).dot(g2)};
        }
        const Tensor db = a.transpose(-2, -1).matmul(grad).sum_to_shape(b.shape());
        return {da, db};
    }

    // tensor/gradient/vjp_matrix.rs:46-67
    static Grads dot_vjp(const Tensor &a, const Tensor &b, const Tensor &grad) {
        return {grad.dot(b.transpose(-2, -1)), a.transpose(-2, -1).dot(grad)};
    }

    // ---- attention's middle step and the function around it ---------------------------------------------------
    // tensor/ops/normalization.rs:4-21, one launch instead of five.
    // causal: the masked_fill(-inf) of attention.rs:40-48 folded in (last dim only).
    Tensor softmax(int dim, bool causal = false) const {
        const size_t d = layout_.axis(dim);
        if (causal && d + 1 != layout_.ndim())
            throw Error(ErrorKind::InvalidArgument, "softmax: the causal mask applies to the last dim");
        auto out = std::make_shared<RocmStorage>(storage_->call_ops_softmax(layout_, d, causal));
        return Tensor(out, Layout::from_shape(shape()));
    }

    // softmax(-1) of masked_fill(mask.eq_scalar(0), get_neg_inf(dtype)) (attention.rs:50-56, :88-96) as one launch: the
    // mask broadcasts against the scores the way masked_fill's where3 broadcasts it (right-aligned, extent 1 repeats)
    Tensor softmax_masked(const Tensor &mask_any, bool causal = false) const {
        if (layout_.ndim() == 0) throw Error(ErrorKind::InvalidArgument, "softmax: a scalar has no last dim");
        const Tensor mask = mask_any.as_mask_bytes();
        const Layout ml = mask.layout().broadcast_to(shape());
        auto out = std::make_shared<RocmStorage>(storage_->call_ops_softmax_masked(layout_, causal, *mask.storage_, ml));
        return Tensor(out, Layout::from_shape(shape()));
    }
    // `mask.eq_scalar(0)` (attention.rs:52) takes a mask of any dtype; the kernels read one byte per element, 0 = masked
    // out.  bool / u8 / i8 are that already; anything else goes through to_dtype(BOOL), whose x != 0 is the same predicate
    // (-0.0 masks, a NaN attends).
    Tensor as_mask_bytes() const {
        const DType d = dtype();
        const bool bytes = (d == DType::BOOL || d == DType::U8 || d == DType::I8) && !storage_->deferred();
        return bytes ? *this : to_dtype(DType::BOOL);
    }

    // `value` as a scalar of dtype `dt`, round-to-nearest-even (what Scalar::to_dtype does through the `half` crate's
    // from_f32 for bf16 / f16: scalar.rs:391-404); only the floating dtypes
    static size_t scalar_bits(DType dt, double value, unsigned char out[8]) {
        std::memset(out, 0, 8);
        const float f = (float)value;
        uint32_t u;
        std::memcpy(&u, &f, 4);
        switch (dt) {
        case DType::F64: std::memcpy(out, &value, 8); return 8;
        case DType::F32: std::memcpy(out, &f, 4); return 4;
        case DType::BF16: {
            const uint16_t h = (u & 0x7F800000u) == 0x7F800000u ? (uint16_t)(u >> 16) : (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
            std::memcpy(out, &h, 2);
            return 2;
        }
        case DType::F16: {
            const uint32_t sign = (u >> 16) & 0x8000u, absu = u & 0x7FFFFFFFu;
            uint16_t h;
            if (absu >= 0x7F800000u) h = (uint16_t)(sign | 0x7C00u | (absu > 0x7F800000u ? 0x200u : 0u));
            else if (absu >= 0x477FF000u) h = (uint16_t)(sign | 0x7C00u);  // rounds to infinity
            else if (absu < 0x33000001u) h = (uint16_t)sign;                // below half the smallest subnormal
            else {
                int e = (int)(absu >> 23) - 127;
                uint32_t m = (absu & 0x7FFFFFu) | 0x800000u;
                int shift = e < -14 ? 13 + (-14 - e) : 13;                   // subnormal results lose more bits
                uint32_t r = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
                if (rem > half || (rem == half && (r & 1u))) r++;
                h = e < -14 ? (uint16_t)(sign | r) : (uint16_t)(sign | (((uint32_t)(e + 15) << 10) + (r - 0x400u)));
            }
            std::memcpy(out, &h, 2);
            return 2;
        }
        default: throw Error(ErrorKind::UnsupportedDTypeForOp, "attention: floating dtypes only");
        }
    }

    // scaled_dot_product_attention (hodu_nn/src/modules/attention.rs:25-70) without dropout:
    // softmax(Q K^T / sqrt(d_k) [+ causal mask] [+ attn_mask]) V.  One launch where the fused kernel applies (bf16 / f16,
    // head dim 64 or 128, dense aligned rows); otherwise three -- the scale rides in the first product's store, the masks
    // and the five softmax kernels are one kernel, the second product is plain.
    static Tensor scaled_dot_product_attention(const Tensor &q, const Tensor &k, const Tensor &v, bool is_causal,
                                               const Tensor *attn_mask = nullptr) {
        if (q.layout().ndim() < 2) throw Error(ErrorKind::InvalidArgument, "attention: query needs at least two dimensions");
        const double scale = 1.0 / std::sqrt((double)q.shape().back());
        unsigned char bits[8];
        const size_t n = scalar_bits(q.dtype(), scale, bits);
        const Tensor mask_bytes = attn_mask ? attn_mask->as_mask_bytes() : q;  // (q: a placeholder nobody reads)
        // one kernel where it applies: q [.., Sq, D], k and v [.., Sk, D] with the batch dims broadcast the way the
        // two matmuls would broadcast them; an attn_mask (1 = attend, 0 = mask out; attention.rs:50-56) is read in
        // place, broadcast against the scores the way masked_fill's where3 broadcasts it
        const size_t qn = q.layout().ndim(), kn = k.layout().ndim(), vn = v.layout().ndim();
        if (kn >= 2 && vn >= 2 && q.shape()[qn - 1] == k.shape()[kn - 1] && k.shape()[kn - 2] == v.shape()[vn - 2] &&
            v.shape()[vn - 1] == q.shape()[qn - 1]) {
            const size_t bn = std::max({qn, kn, vn}) - 2;
            Dims batch(bn, 1);
            bool ok = true;
            for (const Tensor *t : {&q, &k, &v}) {
                const size_t tb = t->layout().ndim() - 2;
                for (size_t i = 0; i < tb; i++) {
                    const size_t ext = t->shape()[tb - 1 - i];
                    size_t &slot = batch[bn - 1 - i];
                    if (slot == 1) slot = ext;
                    else if (ext != 1 && ext != slot) ok = false;
                }
            }
            if (ok) {
                auto spread = [&](const Tensor &t, size_t rows) {
                    Dims s = batch;
                    s.push_back(rows);
                    s.push_back(q.shape()[qn - 1]);
                    return t.layout().broadcast_to(s);
                };
                const Layout ql = spread(q, q.shape()[qn - 2]), kl = spread(k, k.shape()[kn - 2]), vl = spread(v, v.shape()[vn - 2]);
                Metadata md{bn};
                md.insert(md.end(), batch.begin(), batch.end());
                md.push_back(q.shape()[qn - 2]);
                md.push_back(k.shape()[kn - 2]);
                md.push_back(q.shape()[qn - 1]);
                for (const Layout *l : {&ql, &kl, &vl}) md.insert(md.end(), l->strides().begin(), l->strides().end());
                md.push_back(ql.offset());
                md.push_back(kl.offset());
                md.push_back(vl.offset());
                Dims out_shape = batch;
                out_shape.push_back(q.shape()[qn - 2]);
                out_shape.push_back(q.shape()[qn - 1]);
                bool taken = false, mask_fits = true;
                Layout ml;
                if (attn_mask) {
                    Dims scores_shape = batch;
                    scores_shape.push_back(q.shape()[qn - 2]);
                    scores_shape.push_back(k.shape()[kn - 2]);
                    try {
                        ml = mask_bytes.layout().broadcast_to(scores_shape);
                    } catch (const Error &) {
                        mask_fits = false;  // the three launches below report it
                    }
                }
                if (mask_fits) {
                    auto out = std::make_shared<RocmStorage>(q.storage_->call_ops_attention(
                        *k.storage_, *v.storage_, ql, kl, vl, md, product(out_shape), bits, is_causal, &taken,
                        attn_mask ? mask_bytes.storage_.get() : nullptr, attn_mask ? &ml : nullptr));
                    if (taken) return Tensor(out, Layout::from_shape(out_shape));
                }
            }
        }
        // three launches: the scale rides in the first product's store, the masks and the softmax are one kernel
        const Tensor scores = q.matmul_then(k.transpose(-2, -1), {Then::mul_scalar(bits, n)});
        if (attn_mask) return scores.softmax_masked(mask_bytes, is_causal).matmul(v);
        return scores.softmax(-1, is_causal).matmul(v);
    }

private:
    // tensor/utils.rs broadcast_tensors2 as Tensor::add applies it to (output, operand): the operand's shape is
    // right-aligned against the output's; a fused add needs every axis but the last to be broadcast (extent 1
    // or missing), so that the operand is a vector along the output's last axis
    FusedSteps lower(const std::vector<Then> &then, const Dims &out_shape) const {
        FusedSteps steps;
        for (const Then &t : then) {
            FusedStep f;
            f.op = t.op;
            std::memcpy(f.scalar, t.scalar, 8);
            if (t.op == HODU_ROCM_EPI_ADD_ROW) {
                if (!t.operand) throw Error(ErrorKind::InvalidArgument, "fused add: no operand");
                const Layout &bl = t.operand->layout();
                const size_t bn = bl.ndim(), on = out_shape.size();
                if (bn > on) throw Error(ErrorKind::IncompatibleShapes, "fused add: " + dims_str(out_shape) + " vs " + dims_str(bl.shape()));
                for (size_t i = 0; i < bn; i++) {
                    const size_t ext = bl.shape()[bn - 1 - i], want = out_shape[on - 1 - i];
                    if (i == 0 ? (ext != want && ext != 1) : ext != 1)
                        throw Error(ErrorKind::IncompatibleShapes,
                                    "fused add: the operand must be a vector along the last axis: " + dims_str(out_shape) + " vs " + dims_str(bl.shape()));
                }
                if (bl.span() > t.operand->storage_->elems())
                    throw Error(ErrorKind::InvalidLayout, "fused add: operand layout reaches past its storage");
                f.vector = t.operand->storage_.get();
                f.stride = bn == 0 || bl.shape()[bn - 1] == 1 ? 0 : bl.strides()[bn - 1];
                f.offset = bl.offset();
            }
            steps.push_back(f);
        }
        return steps;
    }

    Error incompatible(const Tensor &o, const char *op) const {
        return Error(ErrorKind::IncompatibleShapes, std::string(op) + ": " + dims_str(shape()) + " vs " + dims_str(o.shape()));
    }

    // matrix.rs:38-47 computes mul + sum_all for two vectors.  Element-wise ops are not part of this
    // backend; the same number is produced as the [1,K] x [K,1] product (for floating point the
    // summation order may differ from the reference's reduce kernel).  Result shape: scalar [].
    Tensor inner(const Tensor &other, const char *op) const {
        if (shape()[0] != other.shape()[0]) throw incompatible(other, op);
        const size_t k = shape()[0];
        return reshape({1, k}).dot_2d(other.reshape({k, 1})).reshape({});
    }

    // matrix.rs:302-371: both layouts go to the kernel unchanged
    Tensor dot_2d(const Tensor &other, const std::vector<Then> *then = nullptr) const {
        if (shape()[1] != other.shape()[0]) throw incompatible(other, "dot");
        const FusedSteps fused = then ? lower(*then, {shape()[0], other.shape()[1]}) : FusedSteps{};
        auto out = std::make_shared<RocmStorage>(storage_->call_ops_dot(*other.storage_, layout_, other.layout_, fused));
        return Tensor(out, Layout::from_shape({shape()[0], other.shape()[1]}));
    }

    // matrix.rs:95-224
    Tensor matmul_batched(const Tensor &other, const std::vector<Then> *then = nullptr) const {
        const Dims &ld = shape(), &rd = other.shape();
        const size_t ln = ld.size(), rn = rd.size();
        if (ln < 2 || rn < 2 || ld[ln - 1] != rd[rn - 2]) throw incompatible(other, "matmul");
        const size_t lb = ln - 2, rb = rn - 2, bn = std::max(lb, rb);
        Dims batch(bn);
        for (size_t i = 0; i < bn; i++) {  // i counts from the innermost batch dim
            const size_t a = i < lb ? ld[lb - 1 - i] : 1, b = i < rb ? rd[rb - 1 - i] : 1;
            if (a != 1 && b != 1 && a != b) throw incompatible(other, "matmul");
            batch[bn - 1 - i] = std::max(a, b);
        }
        Dims ls = batch, rs = batch;
        ls.push_back(ld[ln - 2]); ls.push_back(ld[ln - 1]);
        rs.push_back(rd[rn - 2]); rs.push_back(rd[rn - 1]);
        const bool copy = matmul_mode() == MatmulMode::Reference;
        const Tensor l = copy ? broadcast(ls) : view(layout_.broadcast_to(ls));
        const Tensor r = copy ? other.broadcast(rs) : other.view(other.layout_.broadcast_to(rs));
        Dims out_shape = batch;
        out_shape.push_back(ld[ln - 2]);
        out_shape.push_back(rd[rn - 1]);
        const FusedSteps fused = then ? lower(*then, out_shape) : FusedSteps{};
        auto out = std::make_shared<RocmStorage>(l.storage_->call_ops_matmul(*r.storage_, l.layout_, r.layout_, fused));
        return Tensor(out, Layout::from_shape(out_shape));
    }

    std::shared_ptr<const RocmStorage> storage_;
    Layout layout_;
};

}  // namespace hodu_host
