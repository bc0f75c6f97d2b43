// Host-side mirror of hodu's Layout (crates/hodu_core/src/types/layout.rs:15-19): a shape, strides in
// ELEMENTS and an element offset into a flat storage.  View operations never touch data; they return a
// new Layout over the same storage.  Header-only and free of any GPU dependency.
#pragma once

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace hodu_host {

// Error kinds follow the HoduError variants the reference raises on this path
// (crates/hodu_core/src/error.rs): callers and tests match on the kind, not on the text.
enum class ErrorKind {
    IncompatibleShapes,
    InvalidLayout,
    InvalidArgument,
    InvalidAxis,
    DTypeMismatch,
    UnsupportedDTypeForOp,
    DeviceMismatch,
    InternalError,
    RocmKernelError,
};

struct Error : std::runtime_error {
    ErrorKind kind;
    Error(ErrorKind k, const std::string &what) : std::runtime_error(what), kind(k) {}
};

using Dims = std::vector<size_t>;

inline size_t product(const Dims &d) {
    size_t n = 1;
    for (size_t v : d) n *= v;
    return n;
}

inline std::string dims_str(const Dims &d) {
    std::string s = "[";
    for (size_t i = 0; i < d.size(); i++) s += (i ? ", " : "") + std::to_string(d[i]);
    return s + "]";
}

class Layout {
public:
    Layout() = default;
    Layout(Dims shape, Dims strides, size_t offset = 0)
        : shape_(std::move(shape)), strides_(std::move(strides)), offset_(offset) {
        if (shape_.size() != strides_.size())
            throw Error(ErrorKind::InvalidArgument, "Layout: shape and strides differ in rank");
    }

    // layout.rs:33-40: row-major strides, offset 0
    static Layout from_shape(const Dims &shape) { return Layout(shape, compute_strides(shape), 0); }

    // layout.rs:123-134
    static Dims compute_strides(const Dims &shape) {
        Dims s(shape.size(), 1);
        for (size_t i = shape.size(); i-- > 1;) s[i - 1] = s[i] * shape[i];
        return s;
    }

    const Dims &shape() const { return shape_; }
    const Dims &strides() const { return strides_; }
    size_t offset() const { return offset_; }
    size_t ndim() const { return shape_.size(); }
    size_t size() const { return product(shape_); }
    size_t buffer_size() const { return offset_ + size(); }  // layout.rs:86-88

    // layout.rs:105-120: exact row-major strides; the offset is NOT part of the test and a size-1
    // dim with a foreign stride is NOT forgiven (the C kernels' own is_contiguous is more lenient)
    bool is_contiguous() const {
        size_t expected = 1;
        for (size_t i = ndim(); i-- > 0;) {
            if (strides_[i] != expected) return false;
            expected *= shape_[i];
        }
        return true;
    }

    // number of storage elements the view can reach, counted from element 0 of the storage
    size_t span() const {
        if (size() == 0) return 0;
        size_t last = offset_;
        for (size_t i = 0; i < ndim(); i++) last += (shape_[i] - 1) * strides_[i];
        return last + 1;
    }

    // layout.rs:137-165: only a contiguous layout reshapes; the offset is kept
    Layout reshape(const Dims &new_shape) const {
        if (size() != product(new_shape))
            throw Error(ErrorKind::IncompatibleShapes, "reshape " + dims_str(shape_) + " -> " + dims_str(new_shape));
        if (!is_contiguous())
            throw Error(ErrorKind::InvalidLayout,
                        "Cannot reshape a non-contiguous tensor. Use .contiguous() before .reshape()");
        return Layout(new_shape, compute_strides(new_shape), offset_);
    }

    // layout.rs:190-247: empty `dims` drops every size-1 dim; a named dim must have size 1
    Layout squeeze(const std::vector<int> &dims) const {
        if (!is_contiguous())
            throw Error(ErrorKind::InvalidLayout,
                        "Cannot squeeze a non-contiguous tensor. Use .contiguous() before .squeeze()");
        Dims out;
        if (dims.empty()) {
            for (size_t v : shape_)
                if (v != 1) out.push_back(v);
        } else {
            std::vector<bool> drop(ndim(), false);
            for (int d : dims) {
                const size_t a = d < 0 ? (size_t)((int)ndim() + d) : (size_t)d;
                if (a >= ndim()) throw Error(ErrorKind::InvalidAxis, "squeeze: axis " + std::to_string(d));
                if (shape_[a] != 1)
                    throw Error(ErrorKind::InvalidLayout, "Cannot squeeze dimension " + std::to_string(d) +
                                                              " with size " + std::to_string(shape_[a]));
                drop[a] = true;
            }
            for (size_t i = 0; i < ndim(); i++)
                if (!drop[i]) out.push_back(shape_[i]);
        }
        return Layout(out, compute_strides(out), offset_);
    }

    // layout.rs:250-288: insert a size-1 dim; a negative position counts from one past the end
    Layout unsqueeze(int dim) const {
        const size_t a = dim < 0 ? (size_t)((int)ndim() + dim + 1) : (size_t)dim;
        if (a > ndim()) throw Error(ErrorKind::InvalidAxis, "unsqueeze: axis " + std::to_string(dim));
        if (!is_contiguous())
            throw Error(ErrorKind::InvalidLayout,
                        "Cannot unsqueeze a non-contiguous tensor. Use .contiguous() before .unsqueeze()");
        Dims out = shape_;
        out.insert(out.begin() + (long)a, 1);
        return Layout(out, compute_strides(out), offset_);
    }

    // layout.rs:291-337: right-aligned; a new leading dim or a size-1 dim gets stride 0
    Layout broadcast_to(const Dims &target) const {
        if (ndim() > target.size())
            throw Error(ErrorKind::IncompatibleShapes, "broadcast " + dims_str(shape_) + " -> " + dims_str(target));
        const size_t diff = target.size() - ndim();
        Dims st(target.size(), 0);
        for (size_t i = 0; i < target.size(); i++) {
            const size_t src = i < diff ? 1 : shape_[i - diff];
            if (src == target[i]) {
                st[i] = i < diff ? 0 : strides_[i - diff];
            } else if (src == 1) {
                st[i] = 0;
            } else {
                throw Error(ErrorKind::IncompatibleShapes,
                            "broadcast " + dims_str(shape_) + " -> " + dims_str(target));
            }
        }
        return Layout(target, st, offset_);
    }

    // layout.rs:352-380
    Layout transpose(int d1, int d2) const {
        if (ndim() < 2) throw Error(ErrorKind::InternalError, "transpose requires at least 2 dimensions");
        const size_t a = axis(d1), b = axis(d2);
        Layout out = *this;
        std::swap(out.shape_[a], out.shape_[b]);
        std::swap(out.strides_[a], out.strides_[b]);
        return out;
    }

    // layout.rs:383-429
    Layout permute(const std::vector<int> &axes) const {
        if (axes.size() != ndim()) throw Error(ErrorKind::InternalError, "permute: axes length differs from rank");
        std::vector<bool> seen(ndim(), false);
        Dims sh, st;
        for (int ax : axes) {
            const size_t a = axis(ax);
            if (seen[a]) throw Error(ErrorKind::InternalError, "permute: axis appears more than once");
            seen[a] = true;
            sh.push_back(shape_[a]);
            st.push_back(strides_[a]);
        }
        return Layout(sh, st, offset_);
    }

    // layout.rs:432-511.  `has_end` false means "to the end in the direction of step".  Strides stay
    // unsigned: a negative step keeps the start offset and multiplies the stride by |step|, exactly as
    // the reference does (it does not walk backwards).
    Layout slice(int dim, int start, bool has_end, int end, int step) const {
        const size_t a = dim < 0 ? (size_t)((int)ndim() + dim) : (size_t)dim;
        if (a >= ndim()) throw Error(ErrorKind::InvalidAxis, "slice: axis " + std::to_string(dim));
        if (step == 0) throw Error(ErrorKind::InternalError, "slice step cannot be zero");
        const int n = (int)shape_[a];
        const int s = start < 0 ? n + start : start;
        const int e = has_end ? (end < 0 ? n + end : end) : (step > 0 ? n : -1);
        const int cs = std::clamp(s, 0, n);
        const int ce = step > 0 ? std::clamp(e, 0, n) : std::clamp(e, -1, n - 1);
        int len = 0;
        if (step > 0 && ce > cs) len = (ce - cs + step - 1) / step;
        if (step < 0 && cs > ce) len = (cs - ce + (-step) - 1) / (-step);
        if (len <= 0) throw Error(ErrorKind::InternalError, "slice results in empty tensor");
        Layout out = *this;
        out.shape_[a] = (size_t)len;
        out.strides_[a] = strides_[a] * (size_t)(step < 0 ? -step : step);
        out.offset_ = offset_ + (size_t)cs * strides_[a];
        return out;
    }

    bool operator==(const Layout &o) const {
        return shape_ == o.shape_ && strides_ == o.strides_ && offset_ == o.offset_;
    }

    // negative axes count from the end
    size_t axis(int d) const {
        const int n = (int)ndim();
        const int a = d < 0 ? n + d : d;
        if (a < 0 || a >= n) throw Error(ErrorKind::InternalError, "invalid axis: " + std::to_string(d));
        return (size_t)a;
    }

private:

    Dims shape_, strides_;
    size_t offset_ = 0;
};

}  // namespace hodu_host
