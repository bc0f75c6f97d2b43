// Encoders of the metadata arrays the kernels consume, word for word what hodu_core builds
// (crates/hodu_core/src/op_metadatas.rs).  Header-only, no GPU dependency.
#pragma once

#include <algorithm>

#include "layout.hpp"

namespace hodu_host {

using Metadata = std::vector<size_t>;

// op_metadatas.rs:192-291
//   [num_els, l_nd, r_nd, b_nd, l_shape.., r_shape.., batch_shape.., l_strides.., r_strides..,
//    l_offset, r_offset, M, K, N]
inline Metadata matmul_metadata(const Layout &lhs, const Layout &rhs, const Layout &out) {
    const size_t ln = lhs.ndim(), rn = rhs.ndim();
    if (ln < 2 || rn < 2) throw Error(ErrorKind::InvalidArgument, "matmul requires at least 2D tensors");
    const size_t m = lhs.shape()[ln - 2], kl = lhs.shape()[ln - 1], kr = rhs.shape()[rn - 2], n = rhs.shape()[rn - 1];
    if (kl != kr)
        throw Error(ErrorKind::InvalidArgument,
                    "matmul inner dimensions mismatch: " + std::to_string(kl) + " vs " + std::to_string(kr));
    const size_t lb = ln - 2, rb = rn - 2, bn = std::max(lb, rb);
    Dims batch;
    for (size_t i = 0; i < bn; i++) {
        // right-aligned batch dims; a missing leading dim counts as 1
        const size_t ld = i + lb >= bn ? lhs.shape()[i + lb - bn] : 1;
        const size_t rd = i + rb >= bn ? rhs.shape()[i + rb - bn] : 1;
        if (ld != rd && ld != 1 && rd != 1)
            throw Error(ErrorKind::InvalidArgument, "matmul batch dimension mismatch at index " + std::to_string(i) +
                                                        ": " + std::to_string(ld) + " vs " + std::to_string(rd));
        batch.push_back(std::max(ld, rd));
    }
    Metadata md{out.size(), ln, rn, bn};
    md.insert(md.end(), lhs.shape().begin(), lhs.shape().end());
    md.insert(md.end(), rhs.shape().begin(), rhs.shape().end());
    md.insert(md.end(), batch.begin(), batch.end());
    md.insert(md.end(), lhs.strides().begin(), lhs.strides().end());
    md.insert(md.end(), rhs.strides().begin(), rhs.strides().end());
    md.push_back(lhs.offset());
    md.push_back(rhs.offset());
    md.push_back(m);
    md.push_back(kl);
    md.push_back(n);
    return md;
}

// op_metadatas.rs:464-506: [M, K, N, lhs_stride_m, lhs_stride_k, rhs_stride_k, rhs_stride_n, l_offset, r_offset]
inline Metadata dot_metadata(const Layout &lhs, const Layout &rhs) {
    if (lhs.ndim() != 2 || rhs.ndim() != 2) throw Error(ErrorKind::InvalidArgument, "dot requires exactly 2D tensors");
    if (lhs.shape()[1] != rhs.shape()[0])
        throw Error(ErrorKind::InvalidArgument, "dot inner dimensions mismatch: " + std::to_string(lhs.shape()[1]) +
                                                    " vs " + std::to_string(rhs.shape()[0]));
    return {lhs.shape()[0],   lhs.shape()[1],   rhs.shape()[1], lhs.strides()[0], lhs.strides()[1],
            rhs.strides()[0], rhs.strides()[1], lhs.offset(),   rhs.offset()};
}

// op_metadatas.rs:1615-1640: [num_els, nd, shape.., strides.., offset]
inline Metadata cast_metadata(const Layout &l) {
    Metadata md{l.size(), l.ndim()};
    md.insert(md.end(), l.shape().begin(), l.shape().end());
    md.insert(md.end(), l.strides().begin(), l.strides().end());
    md.push_back(l.offset());
    return md;
}

// op_metadatas.rs:1654-1656
inline Metadata contiguous_metadata(const Layout &l) { return cast_metadata(l); }

// op_metadatas.rs:525-586: [nd, shape.., strides.., offset, out_nd, out_shape.., n_reduce, reduce_dims.., keep_dim,
// reduce_size]; reducing everything without keep_dim still encodes the output shape [1]
inline Metadata reduce_metadata(const Layout &l, const std::vector<size_t> &dims, bool keep_dim) {
    const size_t nd = l.ndim();
    Dims out;
    size_t reduce_size = 1;
    for (size_t i = 0; i < nd; i++) {
        const bool reduced = std::find(dims.begin(), dims.end(), i) != dims.end();
        if (reduced) {
            if (keep_dim) out.push_back(1);
        } else {
            out.push_back(l.shape()[i]);
        }
    }
    if (out.empty()) out.push_back(1);
    for (size_t d : dims) {
        if (d >= nd) throw Error(ErrorKind::InvalidAxis, "sum: dim " + std::to_string(d) + " of " + std::to_string(nd));
        reduce_size *= l.shape()[d];
    }
    Metadata md{nd};
    md.insert(md.end(), l.shape().begin(), l.shape().end());
    md.insert(md.end(), l.strides().begin(), l.strides().end());
    md.push_back(l.offset());
    md.push_back(out.size());
    md.insert(md.end(), out.begin(), out.end());
    md.push_back(dims.size());
    md.insert(md.end(), dims.begin(), dims.end());
    md.push_back(keep_dim ? 1 : 0);
    md.push_back(reduce_size);
    return md;
}

}  // namespace hodu_host
