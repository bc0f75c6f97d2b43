// CPU-only checks of the host mirror's Layout algebra and metadata encoders.  The expected vectors are
// the literals the reference's own kernel tests build by hand
// (crates/hodu_cpu_kernels/tests/ops_matrix.rs:8-147, crates/hodu_cuda_kernels/tests/ops_matrix.rs:188-262,
//  crates/hodu_cuda_kernels/tests/ops_cast.rs:48-89); everything else follows from the definition of a
// strided view and is checked by brute-force index enumeration.
#include <cstdio>
#include <functional>

#include "metadata.hpp"

using namespace hodu_host;

static int g_failed = 0;
#define CHECK(cond)                                                       \
    do {                                                                  \
        if (!(cond)) {                                                    \
            std::printf("FAIL %s:%d  %s\n", __FILE__, __LINE__, #cond);   \
            g_failed++;                                                   \
        }                                                                 \
    } while (0)

static bool throws(ErrorKind kind, const std::function<void()> &f) {
    try {
        f();
    } catch (const Error &e) {
        return e.kind == kind;
    }
    return false;
}

// storage indices a layout visits, in row-major order of its shape
static std::vector<size_t> visit(const Layout &l) {
    std::vector<size_t> out;
    Dims idx(l.ndim(), 0);
    const size_t n = l.size();
    for (size_t e = 0; e < n; e++) {
        size_t pos = l.offset();
        for (size_t d = 0; d < l.ndim(); d++) pos += idx[d] * l.strides()[d];
        out.push_back(pos);
        for (size_t d = l.ndim(); d-- > 0;) {
            if (++idx[d] < l.shape()[d]) break;
            idx[d] = 0;
        }
    }
    return out;
}

int main() {
    // ---- metadata literals of the reference tests ------------------------------------------------
    {  // test_matmul_f32_2d: [2,3] x [3,2]
        Layout l = Layout::from_shape({2, 3}), r = Layout::from_shape({3, 2}), o = Layout::from_shape({2, 2});
        CHECK((matmul_metadata(l, r, o) == Metadata{4, 2, 2, 0, 2, 3, 3, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2}));
        CHECK((dot_metadata(l, r) == Metadata{2, 3, 2, 3, 1, 2, 1, 0, 0}));  // test_dot_f32_simple
    }
    {  // test_matmul_f32_batch: [2,2,2] x [2,2,2]
        Layout l = Layout::from_shape({2, 2, 2}), o = Layout::from_shape({2, 2, 2});
        CHECK((matmul_metadata(l, l, o) == Metadata{8, 3, 3, 1, 2, 2, 2, 2, 2, 2, 2, 4, 2, 1, 4, 2, 1, 0, 0, 2, 2, 2}));
    }
    {  // matmul_f32_batch (shared weight): lhs [2,2,3], rhs [3,2] without a batch dim
        Layout l = Layout::from_shape({2, 2, 3}), r = Layout::from_shape({3, 2}), o = Layout::from_shape({2, 2, 2});
        CHECK((matmul_metadata(l, r, o) == Metadata{8, 3, 2, 1, 2, 2, 3, 3, 2, 2, 6, 3, 1, 2, 1, 0, 0, 2, 3, 2}));
    }
    {  // cast tests: [n, 1, n, 1, 0]
        CHECK((cast_metadata(Layout::from_shape({4})) == Metadata{4, 1, 4, 1, 0}));
        CHECK((contiguous_metadata(Layout::from_shape({2, 3}).transpose(0, 1)) == Metadata{6, 2, 3, 2, 1, 3, 0}));
    }
    CHECK(throws(ErrorKind::InvalidArgument, [] { matmul_metadata(Layout::from_shape({3}), Layout::from_shape({3, 2}), Layout::from_shape({2})); }));
    CHECK(throws(ErrorKind::InvalidArgument, [] { matmul_metadata(Layout::from_shape({2, 3}), Layout::from_shape({4, 2}), Layout::from_shape({2, 2})); }));
    CHECK(throws(ErrorKind::InvalidArgument, [] { matmul_metadata(Layout::from_shape({2, 2, 3}), Layout::from_shape({3, 3, 2}), Layout::from_shape({3, 2, 2})); }));
    CHECK(throws(ErrorKind::InvalidArgument, [] { dot_metadata(Layout::from_shape({2, 2, 3}), Layout::from_shape({3, 2})); }));
    CHECK(throws(ErrorKind::InvalidArgument, [] { dot_metadata(Layout::from_shape({2, 3}), Layout::from_shape({2, 2})); }));
    {  // batch broadcast in the encoder: lhs [4,1,2,3] x rhs [5,3,2] -> batch [4,5]
        Layout l = Layout::from_shape({4, 1, 2, 3}), r = Layout::from_shape({5, 3, 2}), o = Layout::from_shape({4, 5, 2, 2});
        Metadata md = matmul_metadata(l, r, o);
        CHECK(md[3] == 2 && md[4 + 4 + 3] == 4 && md[4 + 4 + 3 + 1] == 5);
        CHECK(md.size() == 4 + 4 + 3 + 2 + 4 + 3 + 5);
    }

    // ---- Layout algebra ------------------------------------------------------------------------------
    Layout a = Layout::from_shape({2, 3, 4});
    CHECK((a.strides() == Dims{12, 4, 1}) && a.offset() == 0 && a.is_contiguous() && a.size() == 24 && a.span() == 24);
    CHECK(Layout::from_shape({}).is_contiguous() && Layout::from_shape({}).size() == 1);

    Layout t = a.transpose(-2, -1);
    CHECK((t.shape() == Dims{2, 4, 3}) && (t.strides() == Dims{12, 1, 4}) && !t.is_contiguous());
    CHECK(t.transpose(1, 2) == a);
    {  // a transposed view visits the transposed positions
        std::vector<size_t> v = visit(Layout::from_shape({2, 3}).transpose(0, 1));
        CHECK((v == std::vector<size_t>{0, 3, 1, 4, 2, 5}));
    }
    CHECK(throws(ErrorKind::InternalError, [&] { Layout::from_shape({3}).transpose(0, 1); }));
    CHECK(throws(ErrorKind::InternalError, [&] { a.transpose(0, 3); }));

    Layout b = Layout::from_shape({3, 4}).broadcast_to({5, 3, 4});
    CHECK((b.strides() == Dims{0, 4, 1}) && b.size() == 60 && b.span() == 12);
    CHECK((Layout::from_shape({3, 1}).broadcast_to({2, 3, 4}).strides() == Dims{0, 1, 0}));
    CHECK(throws(ErrorKind::IncompatibleShapes, [&] { a.broadcast_to({3, 4}); }));
    CHECK(throws(ErrorKind::IncompatibleShapes, [&] { Layout::from_shape({3, 4}).broadcast_to({5, 4, 4}); }));
    {  // broadcasting a transposed layout keeps its strides (what the no-copy matmul relies on)
        Layout w = Layout::from_shape({4, 6}).transpose(0, 1).broadcast_to({8, 6, 4});
        CHECK((w.strides() == Dims{0, 1, 6}));
        std::vector<size_t> v = visit(w);
        CHECK(v[0] == 0 && v[1] == 6 && v[4] == 1 && v[24] == 0);
    }

    // is_contiguous: exact strides, the offset does not matter, size-1 dims are not forgiven
    CHECK(Layout({2, 3}, {3, 1}, 7).is_contiguous());
    CHECK(!Layout({1, 3}, {5, 1}, 0).is_contiguous());
    CHECK(!Layout({2, 3}, {4, 1}, 0).is_contiguous());

    // reshape / squeeze / unsqueeze need a contiguous layout and keep the offset
    CHECK(a.reshape({6, 4}) == Layout({6, 4}, {4, 1}, 0));
    CHECK(Layout({2, 3}, {3, 1}, 5).reshape({6}).offset() == 5);
    CHECK(throws(ErrorKind::IncompatibleShapes, [&] { a.reshape({5, 5}); }));
    CHECK(throws(ErrorKind::InvalidLayout, [&] { t.reshape({24}); }));
    CHECK((Layout::from_shape({1, 3, 1}).squeeze({}).shape() == Dims{3}));
    CHECK((Layout::from_shape({1, 3, 1}).squeeze({-1}).shape() == Dims{1, 3}));
    CHECK((Layout::from_shape({1, 3, 1}).squeeze({0}).shape() == Dims{3, 1}));
    CHECK(throws(ErrorKind::InvalidLayout, [&] { Layout::from_shape({1, 3}).squeeze({1}); }));
    CHECK(throws(ErrorKind::InvalidAxis, [&] { Layout::from_shape({1, 3}).squeeze({2}); }));
    CHECK(throws(ErrorKind::InvalidLayout, [&] { t.squeeze({}); }));
    CHECK((Layout::from_shape({3}).unsqueeze(0).shape() == Dims{1, 3}));
    CHECK((Layout::from_shape({3}).unsqueeze(-1).shape() == Dims{3, 1}));
    CHECK(throws(ErrorKind::InvalidAxis, [&] { Layout::from_shape({3}).unsqueeze(2); }));

    // slice: offset + stride * step, clamped bounds, negative indices
    {
        Layout s = Layout::from_shape({10, 4}).slice(0, 2, true, 9, 3);
        CHECK((s.shape() == Dims{3, 4}) && (s.strides() == Dims{12, 1}) && s.offset() == 8);
        CHECK((visit(s)[4] == 8 + 12));
        Layout c = Layout::from_shape({10, 4}).slice(-1, 1, false, 0, 1);
        CHECK((c.shape() == Dims{10, 3}) && c.offset() == 1 && !c.is_contiguous());
        Layout neg = Layout::from_shape({10}).slice(0, -4, true, -1, 1);
        CHECK((neg.shape() == Dims{3}) && neg.offset() == 6);
        Layout clamp = Layout::from_shape({10}).slice(0, 5, true, 100, 2);
        CHECK((clamp.shape() == Dims{3}) && clamp.offset() == 5 && (clamp.strides() == Dims{2}));
        CHECK(throws(ErrorKind::InternalError, [&] { Layout::from_shape({10}).slice(0, 5, true, 5, 1); }));
        CHECK(throws(ErrorKind::InternalError, [&] { Layout::from_shape({10}).slice(0, 0, false, 0, 0); }));
        CHECK(throws(ErrorKind::InvalidAxis, [&] { Layout::from_shape({10}).slice(1, 0, false, 0, 1); }));
        // a negative step keeps the start offset and an unsigned stride of |step| (strides are never negative)
        Layout back = Layout::from_shape({10}).slice(0, 8, true, 2, -2);
        CHECK((back.shape() == Dims{3}) && back.offset() == 8 && (back.strides() == Dims{2}));
    }

    // permute
    CHECK((a.permute({2, 0, 1}).shape() == Dims{4, 2, 3}) && (a.permute({2, 0, 1}).strides() == Dims{1, 12, 4}));
    CHECK(throws(ErrorKind::InternalError, [&] { a.permute({0, 0, 1}); }));
    CHECK(throws(ErrorKind::InternalError, [&] { a.permute({0, 1}); }));

    // span: the last reachable storage element + 1
    CHECK(Layout({2, 3}, {0, 2}, 4).span() == 4 + 2 * 2 + 1);
    CHECK(Layout({0, 3}, {3, 1}, 0).span() == 0);

    if (g_failed) {
        std::printf("%d check(s) failed\n", g_failed);
        return 1;
    }
    std::printf("host layout/metadata checks passed\n");
    return 0;
}
