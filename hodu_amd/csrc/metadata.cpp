// Host-side parsing and validation of the reference's metadata vectors.  Nothing here touches the
// device: only the derived scalars travel to a kernel, as kernel arguments.
//
// Formats: crates/hodu_core/src/op_metadatas.rs:192-291 (matmul), :464-506 (dot),
// :1615-1656 (cast / contiguous); consumers crates/hodu_cpu_kernels/kernels/ops_matrix.c:76-93,
// :429-437 and ops_cast.c:55-63.
#include "common.hpp"

namespace hodu {

namespace {
constexpr size_t kMaxExtent = (size_t)1 << 40;  // sanity bound on any extent / stride / offset

bool sane(size_t v) { return v <= kMaxExtent; }
}  // namespace

int parse_dot_metadata(const size_t *md, size_t len, Product *p) {
    if (!md) return fail(HODU_ROCM_INVALID_ARG, "dot: metadata is null");
    if (len != 9) return fail(HODU_ROCM_INVALID_ARG, "dot: metadata has %zu words, expected 9", len);
    for (size_t i = 0; i < 9; i++)
        if (!sane(md[i])) return fail(HODU_ROCM_INVALID_ARG, "dot: metadata[%zu] out of range", i);
    *p = Product();
    p->M = (long)md[0]; p->K = (long)md[1]; p->N = (long)md[2];
    p->a_m = (long)md[3]; p->a_k = (long)md[4]; p->b_k = (long)md[5]; p->b_n = (long)md[6];
    p->a_off = (long)md[7]; p->b_off = (long)md[8];
    p->nb = 0; p->batches = 1;
    return HODU_ROCM_OK;
}

int parse_matmul_metadata(const size_t *md, size_t len, Product *p) {
    if (!md) return fail(HODU_ROCM_INVALID_ARG, "matmul: metadata is null");
    if (len < 4) return fail(HODU_ROCM_INVALID_ARG, "matmul: metadata has %zu words (< 4)", len);
    const size_t num_els = md[0], l_nd = md[1], r_nd = md[2], b_nd = md[3];
    if (l_nd < 2 || r_nd < 2)
        return fail(HODU_ROCM_INVALID_ARG, "matmul requires at least 2D tensors (got %zu-D, %zu-D)", l_nd, r_nd);
    if (l_nd > 18 || r_nd > 18 || b_nd > (size_t)kMaxBatchDims)
        return fail(HODU_ROCM_UNSUPPORTED, "matmul: more than %d batch dims", kMaxBatchDims);
    const size_t want = 4 + 2 * l_nd + 2 * r_nd + b_nd + 5;
    if (len != want)
        return fail(HODU_ROCM_INVALID_ARG, "matmul: metadata has %zu words, layout implies %zu", len, want);
    for (size_t i = 0; i < len; i++)
        if (!sane(md[i])) return fail(HODU_ROCM_INVALID_ARG, "matmul: metadata[%zu] out of range", i);
    const size_t *l_shape = md + 4, *r_shape = l_shape + l_nd, *b_shape = r_shape + r_nd;
    const size_t *l_str = b_shape + b_nd, *r_str = l_str + l_nd, *tail = r_str + r_nd;
    const size_t l_bnd = l_nd - 2, r_bnd = r_nd - 2;
    if (l_bnd > b_nd || r_bnd > b_nd)
        return fail(HODU_ROCM_INVALID_ARG, "matmul: operand has more batch dims than the output");

    *p = Product();
    p->a_off = (long)tail[0]; p->b_off = (long)tail[1];
    p->M = (long)tail[2]; p->K = (long)tail[3]; p->N = (long)tail[4];
    if (l_shape[l_nd - 2] != tail[2] || l_shape[l_nd - 1] != tail[3] || r_shape[r_nd - 2] != tail[3] ||
        r_shape[r_nd - 1] != tail[4])
        return fail(HODU_ROCM_INVALID_ARG,
                    "matmul inner dimensions mismatch: lhs [..,%zu,%zu] rhs [..,%zu,%zu] vs M,K,N = %zu,%zu,%zu",
                    l_shape[l_nd - 2], l_shape[l_nd - 1], r_shape[r_nd - 2], r_shape[r_nd - 1], tail[2], tail[3],
                    tail[4]);
    p->a_m = (long)l_str[l_nd - 2]; p->a_k = (long)l_str[l_nd - 1];
    p->b_k = (long)r_str[r_nd - 2]; p->b_n = (long)r_str[r_nd - 1];

    // batch dims: an operand dim of extent 1 (or a missing leading dim) stays at index 0
    long shape[kMaxBatchDims], as[kMaxBatchDims], bs[kMaxBatchDims];
    size_t total = 1;
    for (size_t d = 0; d < b_nd; d++) {
        const size_t ext = b_shape[d];
        long sa = 0, sb = 0;
        if (d + l_bnd >= b_nd) {
            const size_t li = d - (b_nd - l_bnd);
            if (l_shape[li] != 1) {
                if (l_shape[li] != ext)
                    return fail(HODU_ROCM_INVALID_ARG, "matmul batch dimension mismatch at index %zu: %zu vs %zu", d,
                                l_shape[li], ext);
                sa = (long)l_str[li];
            }
        }
        if (d + r_bnd >= b_nd) {
            const size_t ri = d - (b_nd - r_bnd);
            if (r_shape[ri] != 1) {
                if (r_shape[ri] != ext)
                    return fail(HODU_ROCM_INVALID_ARG, "matmul batch dimension mismatch at index %zu: %zu vs %zu", d,
                                r_shape[ri], ext);
                sb = (long)r_str[ri];
            }
        }
        shape[d] = (long)ext; as[d] = sa; bs[d] = sb;
        total *= ext;
    }
    if (num_els != total * tail[2] * tail[4])
        return fail(HODU_ROCM_INVALID_ARG, "matmul: num_els %zu != batch %zu * M %zu * N %zu", num_els, total, tail[2],
                    tail[4]);
    p->batches = (long)total;

    // drop extent-1 dims, then merge neighbours whose strides nest for both operands
    int nb = 0;
    for (size_t d = 0; d < b_nd; d++) {
        if (shape[d] == 1) continue;
        if (nb > 0 && p->a_bs[nb - 1] == as[d] * shape[d] && p->b_bs[nb - 1] == bs[d] * shape[d]) {
            p->bshape[nb - 1] *= shape[d];
            p->a_bs[nb - 1] = as[d];
            p->b_bs[nb - 1] = bs[d];
        } else {
            p->bshape[nb] = shape[d]; p->a_bs[nb] = as[d]; p->b_bs[nb] = bs[d];
            nb++;
        }
    }
    p->nb = nb;

    // a shared right operand turns the batch into extra rows of one product:
    // [B, M, K] x [K, N] == [B*M, K] x [K, N] when the lhs batch stride continues its row stride
    if (p->nb == 1 && p->b_bs[0] == 0) {
        if (p->M == 1) p->a_m = p->a_bs[0];
        if (p->a_bs[0] == p->M * p->a_m) {
            p->M *= p->bshape[0];
            p->nb = 0;
            p->batches = 1;
        }
    }
    return HODU_ROCM_OK;
}

int parse_cast_metadata(const size_t *md, size_t len, Strided *s) {
    if (!md) return fail(HODU_ROCM_INVALID_ARG, "cast: metadata is null");
    if (len < 2) return fail(HODU_ROCM_INVALID_ARG, "cast: metadata has %zu words (< 2)", len);
    const size_t n = md[0], nd = md[1];
    if (nd > 16) return fail(HODU_ROCM_UNSUPPORTED, "cast: %zu dims (> 16)", nd);
    // a 0-d tensor carries no offset word in the reference's reader (ops_cast.c:63) but the
    // encoder always appends one (op_metadatas.rs:1637); accept both
    if (len != 2 + 2 * nd + 1 && !(nd == 0 && len == 2))
        return fail(HODU_ROCM_INVALID_ARG, "cast: metadata has %zu words, layout implies %zu", len, 2 + 2 * nd + 1);
    for (size_t i = 0; i < len; i++)
        if (!sane(md[i])) return fail(HODU_ROCM_INVALID_ARG, "cast: metadata[%zu] out of range", i);
    size_t total = 1;
    for (size_t d = 0; d < nd; d++) total *= md[2 + d];
    if (total != n) return fail(HODU_ROCM_INVALID_ARG, "cast: num_els %zu != product of shape %zu", n, total);
    s->n = (long)n; s->nd = (int)nd;
    s->offset = (nd > 0) ? (long)md[2 + 2 * nd] : 0;
    long expect = 1;
    bool dense = true;
    for (size_t r = nd; r-- > 0;) {
        s->shape[r] = (long)md[2 + r];
        s->strides[r] = (long)md[2 + nd + r];
        if (s->shape[r] > 1 && s->strides[r] != expect) dense = false;
        expect *= s->shape[r];
    }
    s->contiguous = dense;
    return HODU_ROCM_OK;
}

// reduce metadata (crates/hodu_core/src/op_metadatas.rs:525-586, read by kernels/ops_reduce.c:51-66):
// [nd, shape.., strides.., offset, out_nd, out_shape.., n_reduce, reduce_dims.., keep_dim, reduce_size]
int parse_reduce_metadata(const size_t *md, size_t len, Reduction *r) {
    if (!md) return fail(HODU_ROCM_INVALID_ARG, "sum: metadata is null");
    if (len < 1) return fail(HODU_ROCM_INVALID_ARG, "sum: metadata is empty");
    for (size_t i = 0; i < len; i++)
        if (!sane(md[i])) return fail(HODU_ROCM_INVALID_ARG, "sum: metadata[%zu] out of range", i);
    const size_t nd = md[0];
    if (nd > 16) return fail(HODU_ROCM_UNSUPPORTED, "sum: %zu dims (> 16)", nd);
    if (len < 3 + 2 * nd) return fail(HODU_ROCM_INVALID_ARG, "sum: metadata has %zu words, too few for %zu dims", len, nd);
    const size_t *shape = md + 1, *strides = md + 1 + nd;
    const size_t offset = md[1 + 2 * nd], out_nd = md[2 + 2 * nd];
    if (out_nd > 16 || len < 4 + 2 * nd + out_nd) return fail(HODU_ROCM_INVALID_ARG, "sum: output shape does not fit the metadata");
    const size_t *out_shape = md + 3 + 2 * nd;
    const size_t n_red = md[3 + 2 * nd + out_nd];
    if (n_red > nd) return fail(HODU_ROCM_INVALID_ARG, "sum: %zu reduce dims of %zu", n_red, nd);
    if (len != 6 + 2 * nd + out_nd + n_red)
        return fail(HODU_ROCM_INVALID_ARG, "sum: metadata has %zu words, layout implies %zu", len, 6 + 2 * nd + out_nd + n_red);
    const size_t *red = md + 4 + 2 * nd + out_nd;
    const bool keep = md[4 + 2 * nd + out_nd + n_red] != 0;
    const size_t reduce_size = md[5 + 2 * nd + out_nd + n_red];
    bool is_red[16] = {false};
    size_t rs = 1;
    for (size_t i = 0; i < n_red; i++) {
        if (red[i] >= nd || is_red[red[i]]) return fail(HODU_ROCM_INVALID_ARG, "sum: bad reduce dim %zu", red[i]);
        is_red[red[i]] = true;
        rs *= shape[red[i]];
    }
    if (rs != reduce_size) return fail(HODU_ROCM_INVALID_ARG, "sum: reduce_size %zu != product of the reduced extents %zu", reduce_size, rs);
    // the output shape the encoder derives: kept dims in order, reduced dims as 1 when keep_dim, [1] if nothing is left
    size_t want[16], wn = 0, n_out = 1;
    for (size_t d = 0; d < nd; d++) {
        if (!is_red[d]) { want[wn++] = shape[d]; n_out *= shape[d]; }
        else if (keep) want[wn++] = 1;
    }
    if (wn == 0) want[wn++] = 1;
    if (wn != out_nd) return fail(HODU_ROCM_INVALID_ARG, "sum: output has %zu dims, the reduction leaves %zu", out_nd, wn);
    for (size_t d = 0; d < wn; d++)
        if (want[d] != out_shape[d]) return fail(HODU_ROCM_INVALID_ARG, "sum: output extent %zu of dim %zu, expected %zu", out_shape[d], d, want[d]);
    *r = Reduction{};
    r->n_out = (long)n_out;
    r->reduce_size = (long)reduce_size;
    r->offset = (long)offset;
    // split and merge: a dim joins its predecessor in the same list when stride_prev == extent * stride
    auto push = [](long *sh, long *st, int &n, long extent, long stride) {
        if (extent == 1) return;
        if (n > 0 && st[n - 1] == extent * stride) { sh[n - 1] *= extent; st[n - 1] = stride; return; }
        sh[n] = extent; st[n] = stride; n++;
    };
    for (size_t d = 0; d < nd; d++) {
        if (is_red[d]) push(r->red_shape, r->red_stride, r->red_n, (long)shape[d], (long)strides[d]);
        else push(r->kept_shape, r->kept_stride, r->kept_n, (long)shape[d], (long)strides[d]);
    }
    return HODU_ROCM_OK;
}

// attention metadata (this library's own: the reference has no single kernel for the function):
// [nb, batch_shape (nb).., Sq, Sk, D, q_strides (nb + 2).., k_strides (nb + 2).., v_strides (nb + 2).., q_off, k_off, v_off]
// strides and offsets in elements; the batch dims of q, k and v are already broadcast to batch_shape (stride 0 where
// an operand does not have the dim)
int parse_attention_metadata(const size_t *md, size_t len, AttentionArgs *a) {
    if (!md) return fail(HODU_ROCM_INVALID_ARG, "attention: metadata is null");
    if (len < 1) return fail(HODU_ROCM_INVALID_ARG, "attention: metadata is empty");
    for (size_t i = 0; i < len; i++)
        if (!sane(md[i])) return fail(HODU_ROCM_INVALID_ARG, "attention: metadata[%zu] out of range", i);
    const size_t nb = md[0];
    if (nb > 14) return fail(HODU_ROCM_UNSUPPORTED, "attention: %zu batch dims (> 14)", nb);
    const size_t want = 1 + nb + 3 + 3 * (nb + 2) + 3;
    if (len != want) return fail(HODU_ROCM_INVALID_ARG, "attention: metadata has %zu words, layout implies %zu", len, want);
    *a = AttentionArgs{};
    a->nb = (int)nb;
    a->batches = 1;
    for (size_t d = 0; d < nb; d++) {
        a->bshape[d] = (long)md[1 + d];
        a->batches *= a->bshape[d];
    }
    a->sq = (long)md[1 + nb]; a->sk = (long)md[2 + nb]; a->d = (long)md[3 + nb];
    const size_t *qs = md + 4 + nb, *ks = qs + nb + 2, *vs = ks + nb + 2;
    if (a->d > 1 && (qs[nb + 1] != 1 || ks[nb + 1] != 1 || vs[nb + 1] != 1))
        return fail(HODU_ROCM_UNSUPPORTED, "attention: the head dim must be dense in q, k and v");
    for (size_t d = 0; d < nb; d++) {
        a->q_bs[d] = (long)qs[d]; a->k_bs[d] = (long)ks[d]; a->v_bs[d] = (long)vs[d];
    }
    a->q_row = (long)qs[nb]; a->k_row = (long)ks[nb]; a->v_row = (long)vs[nb];
    a->q_off = (long)md[want - 3]; a->k_off = (long)md[want - 2]; a->v_off = (long)md[want - 1];
    return HODU_ROCM_OK;
}

}  // namespace hodu