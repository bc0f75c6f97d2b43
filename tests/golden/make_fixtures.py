"""Writes the golden fixtures of this directory from the reference's own C kernels.

Run in the build container only (needs oracle/_ref/libhodu_cpu_ref.so, i.e. `make -C oracle ref`,
which compiles crates/hodu_cpu_kernels/kernels/{ops_matrix,ops_cast,ops_memory,ops_binary,ops_unary,ops_reduce}.c where they lie
under /root/reference):

    python tests/golden/make_fixtures.py

Each fixture is data only: seeded inputs (bit patterns), the metadata vector handed to the
reference kernel and the bytes it returned.  The fixtures let the oracle be checked against the
reference on machines where the reference tree does not exist.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import helpers as H  # noqa: E402
import oracle  # noqa: E402


def product_cases():
    """(name, op, lhs view, rhs view) -- one per branch of the reference kernels."""
    V = H.View
    cases = [
        # dot, contiguous, M < 512: blocked 32x32x256 path with 4x4 register tiles (ops_matrix.c:486-525)
        ("dot_blocked", "dot", V([37, 300]), V([300, 29])),
        # dot, contiguous, M >= 512: pthread row split (ops_matrix.c:455-484)
        ("dot_threaded", "dot", V([520, 24]), V([24, 20])),
        # dot, rhs is a transposed view: strided i-k-j path (ops_matrix.c:527-548)
        ("dot_rhs_t", "dot", V([19, 40]), V([23, 40]).t()),
        # dot, lhs transposed, both with offsets into a larger buffer
        ("dot_lhs_t_offset", "dot", V([40, 17], offset=5).t(), V([40, 21], offset=3)),
        # dot, row-sliced lhs (stride != K) and column-strided rhs
        ("dot_sliced", "dot", V([30, 64]).slice(1, 4, 36), V([32, 50]).slice(1, 1, 49, 2)),
        # matmul, 2-D contiguous: fast path (ops_matrix.c:100-143)
        ("matmul_2d", "matmul", V([33, 47]), V([47, 18])),
        # matmul, M >= 256: threaded fast path (get_optimal_threads(M,128))
        ("matmul_2d_threaded", "matmul", V([260, 16]), V([16, 12])),
        # matmul, batched contiguous: general path (ops_matrix.c:144-192)
        ("matmul_batched", "matmul", V([3, 9, 20]), V([3, 20, 11])),
        # matmul, rhs has no batch dim
        ("matmul_rhs_2d", "matmul", V([2, 3, 8, 16]), V([16, 10])),
        # matmul, stride-0 broadcast of a transposed weight (what Linear on a 3-D input produces
        # once the forced copy in Tensor::broadcast is removed)
        ("matmul_bcast_t", "matmul", V([4, 6, 24]), V([13, 24]).t().broadcast_to([4, 24, 13])),
        # matmul, size-1 batch dims on both sides, transposed batched rhs
        ("matmul_b1_t", "matmul", V([1, 5, 7, 12]), V([2, 1, 9, 12]).t()),
    ]
    return cases


PRODUCT_DTYPES = ["bf16", "f16", "f8e4m3", "f8e5m2", "f32", "f64", "i8", "i32", "i64", "u8", "u32", "u16", "i16", "u64"]


# the dtypes behind hodu's optional cargo features are pinned on one case per kernel branch
RARE_DTYPES = {"f64", "i64", "u64", "u16", "i16", "f8e5m2"}
RARE_CASES = {"dot_rhs_t", "dot_threaded", "matmul_2d", "matmul_b1_t"}


def scale_for(dt):
    # keep narrow floats inside the range where the hodu decoder and OCP agree (|v| < 256)
    return {"f8e4m3": 2.0, "f8e5m2": 2.0}.get(dt, 1.0)


def write_products(ref):
    out = {}
    names = []
    for name, op, lv, rv in product_cases():
        for dt in PRODUCT_DTYPES:
            key = f"{name}__{dt}"
            if dt in RARE_DTYPES and name not in RARE_CASES:
                continue
            seed = (sum(map(ord, key)) * 7919) % 100003
            a = H.random_storage(dt, lv.span(), seed, scale_for(dt))
            b = H.random_storage(dt, rv.span(), seed + 1, scale_for(dt))
            md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
            got = ref.dot(dt, a, b, md) if op == "dot" else ref.matmul(dt, a, b, md)
            out[key + "__lhs"] = a
            out[key + "__rhs"] = b
            out[key + "__md"] = np.asarray(md, dtype=np.uint64)
            out[key + "__out"] = got
            names.append(f"{key}|{op}|{dt}")
    out["index"] = np.array(names)
    np.savez_compressed(os.path.join(HERE, "products.npz"), **out)
    return len(names)


def sample_floats():
    g = H.rng(77)
    parts = [
        g.standard_normal(3000).astype(np.float32),
        (g.standard_normal(2000) * 100).astype(np.float32),
        (g.standard_normal(2000) * 1e-3).astype(np.float32),
        np.exp(g.uniform(-20, 12, 3000)).astype(np.float32) * np.where(g.random(3000) < 0.5, -1, 1).astype(np.float32),
        np.array([0.0, -0.0, 1.0, -1.0, 0.5, 448.0, 449.0, 240.0, 256.0, 255.9, 447.9, 1e-3, 0.001953125,
                  0.0019531, 0.015625, 0.0156, 65504.0, 65505.0, 65520.0, 6.1e-5, 6.103515625e-05, 5.9e-8,
                  57344.0, 57345.0, 1.52587890625e-05, 1.5e-5, np.inf, -np.inf, np.nan, 3.0e38, 1.17e-38,
                  1.0039062, 1.00390625, 1.0078125, 0.99609375, 1.9999, 3.9999, 0.12499, 2.5, 3.5, 4.5, 5.5, 6.5, 7.5],
                 dtype=np.float32),
    ]
    return np.concatenate(parts)


def write_tables(ref):
    one = lambda n: H.cast_md(H.View([n]))  # noqa: E731
    out = {}
    codes = np.arange(256, dtype=np.uint8)
    out["f8e4m3_to_f32"] = ref.cast("f8e4m3", "f32", codes, one(256)).view(np.uint32)
    out["f8e5m2_to_f32"] = ref.cast("f8e5m2", "f32", codes, one(256)).view(np.uint32)
    out["f8e4m3_to_bf16"] = ref.cast("f8e4m3", "bf16", codes, one(256))
    out["f8e4m3_to_f16"] = ref.cast("f8e4m3", "f16", codes, one(256))
    h = np.arange(65536, dtype=np.uint16)
    out["f16_to_f32"] = ref.cast("f16", "f32", h, one(65536)).view(np.uint32)
    out["bf16_to_f16"] = ref.cast("bf16", "f16", h, one(65536))
    out["bf16_to_f8e4m3"] = ref.cast("bf16", "f8e4m3", h, one(65536))
    out["bf16_to_f8e5m2"] = ref.cast("bf16", "f8e5m2", h, one(65536))
    out["f16_to_f8e4m3"] = ref.cast("f16", "f8e4m3", h, one(65536))
    x = sample_floats()
    out["f32_samples"] = x.view(np.uint32)
    for dst in ("bf16", "f16", "f8e4m3", "f8e5m2"):
        out[f"f32_to_{dst}"] = ref.cast("f32", dst, x, one(x.size))
    np.savez_compressed(os.path.join(HERE, "tables.npz"), **out)


def cast_cases():
    V = H.View
    return [
        ("flat", V([257])),
        ("t2d", V([13, 21]).t()),
        ("sliced", V([6, 10, 12], offset=7).slice(2, 1, 11, 3)),
        ("bcast", V([1, 9]).broadcast_to([5, 9])),
    ]


CAST_PAIRS = [
    ("f8e4m3", "bf16"), ("f8e4m3", "f32"), ("f8e4m3", "f16"), ("i8", "i32"), ("bf16", "f32"), ("f32", "bf16"),
    ("f32", "f16"), ("f16", "f32"), ("f16", "bf16"), ("bf16", "f16"), ("f32", "i32"), ("i32", "f32"), ("f32", "u32"),
    ("u32", "f32"), ("f64", "f32"), ("f32", "f64"), ("f32", "f8e4m3"), ("bf16", "f8e4m3"), ("u8", "f32"),
    ("f32", "u8"), ("f32", "i8"), ("i32", "i8"), ("i32", "u8"), ("u8", "i32"), ("bool", "f32"), ("f32", "bool"),
    ("i32", "bool"), ("bool", "bool"), ("u32", "i32"), ("i32", "u32"), ("i8", "bf16"), ("i32", "bf16"),
    ("i64", "i32"), ("i32", "i64"), ("u16", "f16"), ("i16", "f32"), ("u64", "f32"), ("f64", "bf16"),
    ("f8e5m2", "f32"), ("f32", "f8e5m2"), ("bf16", "i32"), ("f16", "i32"), ("bf16", "bf16"), ("f32", "f32"),
]


def cast_input(src, n, seed):
    if src in ("f32", "f64"):
        g = H.rng(seed)
        x = g.standard_normal(n) * g.choice([0.5, 3.0, 40.0], n)  # in range for every integer target >= 8 bit
        return x.astype(np.float32) if src == "f32" else x
    if src == "bool":
        return H.rng(seed).integers(0, 4, n).astype(np.uint8)  # non-canonical truthy bytes too
    return H.random_storage(src, n, seed, 2.0)


def write_casts(ref):
    out, names = {}, []
    for cname, v in cast_cases():
        for src, dst in CAST_PAIRS:
            key = f"{cname}__{src}__{dst}"
            x = cast_input(src, v.span(), (sum(map(ord, key)) * 104729) % 100003)
            if dst in ("u8", "u32", "bool") and src in ("f32", "f64", "bf16", "f16"):
                # negative float -> unsigned is undefined in C; keep the pinned domain defined
                if src in ("f32", "f64"):
                    x = np.abs(x)
                else:
                    x = x & 0x7FFF
            md = H.cast_md(v)
            out[key + "__in"] = x
            out[key + "__md"] = np.asarray(md, dtype=np.uint64)
            out[key + "__out"] = ref.cast(src, dst, x, md)
            names.append(f"{key}|{src}|{dst}")
        for dt in ("bf16", "f8e4m3", "f32", "i32", "i8", "u8", "f64"):
            key = f"{cname}__contig__{dt}"
            x = H.random_storage(dt, v.span(), 991)
            md = H.cast_md(v)
            out[key + "__in"] = x
            out[key + "__md"] = np.asarray(md, dtype=np.uint64)
            out[key + "__out"] = ref.contiguous(dt, x, md)
            names.append(f"{key}|contiguous|{dt}")
    out["index"] = np.array(names)
    np.savez_compressed(os.path.join(HERE, "casts.npz"), **out)
    return len(names)


ELEMENTWISE_FLOATS = ["f8e4m3", "f8e5m2", "bf16", "f16", "f32", "f64"]
ELEMENTWISE_INTS = ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]


def elementwise_input(dt, n, seed):
    """values spread over the dtype's range, so that narrowing overflows, underflows and ties all occur"""
    g = H.rng(seed)
    if dt in ELEMENTWISE_INTS:
        info = np.iinfo(oracle.STORAGE[dt])
        return g.integers(info.min, info.max, n, dtype=info.dtype, endpoint=True)
    mag = {"f8e4m3": 6.0, "f8e5m2": 12.0, "bf16": 30.0, "f16": 14.0, "f32": 30.0, "f64": 30.0}[dt]
    x = g.standard_normal(n) * np.exp2(g.uniform(-mag, mag, n))
    x[:: 37] = 0.0
    if dt == "f64":
        return x
    if dt == "f32":
        return x.astype(np.float32)
    return cast_input_from_f32(dt, x.astype(np.float32))


def cast_input_from_f32(dt, x):
    md = H.cast_md(H.View([x.size]))
    return oracle.RefLib().cast("f32", dt, np.clip(x, -3e38, 3e38), md)


def write_elementwise(ref):
    """add (a contiguous [.., M, N] plus a vector broadcast along the last axis -- what Linear::forward adds --,
    and two contiguous operands), mul_scalar and relu of every dtype the reference defines them for"""
    V = H.View
    out, names = {}, []
    for dt in ELEMENTWISE_FLOATS + ELEMENTWISE_INTS:
        lv = V([3, 7, 19])
        for tag, rv in (("bias", V([19], offset=2).broadcast_to([3, 7, 19])), ("bias_strided", V([19], [3], 1).broadcast_to([3, 7, 19])),
                        ("full", V([3, 7, 19], offset=4))):
            a, b = elementwise_input(dt, lv.span(), 11), elementwise_input(dt, rv.span(), 12)
            md = np.array(H.binary_md(lv, rv), dtype=np.uint64)
            key = f"add_{tag}__{dt}"
            out[key + "__lhs"], out[key + "__rhs"], out[key + "__md"] = a, b, md
            out[key + "__out"] = ref.add(dt, a, b, md)
            names.append(f"{key}|add|{dt}")
        x = elementwise_input(dt, 1024, 13)
        md = np.array(H.cast_md(V([1024])), dtype=np.uint64)
        for j, c in enumerate(elementwise_input(dt, 64, 14)[[3, 5, 8]]):
            key = f"mul_scalar{j}__{dt}"
            out[key + "__in"], out[key + "__md"], out[key + "__scalar"] = x, md, np.array([c], dtype=x.dtype)
            out[key + "__out"] = ref.mul_scalar(dt, x, md, np.array([c], dtype=x.dtype))
            names.append(f"{key}|mul_scalar|{dt}")
        if dt in ELEMENTWISE_FLOATS:
            key = f"relu__{dt}"
            out[key + "__in"], out[key + "__md"] = x, md
            out[key + "__out"] = ref.relu(dt, x, md)
            names.append(f"{key}|relu|{dt}")
    out["index"] = np.array(names)
    np.savez_compressed(os.path.join(HERE, "elementwise.npz"), **out)
    return len(names)


def sum_cases():
    """(name, view, dims, keep_dim): what sum_to_shape runs on a matmul's gradients (leading dims, one at a time, and
    kept extent-1 dims) plus the other shapes of the reference's walker"""
    V = H.View
    return [
        ("lead", V([5, 7, 12]), [0], False),           # [B, K, N] -> [K, N]
        ("lead_keep", V([5, 7, 12]), [0], True),       # -> [1, K, N]
        ("middle_keep", V([3, 4, 6, 5]), [1], True),   # a broadcast batch dim of extent 1 in the target
        ("two", V([3, 4, 6, 5]), [0, 1], False),
        ("last", V([9, 33]), [1], False),              # strided rows: the reference's sequential order
        ("last_keep_strided", V([9, 40]).slice(1, 1, 40, 3), [1], True),
        ("transposed", V([6, 8, 10], offset=3).t(0, 2), [0], False),
        ("all", V([4, 5, 6]), [0, 1, 2], False),
    ]


def write_sums(ref):
    out, names = {}, []
    for dt in ELEMENTWISE_FLOATS + ELEMENTWISE_INTS:
        for name, v, dims, keep in sum_cases():
            x = H.random_storage(dt, v.span(), 21, 2.0)
            md = np.array(H.reduce_md(v, dims, keep), dtype=np.uint64)
            key = f"sum_{name}__{dt}"
            out[key + "__in"], out[key + "__md"] = x, md
            out[key + "__out"] = ref.sum(dt, x, md)
            names.append(f"{key}|{dt}")
    out["index"] = np.array(names)
    np.savez_compressed(os.path.join(HERE, "sums.npz"), **out)
    return len(names)


def main():
    if not oracle.RefLib.available():
        raise SystemExit("oracle/_ref/libhodu_cpu_ref.so missing: run `make -C oracle ref` first")
    ref = oracle.RefLib()
    n = write_products(ref)
    write_tables(ref)
    m = write_casts(ref)
    e = write_elementwise(ref)
    k = write_sums(ref)
    print(f"wrote {n} product cases, {m} cast/contiguous cases, {e} element-wise cases, {k} sum cases, tables")


if __name__ == "__main__":
    main()
