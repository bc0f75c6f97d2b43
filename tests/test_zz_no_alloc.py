"""The one entry point that allocates nothing (hodu_rocm_dot_bf16_f8e4m3w_noalloc) against the entry point it is a
variant of (hodu_rocm_dot_bf16_f8e4m3w), bit for bit, through the C ABI: two calls in a row on kernels that use the
scratch (the split-K kernel for M <= 16: partial sums and arrival counters), the second with a smaller input;
then the decode shapes without scratch, a product whose scratch does not fit (refused, with both sizes in the
message), and the same calls captured into a HIP graph and replayed."""
import numpy as np
import pytest

import helpers as H
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.force_tile(-1)
    c.force_splitk(-1)
    c.close()


def both(ctx, m, n, k, seed, expect=None):
    x = H.random_storage("bf16", m * k, seed)
    w = H.random_storage("f8e4m3", n * k, seed + 1, 30.0)
    md = H.dot_md(V([m, k]), V([n, k]).t())
    dx, dw = ctx.upload(x), ctx.upload(w)
    out_a, out_b = ctx.alloc(m * n * 2), ctx.alloc(m * n * 2)
    ctx.fill(out_a, 0xFF)
    ctx.fill(out_b, 0xEE)
    ctx.product("dot", "bf16_f8e4m3w", dx, dw, out_a, md)
    k_alloc = ctx.last_kernel()
    ctx.dot_noalloc(dx, dw, out_b, md)
    k_fixed = ctx.last_kernel()
    a, b = ctx.download(out_a, np.uint16), ctx.download(out_b, np.uint16)
    for d in (dx, dw, out_a, out_b):
        d.free()
    assert k_alloc == k_fixed
    if expect:
        assert k_fixed == expect, k_fixed
    assert np.array_equal(a, b), f"{k_fixed}: {np.count_nonzero(a != b)} of {a.size} outputs differ"
    return a


def test_two_calls_in_a_row_the_second_smaller(ctx):
    both(ctx, 16, 4096, 4096, 1, expect="skinny_bf16_f8w_splitk")   # config 3, M = 16: 8 slices, 2 MiB of partial sums
    both(ctx, 12, 1024, 4096, 3, expect="skinny_bf16_f8w_splitk")   # smaller: fewer column blocks, other slice count
    both(ctx, 16, 4096, 4096, 1, expect="skinny_bf16_f8w_splitk")   # and the first again, after the smaller one


def test_a_fresh_context_allocates_nothing_for_it():
    """the split-K shapes on a context that has never run a product: after the calls the context still owns no
    partial-sum workspace and no arrival counters (had the entry point grown them, they would be there), while the
    allocating entry point on the same context does grow them"""
    fresh = ffi.Context(0)
    try:
        assert fresh.scratch_state() == {"workspace_bytes": 0, "arrival_allocated": False, "fixed": False}
        m, n, k = 16, 4096, 4096
        x = H.random_storage("bf16", m * k, 31)
        w = H.random_storage("f8e4m3", n * k, 32, 30.0)
        md = H.dot_md(V([m, k]), V([n, k]).t())
        dx, dw, out_a, out_b = fresh.upload(x), fresh.upload(w), fresh.alloc(m * n * 2), fresh.alloc(m * n * 2)
        for _ in range(2):
            fresh.fill(out_b, 0xEE)
            fresh.dot_noalloc(dx, dw, out_b, md)
            assert fresh.last_kernel() == "skinny_bf16_f8w_splitk"
            assert fresh.scratch_state() == {"workspace_bytes": 0, "arrival_allocated": False, "fixed": False}
        fresh.force_splitk(4)
        x2 = H.random_storage("bf16", 128 * k, 33)
        dx2, out2 = fresh.upload(x2), fresh.alloc(128 * 512 * 2)
        fresh.dot_noalloc(dx2, dw, out2, H.dot_md(V([128, k]), V([512, k]).t()))  # the pipelined kernel cut along K
        assert "splitk" in fresh.last_kernel()
        assert fresh.scratch_state() == {"workspace_bytes": 0, "arrival_allocated": False, "fixed": False}
        fresh.force_splitk(-1)
        got_b = fresh.download(out_b, np.uint16)
        fresh.product("dot", "bf16_f8e4m3w", dx, dw, out_a, md)
        state = fresh.scratch_state()
        assert state["workspace_bytes"] > 0 and state["arrival_allocated"] and not state["fixed"]
        assert np.array_equal(fresh.download(out_a, np.uint16), got_b)
        for d in (dx, dw, out_a, out_b, dx2, out2):
            d.free()
    finally:
        fresh.force_splitk(-1)
        fresh.close()


def test_shapes_without_scratch(ctx):
    both(ctx, 1, 4096, 4096, 5, expect="gemv_bf16_f8w_walk")
    both(ctx, 8, 640, 1024, 7)
    both(ctx, 512, 512, 1024, 9)


def test_pipelined_split_k_within_the_limit(ctx):
    ctx.force_splitk(4)
    try:
        both(ctx, 128, 512, 4096, 11)   # 4 x 128 x 512 x 4 bytes = 1 MiB
        assert "splitk" in ctx.last_kernel()
    finally:
        ctx.force_splitk(-1)


def test_scratch_beyond_the_limit_is_refused(ctx):
    m, n, k = 256, 4096, 4096  # cut four ways: 16 MiB of partial sums against 8 MiB of static scratch
    dx, dw, out = ctx.alloc(m * k * 2), ctx.alloc(n * k), ctx.alloc(m * n * 2)
    ctx.fill(dx, 0)
    ctx.fill(dw, 0)
    md = H.dot_md(V([m, k]), V([n, k]).t())
    ctx.force_splitk(4)
    try:
        with pytest.raises(ffi.HoduRocmError) as e:
            ctx.dot_noalloc(dx, dw, out, md)
        assert e.value.status == ffi.SCRATCH
        assert "16777216" in e.value.message and "8388608" in e.value.message
        assert not ctx.scratch_state()["fixed"]  # the refused call put the context's own scratch pointers back
        ctx.product("dot", "bf16_f8e4m3w", dx, dw, out, md)  # the allocating entry point still takes it
        ctx.sync()
        ctx.force_splitk(-1)
        both(ctx, 16, 4096, 4096, 1, expect="skinny_bf16_f8w_splitk")  # and a split-K product after the refusal matches
    finally:
        ctx.force_splitk(-1)
        for d in (dx, dw, out):
            d.free()


def test_captured_into_a_graph_and_replayed(ctx):
    """the calls launch kernels only, so they can be recorded; every replay equals the eager result"""
    m, n, k = 16, 4096, 4096
    x = H.random_storage("bf16", m * k, 21)
    w = H.random_storage("f8e4m3", n * k, 22, 30.0)
    md = H.dot_md(V([m, k]), V([n, k]).t())
    dx, dw, out = ctx.upload(x), ctx.upload(w), ctx.alloc(m * n * 2)
    ctx.dot_noalloc(dx, dw, out, md)
    eager = ctx.download(out, np.uint16)
    for _ in range(3):
        ctx.fill(out, 0xFF)
        ms = ctx.time_noalloc(dx, [dw], out, md, 5, graph=True)
        assert ms > 0
        assert np.array_equal(ctx.download(out, np.uint16), eager)
        both(ctx, 12, 1024, 4096, 3)  # eager work between the replays
    for d in (dx, dw, out):
        d.free()
