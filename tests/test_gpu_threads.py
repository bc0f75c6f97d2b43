"""Several host threads on ONE context (the contract of the boundary: any host thread may call, calls on a context are
serialised inside the library).  The products chosen share context-owned state -- the split-K workspace and the
arrival counters of the M <= 16 kernel -- and are deterministic, so every thread must reproduce, bit for bit, what a
single thread computed first."""
import threading

import numpy as np
import pytest

import helpers as H
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View


def test_threads_share_a_context():
    ctx = ffi.Context(0)
    g = H.rng(77)
    cases = []
    for name, lv, rv, kind in (("bf16", V([128, 2048]), V([256, 2048]).t(), "splitk"),
                               ("bf16_f8e4m3w", V([16, 4096]), V([4096, 4096]).t(), "_splitk"),
                               ("bf16", V([3, 200, 256]), V([3, 136, 256]).t(), "")):
        l_dt, r_dt = ("bf16", "f8e4m3") if name == "bf16_f8e4m3w" else ("bf16", "bf16")
        a = ctx.upload(H.random_storage(l_dt, lv.span(), int(g.integers(1 << 30)), 1.0))
        b = ctx.upload(H.random_storage(r_dt, rv.span(), int(g.integers(1 << 30)), 2.0 if r_dt == "f8e4m3" else 1.0))
        op = "dot" if lv.ndim == 2 else "matmul"
        md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
        n = int(np.prod(lv.shape[:-1])) * rv.shape[-1]
        out = ctx.alloc(n * 2)
        ctx.product(op, name, a, b, out, md)
        assert kind in ctx.last_kernel(), ctx.last_kernel()
        cases.append((op, name, a, b, md, n, ctx.download(out, np.uint16, n)))
        out.free()
    errors = []

    def worker(seed):
        try:
            order = np.random.default_rng(seed).permutation(len(cases) * 8) % len(cases)
            for i in order:
                op, name, a, b, md, n, want = cases[i]
                out = ctx.alloc(n * 2)
                ctx.product(op, name, a, b, out, md)
                got = ctx.download(out, np.uint16, n)
                out.free()
                if not np.array_equal(got, want):
                    errors.append((seed, name, int((got != want).sum())))
        except Exception as e:  # noqa: BLE001
            errors.append((seed, repr(e)))

    threads = [threading.Thread(target=worker, args=(s,)) for s in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    ctx.close()
    assert not errors, errors[:5]
