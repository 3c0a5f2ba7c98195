"""The arg-max entry point that allocates nothing (shv_argmax_static): same results as shv_argmax,
its partial results in the library's static device array.  Two calls in a row, the second with a
smaller input, so that what the first call left in the array must not show in the second."""
import ctypes as C

import numpy as np
import pytest

import shv

pytestmark = pytest.mark.gpu
A = shv.api


def _both(ctx, logits):
    """(shv_argmax, shv_argmax_static) over the same device rows, both through the C ABI."""
    L = A.load()
    logits = np.ascontiguousarray(logits, np.float32)
    rows, n = logits.shape
    dev = ctx.upload(logits)
    out = []
    for fn in (L.shv_argmax, L.shv_argmax_static):
        best = ctx.upload(np.full(rows, -7, np.int32))
        args = A.ArgmaxArgs(dev.ptr, best.ptr, None, None, rows, n, n)
        A.check(fn(ctx.h, C.byref(args)))
        out.append(list(best.read(np.int32, rows)))
    return out


def test_static_argmax_equals_argmax_on_two_calls_in_a_row(ctx):
    rng = np.random.default_rng(11)
    big = rng.standard_normal((3, 151936)).astype(np.float32)
    big[1, [40, 150000]] = 9.0          # a tie across blocks goes to the lower index
    want, got = _both(ctx, big)
    assert got == want == list(np.argmax(big, axis=1))
    small = rng.standard_normal((2, 1500)).astype(np.float32)   # two blocks a row where there were 149
    small[0, 1499] = 8.0
    want, got = _both(ctx, small)
    assert got == want == list(np.argmax(small, axis=1))
    one = np.full((1, 7), -np.inf, np.float32)                  # nothing above -inf: 0, as the reference returns
    want, got = _both(ctx, one)
    assert got == want == [0]


def test_static_argmax_stores_the_next_token_and_refuses_too_many_rows(ctx):
    L = A.load()
    logits = np.zeros((1, 5000), np.float32)
    logits[0, 4321] = 1.0
    ids = ctx.upload(np.array([11, 22, 33, -1, -1], np.int32))
    pos = ctx.upload(np.array([2], np.int32))
    best = ctx.alloc(4)
    args = A.ArgmaxArgs(ctx.upload(logits).ptr, best.ptr, ids.ptr, pos.ptr, 1, 5000, 5000)
    A.check(L.shv_argmax_static(ctx.h, C.byref(args)))
    assert best.read(np.int32, 1)[0] == 4321
    assert list(ids.read(np.int32, 5)) == [11, 22, 33, 4321, -1]
    assert pos.read(np.int32, 1)[0] == 3
    rows = 15
    x = ctx.upload(np.zeros((rows, 64), np.float32))
    out = ctx.alloc(rows * 4)
    args = A.ArgmaxArgs(x.ptr, out.ptr, None, None, rows, 64, 64)
    assert L.shv_argmax_static(ctx.h, C.byref(args)) == -1
    assert b"at most 14 rows" in L.shv_last_error()


def test_static_argmax_recorded_into_a_graph_and_replayed(ctx):
    """Its stated callers record it: the op (counters cleared by a kernel, then the arg-max) goes into a
    recorded sequence of the library, which replays as a HIP graph; three replays, with other eager
    work and new logits in the same buffer between them, each against shv_argmax on the same rows."""
    L = A.load()
    rng = np.random.default_rng(5)
    rows, n = 3, 151936
    dev = ctx.upload(np.zeros((rows, n), np.float32))
    best = ctx.upload(np.full(rows, -7, np.int32))
    rec = ctx.prerecord([A.make_op(A.OP_ARGMAX_STATIC, A.ArgmaxArgs(dev.ptr, best.ptr, None, None, rows, n, n))])
    try:
        for rep in range(3):
            logits = rng.standard_normal((rows, n)).astype(np.float32)
            logits[rep % rows, [rep, n - 1 - rep]] = 7.0        # a tie across blocks: the lower index
            dev.write(logits)
            best.write(np.full(rows, -7, np.int32))
            rec.submit(1)
            got = list(best.read(np.int32, rows))
            eager = ctx.upload(np.full(rows, -7, np.int32))
            A.check(L.shv_argmax(ctx.h, C.byref(A.ArgmaxArgs(dev.ptr, eager.ptr, None, None, rows, n, n))))
            assert got == list(eager.read(np.int32, rows)) == list(np.argmax(logits, axis=1)), rep
    finally:
        rec.destroy()
