"""Q4_K projections of two to eight rows through the kernel that forms each weight once for all
rows (binary16 operands on the matrix cores): float32 accuracy whatever the activations'
magnitude, every way the launcher splits a matrix into blocks, and agreement with the kernels
it took over from.  The reference's form is matvec over dequantised rows, one row of
activations at a time (llm/hc.go:255-264, gguf/dequant.go:252-276)."""
import os

import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu
A = shv.api


def _weights(rng, n, k, std=0.02):
    return O.quantize_q4k((rng.standard_normal((n, k)) * std).astype(np.float32))


@pytest.fixture(scope="module")
def old_ctx():
    """A context with the kernel switched off: the side-by-side row kernel and the tiled ones."""
    os.environ["SHV_MROWS"] = "0"
    try:
        c = A.Context(0)
    finally:
        del os.environ["SHV_MROWS"]
    yield c
    c.destroy()


@pytest.mark.parametrize("n,k", [(1024, 2048), (2048, 4096)])
@pytest.mark.parametrize("scale", [1e-5, 1e-3, 0.02, 1.0, 100.0, 3e4])
def test_accuracy_does_not_depend_on_the_activations_magnitude(ctx, n, k, scale):
    """The activations go through binary16 as a high part and a remainder.  Unscaled, a remainder below
    6e-5 is a subnormal number (rows of magnitude 0.02 came out 4e-5 off, of 1e-5 half a percent);
    each wave scales its part of a row by a power of two first, and the result is good to a few
    1e-7 from 1e-5 to 3e4 (the bar here leaves room for the side-by-side row kernel's 3e-6, which takes
    two to four rows of 4096 columns).  Against float64 over the dequantised weights."""
    rng = np.random.default_rng(int(n + 1000 * np.log10(scale) + 7000))
    wq = _weights(rng, n, k)
    w64 = O.dequant_q4k(wq, k).astype(np.float64)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    dw, dg = ctx.upload(wq), ctx.upload(gamma)
    for rows in (2, 3, 5, 8):
        x = (rng.standard_normal((rows, k)) * scale).astype(np.float32)
        # one row of a few large entries among small ones: the scale follows the largest
        x[0, ::97] *= 50
        dx, dy = ctx.upload(x), ctx.alloc(rows * n * 4)
        for pro in (A.PRO_NONE, A.PRO_RMSNORM):
            ctx.gemv_q4k(dw, dx, dy, n, k, n_tok=rows, prologue=pro, gamma=dg if pro else None, eps=1e-6)
            got = dy.read(np.float32, rows * n).reshape(rows, n)
            x64 = x.astype(np.float64)
            if pro:
                x64 = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * gamma.astype(np.float64)
            want = x64 @ w64.T
            for t in range(rows):
                assert O.rel_l2(got[t], want[t]) <= 1e-5, (rows, pro, t)


def test_rows_of_zeros_and_a_zero_quarter(ctx):
    """A row of zeros (a padded sequence) and a row whose first 512 columns are zero: a wave whose
    part of a row holds nothing scales by the largest finite power of two and must add 0, not NaN."""
    rng = np.random.default_rng(11)
    n, k, rows = 512, 2048, 4
    wq = _weights(rng, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[1] = 0
    x[2, :512] = 0
    x[3, 512:] = 0
    x[3, :512] *= 1e-30
    dy = ctx.alloc(rows * n * 4)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(x), dy, n, k, n_tok=rows)
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    w64 = O.dequant_q4k(wq, k).astype(np.float64)
    want = x.astype(np.float64) @ w64.T
    assert np.all(np.isfinite(got))
    assert np.all(got[1] == 0)
    for t in (0, 2, 3):
        assert O.rel_l2(got[t], want[t]) <= 3e-6, t


@pytest.mark.parametrize("n,rows", [(8192 + 16, 6), (8192 + 40, 8), (8200, 5),      # four tiles a block from six rows on, ragged tails
                                    (32768 + 48, 2), (32768 + 48, 3), (32768 + 8, 4),  # a stream: two and four tiles a block
                                    (32768, 7),                                   # a stream of five rows and more stays with the tiled kernel
                                    (16, 2), (20, 8), (4080, 4),                  # one tile, a ragged only tile, one tile a block
                                    # eight waves a block from four rows on: four, two and one tile a block, ragged tails
                                    (12352, 4), (12352, 8), (4096 + 24, 5), (6000, 7), (3000, 6)])
def test_every_split_of_a_matrix_into_blocks(ctx, old_ctx, n, rows):
    """The launcher gives a block one, two or four tiles of sixteen weight rows and four or eight waves depending on
    how many tiles there are and how many activation rows; the last block's tiles may be ragged or absent."""
    rng = np.random.default_rng(n + rows)
    k = 2048
    wq = _weights(rng, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    res = rng.standard_normal((rows, n)).astype(np.float32)
    want = (x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6) * gamma) @ \
        O.dequant_q4k(wq, k).astype(np.float64).T + res
    dw, dx, dg = ctx.upload(wq), ctx.upload(x), ctx.upload(gamma)
    dy = ctx.upload(res)
    ctx.gemv_q4k(dw, dx, dy, n, k, n_tok=rows, prologue=A.PRO_RMSNORM, gamma=dg, eps=1e-6, residual=dy)   # in place
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    for t in range(rows):
        assert O.rel_l2(got[t], want[t]) <= 3e-6, t
    # the kernels it took over from, on the same buffers
    dy2 = old_ctx.upload(res)
    old_ctx.gemv_q4k(old_ctx.upload(wq), old_ctx.upload(x), dy2, n, k, n_tok=rows, prologue=A.PRO_RMSNORM, gamma=old_ctx.upload(gamma),
                     eps=1e-6, residual=dy2)
    old = dy2.read(np.float32, rows * n).reshape(rows, n)
    for t in range(rows):
        assert O.rel_l2(got[t], old[t]) <= 1e-5, t


@pytest.mark.parametrize("rows", [2, 3, 4, 6, 8])
def test_two_sequences_and_more_write_their_own_ring_rows(ctx, rows):
    """Ring output with a slot table: `rows` sequences of one row each (a batched decode pass) and one
    sequence of `rows` rows, at positions that wrap around the ring."""
    rng = np.random.default_rng(40 + rows)
    n, k, slots_ring, n_slots = 12352, 2048, 8, 9
    wq = _weights(rng, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    want = [O.gemv_q4k(wq, O.rmsnorm(x[t:t + 1], gamma, 1e-6)[0], n, k, threads=8) for t in range(rows)]
    dw, dx, dg = ctx.upload(wq), ctx.upload(x), ctx.upload(gamma)
    # one row each of `rows` sequences
    pos = rng.integers(0, 50, size=rows).astype(np.int32)
    slot = rng.permutation(n_slots)[:rows].astype(np.int32)
    ring = ctx.upload(np.zeros((n_slots, slots_ring, n), np.float32))
    ctx.gemv_q4k(dw, dx, ring, n, k, n_tok=rows, prologue=A.PRO_RMSNORM, gamma=dg, eps=1e-6, pos=ctx.upload(pos), slot=ctx.upload(slot),
                 seq_len=1, ring_slots=slots_ring, ring_stride=n)
    got = ring.read(np.float32, n_slots * slots_ring * n).reshape(n_slots, slots_ring, n)
    for t in range(rows):
        assert O.rel_l2(got[slot[t], pos[t] % slots_ring], want[t]) <= 1e-3, t
    assert np.count_nonzero(got.any(axis=2)) == rows
    # one sequence of `rows` rows from position 6: rows wrap to the ring's start
    ring2 = ctx.upload(np.zeros((n_slots, slots_ring, n), np.float32))
    ctx.gemv_q4k(dw, dx, ring2, n, k, n_tok=rows, prologue=A.PRO_RMSNORM, gamma=dg, eps=1e-6, pos=ctx.upload(np.array([6], np.int32)),
                 slot=ctx.upload(np.array([4], np.int32)), seq_len=rows, ring_slots=slots_ring, ring_stride=n)
    got = ring2.read(np.float32, n_slots * slots_ring * n).reshape(n_slots, slots_ring, n)
    for t in range(rows):
        assert O.rel_l2(got[4, (6 + t) % slots_ring], want[t]) <= 1e-3, t
    assert np.count_nonzero(got.any(axis=2)) == rows


# The output projections' prologues through this kernel (the library's own context; the tests of these names in
# test_gemm_q4k_gpu.py run on a context that sends every pass to the tiled matrix-core kernels): five rows and more
# of 4096 columns spread a row over sixteen waves, two rows to a wave's lanes.
import test_gemm_q4k_gpu as G


@pytest.mark.parametrize("rows,slots", [(2, 8), (5, 8), (6, 8), (7, 8), (8, 8)])
def test_gated_norm_prologue_with_the_gate_from_the_ring(ctx, rows, slots):
    G.test_gated_norm_prologue_with_ring_gate_and_wide_rows(ctx, rows, slots)


@pytest.mark.parametrize("rows", [2, 5, 6, 7, 8])
def test_sigmoid_gate_prologue(ctx, rows):
    G.test_sigmoid_gate_prologue_with_fused_query_rows(ctx, rows)


@pytest.mark.parametrize("rows", [5, 7, 8])
def test_sixteen_waves_equal_four(ctx, rows):
    """2048 x 4096 with the RMSNorm in front and a residual behind: the block of sixteen waves against the block of
    four (SHV_MROWS_WAVES=4) to rounding, both against float64."""
    os.environ["SHV_MROWS_WAVES"] = "4"
    try:
        four = A.Context(0)
    finally:
        del os.environ["SHV_MROWS_WAVES"]
    try:
        rng = np.random.default_rng(900 + rows)
        n, k = 2048, 4096
        wq = _weights(rng, n, k)
        w64 = O.dequant_q4k(wq, k).astype(np.float64)
        gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
        x = (rng.standard_normal((rows, k)) * 3).astype(np.float32)
        res = rng.standard_normal((rows, n)).astype(np.float32)
        outs = []
        for c in (ctx, four):
            dy = c.upload(res)
            c.gemv_q4k(c.upload(wq), c.upload(x), dy, n, k, n_tok=rows, prologue=A.PRO_RMSNORM, gamma=c.upload(gamma), eps=1e-6, residual=dy)
            outs.append(dy.read(np.float32, rows * n).reshape(rows, n))
        x64 = x.astype(np.float64)
        want = (x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * gamma) @ w64.T + res
        for t in range(rows):
            assert O.rel_l2(outs[0][t], want[t]) <= 1e-5 and O.rel_l2(outs[1][t], want[t]) <= 1e-5, t
            assert O.rel_l2(outs[0][t], outs[1][t]) <= 3e-6, t
    finally:
        four.destroy()


@pytest.mark.parametrize("n_seq", [2, 3, 4, 5, 8])
def test_one_row_each_of_several_sequences(ctx, n_seq):
    """Several sequences' steps in one pass on the library's own context: two to four go through the side-by-side
    row kernel at 4096 columns (each row's gate from its own sequence's ring row) and this kernel at 2048, five and
    eight through the wider blocks."""
    G.test_one_row_each_of_several_sequences(ctx, n_seq)
