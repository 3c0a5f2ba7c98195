"""Q4_K projections of several rows run on the matrix cores (gemm_q4k.hip); these tests hold
that kernel to the oracle's GEMV row by row (matvec over dequantised rows, llm/hc.go:255-264), to a
float64 product, and to the one-row kernel it replaces, over the shapes, prologues and output
layouts the token loop uses (verification passes, batched decode rows, prompt chunks)."""
import os

import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu
A = shv.api
TOL = 1e-3      # the bar against the oracle (its own sequential float32 sums are ~1e-6 off)
TOL64 = 1e-5    # against float64: the activations go in as two halves, the products are exact


def _weights(rng, n, k, std=0.02):
    return O.quantize_q4k((rng.standard_normal((n, k)) * std).astype(np.float32))


@pytest.fixture(scope="module")
def ctx():
    """A context that sends every pass of two rows and more to the matrix-core kernel (the
    library's own threshold is tuned to where that kernel starts to win)."""
    os.environ["SHV_MFMA_MIN_ROWS"] = "2"
    try:
        c = A.Context(0)
    finally:
        del os.environ["SHV_MFMA_MIN_ROWS"]
    yield c
    c.destroy()


@pytest.fixture(scope="module")
def row_ctx():
    """A second context that keeps every pass on the row kernel, to compare the two."""
    os.environ["SHV_MFMA_MIN_ROWS"] = "1000"
    try:
        c = A.Context(0)
    finally:
        del os.environ["SHV_MFMA_MIN_ROWS"]
    yield c
    c.destroy()


@pytest.mark.parametrize("n,k,rows", [(1024, 2048, 2), (4096, 2048, 3), (2048, 4096, 4), (2048, 512, 16),
                                      (48, 1024, 5), (7, 2048, 2), (33, 256, 9), (12352, 2048, 16),
                                      (2048, 4096, 17), (512, 2048, 40),
                                      # passes of more rows than a block keeps in LDS stream their operands:
                                      # whole and ragged groups of 64, split columns, rows not a multiple of 128
                                      (12352, 2048, 64), (2048, 4096, 64), (9216, 2048, 33), (1000, 1024, 50),
                                      (512, 2048, 57), (2048, 4096, 9), (40, 256, 20),
                                      # 5..16 rows of the decode step's widths (8 where rows are 4096 wide): sixteen waves
                                      # a block, the rows staged under the weight loads; ragged tiles, one to three rounds
                                      (4096, 2048, 5), (12352, 2048, 8), (1000, 2048, 7), (7, 2048, 6), (2048, 2048, 13),
                                      (2048, 4096, 8), (2048, 4096, 5), (33, 4096, 6), (9216, 2048, 16), (70000, 2048, 8)])
def test_rows_match_oracle_and_float64(ctx, row_ctx, n, k, rows):
    rng = np.random.default_rng(n + k + rows)
    wq = _weights(rng, n, k)
    x = (rng.standard_normal((rows, k)) * rng.uniform(0.01, 30.0, size=(rows, 1))).astype(np.float32)
    w64 = O.dequant_q4k(wq, k).astype(np.float64)
    dy = ctx.alloc(rows * n * 4)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(x), dy, n, k, n_tok=rows)
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    ref = None
    if k >= 512:  # the row kernel's narrowest matrix
        dy2 = row_ctx.alloc(rows * n * 4)
        row_ctx.gemv_q4k(row_ctx.upload(wq), row_ctx.upload(x), dy2, n, k, n_tok=rows)
        ref = dy2.read(np.float32, rows * n).reshape(rows, n)
    worst = 0.0
    for t in range(rows):
        assert O.rel_l2(got[t], O.gemv_q4k(wq, x[t], n, k, threads=8)) <= TOL, t
        e64 = O.rel_l2(got[t], w64 @ x[t].astype(np.float64))
        worst = max(worst, e64)
        assert e64 <= TOL64, (t, e64)
        assert ref is None or O.rel_l2(got[t], ref[t]) <= TOL64, t
    print(f"gemm {n}x{k} x{rows}: worst rel-L2 vs float64 {worst:.2e}")


@pytest.mark.parametrize("n,k,rows", [(1000, 256, 256), (513, 512, 300), (2048, 1024, 193), (12352, 2048, 257),
                                      (2048, 4096, 320), (2048, 2048, 2048)])
def test_long_pass_matches_float64_and_oracle(ctx, n, k, rows):
    """A pass of four groups of 64 rows and more goes to the kernel that walks every group in one
    launch and takes Q4_K's min term on the matrix cores as well; here whole and ragged groups, every
    width of a super-block count that kernel has a case for, and columns not a multiple of 128.  Every
    row is held to a float64 product; the oracle's GEMV (llm/hc.go:255-264) takes a sample of rows, the
    first and last of each group among them."""
    rng = np.random.default_rng(n + k + rows)
    wq = _weights(rng, n, k)
    x = (rng.standard_normal((rows, k)) * rng.uniform(0.01, 30.0, size=(rows, 1))).astype(np.float32)
    w64 = O.dequant_q4k(wq, k).astype(np.float64)
    dy = ctx.alloc(rows * n * 4)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(x), dy, n, k, n_tok=rows)
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    want = x.astype(np.float64) @ w64.T
    err = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
    assert err.max() <= TOL64, (int(err.argmax()), float(err.max()))
    sample = sorted({t for g in range(0, rows, 64) for t in (g, min(g + 63, rows - 1))} | {rows // 2})[:24]
    for t in sample:
        assert O.rel_l2(got[t], O.gemv_q4k(wq, x[t], n, k, threads=8)) <= TOL, t
    print(f"gemm {n}x{k} x{rows}: worst rel-L2 vs float64 {err.max():.2e}")


@pytest.mark.parametrize("rows", [256, 333])
def test_long_pass_rmsnorm_prologue_residual_in_place(ctx, rows):
    """The long pass with the norm folded in and the residual stream updated in place (the MoE block's
    shared expert and the output projections of a prompt chunk run this way)."""
    rng = np.random.default_rng(310 + rows)
    n, k, eps = 2048, 2048, 1e-6
    wq = _weights(rng, n, k)
    h = (rng.standard_normal((rows, k)) * 3).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    res = rng.standard_normal((rows, n)).astype(np.float32)
    dy = ctx.upload(res)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(h), dy, n, k, n_tok=rows, prologue=A.PRO_RMSNORM,
                 gamma=ctx.upload(gamma), residual=dy, eps=eps)
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    for t in list(range(0, rows, 17)) + [rows - 1]:
        want = O.gemv_q4k(wq, O.rmsnorm(h[t], gamma, eps), n, k, threads=8) + res[t]
        assert O.rel_l2(got[t], want) <= TOL, t


@pytest.mark.parametrize("rows", [3, 6, 8, 11, 64])
def test_rmsnorm_prologue_residual_in_place(ctx, rows):
    """The residual stream's own rows are the residual and the destination (dn.out, attn.out, the
    MoE down projection write x in place)."""
    rng = np.random.default_rng(31)
    n, k, eps = 2048, 2048, 1e-6
    wq = _weights(rng, n, k)
    h = (rng.standard_normal((rows, k)) * 3).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    res = rng.standard_normal((rows, n)).astype(np.float32)
    dy = ctx.upload(res)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(h), dy, n, k, n_tok=rows, prologue=A.PRO_RMSNORM,
                 gamma=ctx.upload(gamma), residual=dy, eps=eps)
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    for t in range(rows):
        want = O.gemv_q4k(wq, O.rmsnorm(h[t], gamma, eps), n, k, threads=8) + res[t]
        assert O.rel_l2(got[t], want) <= TOL, t


@pytest.mark.parametrize("rows,slots", [(4, 8), (5, 8), (8, 8), (37, 64), (260, 512)])
def test_gated_norm_prologue_with_ring_gate_and_wide_rows(ctx, rows, slots):
    """DeltaNet's output projection at its real shape: 4096 columns (two column ranges), per-head
    norm, the gate z read from the projection ring at each row's position, residual in place."""
    rng = np.random.default_rng(32)
    n, k, d, eps = 2048, 4096, 128, 1e-6
    ring_stride, z_col = 12352, 8192
    wq = _weights(rng, n, k)
    o = rng.standard_normal((rows, k)).astype(np.float32)
    ring = rng.standard_normal((2, slots, ring_stride)).astype(np.float32)   # two sequence slots
    gamma = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    res = rng.standard_normal((rows, n)).astype(np.float32)
    pos, slot = 13, 1
    L = O.lib()
    dring, dy = ctx.upload(ring), ctx.upload(res)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(o), dy, n, k, n_tok=rows, prologue=A.PRO_GATED_NORM,
                 gamma=ctx.upload(gamma), z=dring.at(z_col * 4), head_dim=d, eps=eps, residual=dy,
                 pos=ctx.upload(np.array([pos], np.int32)), slot=ctx.upload(np.array([slot], np.int32)),
                 seq_len=rows, ring_slots=slots, ring_stride=ring_stride, z_ring=1)
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    for t in (range(rows) if rows <= 64 else list(range(0, rows, 13)) + [rows - 1]):
        z = ring[slot, (pos + t) % slots, z_col:z_col + k]
        xn = O.rmsnorm(o[t].reshape(-1, d), gamma, eps).ravel()
        sig = np.array([L.shv_ref_sigmoid(float(v)) for v in z], dtype=np.float32)
        want = O.gemv_q4k(wq, (xn * sig).astype(np.float32), n, k, threads=8) + res[t]
        assert O.rel_l2(got[t], want) <= TOL, t


@pytest.mark.parametrize("rows", [3, 7, 8, 64])
def test_sigmoid_gate_prologue_with_fused_query_rows(ctx, rows):
    """Attention's output projection: x * sigmoid(gate), the gate being the second half of each
    head's [q | gate] rows in the fused projection (llm/attn.go:162-166,198-205)."""
    rng = np.random.default_rng(33)
    n, k, d = 2048, 4096, 256
    heads, zw = k // d, 2 * k + 1024
    wq = _weights(rng, n, k)
    c = rng.standard_normal((rows, k)).astype(np.float32)
    qkv = rng.standard_normal((rows, zw)).astype(np.float32)
    L = O.lib()
    dy = ctx.alloc(rows * n * 4)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(c), dy, n, k, n_tok=rows, prologue=A.PRO_MUL_SIGMOID,
                 z=ctx.upload(qkv), head_dim=d, z_stride=zw)
    got = dy.read(np.float32, rows * n).reshape(rows, n)
    for t in range(rows):
        gate = np.concatenate([qkv[t, h * 2 * d + d:(h + 1) * 2 * d] for h in range(heads)])
        sig = np.array([L.shv_ref_sigmoid(float(v)) for v in gate], dtype=np.float32)
        want = O.gemv_q4k(wq, (c[t] * sig).astype(np.float32), n, k, threads=8)
        assert O.rel_l2(got[t], want) <= TOL, t


@pytest.mark.parametrize("seq_len,slots", [(3, 8), (20, 32)])
def test_ring_output_for_sequences_and_slots(ctx, seq_len, slots):
    """The DeltaNet input projection writes each row into its sequence's ring at its position:
    here two sequences of three rows each, on slots 2 and 0, wrapping around an 8-row ring."""
    rng = np.random.default_rng(34)
    n, k, n_slots = 528, 2048, 3
    wq = _weights(rng, n, k)
    x = rng.standard_normal((2 * seq_len, k)).astype(np.float32)
    pos, slot = np.array([6, 17], np.int32), np.array([2, 0], np.int32)
    ring = ctx.upload(np.full(n_slots * slots * n, -7.0, dtype=np.float32))
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(x), ring, n, k, n_tok=2 * seq_len, pos=ctx.upload(pos),
                 slot=ctx.upload(slot), seq_len=seq_len, ring_slots=slots, ring_stride=n)
    got = ring.read(np.float32, n_slots * slots * n).reshape(n_slots, slots, n)
    written = np.zeros((n_slots, slots), bool)
    for s in range(2):
        for i in range(seq_len):
            row = got[slot[s], (pos[s] + i) % slots]
            assert O.rel_l2(row, O.gemv_q4k(wq, x[s * seq_len + i], n, k, threads=8)) <= TOL, (s, i)
            written[slot[s], (pos[s] + i) % slots] = True
    assert (got[~written] == -7.0).all()


@pytest.mark.parametrize("n_seq", [5, 8, 12])
def test_one_row_each_of_several_sequences(ctx, n_seq):
    """Several sequences decoded together: a row each, every sequence at its own position on its own slot.  The DeltaNet
    input projection (norm folded in) writes each row into its sequence's ring; the output projection takes each row's
    gate from that ring at the sequence's position, norms per head and adds the residual in place."""
    rng = np.random.default_rng(35 + n_seq)
    H, W, d, eps, slots, n_slots = 2048, 12352, 128, 1e-6, 8, 13
    z_col, k2 = 8192, 4096
    w_in, w_out = _weights(rng, W, H), _weights(rng, H, k2)
    x = (rng.standard_normal((n_seq, H)) * 2).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    pos = rng.integers(0, 40, size=n_seq).astype(np.int32)
    slot = rng.permutation(n_slots)[:n_seq].astype(np.int32)
    ring0 = rng.standard_normal((n_slots, slots, W)).astype(np.float32)
    dring = ctx.upload(ring0)
    dpos, dslot = ctx.upload(pos), ctx.upload(slot)
    ctx.gemv_q4k(ctx.upload(w_in), ctx.upload(x), dring, W, H, n_tok=n_seq, prologue=A.PRO_RMSNORM, gamma=ctx.upload(gamma),
                 eps=eps, pos=dpos, slot=dslot, seq_len=1, ring_slots=slots, ring_stride=W)
    ring = dring.read(np.float32, ring0.size).reshape(ring0.shape)
    written = np.zeros((n_slots, slots), bool)
    for s in range(n_seq):
        want = O.gemv_q4k(w_in, O.rmsnorm(x[s], gamma, eps), W, H, threads=8)
        assert O.rel_l2(ring[slot[s], pos[s] % slots], want) <= TOL, s
        written[slot[s], pos[s] % slots] = True
    assert (ring[~written] == ring0[~written]).all()
    o = rng.standard_normal((n_seq, k2)).astype(np.float32)
    g2 = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    res = rng.standard_normal((n_seq, H)).astype(np.float32)
    dy = ctx.upload(res)
    ctx.gemv_q4k(ctx.upload(w_out), ctx.upload(o), dy, H, k2, n_tok=n_seq, prologue=A.PRO_GATED_NORM, gamma=ctx.upload(g2),
                 z=dring.at(z_col * 4), head_dim=d, eps=eps, residual=dy, pos=dpos, slot=dslot, seq_len=1, ring_slots=slots,
                 ring_stride=W, z_ring=1)
    got = dy.read(np.float32, n_seq * H).reshape(n_seq, H)
    L = O.lib()
    for s in range(n_seq):
        z = ring[slot[s], pos[s] % slots, z_col:z_col + k2]
        xn = O.rmsnorm(o[s].reshape(-1, d), g2, eps).ravel()
        sig = np.array([L.shv_ref_sigmoid(float(v)) for v in z], dtype=np.float32)
        want = O.gemv_q4k(w_out, (xn * sig).astype(np.float32), H, k2, threads=8) + res[s]
        assert O.rel_l2(got[s], want) <= TOL, s
