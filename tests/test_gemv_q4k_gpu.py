"""Q4_K GEMV on the GPU against the oracle (matvec over dequantised rows, llm/hc.go:255-264,
gguf/dequant.go:252-276), plus the bit-exact format kernels (dequantise, quantise)."""
import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu
A = shv.api
TOL = 1e-3  # relative L2, the bar for fp32-accumulated outputs; typical result is ~1e-6


def _weights(rng, n, k, std=0.02):
    return O.quantize_q4k((rng.standard_normal((n, k)) * std).astype(np.float32))


@pytest.mark.parametrize("n,k", [(4096, 2048), (2048, 4096), (2048, 512), (1024, 1024), (64, 2048),
                                 (12352, 2048), (7, 2048), (33, 512)])
def test_gemv_matches_oracle(ctx, n, k):
    rng = np.random.default_rng(1000 + n + k)
    wq = _weights(rng, n, k)
    x = rng.standard_normal(k).astype(np.float32)
    want = O.gemv_q4k(wq, x, n, k, threads=8)
    dw, dx, dy = ctx.upload(wq), ctx.upload(x), ctx.alloc(n * 4)
    ctx.gemv_q4k(dw, dx, dy, n, k)
    got = dy.read(np.float32, n)
    err = O.rel_l2(got, want)
    print(f"gemv {n}x{k}: rel-L2 {err:.3e}")
    assert err <= TOL
    # float64 cross-check of both: the oracle's sequential float32 sum is itself ~1e-6 off
    w64 = O.dequant_q4k(wq, k).astype(np.float64)
    assert O.rel_l2(got, w64 @ x.astype(np.float64)) <= 1e-5


def test_config1_exact_shape_and_seeded_inputs(ctx):
    """W 4096x2048 ~ N(0,0.02) quantised by the reference's quantiser, x ~ N(0,1)."""
    rng = np.random.default_rng(20260101)
    n, k = 4096, 2048
    wq = _weights(rng, n, k)
    assert wq.nbytes == 4718592
    x = rng.standard_normal(k).astype(np.float32)
    dw, dx, dy = ctx.upload(wq), ctx.upload(x), ctx.alloc(n * 4)
    ctx.gemv_q4k(dw, dx, dy, n, k)
    got = dy.read(np.float32, n)
    assert O.rel_l2(got, O.gemv_q4k(wq, x, n, k, threads=8)) <= TOL
    # linearity, a size-independent property: W(a*x1 + x2) = a*W x1 + W x2
    x2 = rng.standard_normal(k).astype(np.float32)
    dx2, dy2, dy3 = ctx.upload(x2), ctx.alloc(n * 4), ctx.alloc(n * 4)
    ctx.gemv_q4k(dw, dx2, dy2, n, k)
    ctx.gemv_q4k(dw, ctx.upload((0.5 * x + x2).astype(np.float32)), dy3, n, k)
    lin = 0.5 * got + dy2.read(np.float32, n)
    assert O.rel_l2(dy3.read(np.float32, n), lin) <= 1e-5


@pytest.mark.parametrize("n_tok", [2, 3, 4, 8, 13])
def test_gemv_rows_share_one_weight_pass(ctx, n_tok):
    rng = np.random.default_rng(7 + n_tok)
    n, k = 1024, 2048
    wq = _weights(rng, n, k)
    x = rng.standard_normal((n_tok, k)).astype(np.float32)
    dw, dx, dy = ctx.upload(wq), ctx.upload(x), ctx.alloc(n_tok * n * 4)
    ctx.gemv_q4k(dw, dx, dy, n, k, n_tok=n_tok)
    got = dy.read(np.float32, n_tok * n).reshape(n_tok, n)
    for t in range(n_tok):
        assert O.rel_l2(got[t], O.gemv_q4k(wq, x[t], n, k, threads=8)) <= TOL


def test_gemv_rmsnorm_prologue_and_residual(ctx):
    rng = np.random.default_rng(5)
    n, k, eps = 2048, 2048, 1e-6
    wq = _weights(rng, n, k)
    h = rng.standard_normal(k).astype(np.float32) * 3
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    res = rng.standard_normal(n).astype(np.float32)
    want = O.gemv_q4k(wq, O.rmsnorm(h, gamma, eps), n, k, threads=8) + res
    dy = ctx.alloc(n * 4)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(h), dy, n, k, prologue=A.PRO_RMSNORM,
                 gamma=ctx.upload(gamma), residual=ctx.upload(res), eps=eps)
    assert O.rel_l2(dy.read(np.float32, n), want) <= TOL


def test_gemv_gated_norm_prologue(ctx):
    """DeltaNet's output norm (llm/deltanet.go:329-341) applied while staging x."""
    rng = np.random.default_rng(6)
    n, k, d, eps = 2048, 4096, 128, 1e-6
    wq = _weights(rng, n, k)
    o = rng.standard_normal(k).astype(np.float32)
    z = rng.standard_normal(k).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    L = O.lib()
    xn = O.rmsnorm(o.reshape(-1, d), gamma, eps).ravel()
    sig = np.array([L.shv_ref_sigmoid(float(v)) for v in z], dtype=np.float32)
    want = O.gemv_q4k(wq, (xn * sig).astype(np.float32), n, k, threads=8)
    dy = ctx.alloc(n * 4)
    ctx.gemv_q4k(ctx.upload(wq), ctx.upload(o), dy, n, k, prologue=A.PRO_GATED_NORM,
                 gamma=ctx.upload(gamma), z=ctx.upload(z), head_dim=d, eps=eps)
    assert O.rel_l2(dy.read(np.float32, n), want) <= TOL


def test_gemv_ring_output(ctx):
    rng = np.random.default_rng(8)
    n, k, slots = 512, 2048, 4
    wq = _weights(rng, n, k)
    x = rng.standard_normal(k).astype(np.float32)
    want = O.gemv_q4k(wq, x, n, k, threads=8)
    dw, dx = ctx.upload(wq), ctx.upload(x)
    for p in (0, 1, 6, 11):
        ring = ctx.upload(np.full(slots * n, -7.0, dtype=np.float32))
        ctx.gemv_q4k(dw, dx, ring, n, k, pos=ctx.upload(np.array([p], dtype=np.int32)),
                     ring_slots=slots, ring_stride=n)
        got = ring.read(np.float32, slots * n).reshape(slots, n)
        assert O.rel_l2(got[p % slots], want) <= TOL
        assert (np.delete(got, p % slots, axis=0) == -7.0).all()


def test_gemv_refuses_shapes_it_does_not_cover(ctx):
    d = ctx.alloc(1 << 20)
    with pytest.raises(shv.pkg.ShvError):
        ctx.gemv_q4k(d, d, d, 16, 768)
    with pytest.raises(shv.pkg.ShvError):
        ctx.gemv_q4k(d, d, d, 16, 2048, n_tok=4097)   # a pass carries up to 4096 rows
    with pytest.raises(shv.pkg.ShvError):
        ctx.gemv_q4k(d.at(4), d, d, 16, 2048)


def test_dequant_is_bit_exact(ctx, golden_dir):
    import os
    import struct
    b = open(os.path.join(golden_dir, "dequant_q4k_in.bin"), "rb").read()
    r = open(os.path.join(golden_dir, "dequant_q4k_ref.bin"), "rb").read()
    payload = np.frombuffer(b[16:], dtype=np.uint8)
    want = np.frombuffer(r[16:], dtype=np.float32)
    a = A.DequantQ4KArgs(ctx.upload(payload).ptr, ctx.alloc(want.nbytes).ptr, 1, 1024)
    dst = a.dst
    ctx.enqueue(A.OP_DEQUANT_Q4K, a)
    ctx.sync()
    got = np.empty(1024, dtype=np.float32)
    shv.api.check(ctx.L.shv_download(ctx.h, got.ctypes.data, dst, got.nbytes))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and on a larger seeded matrix against the oracle
    rng = np.random.default_rng(9)
    wq = _weights(rng, 256, 2048)
    dd = ctx.alloc(256 * 2048 * 4)
    ctx.enqueue(A.OP_DEQUANT_Q4K, A.DequantQ4KArgs(ctx.upload(wq).ptr, dd.ptr, 256, 2048))
    got = dd.read(np.float32, 256 * 2048)
    assert np.array_equal(got.view(np.uint32), O.dequant_q4k(wq).view(np.uint32))


def test_quantiser_is_bit_exact(ctx, golden_dir):
    """The device quantiser must produce the reference quantiser's bytes: on the real weight
    rows the reference's fixture holds, and on seeded N(0, 0.02) including degenerate groups."""
    import os
    import struct
    rng = np.random.default_rng(10)
    cases = []
    b = open(os.path.join(golden_dir, "quant_q4k_in.bin"), "rb").read()
    typ, rows, k, im = struct.unpack_from("<IIII", b, 0)
    cases.append(np.frombuffer(b, dtype=np.float32, count=rows * k, offset=16).reshape(rows, k))
    w = (rng.standard_normal((64, 2048)) * 0.02).astype(np.float32)
    w[3, :256] = 0          # an all-zero super-block
    w[4, 32:64] = 0.01      # a constant group
    w[5, :32] = np.abs(w[5, :32])  # an all-positive group (min clamps to 0)
    w[6] *= 1e-6            # halves that land in the subnormal range
    cases.append(w)
    for x in cases:
        rows, k = x.shape
        want = O.quantize_q4k(x)
        dq = ctx.alloc(want.nbytes)
        ctx.enqueue(A.OP_QUANTIZE_Q4K, A.QuantizeQ4KArgs(ctx.upload(x).ptr, dq.ptr, rows, k))
        got = dq.read(np.uint8, want.size).reshape(want.shape)
        bad = np.argwhere(got != want)
        assert bad.size == 0, f"{len(bad)} bytes differ, first at {bad[0]}"


def test_fill_normal_statistics(ctx):
    n = 1 << 22
    d = ctx.alloc(n * 4)
    ctx.enqueue(A.OP_FILL_NORMAL, A.FillNormalArgs(d.ptr, n, 1234, 0.0, 0.02))
    v = d.read(np.float32, n)
    assert abs(v.mean()) < 1e-4 and abs(v.std() - 0.02) < 2e-4
    assert np.isfinite(v).all() and np.abs(v).max() < 0.02 * 7
    d2 = ctx.alloc(n * 4)
    ctx.enqueue(A.OP_FILL_NORMAL, A.FillNormalArgs(d2.ptr, n, 1234, 0.0, 0.02))
    assert np.array_equal(v, d2.read(np.float32, n))


def test_prerecorded_sequence_replays(ctx):
    """vk.Prerecorded's contract (vk/engine.go:997-1086): record once, replay, same answer;
    replays interleaved with eager work and synchronisation."""
    rng = np.random.default_rng(12)
    n, k = 2048, 2048
    wq = _weights(rng, n, k)
    x = rng.standard_normal(k).astype(np.float32)
    dw, dx, dy, dy2 = ctx.upload(wq), ctx.upload(x), ctx.alloc(n * 4), ctx.alloc(n * 4)
    ops = [A.make_op(A.OP_GEMV_Q4K, A.gemv_args(dw, dx, dy, n, k)),
           A.make_op(A.OP_GEMV_Q4K, A.gemv_args(dw, dy, dy2, n, k))]
    total, per = ctx.dispatch_multi(ops, per_op=True)
    assert total > 0 and len(per) == 2
    eager = dy2.read(np.float32, n)
    pre = ctx.prerecord(ops)
    assert pre.count() == 2
    for i in range(3):
        dy2.write(np.zeros(n, dtype=np.float32))
        ns = pre.submit()
        assert ns > 0
        assert np.array_equal(dy2.read(np.float32, n), eager)
        ctx.gemv_q4k(dw, dx, dy, n, k)
        ctx.sync()
    pre.destroy()
