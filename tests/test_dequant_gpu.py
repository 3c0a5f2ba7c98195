"""The device dequantiser for every tensor type the reference's loader accepts
(gguf/dequant.go:52-98,103-110), bit for bit against ggml's own vectors
(gguf/dequant_test.go:40-92) and against the CPU restatement on random blocks."""
import os
import struct

import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu


def _records(path):
    b = open(path, "rb").read()
    o, out = 0, []
    while o < len(b):
        typ, n, nbytes = struct.unpack_from("<IIQ", b, o)
        out.append((typ, n, b[o + 16:o + 16 + nbytes]))
        o += 16 + nbytes
    return out


def _device(ctx, typ, payload, n):
    dst = ctx.alloc(n * 4)
    ctx.dequant(typ, ctx.upload(np.frombuffer(payload, dtype=np.uint8).copy()), dst, n)
    return dst.read(np.float32, n)


def test_ggml_vectors_bit_for_bit(ctx, golden_dir):
    ins = _records(os.path.join(golden_dir, "dequant_in.bin"))
    refs = _records(os.path.join(golden_dir, "dequant_ref.bin"))
    for (typ, n, payload), (_, _, rpayload) in zip(ins, refs):
        got = _device(ctx, typ, payload, n)
        want = np.frombuffer(rpayload, dtype=np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), typ


def random_tensor(name, n, seed=None, scale=0.05):
    """`n` elements of tensor type `name`: random bytes with finite half scales (normal, sigma `scale`), so
    every bit pattern of levels, fifth/sixth-bit planes and packed scales occurs."""
    typ = O.GGML_TYPES[name]
    rng = np.random.default_rng(typ if seed is None else seed)
    raw = rng.integers(0, 256, size=O.type_bytes(typ, n), dtype=np.uint8)
    if name in ("F32", "F16", "BF16"):
        vals = rng.standard_normal(n).astype(np.float32)
        return {"F32": vals.view(np.uint8), "F16": vals.astype(np.float16).view(np.uint8),
                "BF16": (vals.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)}[name].copy()
    # put finite halves where the formats keep their scales
    blk = {"Q8_0": (34, [0]), "Q4_1": (20, [0, 2]), "Q5_0": (22, [0]), "Q5_1": (24, [0, 2]), "IQ4_NL": (18, [0]),
           "Q4_K": (144, [0, 2]), "Q5_K": (176, [0, 2]), "Q6_K": (210, [208])}[name]
    rows = raw.reshape(-1, blk[0])
    for off in blk[1]:
        h = (rng.standard_normal(rows.shape[0]) * scale).astype(np.float16).view(np.uint16)
        rows[:, off] = h & 0xFF
        rows[:, off + 1] = h >> 8
    return raw


@pytest.mark.parametrize("name", sorted(O.GGML_TYPES))
def test_random_blocks_match_the_cpu(ctx, name):
    typ, n = O.GGML_TYPES[name], 65536
    raw = random_tensor(name, n)
    want = O.dequant(typ, raw, n)
    got = _device(ctx, typ, raw.tobytes(), n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("k", [256, 2048, 4096])
@pytest.mark.parametrize("name", sorted(O.GGML_TYPES))
def test_gemv_of_every_type_matches_matvec_over_dequantised_rows(ctx, name, k):
    """y = W x as the CPU path forms it (llm/hc.go:255-264 over gguf/dequant.go:119-124): rows
    dequantised by the fixture-pinned restatement, dotted in float64.  fp32 accumulation, so 1e-5
    relative L2 (the path's bar is 1e-3); 37 rows leave the last block ragged."""
    typ, n = O.GGML_TYPES[name], 37
    raw = random_tensor(name, n * k, seed=1000 + typ + k)
    rng = np.random.default_rng(k)
    x = rng.standard_normal(k).astype(np.float32)
    res = rng.standard_normal(n).astype(np.float32)
    w = O.dequant(typ, raw, n * k).reshape(n, k).astype(np.float64)
    y = ctx.alloc(n * 4)
    ctx.gemv(typ, ctx.upload(raw), ctx.upload(x), y, n, k)
    assert O.rel_l2(y.read(np.float32, n), w @ x) <= 1e-5
    ctx.gemv(typ, ctx.upload(raw), ctx.upload(x), y, n, k, residual=ctx.upload(res))
    assert O.rel_l2(y.read(np.float32, n), w @ x + res) <= 1e-5


def test_gemv_at_vocabulary_height_agrees_with_the_q4k_kernel(ctx):
    """151936 x 2048 Q4_K through both kernels: same weights, same x, results equal to rounding."""
    n, k = 151936, 2048
    raw = random_tensor("Q4_K", n * k, seed=5)
    x = np.random.default_rng(6).standard_normal(k).astype(np.float32)
    w, xd, y0, y1 = ctx.upload(raw), ctx.upload(x), ctx.alloc(n * 4), ctx.alloc(n * 4)
    ctx.gemv(O.GGML_TYPES["Q4_K"], w, xd, y0, n, k)
    ctx.gemv_q4k(w, xd, y1, n, k)
    assert O.rel_l2(y0.read(np.float32, n), y1.read(np.float32, n)) <= 1e-5


def test_refusals(ctx):
    src, dst = ctx.alloc(1024), ctx.alloc(4096)
    with pytest.raises(shv.api.ShvError):
        ctx.dequant(2, src, dst, 32)      # Q4_0: not a type the loader accepts
    with pytest.raises(shv.api.ShvError):
        ctx.dequant(12, src, dst, 100)    # not whole super-blocks
    with pytest.raises(shv.api.ShvError):
        ctx.gemv(2, src, src, dst, 4, 32)     # Q4_0
    with pytest.raises(shv.api.ShvError):
        ctx.gemv(14, src, src, dst, 1, 128)   # Q6_K rows are whole super-blocks
    with pytest.raises(shv.api.ShvError):
        ctx.gemv(8, src, src, dst, 1, 32768)  # x would not fit its staging


@pytest.mark.parametrize("name", ["Q6_K", "Q8_0", "F16", "Q5_K"])
@pytest.mark.parametrize("rows", [1, 3, 6])
def test_gemv_rows_with_the_rmsnorm_prologue(ctx, name, rows):
    """The any-type GEMV as a vocabulary projection takes it: rows of a pass, the final RMSNorm as its prologue
    (llm/hc.go:176-190), strides wider than the rows, a residual in place; the weights read once per four rows."""
    typ, n, k, eps = O.GGML_TYPES[name], 200, 2048, 1e-6
    rng = np.random.default_rng(typ + rows)
    raw = random_tensor(name, n * k, seed=typ + 31)
    w = O.dequant(typ, raw, n * k).reshape(n, k).astype(np.float64)
    xs, ys = k + 64, n + 8
    x = np.zeros((rows, xs), np.float32)
    x[:, :k] = rng.standard_normal((rows, k)) * 3
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    res = np.zeros((rows, ys), np.float32)
    res[:, :n] = rng.standard_normal((rows, n))
    dy = ctx.upload(res)
    ctx.gemv(typ, ctx.upload(raw), ctx.upload(x), dy, n, k, residual=dy, n_tok=rows, gamma=ctx.upload(gamma), eps=eps, x_stride=xs, y_stride=ys)
    got = dy.read(np.float32, rows * ys).reshape(rows, ys)
    x64 = x[:, :k].astype(np.float64)
    xn = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * gamma
    want = xn @ w.T + res[:, :n]
    for t in range(rows):
        assert O.rel_l2(got[t, :n], want[t]) <= 1e-5, t
    assert np.all(got[:, n:] == 0)     # nothing written past a row's n outputs
