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


@pytest.mark.parametrize("name", sorted(O.GGML_TYPES))
def test_random_blocks_match_the_cpu(ctx, name):
    """Random bytes with finite half scales: every bit pattern of levels, fifth/sixth-bit planes and
    packed scales, 64 Ki elements a type."""
    typ, n = O.GGML_TYPES[name], 65536
    rng = np.random.default_rng(typ)
    nbytes = O.type_bytes(typ, n)
    raw = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
    if name in ("F32", "F16", "BF16"):
        width = {"F32": 4, "F16": 2, "BF16": 2}[name]
        vals = rng.standard_normal(n).astype(np.float32)
        raw = {"F32": vals.view(np.uint8), "F16": vals.astype(np.float16).view(np.uint8),
               "BF16": (vals.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)}[name].copy()
        assert raw.size == n * width
    else:
        # put finite halves where the formats keep their scales
        blk = {"Q8_0": (34, [0]), "Q4_1": (20, [0, 2]), "Q5_0": (22, [0]), "Q5_1": (24, [0, 2]), "IQ4_NL": (18, [0]),
               "Q4_K": (144, [0, 2]), "Q5_K": (176, [0, 2]), "Q6_K": (210, [208])}[name]
        rows = raw.reshape(-1, blk[0])
        for off in blk[1]:
            h = (rng.standard_normal(rows.shape[0]) * 0.05).astype(np.float16).view(np.uint16)
            rows[:, off] = h & 0xFF
            rows[:, off + 1] = h >> 8
    want = O.dequant(typ, raw, n)
    got = _device(ctx, typ, raw.tobytes(), n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_refusals(ctx):
    src, dst = ctx.alloc(1024), ctx.alloc(4096)
    with pytest.raises(shv.api.ShvError):
        ctx.dequant(2, src, dst, 32)      # Q4_0: not a type the loader accepts
    with pytest.raises(shv.api.ShvError):
        ctx.dequant(12, src, dst, 100)    # not whole super-blocks
