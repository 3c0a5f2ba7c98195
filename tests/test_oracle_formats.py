"""Pins the oracle's format layer against the vectors the reference's own tests hold:
fp16 conversion (safetensors/safetensors_test.go:20-61), Q4_K dequantisation
(gguf/dequant_test.go:40-92) and the Q4_K quantiser (llm/quantref_test.go:106-174)."""
import os
import struct

import numpy as np
import pytest

import oracle_lib as O


def test_f32_to_f16_golden_table(golden_dir):
    L = O.lib()
    n = bad = 0
    for line in open(os.path.join(golden_dir, "f32_to_f16.txt")):
        line = line.strip()
        if not line or line.startswith("#"):
            continue
        a, b = line.split()
        f = struct.unpack("<f", struct.pack("<I", int(a, 16)))[0]
        got = L.shv_ref_f32_to_f16(f)
        bad += got != int(b, 16)
        n += 1
    assert n >= 10000, n
    assert bad == 0, f"{bad} of {n} golden pairs wrong"


def test_f16_all_halves_against_numpy():
    """Independent routine: numpy's float16 is IEEE binary16.  Widening must be exact for all
    65 536 patterns, and narrowing the widened value must return the pattern (NaNs quieted)."""
    L = O.lib()
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([L.shv_ref_f16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all()
    back = np.array([L.shv_ref_f32_to_f16(float(v)) for v in want[~nan]], dtype=np.uint16)
    assert np.array_equal(back, h[~nan])


def test_f16_round_matches_numpy_on_random_floats():
    L = O.lib()
    rng = np.random.default_rng(11)
    bits = rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[np.isfinite(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).astype(np.float32)
    got = np.array([L.shv_ref_f16_round(float(v)) for v in x], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    narrow = np.array([L.shv_ref_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    with np.errstate(over="ignore"):
        assert np.array_equal(narrow, x.astype(np.float16).view(np.uint16))


def _dequant_record(path):
    b = open(path, "rb").read()
    typ, n, nbytes = struct.unpack_from("<IIQ", b, 0)
    return typ, n, b[16:16 + nbytes]


def _records(path):
    b = open(path, "rb").read()
    o, out = 0, []
    while o < len(b):
        typ, n, nbytes = struct.unpack_from("<IIQ", b, o)
        out.append((typ, n, b[o + 16:o + 16 + nbytes]))
        o += 16 + nbytes
    return out


def test_every_tensor_type_matches_ggml_bit_for_bit(golden_dir):
    """All eleven types the reference's loader accepts (gguf/dequant.go:103-110), each against
    ggml's own to_float of the same bytes (gguf/dequant_test.go:40-92)."""
    ins = _records(os.path.join(golden_dir, "dequant_in.bin"))
    refs = _records(os.path.join(golden_dir, "dequant_ref.bin"))
    assert len(ins) == len(refs) == 11
    assert {t for t, _, _ in ins} == set(O.GGML_TYPES.values())
    for (typ, n, payload), (rtyp, rn, rpayload) in zip(ins, refs):
        assert (typ, n) == (rtyp, rn) and len(payload) == O.type_bytes(typ, n)
        got = O.dequant(typ, np.frombuffer(payload, dtype=np.uint8), n)
        want = np.frombuffer(rpayload, dtype=np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), typ


def test_dequant_refuses_what_the_loader_refuses():
    assert O.type_bytes(2, 32) == -1        # Q4_0 is not among the loader's types
    assert O.type_bytes(12, 100) == -1      # not whole super-blocks
    with pytest.raises((ValueError, AssertionError)):
        O.dequant(12, np.zeros(10, np.uint8), 100)


def test_dequant_q4k_matches_ggml_bit_for_bit(golden_dir):
    typ, n, payload = _dequant_record(os.path.join(golden_dir, "dequant_q4k_in.bin"))
    rtyp, rn, rpayload = _dequant_record(os.path.join(golden_dir, "dequant_q4k_ref.bin"))
    assert typ == rtyp == 12 and n == rn == 1024 and len(payload) == 576
    want = np.frombuffer(rpayload, dtype=np.float32)
    got = O.dequant_q4k(np.frombuffer(payload, dtype=np.uint8))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _unpack_scale_min(packed, j):
    L = O.lib()
    sc, m = O.C.c_uint8(), O.C.c_uint8()
    L.shv_ref_scale_min_k4(j, O.B(packed), O.C.byref(sc), O.C.byref(m))
    return sc.value, m.value


def test_scale_min_k4_is_the_inverse_of_the_packing():
    """llm/bank_q4_test.go:130-155: pack then unpack over every 6-bit value in every place.
    The packing is written here from ggml's published layout (low 6 bits of bytes 0..7 for the
    first four pairs; low nibbles in bytes 8..11 and the top two bits in the spare bits of
    bytes 0..7 for the last four)."""
    rng = np.random.default_rng(5)
    for trial in range(200):
        ls = rng.integers(0, 64, size=8)
        lm = rng.integers(0, 64, size=8)
        if trial < 64:
            ls[:] = trial
            lm[:] = 63 - trial
        p = np.zeros(12, dtype=np.uint8)
        for j in range(4):
            p[j] = ls[j] | ((ls[j + 4] >> 4) << 6)
            p[j + 4] = lm[j] | ((lm[j + 4] >> 4) << 6)
            p[j + 8] = (ls[j + 4] & 0xF) | ((lm[j + 4] & 0xF) << 4)
        for j in range(8):
            assert _unpack_scale_min(p, j) == (ls[j], lm[j])


def _quant_records(path):
    b = open(path, "rb").read()
    o, recs = 0, []
    while o < len(b):
        typ, rows, k, im = struct.unpack_from("<IIII", b, o)
        o += 16
        x = np.frombuffer(b, dtype=np.float32, count=rows * k, offset=o).reshape(rows, k)
        o += rows * k * 4
        recs.append((typ, rows, k, im, x))
    return recs


def test_quantiser_matches_ggml_quantize_chunk(golden_dir):
    """quantise with the oracle, dequantise with the oracle, compare with ggml's
    quantize_chunk -> to_float of the same real weight rows.  The reference demands equal
    halves and reports float32-exact counts (llm/quantref_test.go:146-174); both are demanded
    here, since dequant is pinned bit-exact and the quantiser keeps ggml's float32 widths."""
    ins = _quant_records(os.path.join(golden_dir, "quant_q4k_in.bin"))
    refs = _quant_records(os.path.join(golden_dir, "quant_q4k_ref.bin"))
    assert len(ins) == len(refs) == 2
    for (typ, rows, k, im, x), (_, rrows, rk, _, want) in zip(ins, refs):
        assert typ == 12 and im == 0 and (rows, k) == (rrows, rk)
        q = O.quantize_q4k(x)
        got = O.dequant_q4k(q, k)
        same = got.view(np.uint32) == want.view(np.uint32)
        assert same.all(), f"k={k}: {np.count_nonzero(~same)} of {same.size} values differ"


def test_quantiser_invariants():
    """What the format fixes regardless of any vector: levels in [0,15], 6-bit scales, d and
    dmin exact halves, and a round trip within one level of the group's step."""
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((8, 1024)) * 0.02).astype(np.float32)
    q = O.quantize_q4k(w)
    back = O.dequant_q4k(q, 1024)
    blocks = q.reshape(-1, 144)
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).ravel()
    assert np.isfinite(d).all() and (d >= 0).all()
    for bi, blk in enumerate(blocks):
        for j in range(8):
            sc, m = _unpack_scale_min(np.ascontiguousarray(blk[4:16]), j)
            assert 0 <= sc <= 63 and 0 <= m <= 63
            step = d[bi] * sc
            g = slice(bi * 256 + j * 32, bi * 256 + (j + 1) * 32)
            err = np.abs(back.ravel()[g] - w.ravel()[g]).max()
            assert err <= step * 1.01 + 1e-7, (bi, j, err, step)
    # all-zero and constant groups (the `if (!d) continue` arm, llm/quantk.go:158-166)
    z = np.zeros((1, 256), dtype=np.float32)
    assert np.array_equal(O.dequant_q4k(O.quantize_q4k(z)), z.ravel())
    c = np.full((1, 256), 0.5, dtype=np.float32)
    assert np.allclose(O.dequant_q4k(O.quantize_q4k(c)), 0.5, atol=0.5 / 15)
