"""The GGUF container reader (host/gguf.hpp through its C entry points) on files written by the
tests' own writer: the cases of the reference's gguf/gguf_test.go — metadata of every width,
tensor spans and rows, block geometry, alignment, refused files, split checkpoints."""
import math
import os
import struct

import numpy as np
import pytest

import gguf_file as GF
import shv

G = shv.pkg.gguf_api
ShvError = shv.api.ShvError
T = G.TYPES


def _sample(w):
    w.put("general.architecture", GF.STR, "qwen4exp")
    w.put("qwen4exp.block_count", GF.U32, 48)
    w.put("small.u16", GF.U16, 65535)
    w.put("small.i32", GF.I32, -7)
    w.put("qwen4exp.attention.layer_norm_rms_epsilon", GF.F32, 1e-6)
    w.put("tokenizer.ggml.add_bos_token", GF.BOOL, 1)
    w.put_array("tokenizer.ggml.tokens", GF.STR, ["<s>", "hello", " world"])
    w.put_array("tokenizer.ggml.token_type", GF.I32, [3, 1, 1])
    w.tensor("token_embd.weight", T["Q8_0"], [2560, 64], 0x11)
    w.tensor("blk.0.attn_norm.weight", T["F32"], [2560], 0x22)
    w.tensor("blk.0.ffn_gate_exps.weight", T["Q4_K"], [2560, 4, 8], 0x33)


def test_open_reads_metadata_and_tensors(tmp_path):
    """gguf/gguf_test.go:142-234"""
    w = GF.Writer()
    _sample(w)
    with G.GGUF(w.write(tmp_path / "m.gguf"), single=True) as f:
        assert f.files()[0]["version"] == 3
        assert f.str("general.architecture") == "qwen4exp" and f.arch() == "qwen4exp"
        # every integer width answers to uint
        assert f.uint("qwen4exp.block_count") == 48 and f.uint("small.u16") == 65535
        assert f.int("small.i32") == -7 and f.uint("small.i32") is None   # a negative one is no uint
        assert f.int("small.u16") == 65535 and f.float("small.i32") == -7.0
        assert abs(f.float("qwen4exp.attention.layer_norm_rms_epsilon") - 1e-6) < 1e-12
        assert f.bool("tokenizer.ggml.add_bos_token") is True
        assert f.strings("tokenizer.ggml.tokens") == ["<s>", "hello", " world"]
        assert list(f.ints("tokenizer.ggml.token_type")) == [3, 1, 1]
        assert f.uints("tokenizer.ggml.token_type") is None and f.str("small.u16") is None
        assert f.uint("absent") is None and f.strings("absent") is None
        assert f.keys() == ["general.architecture", "qwen4exp.block_count", "small.u16", "small.i32",
                            "qwen4exp.attention.layer_norm_rms_epsilon", "tokenizer.ggml.add_bos_token",
                            "tokenizer.ggml.tokens", "tokenizer.ggml.token_type"]

        tn = f.get("token_embd.weight")
        assert tn.nbytes == 2560 * 64 // 32 * 34       # Q8_0: 32 elements in 34 bytes
        d = tn.data()
        assert d[0] == 0x11 and d[-1] == 0x11
        assert tn.rows == 64 and tn.row_bytes == 2560 // 32 * 34 and tn.elems() == 2560 * 64
        r = tn.row(63)
        assert len(r) == tn.row_bytes and r[0] == 0x11
        assert f.get("blk.0.attn_norm.weight").data()[0] == 0x22 and f.get("blk.0.attn_norm.weight").rows == 1

        # a 3-D expert bank: rows are the product of every axis but the first
        ex = f.get("blk.0.ffn_gate_exps.weight")
        assert ex.rows == 32 and ex.nbytes == 2560 * 4 * 8 // 256 * 144 and ex.dims == [2560, 4, 8]
        assert f.has("blk.0.attn_norm.weight") and not f.has("nope")
        with pytest.raises(KeyError):
            f.get("nope")
        assert len(f) == 3 and f.params() == 2560 * 64 + 2560 + 2560 * 32
        assert f.nbytes() == sum(t.nbytes for t in f.tensors())


def test_every_value_width_and_array_kind(tmp_path):
    """The value grammar (gguf/gguf.go:528-651): scalars widen, arrays keep one widened element type."""
    w = GF.Writer()
    for name, vt, v in [("u8", GF.U8, 200), ("i8", GF.I8, -100), ("i16", GF.I16, -30000), ("u64", GF.U64, 2 ** 63 + 5),
                        ("i64", GF.I64, -2 ** 62), ("f64", GF.F64, math.pi), ("no", GF.BOOL, 0), ("empty", GF.STR, "")]:
        w.put(name, vt, v)
    w.put_array("a.u8", GF.U8, [1, 2, 255])
    w.put_array("a.u64", GF.U64, [2 ** 64 - 1])
    w.put_array("a.i16", GF.I16, [-1, 7])
    w.put_array("a.f32", GF.F32, [0.5, -2.0])
    w.put_array("a.f64", GF.F64, [1e300])
    w.put_array("a.none", GF.U32, [])
    w.put("dup", GF.U32, 1)
    w.put("dup", GF.U32, 2)
    w.tensor("x", T["F16"], [4], 0)
    with G.GGUF(w.write(tmp_path / "v.gguf")) as f:
        assert f.uint("u8") == 200 and f.int("i8") == -100 and f.int("i16") == -30000
        assert f.uint("u64") == 2 ** 63 + 5 and f.int("i64") == -2 ** 62 and f.float("f64") == math.pi
        assert f.bool("no") is False and f.str("empty") == ""
        assert list(f.uints("a.u8")) == [1, 2, 255] and list(f.uints("a.u64")) == [2 ** 64 - 1]
        assert list(f.ints("a.i16")) == [-1, 7] and list(f.floats("a.f32")) == [0.5, -2.0] and list(f.floats("a.f64")) == [1e300]
        assert len(f.uints("a.none")) == 0
        assert f.uint("dup") == 2 and f.keys().count("dup") == 1      # a repeated key keeps its first place, last value


def test_type_block_geometry():
    """gguf/gguf_test.go:236-275"""
    for name, elems, nbytes in [("F32", 1, 4), ("F16", 1, 2), ("BF16", 1, 2), ("Q4_K", 256, 144), ("Q5_K", 256, 176),
                                ("Q5_1", 32, 24), ("Q8_0", 32, 34), ("IQ4_NL", 32, 18), ("Q6_K", 256, 210), ("MXFP4", 32, 17)]:
        assert G.type_name(T[name]) == name
        assert G.type_block(T[name]) == (elems, nbytes)
        assert G.size_of(T[name], elems * 10) == nbytes * 10
    with pytest.raises(ShvError):
        G.size_of(T["Q4_K"], 100)      # a partial block
    with pytest.raises(ShvError):
        G.size_of(99, 32)              # an unknown type
    assert G.type_name(99) == "?99" and G.type_block(99) is None
    # the table agrees with the sizes the CPU dequantiser works in, for every type that has one
    import oracle_lib as O
    for name, typ in O.GGML_TYPES.items():
        e, b = G.type_block(typ)
        assert O.type_bytes(typ, e * 256) == b * 256, name


def test_alignment_is_honoured(tmp_path):
    """gguf/gguf_test.go:277-299: general.alignment moves the data section."""
    w = GF.Writer(align=4096)
    w.put("general.alignment", GF.U32, 4096)
    w.tensor("a", T["F32"], [8], 0xAB)
    with G.GGUF(w.write(tmp_path / "m.gguf")) as f:
        info = f.files()[0]
        assert info["alignment"] == 4096 and info["data_start"] % 4096 == 0
        a = f.get("a")
        assert a.nbytes == 32 and a.data()[0] == 0xAB


def test_rejects_bad_files(tmp_path):
    """gguf/gguf_test.go:301-346, plus the bounds the header reader keeps (gguf/gguf.go:436-500,580-583)."""
    def bad(name, b):
        p = tmp_path / name
        p.write_bytes(b)
        with pytest.raises(ShvError) as e:
            G.GGUF(p).close()
        return str(e.value)

    assert "magic" in bad("magic.gguf", bytes(64))
    assert "too short" in bad("short.gguf", b"GGUF")
    w = GF.Writer()
    w.tensor("a", T["F32"], [8], 1)
    good = w.bytes()
    assert "past the end" in bad("truncated.gguf", good[:-16])
    w2 = GF.Writer()
    w2.put("general.alignment", GF.U32, 48)
    w2.tensor("a", T["F32"], [8], 1)
    assert "power of two" in bad("align.gguf", w2.bytes())
    # an unknown ggml type has no block geometry: patch the descriptor's type word
    at = 24 + 8 + 1 + 4 + 8      # header, then the descriptor's name, dimension count and one dimension
    assert good[at:at + 12] == struct.pack("<IQ", T["F32"], 0)
    assert "unknown ggml type 99" in bad("unknown-type.gguf", good[:at] + struct.pack("<I", 99) + good[at + 4:])
    assert "version" in bad("v1.gguf", GF.Writer(version=1).bytes() + bytes(32))
    assert "version" in bad("v4.gguf", GF.Writer(version=4).bytes() + bytes(32))
    # a header that ends inside a key, a string longer than the file, an array longer than the file
    w3 = GF.Writer()
    w3.put("some.long.key.name", GF.U32, 1)
    assert "truncated" in bad("cut.gguf", (w3.bytes() + bytes(8))[:30] + bytes(2))
    hdr = b"GGUF" + struct.pack("<IQQ", 3, 0, 1)
    assert "exceeds the file" in bad("str.gguf", hdr + struct.pack("<Q", 1 << 40) + bytes(32))
    assert "exceeds the file" in bad("arr.gguf", hdr + GF._str("k") + struct.pack("<IIQ", GF.ARRAY, GF.U8, 1 << 40) + bytes(32))
    assert "nested" in bad("nest.gguf", hdr + GF._str("k") + struct.pack("<IIQ", GF.ARRAY, GF.ARRAY, 1) + bytes(32))
    assert "unknown value type" in bad("vt.gguf", hdr + GF._str("k") + struct.pack("<I", 13) + bytes(32))
    # dimensions: none, five, a partial block, a product that wraps, the same name twice
    def one(dims, typ=T["F32"], name=b"a"):
        return (b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + GF._str(name) + struct.pack("<I", len(dims)) +
                b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", typ, 0) + bytes(96))
    assert "dimensions" in bad("d0.gguf", one([]))
    assert "dimensions" in bad("d5.gguf", one([1, 1, 1, 1, 1]))
    assert "whole number" in bad("part.gguf", one([100], T["Q4_K"]))
    assert "overflow" in bad("wrap.gguf", one([1 << 40, 1 << 40]))
    w4 = GF.Writer()
    w4.tensor("a", T["F32"], [8], 1)
    w4.tensor("a", T["F32"], [8], 2)
    assert "twice" in bad("twice.gguf", w4.bytes())
    with pytest.raises(ShvError):
        G.GGUF(tmp_path / "absent.gguf")


def _shard_file(base, i, n):
    return "%s-%05d-of-%05d.gguf" % (base, i + 1, n)


def _shard_tensor(shard, i):
    return "blk.%05d.w%05d" % (shard, i)


def test_open_set_joins_shards(tmp_path):
    """gguf/gguf_test.go:359-421"""
    n = 3
    for i in range(n):
        w = GF.Writer()
        if i == 0:
            w.put("general.architecture", GF.STR, "qwen4exp")
            w.put("qwen4exp.expert_count", GF.U32, 512)
        w.put("split.no", GF.U16, i)
        w.put("split.count", GF.U16, n)
        w.put("split.tensors.count", GF.I32, 6)
        w.tensor(_shard_tensor(i, 0), T["Q8_0"], [256, 2], 0x10 + i)
        w.tensor(_shard_tensor(i, 1), T["Q4_K"], [256, 2], 0x20 + i)
        w.write(tmp_path / _shard_file("model", i, n))
    # openable from any shard: the suffix names the set
    for frm in (_shard_file("model", 0, n), _shard_file("model", 2, n)):
        with G.GGUF(tmp_path / frm) as s:
            assert len(s.files()) == n and len(s) == 6
            assert s.arch() == "qwen4exp" and s.uint("qwen4exp.expert_count") == 512   # metadata from shard 1
            t = s.get(_shard_tensor(2, 1))
            assert t.shard == 2 and t.data()[0] == 0x22
            assert [x.shard for x in s.tensors()] == [0, 0, 1, 1, 2, 2]
    # one file by itself does not join its siblings
    with G.GGUF(tmp_path / _shard_file("model", 1, n), single=True) as f:
        assert len(f.files()) == 1 and len(f) == 2
    # a directory holding one split set resolves to it
    with G.GGUF(tmp_path) as s:
        assert len(s.files()) == n
    # a second checkpoint beside it makes the directory ambiguous
    w = GF.Writer()
    w.tensor("a", T["F32"], [8], 0)
    w.write(tmp_path / "other.gguf")
    with pytest.raises(ShvError, match="holds 2 checkpoints"):
        G.GGUF(tmp_path)
    os.remove(tmp_path / "other.gguf")
    # the failure the check exists for: a download that stopped short
    os.remove(tmp_path / _shard_file("model", 2, n))
    with pytest.raises(ShvError, match="missing"):
        G.GGUF(tmp_path / _shard_file("model", 0, n))


def test_open_set_rejects_inconsistent_shards(tmp_path):
    """gguf/gguf_test.go:423-437 and the other arms of checkSplit (gguf/gguf.go:795-819)."""
    def shards(d, no=(0, 1), count=(2, 2), total=2, names=None):
        os.makedirs(d)
        for i in range(2):
            w = GF.Writer()
            if no[i] is not None:
                w.put("split.no", GF.U16, no[i])
            w.put("split.count", GF.U16, count[i])
            w.put("split.tensors.count", GF.I32, total)
            w.tensor(names[i] if names else _shard_tensor(i, 0), T["F32"], [8], i)
            w.write(d / _shard_file("m", i, 2))
        return d / _shard_file("m", 0, 2)

    G.GGUF(shards(tmp_path / "ok")).close()
    with pytest.raises(ShvError, match="split.tensors.count=5"):
        G.GGUF(shards(tmp_path / "total", total=5))
    with pytest.raises(ShvError, match="expected 1"):
        G.GGUF(shards(tmp_path / "order", no=(0, 0)))
    with pytest.raises(ShvError, match="no split.no"):
        G.GGUF(shards(tmp_path / "nono", no=(0, None)))
    with pytest.raises(ShvError, match="split.count=3"):
        G.GGUF(shards(tmp_path / "count", count=(2, 3)))
    with pytest.raises(ShvError, match="more than one shard"):
        G.GGUF(shards(tmp_path / "dup", names=("same", "same")))
    # a lone file that says it is one of several
    w = GF.Writer()
    w.put("split.count", GF.U16, 4)
    w.tensor("a", T["F32"], [8], 0)
    with pytest.raises(ShvError, match="no siblings"):
        G.GGUF(w.write(tmp_path / "lonely.gguf"))
    with pytest.raises(ShvError, match="no .gguf checkpoint"):
        os.makedirs(tmp_path / "void")
        G.GGUF(tmp_path / "void")


def test_rows_of_a_mapped_tensor_dequantise_like_the_fixture(tmp_path, golden_dir):
    """ggml's own vectors written into a file and read back through the mapping: the container hands
    the dequantiser the bytes it was given (Tensor.Row + DequantizeRow, gguf/dequant.go:119-124)."""
    import oracle_lib as O
    b = open(os.path.join(golden_dir, "dequant_in.bin"), "rb").read()
    r = open(os.path.join(golden_dir, "dequant_ref.bin"), "rb").read()
    w, want, o, ro = GF.Writer(), {}, 0, 0
    while o < len(b):
        typ, n, nbytes = struct.unpack_from("<IIQ", b, o)
        _, _, rbytes = struct.unpack_from("<IIQ", r, ro)
        name = "t%d" % typ
        w.tensor(name, typ, [n // 2, 2] if n % 512 == 0 else [n], b[o + 16:o + 16 + nbytes])
        want[name] = np.frombuffer(r[ro + 16:ro + 16 + rbytes], dtype=np.float32)
        o += 16 + nbytes
        ro += 16 + rbytes
    with G.GGUF(w.write(tmp_path / "vec.gguf")) as f:
        assert len(f) == len(want) == 11
        for t in f.tensors():
            cols = t.dims[0]
            got = np.concatenate([O.dequant(t.type, np.array(t.row(i)), cols) for i in range(t.rows)])
            assert np.array_equal(got.view(np.uint32), want[t.name].view(np.uint32)), t.name


def test_damaged_headers_are_refused_not_followed(tmp_path):
    """A checkpoint is an untrusted file: whatever a header claims, the reader stays inside the
    mapping.  2 000 files made from a good one by overwriting bytes of the header or cutting it
    short either open (and then every tensor's span lies inside the file) or are refused."""
    w = GF.Writer()
    _sample(w)
    good = bytearray(w.bytes())
    header = good.index(b"\x11" * 64)          # the data section starts with token_embd's fill
    rng = np.random.default_rng(99)
    opened = refused = 0
    for trial in range(2000):
        b = bytearray(good)
        for _ in range(int(rng.integers(1, 4))):
            at = int(rng.integers(4, header))
            b[at] = int(rng.integers(0, 256)) if trial % 3 else 0xFF
        if trial % 5 == 0:
            b = b[:int(rng.integers(24, len(b)))]
        p = tmp_path / "f.gguf"
        p.write_bytes(bytes(b))
        try:
            f = G.GGUF(p, single=True)
        except ShvError:
            refused += 1
            continue
        opened += 1
        size = len(b)
        start = f.files()[0]["data_start"]
        for t in f.tensors():
            d = t.data()
            assert t.nbytes == G.size_of(t.type, t.elems()) and len(d) == t.nbytes
            if t.nbytes:
                int(d[0]), int(d[-1])          # both ends are readable
        for k in f.keys():
            f.kind(k), f.uint(k), f.str(k), f.strings(k)
        assert 0 <= start <= size
        f.close()
    assert opened > 100 and refused > 100, (opened, refused)
