"""A GGUF writer and a plain parser for the tests, written from the format's specification and
independent of the library under test: the counterpart of the writer the reference's own tests
keep (gguf/gguf_test.go:17-140)."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}
BLOCK = {0: (1, 4), 1: (1, 2), 30: (1, 2), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 20: (32, 18),
         12: (256, 144), 13: (256, 176), 14: (256, 210),
         10: (256, 84)}     # Q2_K: a type the loader knows the geometry of and the device does not expand


def _str(s):
    b = s.encode() if isinstance(s, str) else s
    return struct.pack("<Q", len(b)) + b


class Writer:
    def __init__(self, align=32, version=3):
        self.align, self.version = align, version
        self.kv, self.n_kv, self.desc, self.n_tensor, self.data = b"", 0, b"", 0, b""

    def put(self, key, vt, value):
        self.kv += _str(key) + struct.pack("<I", vt)
        self.kv += _str(value) if vt == STR else struct.pack(_FMT[vt], value)
        self.n_kv += 1

    def put_array(self, key, et, values):
        self.kv += _str(key) + struct.pack("<IIQ", ARRAY, et, len(values))
        for v in values:
            self.kv += _str(v) if et == STR else struct.pack(_FMT[et], v)
        self.n_kv += 1

    def tensor(self, name, typ, dims, payload):
        """payload: a fill byte, or the tensor's bytes."""
        self.data += b"\0" * (-len(self.data) % self.align)
        off = len(self.data)
        n = int(np.prod(dims, dtype=np.int64))
        e, b = BLOCK[typ]
        assert n % e == 0
        nbytes = n // e * b
        if isinstance(payload, int):
            payload = bytes([payload]) * nbytes
        payload = bytes(payload)
        assert len(payload) == nbytes, (name, len(payload), nbytes)
        self.data += payload
        self.desc += _str(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        self.desc += struct.pack("<IQ", typ, off)
        self.n_tensor += 1

    def bytes(self):
        out = b"GGUF" + struct.pack("<IQQ", self.version, self.n_tensor, self.n_kv) + self.kv + self.desc
        out += b"\0" * (-len(out) % self.align)
        return out + self.data

    def write(self, path):
        with open(path, "wb") as f:
            f.write(self.bytes())
        return str(path)


def parse(path):
    """{'version', 'kv': {key: value}, 'tensors': {name: (type, dims, bytes)}} of a file this
    module's grammar covers; scalars and arrays come back as Python values."""
    b = open(path, "rb").read()
    assert b[:4] == b"GGUF"
    o = [4]

    def rd(fmt):
        v = struct.unpack_from(fmt, b, o[0])
        o[0] += struct.calcsize(fmt)
        return v[0]

    def rs():
        n = rd("<Q")
        s = b[o[0]:o[0] + n]
        o[0] += n
        return s.decode()

    def val(vt):
        if vt == STR:
            return rs()
        if vt == ARRAY:
            et, n = rd("<I"), rd("<Q")
            return [val(et) for _ in range(n)]
        return rd(_FMT[vt])

    version, n_tensor, n_kv = rd("<I"), rd("<Q"), rd("<Q")
    kv = {}
    for _ in range(n_kv):
        k = rs()
        kv[k] = val(rd("<I"))
    descs = []
    for _ in range(n_tensor):
        name = rs()
        dims = [rd("<Q") for _ in range(rd("<I"))]
        descs.append((name, dims, rd("<I"), rd("<Q")))
    align = kv.get("general.alignment", 32)
    start = (o[0] + align - 1) // align * align
    tensors = {}
    for name, dims, typ, off in descs:
        e, bb = BLOCK[typ]
        nbytes = int(np.prod(dims, dtype=np.int64)) // e * bb
        tensors[name] = (typ, dims, b[start + off:start + off + nbytes])
    return dict(version=version, kv=kv, tensors=tensors)
