"""ctypes binding of the GGUF container reader in host/gguf.hpp (the shvgguf_* entry points of
host/shv_llm.h): the reference's gguf.Open / gguf.OpenSet with their tensors and typed metadata
getters.  Nothing here touches a device."""
import ctypes as C

import numpy as np

from . import hip_api, llm_api

TYPES = {"F32": 0, "F16": 1, "Q4_0": 2, "Q4_1": 3, "Q5_0": 6, "Q5_1": 7, "Q8_0": 8, "Q8_1": 9, "Q2_K": 10,
         "Q3_K": 11, "Q4_K": 12, "Q5_K": 13, "Q6_K": 14, "Q8_K": 15, "IQ4_NL": 20, "I8": 24, "I16": 25,
         "I32": 26, "I64": 27, "F64": 28, "BF16": 30, "MXFP4": 39}

_bound = False


def _lib():
    global _bound
    L = llm_api.load()
    if _bound:
        return L
    vp, cp, u64, i64 = C.c_void_p, C.c_char_p, C.c_uint64, C.c_int64
    P = C.POINTER
    L.shvgguf_open.argtypes = [cp, P(vp)]
    L.shvgguf_open_file.argtypes = [cp, P(vp)]
    L.shvgguf_close.argtypes = [vp]
    L.shvgguf_close.restype = None
    L.shvgguf_files.argtypes = [vp]
    L.shvgguf_file_info.argtypes = [vp, C.c_int, P(cp), P(C.c_uint32), P(u64), P(i64)]
    L.shvgguf_len.argtypes = [vp]
    L.shvgguf_params.argtypes = [vp]
    L.shvgguf_params.restype = i64
    L.shvgguf_bytes.argtypes = [vp]
    L.shvgguf_bytes.restype = i64
    L.shvgguf_arch.argtypes = [vp]
    L.shvgguf_arch.restype = cp
    L.shvgguf_tensor_at.argtypes = [vp, C.c_int, P(cp), P(C.c_uint32), P(C.c_int32), P(i64), P(vp), P(u64),
                                    P(C.c_int32), P(i64), P(i64)]
    L.shvgguf_find.argtypes = [vp, cp]
    L.shvgguf_advise_random.argtypes = [vp, C.c_int]
    L.shvgguf_key_count.argtypes = [vp]
    L.shvgguf_key_at.argtypes = [vp, C.c_int]
    L.shvgguf_key_at.restype = cp
    L.shvgguf_kind.argtypes = [vp, cp]
    L.shvgguf_uint.argtypes = [vp, cp, P(u64)]
    L.shvgguf_int.argtypes = [vp, cp, P(i64)]
    L.shvgguf_float.argtypes = [vp, cp, P(C.c_double)]
    L.shvgguf_bool.argtypes = [vp, cp, P(C.c_int32)]
    L.shvgguf_str.argtypes = [vp, cp, P(vp), P(u64)]
    L.shvgguf_array_len.argtypes = [vp, cp, P(u64)]
    L.shvgguf_uints.argtypes = [vp, cp, P(u64), u64]
    L.shvgguf_ints.argtypes = [vp, cp, P(i64), u64]
    L.shvgguf_floats.argtypes = [vp, cp, P(C.c_double), u64]
    L.shvgguf_string_at.argtypes = [vp, cp, u64, P(vp), P(u64)]
    L.shvgguf_type_name.argtypes = [C.c_uint32]
    L.shvgguf_type_name.restype = cp
    L.shvgguf_type_block.argtypes = [C.c_uint32, P(C.c_int32), P(C.c_int32)]
    L.shvgguf_size_of.argtypes = [C.c_uint32, i64]
    L.shvgguf_size_of.restype = i64
    _bound = True
    return L


def type_name(t):
    return _lib().shvgguf_type_name(t).decode()


def type_block(t):
    """(elements, bytes) of one block, or None for a type the table does not know."""
    e, b = C.c_int32(), C.c_int32()
    return (e.value, b.value) if _lib().shvgguf_type_block(t, C.byref(e), C.byref(b)) else None


def size_of(t, n):
    r = _lib().shvgguf_size_of(t, n)
    if r < 0:
        raise hip_api.ShvError(-1, _lib().shvllm_last_error().decode("utf-8", "replace"))
    return r


class Tensor:
    def __init__(self, name, typ, dims, data, nbytes, shard, rows, row_bytes):
        self.name, self.type, self.dims, self.shard = name, typ, dims, shard
        self.ptr, self.nbytes, self.rows, self.row_bytes = data, nbytes, rows, row_bytes

    def data(self):
        """The tensor's bytes: a view of the mapping, valid until the checkpoint is closed."""
        return np.ctypeslib.as_array(C.cast(self.ptr, C.POINTER(C.c_uint8)), shape=(self.nbytes,))

    def row(self, i):
        return self.data()[i * self.row_bytes:(i + 1) * self.row_bytes]

    def elems(self):
        return int(np.prod(self.dims, dtype=np.int64))


class GGUF:
    """gguf.OpenSet (a file, any shard of a split checkpoint, or a directory holding one), or with
    single=True gguf.Open (this file alone)."""

    def __init__(self, path, single=False):
        self.L = _lib()
        h = C.c_void_p()
        op = self.L.shvgguf_open_file if single else self.L.shvgguf_open
        llm_api._check(op(str(path).encode(), C.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            self.L.shvgguf_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def files(self):
        out = []
        for i in range(self.L.shvgguf_files(self.h)):
            p, v, a, d = C.c_char_p(), C.c_uint32(), C.c_uint64(), C.c_int64()
            llm_api._check(self.L.shvgguf_file_info(self.h, i, C.byref(p), C.byref(v), C.byref(a), C.byref(d)))
            out.append(dict(path=p.value.decode("utf-8", "replace"), version=v.value, alignment=a.value, data_start=d.value))
        return out

    def __len__(self):
        return self.L.shvgguf_len(self.h)

    def params(self):
        return self.L.shvgguf_params(self.h)

    def nbytes(self):
        return self.L.shvgguf_bytes(self.h)

    def arch(self):
        return self.L.shvgguf_arch(self.h).decode("utf-8", "replace")

    def tensor_at(self, i):
        name, typ, nd, dims = C.c_char_p(), C.c_uint32(), C.c_int32(), (C.c_int64 * 4)()
        data, nb, shard, rows, rb = C.c_void_p(), C.c_uint64(), C.c_int32(), C.c_int64(), C.c_int64()
        llm_api._check(self.L.shvgguf_tensor_at(self.h, i, C.byref(name), C.byref(typ), C.byref(nd), dims, C.byref(data),
                                                C.byref(nb), C.byref(shard), C.byref(rows), C.byref(rb)))
        return Tensor(name.value.decode("utf-8", "replace"), typ.value, list(dims[:nd.value]), data.value, nb.value, shard.value,
                      rows.value, rb.value)

    def tensors(self):
        return [self.tensor_at(i) for i in range(len(self))]

    def has(self, name):
        return self.L.shvgguf_find(self.h, name.encode()) >= 0

    def get(self, name):
        i = self.L.shvgguf_find(self.h, name.encode())
        if i < 0:
            raise KeyError("gguf: no tensor named %r" % name)
        return self.tensor_at(i)

    def keys(self):
        return [self.L.shvgguf_key_at(self.h, i).decode("utf-8", "replace") for i in range(self.L.shvgguf_key_count(self.h))]

    def kind(self, key):
        return self.L.shvgguf_kind(self.h, key.encode())

    def _scalar(self, fn, ctype, key):
        v = ctype()
        return v.value if fn(self.h, key.encode(), C.byref(v)) else None

    def uint(self, key):
        return self._scalar(self.L.shvgguf_uint, C.c_uint64, key)

    def int(self, key):
        return self._scalar(self.L.shvgguf_int, C.c_int64, key)

    def float(self, key):
        return self._scalar(self.L.shvgguf_float, C.c_double, key)

    def bool(self, key):
        v = self._scalar(self.L.shvgguf_bool, C.c_int32, key)
        return None if v is None else bool(v)

    def str(self, key):
        p, n = C.c_void_p(), C.c_uint64()
        if not self.L.shvgguf_str(self.h, key.encode(), C.byref(p), C.byref(n)):
            return None
        return C.string_at(p.value, n.value).decode("utf-8", "replace")

    def _array(self, fn, dtype, key):
        n = C.c_uint64()
        if not self.L.shvgguf_array_len(self.h, key.encode(), C.byref(n)):
            return None
        out = np.empty(max(1, n.value), dtype)
        if not fn(self.h, key.encode(), out.ctypes.data_as(C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), n.value):
            return None
        return out[:n.value]

    def uints(self, key):
        return self._array(self.L.shvgguf_uints, np.uint64, key)

    def ints(self, key):
        return self._array(self.L.shvgguf_ints, np.int64, key)

    def floats(self, key):
        return self._array(self.L.shvgguf_floats, np.float64, key)

    def strings(self, key):
        n = C.c_uint64()
        if not self.L.shvgguf_array_len(self.h, key.encode(), C.byref(n)) or self.kind(key) != 10:
            return None
        out = []
        for i in range(n.value):
            p, ln = C.c_void_p(), C.c_uint64()
            self.L.shvgguf_string_at(self.h, key.encode(), i, C.byref(p), C.byref(ln))
            out.append(C.string_at(p.value, ln.value).decode("utf-8", "replace"))
        return out
