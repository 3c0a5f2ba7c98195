"""ctypes binding of the host sampler (host/sample.hpp through the shvsampler_* entry points of
host/shv_llm.h): the reference's llm.Sampler."""
import ctypes as C

import numpy as np

from . import llm_api

_bound = False


def _lib():
    global _bound
    L = llm_api.load()
    if _bound:
        return L
    vp, i32p, f32p = C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_float)
    L.shvsampler_new.argtypes = [C.c_float, C.c_int, C.c_float, C.c_int64]
    L.shvsampler_new.restype = vp
    L.shvsampler_free.argtypes = [vp]
    L.shvsampler_free.restype = None
    L.shvsampler_set.argtypes = [vp, C.c_float, C.c_float, C.c_float]
    L.shvsampler_set.restype = None
    L.shvsampler_greedy.argtypes = [vp]
    L.shvsampler_accept.argtypes = [vp, i32p, C.c_int]
    L.shvsampler_accept.restype = None
    L.shvsampler_sample.argtypes = [vp, f32p, C.c_int]
    L.shvsampler_dist.argtypes = [vp, f32p, C.c_int, i32p, f32p, C.c_int]
    L.shvsampler_draft.argtypes = [vp, C.c_int64]
    L.shvsampler_draft.restype = vp
    L.shvsampler_propose.argtypes = [vp, f32p, C.c_int]
    L.shvsampler_last_dist.argtypes = [vp, i32p, f32p, C.c_int]
    L.shvsampler_verify.argtypes = [vp, f32p, C.c_int, C.c_int32, vp]
    L.shvsampler_sample_many.argtypes = [vp, f32p, C.c_int, C.c_int, i32p]
    L.shvsampler_sample_many.restype = None
    L.shvsampler_speculate_many.argtypes = [vp, vp, f32p, f32p, C.c_int, C.c_int, i32p]
    L.shvsampler_speculate_many.restype = C.c_int64
    L.shvsampler_argmax.argtypes = [f32p, C.c_int]
    L.shvsampler_top_n.argtypes = [f32p, C.c_int, C.c_int, i32p]
    L.shvsampler_top_k_of.argtypes = [f32p, C.c_int, C.c_int, i32p]
    _bound = True
    return L


def _f(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _i(a):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


def argmax(row):
    return _lib().shvsampler_argmax(_f(row), len(row))


def top_n(row, k):
    out = np.empty(max(0, min(k, len(row))), np.int32)
    n = _lib().shvsampler_top_n(_f(row), len(row), k, _i(out))
    return out[:n]


def top_k_of(row, k):
    out = np.empty(max(0, k), np.int32)
    n = _lib().shvsampler_top_k_of(_f(row), len(row), k, _i(out))
    return out[:n]


class Sampler:
    def __init__(self, temp, top_k, top_p, seed, min_p=0.0, repeat_penalty=1.0, presence_penalty=0.0, _handle=None):
        self.L = _lib()
        self.h = _handle if _handle is not None else self.L.shvsampler_new(temp, top_k, top_p, seed)
        if _handle is None:
            self.L.shvsampler_set(self.h, min_p, repeat_penalty, presence_penalty)

    def close(self):
        if self.h:
            self.L.shvsampler_free(self.h)
            self.h = None

    def greedy(self):
        return bool(self.L.shvsampler_greedy(self.h))

    def accept(self, *ids):
        a = np.asarray(ids, np.int32)
        self.L.shvsampler_accept(self.h, _i(a), len(a))

    def sample(self, row):
        return self.L.shvsampler_sample(self.h, _f(row), len(row))

    def dist(self, row):
        n = self.L.shvsampler_dist(self.h, _f(row), len(row), None, None, 0)
        ids, p = np.empty(n, np.int32), np.empty(n, np.float32)
        self.L.shvsampler_dist(self.h, _f(row), len(row), _i(ids), _f(p), n)
        return ids, p

    def draft_sampler(self, seed):
        h = self.L.shvsampler_draft(self.h, seed)
        return Sampler(0, 0, 0, 0, _handle=h) if h else None

    def propose(self, row):
        return self.L.shvsampler_propose(self.h, _f(row), len(row))

    def last_dist(self):
        n = self.L.shvsampler_last_dist(self.h, None, None, 0)
        ids, p = np.empty(n, np.int32), np.empty(n, np.float32)
        self.L.shvsampler_last_dist(self.h, _i(ids), _f(p), n)
        return ids, p

    def verify(self, row, draft, proposer=None):
        return self.L.shvsampler_verify(self.h, _f(row), len(row), draft, proposer.h if proposer else None)

    def sample_many(self, row, draws):
        counts = np.zeros(len(row), np.int32)
        self.L.shvsampler_sample_many(self.h, _f(row), len(row), draws, _i(counts))
        return counts

    def speculate_many(self, draft_sampler, pl, ql, draws):
        counts = np.zeros(len(pl), np.int32)
        kept = self.L.shvsampler_speculate_many(self.h, draft_sampler.h, _f(pl), _f(ql), len(pl), draws, _i(counts))
        return counts, kept
