"""ctypes binding of host/shv_llm.h: the C++ host layer (llm::Graph and its blocks) for the tests
and the benchmark.  No arithmetic lives here."""
import ctypes as C
import os

import numpy as np

from . import hip_api

HERE = os.path.dirname(os.path.abspath(__file__))


class Config(C.Structure):
    """shvllm_config; defaults are the synthetic Qwen3-Next-shape model."""
    _fields_ = [("n_layer", C.c_int32), ("n_embd", C.c_int32), ("n_head", C.c_int32),
                ("n_head_kv", C.c_int32), ("head_dim", C.c_int32), ("rope_dims", C.c_int32),
                ("rope_base", C.c_float), ("n_expert", C.c_int32), ("n_expert_used", C.c_int32),
                ("ffn_expert", C.c_int32), ("vocab", C.c_int32), ("rms_eps", C.c_float),
                ("ssm_head_dim", C.c_int32), ("ssm_head_k", C.c_int32), ("ssm_head_v", C.c_int32),
                ("ssm_conv", C.c_int32), ("attn_every", C.c_int32), ("nkv", C.c_int32),
                ("layers", C.c_int32), ("no_head", C.c_int32), ("attn_splits", C.c_int32),
                ("max_tokens", C.c_int32), ("slots", C.c_int32), ("head_rows", C.c_int32),
                ("speculative", C.c_int32), ("spec_rows", C.c_int32), ("nextn", C.c_int32),
                ("idx_heads", C.c_int32), ("idx_dim", C.c_int32), ("idx_top_k", C.c_int32), ("idx_ratio", C.c_int32)]

    def __init__(self, **kw):
        d = dict(n_layer=48, n_embd=2048, n_head=16, n_head_kv=2, head_dim=256, rope_dims=64,
                 rope_base=1e7, n_expert=512, n_expert_used=10, ffn_expert=512, vocab=151936,
                 rms_eps=1e-6, ssm_head_dim=128, ssm_head_k=16, ssm_head_v=32, ssm_conv=4,
                 attn_every=4, nkv=4096, layers=0, no_head=0, attn_splits=0, max_tokens=1, slots=1,
                 head_rows=0, speculative=0, spec_rows=2, nextn=0)
        d.update(kw)
        super().__init__(**d)


_lib = None


SCHED_MAX_ROWS = 64
INTERACTIVE, BACKGROUND = 0, 1  # backend/llm_sched.go:77-80


class SchedOpts(C.Structure):
    _fields_ = [("batch", C.c_int32), ("preempt_chunk", C.c_int32), ("reserve", C.c_int32), ("no_batch_decode", C.c_int32),
                ("coalesce_ms", C.c_double), ("spec_depth", C.c_int32)]


class SchedPass(C.Structure):
    _fields_ = [("kind", C.c_int32), ("unit", C.c_int32), ("slot", C.c_int32), ("pos", C.c_int32), ("n", C.c_int32),
                ("fresh", C.c_int32), ("restore", C.c_int32), ("take", C.c_int32), ("step", C.c_int32), ("n_units", C.c_int32),
                ("units", C.c_int32 * SCHED_MAX_ROWS), ("slots", C.c_int32 * SCHED_MAX_ROWS), ("wait_ms", C.c_double),
                ("prime", C.c_int32), ("tracked", C.c_int32)]


class SchedJob(C.Structure):
    _fields_ = [("cls", C.c_int32), ("slot", C.c_int32), ("reused", C.c_int32), ("restored", C.c_int32), ("stepping", C.c_int32),
                ("served_ms", C.c_double), ("arrival", C.c_uint64)]


def lib_path():
    return os.path.join(HERE, "libshv_llm.so")


def load():
    global _lib
    if _lib is not None:
        return _lib
    hip_api.load()
    p = lib_path()
    if not os.path.exists(p):
        raise hip_api.ShvError(-4, "%s is missing: build it with `python strix-halo-vulkan_amd/build.py`" % p)
    L = C.CDLL(p)
    vp = C.c_void_p
    L.shvllm_last_error.restype = C.c_char_p
    L.shvllm_open.argtypes = [C.c_int, C.POINTER(Config), C.POINTER(vp)]
    L.shvllm_close.argtypes = [vp]
    L.shvllm_close.restype = None
    L.shvllm_ctx.argtypes = [vp]
    L.shvllm_ctx.restype = vp
    L.shvllm_init_synthetic.argtypes = [vp, C.c_uint64]
    L.shvllm_open_gguf.argtypes = [C.c_int, C.c_char_p, C.POINTER(Config), C.POINTER(vp)]
    L.shvllm_get_config.argtypes = [vp, C.POINTER(Config)]
    L.shvllm_save_gguf.argtypes = [vp, C.c_char_p]
    L.shvllm_tensor_type.argtypes = [vp, C.c_char_p, C.POINTER(C.c_int32)]
    L.shvllm_transcoded.argtypes = [vp, C.c_char_p, C.c_size_t]
    L.shvllm_tensor_count.argtypes = [vp]
    L.shvllm_tensor_at.argtypes = [vp, C.c_int, C.POINTER(C.c_char_p), C.POINTER(vp), C.POINTER(C.c_uint64),
                                   C.POINTER(C.c_int32), C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                   C.POINTER(C.c_int32)]
    L.shvllm_tensor.argtypes = [vp, C.c_char_p, C.POINTER(vp), C.POINTER(C.c_uint64)]
    L.shvllm_weight_bytes.argtypes = [vp]
    L.shvllm_weight_bytes.restype = C.c_uint64
    L.shvllm_stage.argtypes = [vp]
    L.shvllm_reset.argtypes = [vp]
    L.shvllm_extend.argtypes = [vp, C.POINTER(C.c_int32), C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.shvllm_generate.argtypes = [vp, C.c_int, C.POINTER(C.c_int32), C.POINTER(C.c_uint64)]
    L.shvllm_past.argtypes = [vp]
    L.shvllm_dispatches.argtypes = [vp]
    L.shvllm_profile_step.argtypes = [vp, C.POINTER(C.c_char * 32), C.POINTER(C.c_uint64), C.c_int,
                                      C.POINTER(C.c_int)]
    L.shvllm_dn_state.argtypes = [vp, C.c_int, C.POINTER(C.c_float)]
    L.shvllm_kv.argtypes = [vp, C.c_int, C.c_int, C.POINTER(C.c_uint16), C.POINTER(C.c_uint16)]
    L.shvllm_gpu_nanos.argtypes = [vp]
    L.shvllm_gpu_nanos.restype = C.c_uint64
    i32p, f32p, u16p = C.POINTER(C.c_int32), C.POINTER(C.c_float), C.POINTER(C.c_uint16)
    L.shvllm_extend_rows.argtypes = [vp, i32p, C.c_int, f32p, f32p, i32p]
    L.shvllm_decode_rows.argtypes = [vp, i32p, i32p, C.c_int, f32p, i32p]
    for name in ("use_slot", "speculate", "speculate_first", "keep", "mtp_rewind", "spec_open"):
        getattr(L, "shvllm_" + name).argtypes = [vp, C.c_int]
    for name in ("commit", "rewind", "plane", "mtp_past"):
        getattr(L, "shvllm_" + name).argtypes = [vp]
    L.shvllm_ids.argtypes = [vp, i32p, C.c_int, C.POINTER(C.c_int)]
    L.shvllm_dn_state_at.argtypes = [vp, C.c_int, C.c_int, C.c_int, f32p]
    L.shvllm_kv_at.argtypes = [vp, C.c_int, C.c_int, C.c_int, u16p, u16p]
    L.shvllm_profile_rows.argtypes = [vp, C.c_int, C.POINTER(C.c_char * 32), C.POINTER(C.c_uint64), C.c_int,
                                      C.POINTER(C.c_int)]
    L.shvllm_checkpoint.argtypes = [vp, C.POINTER(vp)]
    L.shvllm_restore.argtypes = [vp, vp]
    L.shvllm_checkpoint_free.argtypes = [vp]
    L.shvllm_checkpoint_free.restype = None
    L.shvllm_profile_chunk.argtypes = [vp, i32p, C.c_int, C.POINTER(C.c_char * 32), C.POINTER(C.c_uint64), C.c_int,
                                       C.POINTER(C.c_int)]
    L.shvllm_mtp_stage.argtypes = [vp, C.c_int, C.c_int]
    L.shvllm_mtp_rows.argtypes = [vp, f32p, i32p, C.c_int, C.c_int, C.c_int, f32p, f32p]
    L.shvllm_spec_start.argtypes = [vp, i32p, C.c_int, i32p]
    L.shvllm_spec_sampler.argtypes = [vp, C.c_float, C.c_int, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int64, C.c_int64]
    L.shvllm_spec_round.argtypes = [vp, i32p, C.c_int, i32p, C.c_int, C.POINTER(C.c_int)]
    L.shvllm_spec_stats.argtypes = [vp, i32p, C.POINTER(C.c_uint64)]
    dp = C.POINTER(C.c_double)
    ip = C.POINTER(C.c_int)
    L.shvllm_sched_open.argtypes = [vp, C.c_int, C.POINTER(SchedOpts), C.POINTER(vp)]
    L.shvllm_sched_close.argtypes = [vp]
    L.shvllm_sched_close.restype = None
    L.shvllm_sched_acquire.argtypes = [vp, C.c_int, i32p, C.c_int, C.c_int, C.c_double, ip]
    L.shvllm_sched_release.argtypes = [vp, C.c_int, C.c_double]
    L.shvllm_sched_job_info.argtypes = [vp, C.c_int, C.POINTER(SchedJob)]
    L.shvllm_sched_run.argtypes = [vp, C.c_int, i32p, C.c_int, C.c_int, ip]
    L.shvllm_sched_step.argtypes = [vp, C.c_int, C.c_int32, ip]
    L.shvllm_sched_withdraw.argtypes = [vp, C.c_int]
    L.shvllm_sched_next.argtypes = [vp, C.c_double, C.POINTER(SchedPass)]
    L.shvllm_sched_finish.argtypes = [vp, C.c_double, C.c_int, C.c_double]
    L.shvllm_sched_pump.argtypes = [vp, C.POINTER(SchedPass)]
    L.shvllm_sched_unit.argtypes = [vp, C.c_int, ip, ip, dp, f32p, C.c_int]
    L.shvllm_sched_forget.argtypes = [vp, C.c_int]
    L.shvllm_sched_counts.argtypes = [vp, i32p]
    L.shvllm_sched_held.argtypes = [vp, C.c_int, i32p, C.c_int, ip, ip]
    L.shvllm_sched_decode.argtypes = [vp, C.c_int, C.c_int32, C.c_int, ip]
    L.shvllm_sched_decode_sampled.argtypes = [vp, C.c_int, C.c_int32, C.c_int, vp, C.c_int, C.c_int64, ip]
    L.shvllm_sched_unit_tokens.argtypes = [vp, C.c_int, i32p, C.c_int, ip]
    L.shvllm_sched_finish_round.argtypes = [vp, C.c_double, C.c_int, C.c_double, i32p, C.c_int]
    L.shvllm_sched_round_counts.argtypes = [vp, i32p]
    L.shvllm_sched_tracked.argtypes = [vp, C.c_int, ip]
    _lib = L
    return L


def _check(rc):
    if rc != 0:
        raise hip_api.ShvError(rc, load().shvllm_last_error().decode("utf-8", "replace"))


KIND_DTYPE = {0: np.float32, 1: np.uint16, 2: np.uint8, 3: np.uint8}  # F32, F16 (bit patterns), Q4K (bytes), RAW (bytes of another ggml type)


class LLM:
    """llm.Model + llm.Graph behind one handle."""

    def __init__(self, cfg, device=0, gguf=None):
        """With gguf=path the model's shape and weights come from that checkpoint (llm.Open) and
        only the graph fields of cfg (nkv, max_tokens, slots ...) are used."""
        self.L = load()
        self.H = hip_api.load()
        h = C.c_void_p()
        if gguf is None:
            _check(self.L.shvllm_open(device, C.byref(cfg), C.byref(h)))
        else:
            _check(self.L.shvllm_open_gguf(device, str(gguf).encode(), C.byref(cfg), C.byref(h)))
            cfg = Config()
            _check(self.L.shvllm_get_config(h, C.byref(cfg)))
        self.cfg = cfg
        self.h = h
        self.ctx = self.L.shvllm_ctx(h)

    def save_gguf(self, path):
        _check(self.L.shvllm_save_gguf(self.h, str(path).encode()))

    def close(self):
        if self.h:
            self.L.shvllm_close(self.h)
            self.h = None

    def init_synthetic(self, seed):
        _check(self.L.shvllm_init_synthetic(self.h, seed))

    def tensors(self):
        """[(name, device pointer, bytes, kind, rows, cols, is_alias)]"""
        out = []
        for i in range(self.L.shvllm_tensor_count(self.h)):
            name, ptr, nb = C.c_char_p(), C.c_void_p(), C.c_uint64()
            kind, rows, cols, al = C.c_int32(), C.c_int64(), C.c_int64(), C.c_int32()
            _check(self.L.shvllm_tensor_at(self.h, i, C.byref(name), C.byref(ptr), C.byref(nb), C.byref(kind),
                                           C.byref(rows), C.byref(cols), C.byref(al)))
            out.append((name.value.decode(), ptr.value, nb.value, kind.value, rows.value, cols.value, bool(al.value)))
        return out

    def download(self, name):
        ptr, nb = C.c_void_p(), C.c_uint64()
        _check(self.L.shvllm_tensor(self.h, name.encode(), C.byref(ptr), C.byref(nb)))
        kind = next(t[3] for t in self.tensors() if t[0] == name)
        dt = np.dtype(KIND_DTYPE[kind])
        a = np.empty(nb.value // dt.itemsize, dtype=dt)
        hip_api.check(self.H.shv_download(self.ctx, a.ctypes.data, ptr, nb.value))
        return a

    def tensor_type(self, name):
        t = C.c_int32()
        _check(self.L.shvllm_tensor_type(self.h, name.encode(), C.byref(t)))
        return t.value

    def transcoded(self):
        """Names of the matrices that were fitted again as Q4_K when the checkpoint was opened."""
        buf = C.create_string_buffer(1 << 16)
        n = self.L.shvllm_transcoded(self.h, buf, len(buf))
        names = [x for x in buf.value.decode().split("\n") if x]
        assert len(names) == n, (n, names)
        return names

    def upload(self, name, arr):
        ptr, nb = C.c_void_p(), C.c_uint64()
        _check(self.L.shvllm_tensor(self.h, name.encode(), C.byref(ptr), C.byref(nb)))
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes == nb.value, (name, arr.nbytes, nb.value)
        hip_api.check(self.H.shv_upload(self.ctx, ptr, arr.ctypes.data, arr.nbytes))

    def weight_bytes(self):
        return self.L.shvllm_weight_bytes(self.h)

    def stage(self):
        _check(self.L.shvllm_stage(self.h))

    def reset(self):
        _check(self.L.shvllm_reset(self.h))

    def extend(self, ids, want_logits=True, want_hidden=False):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        lg = np.empty(self.cfg.vocab, np.float32) if want_logits else None
        hd = np.empty(self.cfg.n_embd, np.float32) if want_hidden else None
        fp = C.POINTER(C.c_float)
        _check(self.L.shvllm_extend(self.h, ids.ctypes.data_as(C.POINTER(C.c_int32)), len(ids),
                                    lg.ctypes.data_as(fp) if lg is not None else None,
                                    hd.ctypes.data_as(fp) if hd is not None else None))
        return lg, hd

    def generate(self, n):
        out = np.empty(n, np.int32)
        ns = C.c_uint64()
        _check(self.L.shvllm_generate(self.h, n, out.ctypes.data_as(C.POINTER(C.c_int32)), C.byref(ns)))
        return out, ns.value

    def past(self):
        return self.L.shvllm_past(self.h)

    def dispatches(self):
        return self.L.shvllm_dispatches(self.h)

    def profile_step(self):
        labels = (C.c_char * 32 * 64)()
        ns = (C.c_uint64 * 64)()
        n = C.c_int()
        _check(self.L.shvllm_profile_step(self.h, labels, ns, 64, C.byref(n)))
        return [(labels[i].value.decode(), ns[i]) for i in range(n.value)]

    def dn_state(self, layer):
        c = self.cfg
        out = np.empty((c.ssm_head_v, c.ssm_head_dim, c.ssm_head_dim), np.float32)
        _check(self.L.shvllm_dn_state(self.h, layer, out.ctypes.data_as(C.POINTER(C.c_float))))
        return out

    def kv(self, layer, cells):
        c = self.cfg
        k = np.empty((cells, c.n_head_kv, c.head_dim), np.uint16)
        v = np.empty_like(k)
        u16 = C.POINTER(C.c_uint16)
        _check(self.L.shvllm_kv(self.h, layer, cells, k.ctypes.data_as(u16), v.ctypes.data_as(u16)))
        return k, v

    # ---- multi-row passes, slots, rewindable passes ----

    def extend_rows(self, ids, want_logits=False, want_res=False):
        """Graph.ExtendRows: (greedy token per row, logits [n][vocab] or None, residual [n][n_embd] or None)"""
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        n = len(ids)
        lg = np.empty((n, self.cfg.vocab), np.float32) if want_logits else None
        rs = np.empty((n, self.cfg.n_embd), np.float32) if want_res else None
        best = np.empty(n, np.int32)
        fp, ip = C.POINTER(C.c_float), C.POINTER(C.c_int32)
        _check(self.L.shvllm_extend_rows(self.h, ids.ctypes.data_as(ip), n,
                                         lg.ctypes.data_as(fp) if lg is not None else None,
                                         rs.ctypes.data_as(fp) if rs is not None else None, best.ctypes.data_as(ip)))
        return best, lg, rs

    def decode_rows(self, slots, ids, want_logits=False):
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        n = len(ids)
        lg = np.empty((n, self.cfg.vocab), np.float32) if want_logits else None
        best = np.empty(n, np.int32)
        fp, ip = C.POINTER(C.c_float), C.POINTER(C.c_int32)
        _check(self.L.shvllm_decode_rows(self.h, slots.ctypes.data_as(ip), ids.ctypes.data_as(ip), n,
                                         lg.ctypes.data_as(fp) if lg is not None else None, best.ctypes.data_as(ip)))
        return best, lg

    def use_slot(self, s):
        _check(self.L.shvllm_use_slot(self.h, s))

    def speculate(self, on):
        _check(self.L.shvllm_speculate(self.h, int(on)))

    def speculate_first(self, on):
        _check(self.L.shvllm_speculate_first(self.h, int(on)))

    def keep(self, k):
        _check(self.L.shvllm_keep(self.h, k))

    def commit(self):
        _check(self.L.shvllm_commit(self.h))

    def rewind(self):
        _check(self.L.shvllm_rewind(self.h))

    def plane(self):
        return self.L.shvllm_plane(self.h)

    def ids(self):
        n = C.c_int()
        _check(self.L.shvllm_ids(self.h, None, 0, C.byref(n)))
        out = np.empty(max(n.value, 1), np.int32)
        _check(self.L.shvllm_ids(self.h, out.ctypes.data_as(C.POINTER(C.c_int32)), n.value, C.byref(n)))
        return out[:n.value]

    def dn_state_at(self, layer, slot=0, plane=0):
        c = self.cfg
        out = np.empty((c.ssm_head_v, c.ssm_head_dim, c.ssm_head_dim), np.float32)
        _check(self.L.shvllm_dn_state_at(self.h, layer, slot, plane, out.ctypes.data_as(C.POINTER(C.c_float))))
        return out

    def kv_at(self, layer, slot, cells):
        c = self.cfg
        k = np.empty((cells, c.n_head_kv, c.head_dim), np.uint16)
        v = np.empty_like(k)
        u16 = C.POINTER(C.c_uint16)
        _check(self.L.shvllm_kv_at(self.h, layer, slot, cells, k.ctypes.data_as(u16), v.ctypes.data_as(u16)))
        return k, v

    def profile_rows(self, rows):
        labels = (C.c_char * 32 * 64)()
        ns = (C.c_uint64 * 64)()
        n = C.c_int()
        _check(self.L.shvllm_profile_rows(self.h, rows, labels, ns, 64, C.byref(n)))
        return [(labels[i].value.decode(), ns[i]) for i in range(n.value)]

    def checkpoint(self):
        """Graph.Checkpoint: an opaque handle to the live slot's saved sequence (free with checkpoint_free)."""
        c = C.c_void_p()
        _check(self.L.shvllm_checkpoint(self.h, C.byref(c)))
        return c

    def restore(self, c):
        _check(self.L.shvllm_restore(self.h, c))

    def checkpoint_free(self, c):
        self.L.shvllm_checkpoint_free(c)

    def profile_chunk(self, ids):
        """One headless prompt chunk timed op by op; the sequence advances by the chunk."""
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        labels = (C.c_char * 32 * 64)()
        ns = (C.c_uint64 * 64)()
        n = C.c_int()
        _check(self.L.shvllm_profile_chunk(self.h, ids.ctypes.data_as(C.POINTER(C.c_int32)), len(ids), labels, ns, 64, C.byref(n)))
        return [(labels[i].value.decode(), ns[i]) for i in range(n.value)]

    # ---- draft head and speculative loop ----

    def mtp_stage(self, max_tok=4, vocab_prefix=0):
        _check(self.L.shvllm_mtp_stage(self.h, max_tok, vocab_prefix))

    def mtp_rows(self, hs, ids, pos, head=True, want_res=True):
        """MTPHead.Rows with host buffers: (last row's logits or None, residual rows or None)"""
        hs = np.ascontiguousarray(hs, dtype=np.float32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        n = len(ids)
        lg = np.empty(self.cfg.vocab, np.float32) if head else None
        rs = np.empty((n, self.cfg.n_embd), np.float32) if want_res else None
        fp, ip = C.POINTER(C.c_float), C.POINTER(C.c_int32)
        _check(self.L.shvllm_mtp_rows(self.h, hs.ctypes.data_as(fp), ids.ctypes.data_as(ip), n, pos, int(head),
                                      lg.ctypes.data_as(fp) if lg is not None else None,
                                      rs.ctypes.data_as(fp) if rs is not None else None))
        return lg, rs

    def mtp_rewind(self, n):
        _check(self.L.shvllm_mtp_rewind(self.h, n))

    def mtp_past(self):
        return self.L.shvllm_mtp_past(self.h)

    def spec_open(self, depth):
        _check(self.L.shvllm_spec_open(self.h, depth))

    def spec_sampler(self, temp, top_k=0, top_p=0.0, min_p=0.0, repeat_penalty=1.0, presence_penalty=0.0, seed=0, draft_seed=1):
        """Speculator.UseSampler: the loop's tokens are drawn (temp <= 0: arg-max again)."""
        _check(self.L.shvllm_spec_sampler(self.h, temp, top_k, top_p, min_p, repeat_penalty, presence_penalty, seed, draft_seed))

    def spec_start(self, prompt):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        first = C.c_int32()
        _check(self.L.shvllm_spec_start(self.h, prompt.ctypes.data_as(C.POINTER(C.c_int32)), len(prompt), C.byref(first)))
        return first.value

    def spec_round(self, forced=()):
        forced = np.ascontiguousarray(forced, dtype=np.int32)
        out = np.empty(16, np.int32)
        n = C.c_int()
        ip = C.POINTER(C.c_int32)
        _check(self.L.shvllm_spec_round(self.h, forced.ctypes.data_as(ip) if len(forced) else None, len(forced),
                                        out.ctypes.data_as(ip), 16, C.byref(n)))
        return out[:n.value].copy()

    def spec_stats(self):
        counts = np.zeros(17, np.int32)
        nanos = np.zeros(2, np.uint64)
        _check(self.L.shvllm_spec_stats(self.h, counts.ctypes.data_as(C.POINTER(C.c_int32)),
                                        nanos.ctypes.data_as(C.POINTER(C.c_uint64))))
        return dict(rounds=int(counts[0]), drafted=int(counts[1]), accepted=int(counts[2]), tokens=int(counts[3]),
                    passes=counts[4:9].tolist(), drafted_at=counts[9:13].tolist(), accepted_at=counts[13:17].tolist(),
                    draft_ns=int(nanos[0]), verify_ns=int(nanos[1]))


class Sched:
    """The scheduler over one staged graph (backend/llm_sched.go), or, with llm=None, its policy
    alone over `slots` slots: next() says which pass would run and finish() books a duration the
    caller names, with no device involved."""

    def __init__(self, llm=None, slots=1, batch=2048, preempt_chunk=0, reserve=1, no_batch_decode=False, coalesce_ms=5.0,
                 spec_depth=0):
        """spec_depth > 0: decode() units may run as speculative rounds (the model needs mtp_stage() first and a
        configuration with speculative=1, spec_rows >= spec_depth + 1)."""
        self.L = load()
        self.llm = llm
        o = SchedOpts(batch, preempt_chunk, reserve, int(no_batch_decode), coalesce_ms, spec_depth)
        s = C.c_void_p()
        _check(self.L.shvllm_sched_open(llm.h if llm is not None else None, slots, C.byref(o), C.byref(s)))
        self.s = s

    def close(self):
        if self.s:
            self.L.shvllm_sched_close(self.s)
            self.s = None

    def acquire(self, cls, prompt, mark=0, now_ms=0.0):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        job = C.c_int()
        _check(self.L.shvllm_sched_acquire(self.s, cls, prompt.ctypes.data_as(C.POINTER(C.c_int32)), len(prompt), mark, now_ms, C.byref(job)))
        return job.value

    def release(self, job, now_ms=0.0):
        _check(self.L.shvllm_sched_release(self.s, job, now_ms))

    def job(self, job):
        j = SchedJob()
        _check(self.L.shvllm_sched_job_info(self.s, job, C.byref(j)))
        return j

    def run(self, job, ids, fresh):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        u = C.c_int()
        _check(self.L.shvllm_sched_run(self.s, job, ids.ctypes.data_as(C.POINTER(C.c_int32)), len(ids), int(fresh), C.byref(u)))
        return u.value

    def step(self, job, tok):
        u = C.c_int()
        _check(self.L.shvllm_sched_step(self.s, job, int(tok), C.byref(u)))
        return u.value

    def decode(self, job, tok, room, sampler=None, exact=False, draft_seed=1):
        """A decode step that may run as a speculative round (Sched::Decode).  sampler: a sample_api.Sampler, which
        then names a round's tokens and takes them into its window itself (a unit that ran as a plain step leaves
        sampling to the caller, as ever); exact: a seeded request, every verified row one plain draw."""
        u = C.c_int()
        if sampler is None:
            _check(self.L.shvllm_sched_decode(self.s, job, int(tok), int(room), C.byref(u)))
        else:
            _check(self.L.shvllm_sched_decode_sampled(self.s, job, int(tok), int(room), sampler.h, int(exact), int(draft_seed), C.byref(u)))
        return u.value

    def unit_tokens(self, unit, max_ids=16):
        """The tokens a round drew for `unit`; empty for a unit that ran as a plain step."""
        dst = np.empty(max_ids, np.int32)
        n = C.c_int()
        _check(self.L.shvllm_sched_unit_tokens(self.s, unit, dst.ctypes.data_as(C.POINTER(C.c_int32)), max_ids, C.byref(n)))
        return dst[:min(n.value, max_ids)].copy()

    def finish_round(self, took_ms, toks, ok=True, now_ms=0.0):
        toks = np.ascontiguousarray(toks, dtype=np.int32)
        _check(self.L.shvllm_sched_finish_round(self.s, took_ms, int(ok), now_ms, toks.ctypes.data_as(C.POINTER(C.c_int32)), len(toks)))

    def round_counts(self):
        c = np.zeros(2, np.int32)
        _check(self.L.shvllm_sched_round_counts(self.s, c.ctypes.data_as(C.POINTER(C.c_int32))))
        return dict(rounds=int(c[0]), round_tokens=int(c[1]))

    def tracked(self, slot):
        t = C.c_int()
        _check(self.L.shvllm_sched_tracked(self.s, slot, C.byref(t)))
        return bool(t.value)

    def withdraw(self, unit):
        _check(self.L.shvllm_sched_withdraw(self.s, unit))

    def next(self, now_ms=0.0):
        p = SchedPass()
        _check(self.L.shvllm_sched_next(self.s, now_ms, C.byref(p)))
        return p

    def finish(self, took_ms, ok=True, now_ms=0.0):
        _check(self.L.shvllm_sched_finish(self.s, took_ms, int(ok), now_ms))

    def pump(self):
        p = SchedPass()
        _check(self.L.shvllm_sched_pump(self.s, C.byref(p)))
        return p

    def unit(self, unit, want_logits=False):
        """(state, ids left, device ms, logits): state 0 queued, 1 done, 2 failed (self.error then says why)."""
        st, left, busy = C.c_int(), C.c_int(), C.c_double()
        logits = np.empty(self.llm.cfg.vocab, np.float32) if want_logits and self.llm is not None else None
        rc = self.L.shvllm_sched_unit(self.s, unit, C.byref(st), C.byref(left), C.byref(busy),
                                      logits.ctypes.data_as(C.POINTER(C.c_float)) if logits is not None else None,
                                      len(logits) if logits is not None else 0)
        _check(rc)
        self.error = self.L.shvllm_last_error().decode("utf-8", "replace") if st.value == 2 else ""
        return st.value, left.value, busy.value, logits

    def forget(self, unit):
        _check(self.L.shvllm_sched_forget(self.s, unit))

    def counts(self):
        c = np.zeros(6, np.int32)
        _check(self.L.shvllm_sched_counts(self.s, c.ctypes.data_as(C.POINTER(C.c_int32))))
        return dict(restores=int(c[0]), batches=int(c[1]), batch_rows=int(c[2]), passes=int(c[3]), waiting=int(c[4]), pending=int(c[5]))

    def held(self, slot, max_ids=1 << 16):
        dst = np.empty(max_ids, np.int32)
        n, ck = C.c_int(), C.c_int()
        _check(self.L.shvllm_sched_held(self.s, slot, dst.ctypes.data_as(C.POINTER(C.c_int32)), max_ids, C.byref(n), C.byref(ck)))
        return dst[:min(n.value, max_ids)].copy(), ck.value
