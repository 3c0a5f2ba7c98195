"""ctypes binding of include/shv_hip.h.  Mirrors the header one to one; no arithmetic lives here."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
Q4K_BLOCK = 256
Q4K_BYTES = 144

OP_GEMV_Q4K, OP_DEQUANT_Q4K, OP_QUANTIZE_Q4K, OP_FILL_NORMAL = 1, 2, 3, 4
OP_MOE_ROUTER, OP_MOE_UP, OP_MOE_DOWN, OP_DN_STEP, OP_ATTN_DECODE = 5, 6, 7, 8, 9
OP_EMBED, OP_ARGMAX, OP_ADVANCE, OP_DEQUANT, OP_GEMV, OP_RING_ROWS, OP_ROUTER_FOLD, OP_QSA_INDEX = 10, 11, 12, 13, 14, 15, 16, 17
OP_ARGMAX_STATIC = 18
PRO_NONE, PRO_RMSNORM, PRO_GATED_NORM, PRO_MUL_SIGMOID, PRO_RMSNORM_PAIR = 0, 1, 2, 3, 4


class ShvError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("shv error %d: %s" % (code, msg))
        self.code = code


def lib_path():
    return os.path.join(HERE, "libshv_hip.so")


class Props(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 32), ("compute_units", C.c_int32),
                ("wave_size", C.c_int32), ("lds_bytes_per_cu", C.c_int32), ("clock_mhz", C.c_int32),
                ("hbm_bytes", C.c_uint64)]


class GemvQ4KArgs(C.Structure):
    _fields_ = [("w", C.c_void_p), ("x", C.c_void_p), ("y", C.c_void_p), ("residual", C.c_void_p),
                ("gamma", C.c_void_p), ("z", C.c_void_p), ("pos", C.c_void_p), ("slot", C.c_void_p),
                ("n", C.c_int32), ("k", C.c_int32), ("n_tok", C.c_int32), ("prologue", C.c_int32),
                ("head_dim", C.c_int32), ("eps", C.c_float), ("x_stride", C.c_int32),
                ("y_stride", C.c_int32), ("z_stride", C.c_int32), ("seq_len", C.c_int32),
                ("ring_slots", C.c_int32), ("ring_stride", C.c_int32), ("z_ring", C.c_int32),
                ("y_flat", C.c_void_p), ("fold", C.c_void_p), ("fold_out", C.c_void_p), ("fold_rows", C.c_int32), ("fold_stride", C.c_int32),
                ("amax_best", C.c_void_p), ("amax_ids", C.c_void_p), ("amax_pos", C.c_void_p), ("amax_advance", C.c_int32)]


class RouterFoldArgs(C.Structure):
    _fields_ = [("router", C.c_void_p), ("shared_gate", C.c_void_p), ("gamma", C.c_void_p), ("w_out", C.c_void_p),
                ("out", C.c_void_p), ("scratch", C.c_void_p), ("n_expert", C.c_int32), ("n_embd", C.c_int32),
                ("k", C.c_int32)]


class DequantQ4KArgs(C.Structure):
    _fields_ = [("w", C.c_void_p), ("dst", C.c_void_p), ("rows", C.c_int64), ("k", C.c_int32)]


class DequantArgs(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("n", C.c_int64), ("type", C.c_int32)]


class GemvArgs(C.Structure):
    _fields_ = [("w", C.c_void_p), ("x", C.c_void_p), ("y", C.c_void_p), ("residual", C.c_void_p),
                ("n", C.c_int32), ("k", C.c_int32), ("type", C.c_int32), ("n_tok", C.c_int32), ("gamma", C.c_void_p),
                ("eps", C.c_float), ("x_stride", C.c_int32), ("y_stride", C.c_int32)]


class QuantizeQ4KArgs(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("rows", C.c_int64), ("k", C.c_int32)]


class FillNormalArgs(C.Structure):
    _fields_ = [("dst", C.c_void_p), ("n", C.c_int64), ("seed", C.c_uint64), ("mean", C.c_float),
                ("std", C.c_float), ("half", C.c_int32)]


class MoeRouterArgs(C.Structure):
    _fields_ = [("h", C.c_void_p), ("gamma", C.c_void_p), ("router", C.c_void_p),
                ("shared_gate", C.c_void_p), ("xn", C.c_void_p), ("logits", C.c_void_p),
                ("topk", C.c_void_p), ("weights", C.c_void_p), ("n_tok", C.c_int32),
                ("n_embd", C.c_int32), ("n_expert", C.c_int32), ("n_used", C.c_int32),
                ("eps", C.c_float), ("h_stride", C.c_int32), ("defer_route", C.c_int32)]


class MoeUpArgs(C.Structure):
    _fields_ = [("xn", C.c_void_p), ("topk", C.c_void_p), ("gate_exps", C.c_void_p),
                ("up_exps", C.c_void_p), ("gate_sh", C.c_void_p), ("up_sh", C.c_void_p),
                ("act", C.c_void_p), ("n_tok", C.c_int32), ("n_embd", C.c_int32),
                ("n_used", C.c_int32), ("ffn", C.c_int32), ("logits", C.c_void_p),
                ("weights", C.c_void_p), ("n_expert", C.c_int32), ("gate_type", C.c_int32),
                ("up_type", C.c_int32), ("gate_sh_type", C.c_int32), ("up_sh_type", C.c_int32),
                ("group", C.c_void_p), ("no_shared_gate", C.c_int32), ("act_packed", C.c_int32),
                ("gamma", C.c_void_p), ("eps", C.c_float), ("shared_gate", C.c_void_p)]


class MoeDownArgs(C.Structure):
    _fields_ = [("act", C.c_void_p), ("topk", C.c_void_p), ("weights", C.c_void_p),
                ("down_exps", C.c_void_p), ("down_sh", C.c_void_p), ("residual", C.c_void_p),
                ("out", C.c_void_p), ("n_tok", C.c_int32), ("n_embd", C.c_int32),
                ("n_used", C.c_int32), ("ffn", C.c_int32), ("res_stride", C.c_int32),
                ("out_stride", C.c_int32), ("down_type", C.c_int32), ("down_sh_type", C.c_int32),
                ("n_expert", C.c_int32), ("group", C.c_void_p), ("pairs", C.c_void_p), ("group_ready", C.c_int32), ("act_packed", C.c_int32)]


class DnStepArgs(C.Structure):
    _fields_ = [("ring", C.c_void_p), ("conv1d", C.c_void_p), ("a", C.c_void_p),
                ("dt_bias", C.c_void_p), ("state", C.c_void_p), ("out", C.c_void_p),
                ("pos", C.c_void_p), ("slot", C.c_void_p), ("n_seq", C.c_int32),
                ("seq_len", C.c_int32), ("n_head_k", C.c_int32), ("n_head_v", C.c_int32),
                ("head_dim", C.c_int32), ("conv", C.c_int32), ("ring_slots", C.c_int32),
                ("ring_stride", C.c_int32), ("eps", C.c_float), ("qk_norm_max", C.c_int32),
                ("plane", C.c_void_p), ("n_planes", C.c_int32), ("spec", C.c_int32),
                ("work", C.c_void_p), ("work_floats", C.c_int64)]


class AttnDecodeArgs(C.Structure):
    _fields_ = [("qkv", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p),
                ("rope", C.c_void_p), ("kcache", C.c_void_p), ("vcache", C.c_void_p),
                ("partial", C.c_void_p), ("out", C.c_void_p), ("pos", C.c_void_p),
                ("slot", C.c_void_p), ("n_seq", C.c_int32), ("seq_len", C.c_int32),
                ("n_head", C.c_int32), ("n_head_kv", C.c_int32), ("head_dim", C.c_int32),
                ("rope_dims", C.c_int32), ("max_cells", C.c_int32), ("qkv_stride", C.c_int32),
                ("n_splits", C.c_int32), ("eps", C.c_float), ("mask", C.c_void_p), ("mask_stride", C.c_int32)]


class QsaIndexArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("gamma", C.c_void_p), ("w", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p),
                ("rope", C.c_void_p), ("idxcache", C.c_void_p), ("pooled", C.c_void_p), ("pos", C.c_void_p), ("slot", C.c_void_p),
                ("work", C.c_void_p), ("score", C.c_void_p), ("mask", C.c_void_p), ("n_seq", C.c_int32), ("seq_len", C.c_int32),
                ("n_embd", C.c_int32), ("idx_heads", C.c_int32), ("idx_dim", C.c_int32), ("top_k", C.c_int32), ("ratio", C.c_int32),
                ("rope_dims", C.c_int32), ("max_cells", C.c_int32), ("mask_stride", C.c_int32), ("eps", C.c_float)]


class EmbedArgs(C.Structure):
    _fields_ = [("table", C.c_void_p), ("ids", C.c_void_p), ("pos", C.c_void_p), ("x", C.c_void_p),
                ("n_tok", C.c_int32), ("n_embd", C.c_int32), ("vocab", C.c_int32),
                ("x_stride", C.c_int32), ("type", C.c_int32)]


class ArgmaxArgs(C.Structure):
    _fields_ = [("logits", C.c_void_p), ("best", C.c_void_p), ("ids", C.c_void_p),
                ("pos", C.c_void_p), ("n_rows", C.c_int32), ("n", C.c_int32),
                ("logits_stride", C.c_int32), ("advance", C.c_int32)]


class AdvanceArgs(C.Structure):
    _fields_ = [("pos", C.c_void_p), ("n_seq", C.c_int32), ("delta", C.c_int32)]


class RingRowsArgs(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("pos", C.c_void_p), ("src_slots", C.c_int32),
                ("dst_slots", C.c_int32), ("stride", C.c_int32), ("n", C.c_int32), ("first", C.c_int32),
                ("count", C.c_int32)]


class Op(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("flags", C.c_uint32), ("args", C.c_uint8 * 248)]


def make_op(kind, args, flags=0):
    op = Op()
    op.kind, op.flags = kind, flags
    n = C.sizeof(args)
    assert n <= 248, n
    C.memmove(op.args, C.byref(args), n)
    return op


# every symbol include/shv_hip.h declares; the CPU test suite checks the library exports them all
SYMBOLS = [
    "shv_last_error", "shv_device_count", "shv_init", "shv_destroy", "shv_device_props", "shv_sync",
    "shv_submits", "shv_alloc", "shv_free", "shv_upload", "shv_upload_async", "shv_download", "shv_copy", "shv_zero",
    "shv_host_alloc", "shv_host_free", "shv_enqueue", "shv_dispatch_multi", "shv_prerecord",
    "shv_prerecorded_submit", "shv_prerecorded_launch", "shv_stamp", "shv_stamp_elapsed", "shv_prerecorded_count",
    "shv_prerecorded_destroy", "shv_gemv_q4k", "shv_dequant_q4k", "shv_dequant", "shv_gemv", "shv_quantize_q4k",
    "shv_fill_normal", "shv_moe_router", "shv_moe_up", "shv_moe_down", "shv_dn_step", "shv_attn_decode", "shv_embed", "shv_argmax", "shv_advance",
    "shv_argmax_static", "shv_ring_rows", "shv_router_fold", "shv_qsa_index",
]

_lib = None


def load():
    """Load libshv_hip.so.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    p = lib_path()
    if not os.path.exists(p):
        raise ShvError(-4, "%s is missing: build it with `python strix-halo-vulkan_amd/build.py`" % p)
    L = C.CDLL(p)
    vp, vpp = C.c_void_p, C.POINTER(C.c_void_p)
    L.shv_last_error.restype = C.c_char_p
    L.shv_device_count.argtypes = [C.POINTER(C.c_int)]
    L.shv_init.argtypes = [C.c_int, vpp]
    L.shv_destroy.argtypes = [vp]
    L.shv_destroy.restype = None
    L.shv_device_props.argtypes = [vp, C.POINTER(Props)]
    L.shv_sync.argtypes = [vp]
    L.shv_submits.argtypes = [vp, C.POINTER(C.c_uint64)]
    L.shv_alloc.argtypes = [vp, C.c_size_t, vpp]
    L.shv_free.argtypes = [vp, vp]
    L.shv_upload.argtypes = [vp, vp, vp, C.c_size_t]
    L.shv_upload_async.argtypes = [vp, vp, vp, C.c_size_t]
    L.shv_download.argtypes = [vp, vp, vp, C.c_size_t]
    L.shv_copy.argtypes = [vp, vp, vp, C.c_size_t]
    L.shv_zero.argtypes = [vp, vp, C.c_size_t]
    L.shv_host_alloc.argtypes = [vp, C.c_size_t, vpp]
    L.shv_host_free.argtypes = [vp, vp]
    L.shv_enqueue.argtypes = [vp, C.c_uint32, vp, C.c_size_t]
    L.shv_dispatch_multi.argtypes = [vp, C.POINTER(Op), C.c_int, C.c_int, C.POINTER(C.c_uint64),
                                     C.POINTER(C.c_uint64)]
    L.shv_prerecord.argtypes = [vp, C.POINTER(Op), C.c_int, vpp]
    L.shv_prerecorded_submit.argtypes = [vp, vp, C.c_int, C.POINTER(C.c_uint64)]
    L.shv_prerecorded_launch.argtypes = [vp, vp]
    L.shv_stamp.argtypes = [vp, C.c_int]
    L.shv_stamp_elapsed.argtypes = [vp, C.c_int, C.c_int, C.POINTER(C.c_uint64)]
    L.shv_prerecorded_count.argtypes = [vp]
    L.shv_prerecorded_destroy.argtypes = [vp, vp]
    L.shv_prerecorded_destroy.restype = None
    L.shv_gemv_q4k.argtypes = [vp, C.POINTER(GemvQ4KArgs)]
    L.shv_dequant_q4k.argtypes = [vp, C.POINTER(DequantQ4KArgs)]
    L.shv_dequant.argtypes = [vp, C.POINTER(DequantArgs)]
    L.shv_gemv.argtypes = [vp, C.POINTER(GemvArgs)]
    L.shv_quantize_q4k.argtypes = [vp, C.POINTER(QuantizeQ4KArgs)]
    L.shv_fill_normal.argtypes = [vp, C.POINTER(FillNormalArgs)]
    L.shv_moe_router.argtypes = [vp, C.POINTER(MoeRouterArgs)]
    L.shv_moe_up.argtypes = [vp, C.POINTER(MoeUpArgs)]
    L.shv_moe_down.argtypes = [vp, C.POINTER(MoeDownArgs)]
    L.shv_dn_step.argtypes = [vp, C.POINTER(DnStepArgs)]
    L.shv_attn_decode.argtypes = [vp, C.POINTER(AttnDecodeArgs)]
    L.shv_embed.argtypes = [vp, C.POINTER(EmbedArgs)]
    L.shv_argmax.argtypes = [vp, C.POINTER(ArgmaxArgs)]
    L.shv_advance.argtypes = [vp, C.POINTER(AdvanceArgs)]
    L.shv_argmax_static.argtypes = [vp, C.POINTER(ArgmaxArgs)]
    L.shv_ring_rows.argtypes = [vp, C.POINTER(RingRowsArgs)]
    L.shv_router_fold.argtypes = [vp, C.POINTER(RouterFoldArgs)]
    L.shv_qsa_index.argtypes = [vp, C.POINTER(QsaIndexArgs)]
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise ShvError(rc, load().shv_last_error().decode("utf-8", "replace"))


class DeviceBuffer:
    """A device allocation owned by a Context (vk.Buffer's role, vk/engine.go:319-634)."""

    def __init__(self, ctx, nbytes):
        self.ctx, self.nbytes = ctx, int(nbytes)
        p = C.c_void_p()
        check(ctx.L.shv_alloc(ctx.h, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def at(self, byte_offset):
        assert 0 <= byte_offset <= self.nbytes
        return self.ptr + byte_offset

    def write(self, arr, byte_offset=0):
        arr = np.ascontiguousarray(arr)
        assert byte_offset + arr.nbytes <= self.nbytes, (byte_offset, arr.nbytes, self.nbytes)
        check(self.ctx.L.shv_upload(self.ctx.h, self.ptr + byte_offset, arr.ctypes.data, arr.nbytes))
        return self

    def write_async(self, arr, byte_offset=0):
        """write() that does not wait for the device when arr is up to 512 bytes (the array is copied before the
        call returns); ordered before whatever this context does next."""
        arr = np.ascontiguousarray(arr)
        assert byte_offset + arr.nbytes <= self.nbytes, (byte_offset, arr.nbytes, self.nbytes)
        check(self.ctx.L.shv_upload_async(self.ctx.h, self.ptr + byte_offset, arr.ctypes.data, arr.nbytes))
        return self

    def read(self, dtype, count, byte_offset=0):
        out = np.empty(count, dtype=dtype)
        assert byte_offset + out.nbytes <= self.nbytes, (byte_offset, out.nbytes, self.nbytes)
        check(self.ctx.L.shv_download(self.ctx.h, out.ctypes.data, self.ptr + byte_offset, out.nbytes))
        return out

    def zero(self):
        check(self.ctx.L.shv_zero(self.ctx.h, self.ptr, self.nbytes))
        return self

    def free(self):
        if self.ptr:
            check(self.ctx.L.shv_free(self.ctx.h, self.ptr))
            self.ptr = None


class Prerecorded:
    def __init__(self, ctx, ops):
        self.ctx = ctx
        arr = (Op * len(ops))(*ops)
        p = C.c_void_p()
        check(ctx.L.shv_prerecord(ctx.h, arr, len(ops), C.byref(p)))
        self.h = p

    def submit(self, iters=1):
        ns = C.c_uint64()
        check(self.ctx.L.shv_prerecorded_submit(self.ctx.h, self.h, iters, C.byref(ns)))
        return ns.value

    def launch(self):
        check(self.ctx.L.shv_prerecorded_launch(self.ctx.h, self.h))

    def count(self):
        return self.ctx.L.shv_prerecorded_count(self.h)

    def destroy(self):
        if self.h:
            self.ctx.L.shv_prerecorded_destroy(self.ctx.h, self.h)
            self.h = None


class Context:
    """One device, one in-order stream (vk.Device's role, vk/engine.go:266-311)."""

    def __init__(self, device=0):
        self.L = load()
        h = C.c_void_p()
        check(self.L.shv_init(device, C.byref(h)))
        self.h = h
        self._bufs = []

    def props(self):
        p = Props()
        check(self.L.shv_device_props(self.h, C.byref(p)))
        return p

    def alloc(self, nbytes):
        b = DeviceBuffer(self, max(int(nbytes), 16))
        self._bufs.append(b)
        return b

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        return self.alloc(arr.nbytes).write(arr)

    def sync(self):
        check(self.L.shv_sync(self.h))

    def stamp(self, i):
        check(self.L.shv_stamp(self.h, i))

    def stamp_elapsed(self, frm, to):
        ns = C.c_uint64()
        check(self.L.shv_stamp_elapsed(self.h, frm, to, C.byref(ns)))
        return ns.value

    def enqueue(self, kind, args):
        check(self.L.shv_enqueue(self.h, kind, C.byref(args), C.sizeof(args)))

    def dispatch_multi(self, ops, iters=1, per_op=False):
        arr = (Op * len(ops))(*ops)
        total = C.c_uint64()
        per = (C.c_uint64 * len(ops))() if per_op else None
        check(self.L.shv_dispatch_multi(self.h, arr, len(ops), iters, C.byref(total), per))
        return (total.value, list(per)) if per_op else total.value

    def prerecord(self, ops):
        return Prerecorded(self, ops)

    def destroy(self):
        if self.h:
            for b in self._bufs:
                if b.ptr:
                    b.free()
            self._bufs = []
            self.L.shv_destroy(self.h)
            self.h = None

    # ---- convenience wrappers over single ops ----
    def dequant(self, typ, src, dst, n):
        """n elements of ggml tensor type `typ` at src to float32 at dst."""
        a = DequantArgs(_ptr(src), _ptr(dst), n, typ)
        check(self.L.shv_dequant(self.h, C.byref(a)))

    def gemv(self, typ, w, x, y, n, k, residual=None, n_tok=0, gamma=None, eps=0.0, x_stride=0, y_stride=0):
        """y[t] = W pro(x[t]) (+ residual[t]) for W [n][k] of ggml tensor type `typ`; gamma: the RMSNorm prologue."""
        a = GemvArgs(_ptr(w), _ptr(x), _ptr(y), _ptr(residual), n, k, typ, n_tok, _ptr(gamma), eps, x_stride, y_stride)
        check(self.L.shv_gemv(self.h, C.byref(a)))

    def gemv_q4k(self, w, x, y, n, k, n_tok=1, prologue=PRO_NONE, gamma=None, z=None, residual=None,
                 eps=1e-6, head_dim=0, x_stride=None, y_stride=None, z_stride=None, pos=None,
                 ring_slots=0, ring_stride=0, slot=None, seq_len=0, z_ring=0):
        a = gemv_args(w, x, y, n, k, n_tok, prologue, gamma, z, residual, eps, head_dim, x_stride,
                      y_stride, z_stride, pos, ring_slots, ring_stride, slot, seq_len, z_ring)
        check(self.L.shv_gemv_q4k(self.h, C.byref(a)))


def ptr(b):
    """Device address of a DeviceBuffer, an int, or None."""
    return _ptr(b)


def _ptr(b):
    if b is None:
        return None
    return b.ptr if isinstance(b, DeviceBuffer) else int(b)


def gemv_args(w, x, y, n, k, n_tok=1, prologue=PRO_NONE, gamma=None, z=None, residual=None, eps=1e-6,
              head_dim=0, x_stride=None, y_stride=None, z_stride=None, pos=None, ring_slots=0,
              ring_stride=0, slot=None, seq_len=0, z_ring=0):
    a = GemvQ4KArgs()
    a.w, a.x, a.y = _ptr(w), _ptr(x), _ptr(y)
    a.residual, a.gamma, a.z, a.pos = _ptr(residual), _ptr(gamma), _ptr(z), _ptr(pos)
    a.n, a.k, a.n_tok, a.prologue, a.head_dim, a.eps = n, k, n_tok, prologue, head_dim, eps
    a.x_stride = k if x_stride is None else x_stride
    a.y_stride = n if y_stride is None else y_stride
    a.z_stride = k if z_stride is None else z_stride
    a.ring_slots, a.ring_stride, a.slot, a.seq_len = ring_slots, ring_stride, _ptr(slot), seq_len
    a.z_ring = z_ring
    return a
