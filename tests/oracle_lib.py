"""ctypes binding of the CPU oracle (oracle/libshv_oracle.so) for the tests, the smoke check and
the benchmark's CPU-baseline leg.  The oracle is the checker; nothing here is a product path."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB_PATH = os.path.join(ORACLE_DIR, "libshv_oracle.so")

Q4K_BLOCK = 256
Q4K_BYTES = 144

u8p = C.POINTER(C.c_uint8)
u16p = C.POINTER(C.c_uint16)
f32p = C.POINTER(C.c_float)
i32p = C.POINTER(C.c_int32)


def build(force=False):
    src = [os.path.join(ORACLE_DIR, f) for f in ("shv_oracle.c", "shv_oracle.h")]
    if force or not os.path.exists(LIB_PATH) or any(
            os.path.getmtime(s) > os.path.getmtime(LIB_PATH) for s in src):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "-B", "libshv_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return LIB_PATH


class MoeCfg(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("n_embd", "n_expert", "n_used", "ffn_expert", "ffn_shared")]


class MoeW(C.Structure):
    _fields_ = [("router", f32p), ("shared_gate", f32p), ("gate_exps", u8p), ("up_exps", u8p),
                ("down_exps", u8p), ("gate_sh", u8p), ("up_sh", u8p), ("down_sh", u8p)]


class DnCfg(C.Structure):
    _fields_ = [("n_embd", C.c_int), ("head_dim", C.c_int), ("n_head_k", C.c_int),
                ("n_head_v", C.c_int), ("conv", C.c_int), ("eps", C.c_float),
                ("qk_norm_max", C.c_int)]


class DnW(C.Structure):
    _fields_ = [("qkv", u8p), ("z", u8p), ("alpha", u8p), ("beta", u8p), ("out", u8p),
                ("conv1d", f32p), ("a", f32p), ("dt_bias", f32p), ("norm", f32p)]


class AttnCfg(C.Structure):
    _fields_ = [("n_embd", C.c_int), ("n_head", C.c_int), ("n_head_kv", C.c_int),
                ("head_dim", C.c_int), ("rope_dims", C.c_int), ("rope_base", C.c_float),
                ("sections", C.c_int * 4), ("eps", C.c_float)]


class AttnW(C.Structure):
    _fields_ = [("q", u8p), ("k", u8p), ("v", u8p), ("o", u8p), ("q_norm", f32p), ("k_norm", f32p)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(LIB_PATH)
    L.shv_ref_f32_to_f16.restype = C.c_uint16
    L.shv_ref_f32_to_f16.argtypes = [C.c_float]
    L.shv_ref_f16_to_f32.restype = C.c_float
    L.shv_ref_f16_to_f32.argtypes = [C.c_uint16]
    L.shv_ref_f16_round.restype = C.c_float
    L.shv_ref_f16_round.argtypes = [C.c_float]
    L.shv_ref_scale_min_k4.argtypes = [C.c_int, u8p, u8p, u8p]
    L.shv_ref_dequant_q4k.argtypes = [u8p, C.c_int64, f32p]
    L.shv_ref_make_qkx_quants.restype = C.c_float
    L.shv_ref_make_qkx_quants.argtypes = [f32p, C.c_int, C.c_int, f32p, u8p, u8p, C.c_float,
                                          C.c_float, C.c_int, f32p]
    L.shv_ref_quantize_q4k_row.argtypes = [f32p, C.c_int64, u8p]
    L.shv_ref_quantize_q4k.argtypes = [f32p, C.c_int64, C.c_int64, u8p]
    L.shv_ref_matvec.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int]
    L.shv_ref_gemv_q4k.argtypes = [f32p, u8p, f32p, C.c_int, C.c_int, C.c_int]
    for n in ("sigmoid", "silu", "softplus"):
        f = getattr(L, "shv_ref_" + n)
        f.restype = C.c_float
        f.argtypes = [C.c_float]
    L.shv_ref_rmsnorm.argtypes = [f32p, f32p, f32p, C.c_int, C.c_float]
    L.shv_ref_head_norm.argtypes = [f32p, f32p, C.c_int, C.c_int, C.c_float]
    L.shv_ref_argmax.restype = C.c_int32
    L.shv_ref_argmax.argtypes = [f32p, C.c_int64]
    L.shv_ref_softmax.argtypes = [f32p, f32p, C.c_int]
    L.shv_ref_moe_route.argtypes = [C.POINTER(MoeCfg), C.POINTER(MoeW), f32p, C.c_int, f32p, f32p,
                                    i32p, f32p]
    L.shv_ref_moe_block.argtypes = [C.POINTER(MoeCfg), C.POINTER(MoeW), f32p, C.c_int, f32p, f32p,
                                    i32p, f32p, f32p, f32p, f32p, C.c_int]
    L.shv_ref_deltanet_layer.argtypes = [C.POINTER(DnCfg), C.POINTER(DnW), f32p, C.c_int, f32p,
                                         f32p, f32p, f32p, f32p, f32p, f32p, f32p, f32p, f32p,
                                         C.c_int, C.c_int]
    L.shv_ref_delta_rule.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, f32p, f32p, f32p, f32p,
                                     f32p, f32p, f32p, i32p]
    L.shv_ref_rope.argtypes = [C.POINTER(AttnCfg), f32p, i32p, C.c_int, C.c_int, C.c_int]
    L.shv_ref_attn_layer.argtypes = [C.POINTER(AttnCfg), C.POINTER(AttnW), f32p, C.c_int, C.c_int,
                                     u16p, u16p, f32p, f32p, f32p, C.c_int]
    _lib = L
    return L


def _p(a, typ):
    return None if a is None else a.ctypes.data_as(typ)


def F(a):
    assert a is None or (a.dtype == np.float32 and a.flags.c_contiguous)
    return _p(a, f32p)


def B(a):
    assert a is None or (a.dtype == np.uint8 and a.flags.c_contiguous)
    return _p(a, u8p)


def I(a):
    assert a is None or (a.dtype == np.int32 and a.flags.c_contiguous)
    return _p(a, i32p)


def H(a):
    assert a is None or (a.dtype == np.uint16 and a.flags.c_contiguous)
    return _p(a, u16p)


# ---- numpy-level helpers -------------------------------------------------------------------

def q4k_row_bytes(k):
    assert k % Q4K_BLOCK == 0
    return k // Q4K_BLOCK * Q4K_BYTES


def quantize_q4k(w):
    """float32 [rows][k] -> uint8 [rows][k/256*144] with the reference's quantiser."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows, k = w.shape
    out = np.empty((rows, q4k_row_bytes(k)), dtype=np.uint8)
    lib().shv_ref_quantize_q4k(F(w), rows, k, B(out))
    return out


def dequant_q4k(q, k=None):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    nblocks = q.size // Q4K_BYTES
    out = np.empty(nblocks * Q4K_BLOCK, dtype=np.float32)
    lib().shv_ref_dequant_q4k(B(q), nblocks, F(out))
    return out if k is None else out.reshape(-1, k)


def gemv_q4k(wq, x, n, k, threads=1):
    y = np.empty(n, dtype=np.float32)
    lib().shv_ref_gemv_q4k(F(y), B(wq), F(np.ascontiguousarray(x, dtype=np.float32)), n, k, threads)
    return y


def rmsnorm(x, gamma, eps):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    flat, o = x.reshape(-1, x.shape[-1]), out.reshape(-1, x.shape[-1])
    for i in range(flat.shape[0]):
        lib().shv_ref_rmsnorm(F(o[i]), F(flat[i]), F(gamma), x.shape[-1], eps)
    return out


def rel_l2(got, want):
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    den = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / (den if den > 0 else 1.0))
