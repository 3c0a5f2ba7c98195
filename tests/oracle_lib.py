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
                ("down_exps", u8p), ("gate_sh", u8p), ("up_sh", u8p), ("down_sh", u8p), ("types", C.c_int * 6)]


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
                ("sections", C.c_int * 4), ("eps", C.c_float),
                ("idx_heads", C.c_int), ("idx_dim", C.c_int), ("top_k", C.c_int), ("ratio", C.c_int)]


class AttnW(C.Structure):
    _fields_ = [("q", u8p), ("k", u8p), ("v", u8p), ("o", u8p), ("q_norm", f32p), ("k_norm", f32p),
                ("idx_q", f32p), ("idx_k", f32p), ("idx_q_norm", f32p), ("idx_k_norm", f32p)]


class ModelCfg(C.Structure):
    _fields_ = [("n_layer", C.c_int), ("n_embd", C.c_int), ("vocab", C.c_int), ("attn_every", C.c_int),
                ("eps", C.c_float), ("max_cells", C.c_int), ("moe", MoeCfg), ("dn", DnCfg), ("attn", AttnCfg)]


class LayerW(C.Structure):
    _fields_ = [("attn_norm", f32p), ("ffn_norm", f32p), ("dn", DnW), ("attn", AttnW), ("moe", MoeW)]


class ModelW(C.Structure):
    _fields_ = [("embd", u16p), ("out_norm", f32p), ("lm_head", u8p), ("layers", C.POINTER(LayerW))]


class ModelState(C.Structure):
    _fields_ = [("dn_conv", C.POINTER(f32p)), ("dn_s", C.POINTER(f32p)), ("kcache", C.POINTER(u16p)),
                ("vcache", C.POINTER(u16p)), ("past", C.c_int), ("idxcache", C.POINTER(u16p))]


class MtpW(C.Structure):
    _fields_ = [("enorm", f32p), ("hnorm", f32p), ("eh_proj", u8p), ("head_norm", f32p), ("layer", LayerW)]


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
    L.shv_ref_dequant.argtypes = [C.c_int, u8p, C.c_int64, f32p]
    L.shv_ref_dequant.restype = C.c_int
    L.shv_ref_type_bytes.argtypes = [C.c_int, C.c_int64]
    L.shv_ref_type_bytes.restype = C.c_int64
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
    L.shv_ref_f2ui.restype = C.c_uint32
    L.shv_ref_f2ui.argtypes = [C.c_float]
    L.shv_ref_topk_threshold.restype = C.c_uint32
    L.shv_ref_topk_threshold.argtypes = [f32p, C.c_int, C.c_int]
    L.shv_ref_topk.restype = C.c_int
    L.shv_ref_topk.argtypes = [f32p, C.c_int, C.c_int, i32p]
    L.shv_ref_attn_layer_qsa.argtypes = [C.POINTER(AttnCfg), C.POINTER(AttnW), f32p, C.c_int, C.c_int, u16p, u16p, u16p,
                                         C.c_int, f32p, f32p, f32p, i32p, i32p, f32p, C.c_int]
    L.shv_ref_model_extend.argtypes = [C.POINTER(ModelCfg), C.POINTER(ModelW), C.POINTER(ModelState), i32p,
                                       C.c_int, f32p, f32p, C.c_int]
    L.shv_ref_model_extend_rows.argtypes = L.shv_ref_model_extend.argtypes
    L.shv_ref_mtp_rows.argtypes = [C.POINTER(ModelCfg), C.POINTER(ModelW), C.POINTER(MtpW), u16p, u16p, f32p, i32p,
                                   C.c_int, C.c_int, f32p, f32p, C.c_int]
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


GGML_TYPES = {"F32": 0, "F16": 1, "Q4_1": 3, "Q5_0": 6, "Q5_1": 7, "Q8_0": 8, "Q4_K": 12, "Q5_K": 13, "Q6_K": 14,
              "IQ4_NL": 20, "BF16": 30}


def type_bytes(typ, n):
    return int(lib().shv_ref_type_bytes(typ, n))


def dequant(typ, data, n):
    """n elements of a ggml tensor type to float32 (the reference's gguf.Dequantize)."""
    data = np.ascontiguousarray(data, dtype=np.uint8)
    assert data.size == type_bytes(typ, n), (typ, n, data.size)
    out = np.empty(n, dtype=np.float32)
    if lib().shv_ref_dequant(typ, B(data), n, F(out)) != 0:
        raise ValueError("type %d is not dequantisable" % typ)
    return out


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


class OracleModel:
    """The CPU token loop over a model whose tensors are given by GGUF-style name (numpy arrays):
    Q4_K tensors as bytes, the embedding as binary16 bit patterns, the rest float32."""

    def __init__(self, cfg, tensors, max_cells, sections=(11, 11, 10, 0), bank_types=None):
        """cfg: any object with the fields of the host layer's config.  bank_types: {tensor name:
        ggml type} for expert banks held in another type than Q4_K."""
        self.cfg, self.t, self.keep = cfg, tensors, []
        ne, d = cfg.n_embd, cfg.ssm_head_dim
        self.mcfg = ModelCfg(
            cfg.n_layer, ne, cfg.vocab, cfg.attn_every, cfg.rms_eps, max_cells,
            MoeCfg(ne, cfg.n_expert, cfg.n_expert_used, cfg.ffn_expert, cfg.ffn_expert),
            DnCfg(ne, d, cfg.ssm_head_k, cfg.ssm_head_v, cfg.ssm_conv, cfg.rms_eps, 0),
            AttnCfg(ne, cfg.n_head, cfg.n_head_kv, cfg.head_dim, cfg.rope_dims, cfg.rope_base,
                    (C.c_int * 4)(*sections), cfg.rms_eps, getattr(cfg, "idx_heads", 0), getattr(cfg, "idx_dim", 0),
                    getattr(cfg, "idx_top_k", 0), getattr(cfg, "idx_ratio", 0)))
        self.qsa = getattr(cfg, "idx_ratio", 0) > 0
        blk = lambda l, n: tensors["blk.%d.%s.weight" % (l, n)]
        layers = (LayerW * cfg.n_layer)()
        for l in range(cfg.n_layer):
            lw = layers[l]
            lw.attn_norm, lw.ffn_norm = F(blk(l, "attn_norm")), F(blk(l, "post_attention_norm"))
            if (l + 1) % cfg.attn_every == 0:
                lw.attn = AttnW(B(blk(l, "attn_q")), B(blk(l, "attn_k")), B(blk(l, "attn_v")),
                                B(blk(l, "attn_output")), F(blk(l, "attn_q_norm")), F(blk(l, "attn_k_norm")))
                if self.qsa:
                    lw.attn.idx_q, lw.attn.idx_k = F(blk(l, "indexer.q_proj")), F(blk(l, "indexer.k_proj"))
                    lw.attn.idx_q_norm, lw.attn.idx_k_norm = F(blk(l, "indexer.q_norm")), F(blk(l, "indexer.k_norm"))
            else:
                lw.dn = DnW(B(blk(l, "attn_qkv")), B(blk(l, "attn_gate")), B(blk(l, "ssm_alpha")),
                            B(blk(l, "ssm_beta")), B(blk(l, "ssm_out")), F(blk(l, "ssm_conv1d")),
                            F(blk(l, "ssm_a")), F(blk(l, "ssm_dt")), F(blk(l, "ssm_norm")))
            lw.moe = MoeW(F(blk(l, "ffn_gate_inp")), F(blk(l, "ffn_gate_inp_shexp")), B(blk(l, "ffn_gate_exps")),
                          B(blk(l, "ffn_up_exps")), B(blk(l, "ffn_down_exps")), B(blk(l, "ffn_gate_shexp")),
                          B(blk(l, "ffn_up_shexp")), B(blk(l, "ffn_down_shexp")),
                          (C.c_int * 6)(*[(bank_types or {}).get("blk.%d.ffn_%s.weight" % (l, n), 0) for n in
                                          ("gate_exps", "up_exps", "down_exps", "gate_shexp", "up_shexp", "down_shexp")]))
        self.layers = layers
        self.w = ModelW(H(tensors["token_embd.weight"]), F(tensors["output_norm.weight"]),
                        B(tensors["output.weight"]), layers)
        self.max_cells = max_cells
        self.reset()

    def reset(self):
        c, n = self.cfg, self.cfg.n_layer
        cw = 2 * c.ssm_head_k * c.ssm_head_dim + c.ssm_head_v * c.ssm_head_dim
        self.dn_conv, self.dn_s, self.kc, self.vc = [None] * n, [None] * n, [None] * n, [None] * n
        self.ic = [None] * n   # the indexer's raw keys, attention layers of a model that has one
        a_conv, a_s, a_k, a_v, a_i = (f32p * n)(), (f32p * n)(), (u16p * n)(), (u16p * n)(), (u16p * n)()
        for l in range(n):
            if (l + 1) % c.attn_every == 0:
                self.kc[l] = np.zeros((self.max_cells, c.n_head_kv, c.head_dim), np.uint16)
                self.vc[l] = np.zeros_like(self.kc[l])
                a_k[l], a_v[l] = H(self.kc[l]), H(self.vc[l])
                if self.qsa:
                    self.ic[l] = np.zeros((self.max_cells, c.idx_dim), np.uint16)
                    a_i[l] = H(self.ic[l])
            else:
                self.dn_conv[l] = np.zeros((cw, c.ssm_conv - 1), np.float32)
                self.dn_s[l] = np.zeros((c.ssm_head_v, c.ssm_head_dim, c.ssm_head_dim), np.float32)
                a_conv[l], a_s[l] = F(self.dn_conv[l]), F(self.dn_s[l])
        self.arrays = (a_conv, a_s, a_k, a_v, a_i)
        self.state = ModelState(a_conv, a_s, a_k, a_v, 0, a_i if self.qsa else None)

    def extend(self, ids, threads=8):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        logits = np.empty(self.cfg.vocab, np.float32)
        hidden = np.empty(self.cfg.n_embd, np.float32)
        lib().shv_ref_model_extend(C.byref(self.mcfg), C.byref(self.w), C.byref(self.state), I(ids), len(ids),
                                   F(logits), F(hidden), threads)
        return logits, hidden

    @property
    def past(self):
        return self.state.past

    def extend_rows(self, ids, threads=8):
        """every row's logits [n][vocab] and residual [n][n_embd] (the verification pass)"""
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        logits = np.empty((len(ids), self.cfg.vocab), np.float32)
        hidden = np.empty((len(ids), self.cfg.n_embd), np.float32)
        lib().shv_ref_model_extend_rows(C.byref(self.mcfg), C.byref(self.w), C.byref(self.state), I(ids), len(ids),
                                        F(logits), F(hidden), threads)
        return logits, hidden

    def snapshot(self):
        """the carried state, to come back to with restore()"""
        cp = lambda xs: [None if a is None else a.copy() for a in xs]
        return cp(self.dn_conv), cp(self.dn_s), cp(self.kc), cp(self.vc), self.state.past, cp(self.ic)

    def restore(self, snap):
        for dst, src in zip((self.dn_conv, self.dn_s, self.kc, self.vc, self.ic), snap[:4] + (snap[5],)):
            for d, s_ in zip(dst, src):
                if d is not None:
                    d[...] = s_
        self.state.past = snap[4]


class OracleMTP:
    """The draft head on the CPU over the draft block's tensors (block n_layer of the same model)."""

    def __init__(self, om, max_cells):
        cfg, t = om.cfg, om.t
        self.om = om
        blk = lambda n: t["blk.%d.%s.weight" % (cfg.n_layer, n)]
        lw = LayerW()
        lw.attn_norm, lw.ffn_norm = F(blk("attn_norm")), F(blk("post_attention_norm"))
        lw.attn = AttnW(B(blk("attn_q")), B(blk("attn_k")), B(blk("attn_v")), B(blk("attn_output")),
                        F(blk("attn_q_norm")), F(blk("attn_k_norm")))
        lw.moe = MoeW(F(blk("ffn_gate_inp")), F(blk("ffn_gate_inp_shexp")), B(blk("ffn_gate_exps")),
                      B(blk("ffn_up_exps")), B(blk("ffn_down_exps")), B(blk("ffn_gate_shexp")),
                      B(blk("ffn_up_shexp")), B(blk("ffn_down_shexp")))
        self.w = MtpW(F(blk("nextn.enorm")), F(blk("nextn.hnorm")), B(blk("nextn.eh_proj")),
                      F(blk("nextn.shared_head_norm")), lw)
        self.kc = np.zeros((max_cells, cfg.n_head_kv, cfg.head_dim), np.uint16)
        self.vc = np.zeros_like(self.kc)

    def rows(self, hs, ids, pos, threads=8):
        cfg = self.om.cfg
        hs = np.ascontiguousarray(hs, dtype=np.float32).reshape(-1, cfg.n_embd)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        assert hs.shape[0] == len(ids)
        logits = np.empty(cfg.vocab, np.float32)
        res = np.empty((len(ids), cfg.n_embd), np.float32)
        lib().shv_ref_mtp_rows(C.byref(self.om.mcfg), C.byref(self.om.w), C.byref(self.w), H(self.kc), H(self.vc),
                               F(hs), I(ids), len(ids), pos, F(logits), F(res), threads)
        return logits, res
