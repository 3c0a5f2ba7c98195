"""Pins the oracle's block-level functions by what the mathematics fixes, since the reference
holds no vector for them that can be used without its checkpoint: float64 re-derivations written
independently in numpy, closed forms, invariants the reference's own tests state
(llm/deltanet_test.go:234-320, llm/attn_test.go:87-129, llm/sample_test.go:17, llm/moe_test.go),
and constructed edge cases.  Each check is chosen so that a plausible slip (a dropped term, a
transposed state, a wrong head map, the wrong nibble order) fails it."""
import numpy as np
import pytest

import oracle_lib as O

EPS = 1e-6
L = O.lib()


def q4(rng, rows, k, std=0.02):
    return O.quantize_q4k((rng.standard_normal((rows, k)) * std).astype(np.float32))


def deq(q, k):
    return O.dequant_q4k(q, k).astype(np.float64)


# ------------------------------------------------------------------ dense helpers ----------------

def test_gemv_is_dequant_then_dot():
    rng = np.random.default_rng(1)
    n, k = 96, 1024
    wq = q4(rng, n, k)
    x = rng.standard_normal(k).astype(np.float32)
    want = deq(wq, k) @ x.astype(np.float64)
    for threads in (1, 5):
        got = O.gemv_q4k(wq, x, n, k, threads)
        assert O.rel_l2(got, want) < 2e-6
    assert np.array_equal(O.gemv_q4k(wq, x, n, k, 1), O.gemv_q4k(wq, x, n, k, 7))  # threads change no value
    # sequential float32 accumulation, not pairwise and not float64: reproduce it exactly
    w32 = O.dequant_q4k(wq, k)
    s = np.float32(0)
    for i in range(k):
        s = np.float32(s + np.float32(w32[3, i] * x[i]))
    assert O.gemv_q4k(wq, x, n, k, 1)[3] == s


def test_rmsnorm_and_head_norm_against_float64():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((5, 2048)) * 3).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(2048)).astype(np.float32)
    want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + EPS) * g
    assert O.rel_l2(O.rmsnorm(x, g, EPS), want) < 1e-6
    h = x.reshape(-1, 256).copy()
    gh = g[:256].copy()
    wanth = h.astype(np.float64) / np.sqrt((h.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + EPS) * gh
    L.shv_ref_head_norm(O.F(h), O.F(gh), 256, h.shape[0], EPS)
    assert O.rel_l2(h, wanth) < 1e-6
    z = np.zeros((1, 64), np.float32)
    assert np.array_equal(O.rmsnorm(z, np.ones(64, np.float32), EPS), z)  # eps keeps a zero row finite


def test_scalar_activations():
    for v in (-30.0, -3.5, 0.0, 0.7, 12.0):
        assert abs(L.shv_ref_sigmoid(v) - 1 / (1 + np.exp(-v))) < 1e-7
        assert abs(L.shv_ref_silu(v) - v / (1 + np.exp(-v))) < 1e-6 * max(1, abs(v))
    # softplus: the reference's two documented edges (llm/deltanet.go:445-455)
    assert L.shv_ref_softplus(20.5) == np.float32(20.5)          # identity above 20
    assert L.shv_ref_softplus(-17.0) == 0.0                      # float32 add flushes to exactly 0
    assert L.shv_ref_softplus(-16.0) > 0.0
    for v in (-5.0, 0.0, 3.0, 19.9):
        assert abs(L.shv_ref_softplus(v) - np.log1p(np.exp(v))) < 2e-7 * max(1, abs(v)) + 6e-8


def test_argmax_first_maximum():
    rng = np.random.default_rng(3)
    x = rng.standard_normal(5000).astype(np.float32)
    assert L.shv_ref_argmax(O.F(x), x.size) == int(np.argmax(x))
    x[[40, 4000]] = 9.0
    assert L.shv_ref_argmax(O.F(x), x.size) == 40                 # ties go to the lowest id
    n = np.full(10, np.nan, np.float32)
    assert L.shv_ref_argmax(O.F(n), 10) == 0                      # NaN never wins


# --------------------------------------------------------------------------- MoE ---------------

def moe_setup(rng, H=512, E=16, used=4, ffn=256, T=3):
    w = dict(router=(rng.standard_normal((E, H)) * 0.05).astype(np.float32),
             shared_gate=(rng.standard_normal(H) * 0.05).astype(np.float32),
             gate_exps=q4(rng, E * ffn, H), up_exps=q4(rng, E * ffn, H), down_exps=q4(rng, E * H, ffn),
             gate_sh=q4(rng, ffn, H), up_sh=q4(rng, ffn, H), down_sh=q4(rng, H, ffn))
    x = rng.standard_normal((T, H)).astype(np.float32)
    cfg = O.MoeCfg(H, E, used, ffn, ffn)
    mw = O.MoeW(O.F(w["router"]), O.F(w["shared_gate"]), O.B(w["gate_exps"]), O.B(w["up_exps"]),
                O.B(w["down_exps"]), O.B(w["gate_sh"]), O.B(w["up_sh"]), O.B(w["down_sh"]))
    return cfg, mw, w, x


def run_moe(cfg, mw, x):
    T = x.shape[0]
    r = dict(out=np.empty((T, cfg.n_embd), np.float32), logits=np.empty((T, cfg.n_expert), np.float32),
             topk=np.empty((T, cfg.n_used), np.int32), weights=np.empty((T, cfg.n_used), np.float32),
             moe_out=np.empty((T, cfg.n_embd), np.float32), sig=np.empty(T, np.float32))
    L.shv_ref_moe_block(O.C.byref(cfg), O.C.byref(mw), O.F(x), T, O.F(r["out"]), O.F(r["logits"]), O.I(r["topk"]),
                        O.F(r["weights"]), None, O.F(r["moe_out"]), O.F(r["sig"]), 1)
    return r


def test_route_against_numpy():
    rng = np.random.default_rng(4)
    cfg, mw, w, x = moe_setup(rng)
    r = run_moe(cfg, mw, x)
    lg = x.astype(np.float64) @ w["router"].astype(np.float64).T
    assert O.rel_l2(r["logits"], lg) < 1e-6
    p = np.exp(lg - lg.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    order = np.argsort(-p, axis=1, kind="stable")[:, :cfg.n_used]
    assert np.array_equal(r["topk"], order)                       # descending, tie-free input
    sel = np.take_along_axis(p, order, axis=1)
    assert np.allclose(r["weights"], sel / sel.sum(axis=1, keepdims=True), rtol=1e-5)
    assert np.allclose(r["weights"].sum(axis=1), 1, atol=1e-6)
    assert (np.diff(r["weights"], axis=1) <= 0).all()


def test_route_ties_clamp_and_softmax():
    rng = np.random.default_rng(5)
    cfg, mw, w, x = moe_setup(rng)
    w["router"][:] = w["router"][0]                               # every logit equal
    r = run_moe(cfg, mw, x)
    assert np.array_equal(r["topk"], np.tile(np.arange(cfg.n_used, dtype=np.int32), (x.shape[0], 1)))
    assert np.allclose(r["weights"], 1 / cfg.n_used)
    # ties inside the selection keep ascending index order (sort.SliceStable, llm/moe.go:249-252)
    w["router"][:] = 0
    w["router"][[9, 2, 11], 0] = 1.0
    xx = np.zeros_like(x)
    xx[:, 0] = 2.0
    rr = run_moe(cfg, mw, xx)
    assert list(rr["topk"][0][:3]) == [2, 9, 11]
    # softmax alone: sums to one, shift invariant
    src = rng.standard_normal(64).astype(np.float32)
    a, b = np.empty(64, np.float32), np.empty(64, np.float32)
    L.shv_ref_softmax(O.F(a), O.F(src), 64)
    L.shv_ref_softmax(O.F(b), O.F((src + 5).astype(np.float32)), 64)
    assert abs(a.sum() - 1) < 1e-6 and np.allclose(a, b, atol=1e-7)
    # the clamp at 2^-14 is inert unless the selected mass is below it: force it with many experts
    # holding nearly all the mass outside the selection
    cfg2 = O.MoeCfg(cfg.n_embd, cfg.n_expert, 1, cfg.ffn_expert, cfg.ffn_shared)
    logits = np.empty((1, cfg.n_expert), np.float32)
    probs = np.empty_like(logits)
    topk = np.empty((1, 1), np.int32)
    wn = np.empty((1, 1), np.float32)
    L.shv_ref_moe_route(O.C.byref(cfg2), O.C.byref(mw), O.F(xx[:1]), 1, O.F(logits), O.F(probs), O.I(topk), O.F(wn))
    assert abs(wn[0, 0] - 1.0) < 1e-6                             # one expert: weight is p/p = 1


def test_moe_block_against_dense_float64():
    """Brute force: dequantise every expert, mask by the selection, compare."""
    rng = np.random.default_rng(6)
    cfg, mw, w, x = moe_setup(rng)
    r = run_moe(cfg, mw, x)
    H, E, ffn = cfg.n_embd, cfg.n_expert, cfg.ffn_expert
    G, U, D = deq(w["gate_exps"], H).reshape(E, ffn, H), deq(w["up_exps"], H).reshape(E, ffn, H), deq(w["down_exps"], ffn).reshape(E, H, ffn)
    silu = lambda v: v / (1 + np.exp(-v))
    for t in range(x.shape[0]):
        xt = x[t].astype(np.float64)
        routed = np.zeros(H)
        for k in range(cfg.n_used):
            e = r["topk"][t, k]
            routed += r["weights"][t, k] * (D[e] @ (silu(G[e] @ xt) * (U[e] @ xt)))
        assert O.rel_l2(r["moe_out"][t], routed) < 1e-5
        sh = deq(w["down_sh"], ffn) @ (silu(deq(w["gate_sh"], H) @ xt) * (deq(w["up_sh"], H) @ xt))
        gate = 1 / (1 + np.exp(-(w["shared_gate"].astype(np.float64) @ xt)))
        assert abs(r["sig"][t] - gate) < 1e-6
        assert O.rel_l2(r["out"][t], routed + gate * sh) < 1e-5


# ---------------------------------------------------------------------- DeltaNet ---------------

def dn_setup(rng, H=512, hk=2, hv=4, d=128):
    qk, vw = hk * d, hv * d
    cw = 2 * qk + vw
    w = dict(qkv=q4(rng, cw, H, 0.05), z=q4(rng, vw, H, 0.05), alpha=q4(rng, hv, H, 0.05), beta=q4(rng, hv, H, 0.05),
             out=q4(rng, H, vw), conv1d=(rng.standard_normal((cw, 4)) * 0.3).astype(np.float32),
             a=(-np.exp(rng.standard_normal(hv))).astype(np.float32), dt=rng.standard_normal(hv).astype(np.float32),
             norm=(1 + 0.1 * rng.standard_normal(d)).astype(np.float32))
    cfg = O.DnCfg(H, d, hk, hv, 4, EPS, 0)
    dw = O.DnW(O.B(w["qkv"]), O.B(w["z"]), O.B(w["alpha"]), O.B(w["beta"]), O.B(w["out"]), O.F(w["conv1d"]),
               O.F(w["a"]), O.F(w["dt"]), O.F(w["norm"]))
    return cfg, dw, w, (qk, vw, cw)


def run_dn(cfg, dw, x, conv, S, divide=0, traces=False):
    T = x.shape[0]
    hv, hk, d = cfg.n_head_v, cfg.n_head_k, cfg.head_dim
    res = np.empty((T, cfg.n_embd), np.float32)
    tr = dict(qkv=np.empty((T, 2 * hk * d + hv * d), np.float32), qn=np.empty((T, hk, d), np.float32),
              kn=np.empty((T, hk, d), np.float32), gate=np.empty((T, hv), np.float32),
              bsig=np.empty((T, hv), np.float32), attn=np.empty((T, hv, d), np.float32),
              final=np.empty((T, hv * d), np.float32))
    L.shv_ref_deltanet_layer(O.C.byref(cfg), O.C.byref(dw), O.F(x), T, O.F(conv), O.F(S), O.F(res), O.F(tr["qkv"]),
                             O.F(tr["qn"]), O.F(tr["kn"]), O.F(tr["gate"]), O.F(tr["bsig"]), O.F(tr["attn"]),
                             O.F(tr["final"]), divide, 1)
    return (res, tr) if traces else res


def test_deltanet_chunk_split_is_bit_identical():
    """llm/deltanet_test.go:280-320: 3 + 4 tokens == 7 tokens, output and state, bit for bit; and
    the negative control: dropping the carried state must change the answer."""
    rng = np.random.default_rng(7)
    cfg, dw, w, (qk, vw, cw) = dn_setup(rng)
    x = rng.standard_normal((7, cfg.n_embd)).astype(np.float32)
    z = lambda: (np.zeros((cw, 3), np.float32), np.zeros((cfg.n_head_v, 128, 128), np.float32))
    c1, s1 = z()
    whole = run_dn(cfg, dw, x, c1, s1)
    c2, s2 = z()
    a = run_dn(cfg, dw, x[:3], c2, s2)
    b = run_dn(cfg, dw, x[3:], c2, s2)
    assert np.array_equal(np.concatenate([a, b]), whole)
    assert np.array_equal(s1, s2) and np.array_equal(c1, c2)
    c3, s3 = z()
    fresh = run_dn(cfg, dw, x[3:], c3, s3)
    assert not np.allclose(fresh, whole[3:], rtol=1e-3)


def test_deltanet_against_independent_float64_recurrence():
    """The layer re-derived in numpy float64 from the paper's form S <- S*g + k (beta (v - S^T k))^T,
    o = S^T q / sqrt(d), with the state held UNtransposed: catches a transposed state, a wrong
    head map, a conv window slip, a missing beta or decay."""
    rng = np.random.default_rng(8)
    cfg, dw, w, (qk, vw, cw) = dn_setup(rng)
    hk, hv, d, H = cfg.n_head_k, cfg.n_head_v, cfg.head_dim, cfg.n_embd
    T = 6
    x = rng.standard_normal((T, H)).astype(np.float32)
    conv, S = np.zeros((cw, 3), np.float32), np.zeros((hv, d, d), np.float32)
    res, tr = run_dn(cfg, dw, x, conv, S, traces=True)
    X = x.astype(np.float64)
    mixed = X @ deq(w["qkv"], H).T
    zz = X @ deq(w["z"], H).T
    al = X @ deq(w["alpha"], H).T
    be = X @ deq(w["beta"], H).T
    softplus = lambda v: np.where(v > 20, v, np.log1p(np.exp(np.minimum(v, 20))))
    gate = softplus(al + w["dt"]) * w["a"]
    bsig = 1 / (1 + np.exp(-be))
    pad = np.concatenate([np.zeros((3, cw)), mixed])
    convd = sum(pad[j:j + T] * w["conv1d"][:, j].astype(np.float64) for j in range(4))
    act = convd / (1 + np.exp(-convd))
    q, k, v = act[:, :qk].reshape(T, hk, d), act[:, qk:2 * qk].reshape(T, hk, d), act[:, 2 * qk:].reshape(T, hv, d)
    qn = q / np.sqrt((q ** 2).sum(-1, keepdims=True) + EPS)
    kn = k / np.sqrt((k ** 2).sum(-1, keepdims=True) + EPS)
    Sm = np.zeros((hv, d, d))          # S[i][j]: key axis i, value axis j
    out = np.zeros((T, hv, d))
    for t in range(T):
        for h in range(hv):
            kk, qq = kn[t, h % hk], qn[t, h % hk]
            Sm[h] *= np.exp(gate[t, h])
            delta = (v[t, h] - Sm[h].T @ kk) * bsig[t, h]
            Sm[h] += np.outer(kk, delta)
            out[t, h] = Sm[h].T @ qq / np.sqrt(d)
    assert O.rel_l2(tr["qkv"], mixed) < 1e-5
    assert O.rel_l2(tr["gate"], gate) < 1e-5 and O.rel_l2(tr["bsig"], bsig) < 1e-6
    assert O.rel_l2(tr["qn"], qn) < 1e-5 and O.rel_l2(tr["kn"], kn) < 1e-5
    assert O.rel_l2(tr["attn"], out) < 1e-4
    assert O.rel_l2(S, Sm.transpose(0, 2, 1)) < 1e-4              # the oracle stores S transposed
    fin = out / np.sqrt((out ** 2).mean(-1, keepdims=True) + EPS) * w["norm"] * (1 / (1 + np.exp(-zz))).reshape(T, hv, d)
    assert O.rel_l2(tr["final"], fin.reshape(T, -1)) < 1e-4
    assert O.rel_l2(res, fin.reshape(T, -1) @ deq(w["out"], vw).T) < 1e-4
    assert np.array_equal(conv, np.ascontiguousarray(tr["qkv"][-3:].T))  # history = last 3 rows, oldest first


def test_delta_rule_closed_form_and_head_map():
    """g = 0 (no decay), beta = 1, orthonormal keys: after T tokens S = sum_t k_t v_t^T and the
    read-out of a stored key returns its value.  And the modulo head map against the divide map
    (llm/deltanet_test.go:234-268): they must disagree when hv != hk."""
    d, hk, hv, T = 128, 2, 4, 5
    rng = np.random.default_rng(9)
    Q, _ = np.linalg.qr(rng.standard_normal((d, d)))
    kn = np.zeros((T, hk, d), np.float32)
    for t in range(T):
        kn[t, 0], kn[t, 1] = Q[:, t], Q[:, 10 + t]
    v = rng.standard_normal((T, hv, d)).astype(np.float32)
    gate = np.zeros((T, hv), np.float32)
    beta = np.ones((T, hv), np.float32)
    S = np.zeros((hv, d, d), np.float32)
    out = np.empty((T, hv, d), np.float32)
    k_of = np.array([h % hk for h in range(hv)], np.int32)
    L.shv_ref_delta_rule(d, hk, hv, T, O.F(kn), O.F(kn), O.F(v), O.F(gate), O.F(beta), O.F(S), O.F(out), O.I(k_of))
    for h in range(hv):
        want = sum(np.outer(kn[t, h % hk].astype(np.float64), v[t, h].astype(np.float64)) for t in range(T))
        assert np.allclose(S[h].T, want, atol=1e-5)               # S[i][j] lives at [j][i]
        for t in range(T):
            assert np.allclose(out[t, h] * np.sqrt(d), v[t, h], atol=1e-4)   # q = k_t reads v_t back
    cfg, dw, w, (qk, vw, cw) = dn_setup(rng)
    x = rng.standard_normal((3, cfg.n_embd)).astype(np.float32)
    z = lambda: (np.zeros((cw, 3), np.float32), np.zeros((cfg.n_head_v, 128, 128), np.float32))
    a = run_dn(cfg, dw, x, *z(), divide=0)
    b = run_dn(cfg, dw, x, *z(), divide=1)
    assert O.rel_l2(a, b) > 1e-2


# --------------------------------------------------------------------- attention ---------------

def attn_cfg(H=512, nh=4, nkv=2, d=64, rope=32):
    return O.AttnCfg(H, nh, nkv, d, rope, 1e7, (O.C.c_int * 4)(6, 5, 5, 0), EPS)


def test_rope_is_neox_on_the_first_dims_only():
    """llm/attn_test.go:87,129: pairs (i, i + n_rot/2), dims past n_rot untouched, identity at
    position 0, norm preserved; angles pos * base^(-2i/n_rot)."""
    cfg = attn_cfg()
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 4, 64)).astype(np.float32)
    pos = np.array([0, 5, 1000], np.int32)
    y = x.copy()
    L.shv_ref_rope(O.C.byref(cfg), O.F(y), O.I(pos), 4, 64, 3)
    assert np.array_equal(y[0], x[0])                              # position 0
    assert np.array_equal(y[:, :, 32:], x[:, :, 32:])              # dims >= n_rot
    assert np.allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)
    half = 16
    for t in (1, 2):
        for i in range(half):
            th = float(pos[t]) * (1e7 ** (-2.0 * i / 32))
            c, s = np.cos(th), np.sin(th)
            assert np.allclose(y[t, :, i], x[t, :, i] * c - x[t, :, i + half] * s, atol=2e-5)
            assert np.allclose(y[t, :, i + half], x[t, :, i] * s + x[t, :, i + half] * c, atol=2e-5)


def attn_setup(rng, cfg):
    H, nh, nkv, d = cfg.n_embd, cfg.n_head, cfg.n_head_kv, cfg.head_dim
    w = dict(q=q4(rng, nh * 2 * d, H, 0.05), k=q4(rng, nkv * d, H, 0.05), v=q4(rng, nkv * d, H, 0.05),
             o=q4(rng, H, nh * d), qn=(1 + 0.1 * rng.standard_normal(d)).astype(np.float32),
             kn=(1 + 0.1 * rng.standard_normal(d)).astype(np.float32))
    aw = O.AttnW(O.B(w["q"]), O.B(w["k"]), O.B(w["v"]), O.B(w["o"]), O.F(w["qn"]), O.F(w["kn"]))
    return aw, w


def run_attn(cfg, aw, x, past, kc, vc):
    T = x.shape[0]
    out = np.empty((T, cfg.n_embd), np.float32)
    pre = np.empty((T, cfg.n_head * cfg.head_dim), np.float32)
    L.shv_ref_attn_layer(O.C.byref(cfg), O.C.byref(aw), O.F(x), T, past, O.H(kc), O.H(vc), O.F(out), None, O.F(pre), 1)
    return out, pre


def test_attention_against_independent_float64():
    """Causal GQA with a query gate, re-derived in numpy float64 on the half-rounded K and V."""
    cfg = attn_cfg()
    rng = np.random.default_rng(11)
    aw, w = attn_setup(rng, cfg)
    H, nh, nkv, d, T = cfg.n_embd, cfg.n_head, cfg.n_head_kv, cfg.head_dim, 7
    x = rng.standard_normal((T, H)).astype(np.float32)
    kc, vc = np.zeros((16, nkv, d), np.uint16), np.zeros((16, nkv, d), np.uint16)
    out, pre = run_attn(cfg, aw, x, 0, kc, vc)
    X = x.astype(np.float64)
    qg = (X @ deq(w["q"], H).T).reshape(T, nh, 2, d)
    q, gate = qg[:, :, 0], qg[:, :, 1]
    k = (X @ deq(w["k"], H).T).reshape(T, nkv, d)
    v = (X @ deq(w["v"], H).T).reshape(T, nkv, d)
    hn = lambda a, g: a / np.sqrt((a ** 2).mean(-1, keepdims=True) + EPS) * g

    def rope(a):
        a = a.copy()
        for t in range(T):
            for i in range(16):
                th = t * (1e7 ** (-2.0 * i / 32))
                x0, x1 = a[t, :, i].copy(), a[t, :, i + 16].copy()
                a[t, :, i], a[t, :, i + 16] = x0 * np.cos(th) - x1 * np.sin(th), x0 * np.sin(th) + x1 * np.cos(th)
        return a

    q, k = rope(hn(q, w["qn"])), rope(hn(k, w["kn"]))
    k16 = k.astype(np.float16).astype(np.float64)
    v16 = v.astype(np.float16).astype(np.float64)
    want = np.zeros((T, nh, d))
    for t in range(T):
        for h in range(nh):
            s = k16[:t + 1, h // (nh // nkv)] @ q[t, h] / np.sqrt(d)
            p = np.exp(s - s.max())
            want[t, h] = (p / p.sum()) @ v16[:t + 1, h // (nh // nkv)]
    assert O.rel_l2(pre, want.reshape(T, -1)) < 5e-4               # halves of K,V may round apart
    gated = want * (1 / (1 + np.exp(-gate)))
    assert O.rel_l2(out, gated.reshape(T, -1) @ deq(w["o"], nh * d).T) < 5e-4
    assert np.array_equal(vc[:T].view(np.float16), v.astype(np.float32).astype(np.float16)) or \
        np.count_nonzero(vc[:T].view(np.float16) != v.astype(np.float32).astype(np.float16)) < vc[:T].size // 50


def test_attention_cache_steps_equal_one_pass():
    """Seven tokens at once == 4 then 3 over the carried cache, bit for bit: the generalisation to a
    non-empty cache changes nothing about the reference's whole-prompt function."""
    cfg = attn_cfg()
    rng = np.random.default_rng(12)
    aw, w = attn_setup(rng, cfg)
    x = rng.standard_normal((7, cfg.n_embd)).astype(np.float32)
    mk = lambda: (np.zeros((16, cfg.n_head_kv, cfg.head_dim), np.uint16), np.zeros((16, cfg.n_head_kv, cfg.head_dim), np.uint16))
    kc, vc = mk()
    whole, _ = run_attn(cfg, aw, x, 0, kc, vc)
    kc2, vc2 = mk()
    a, _ = run_attn(cfg, aw, x[:4], 0, kc2, vc2)
    b, _ = run_attn(cfg, aw, x[4:], 4, kc2, vc2)
    assert np.array_equal(np.concatenate([a, b]), whole)
    assert np.array_equal(kc, kc2) and np.array_equal(vc, vc2)


# ------------------------------------------------------------------- token loop ----------------

class TinyCfg:
    n_layer, n_embd, vocab, attn_every, rms_eps = 2, 512, 300, 2, EPS
    n_expert, n_expert_used, ffn_expert = 8, 2, 256
    ssm_head_dim, ssm_head_k, ssm_head_v, ssm_conv = 128, 2, 4, 4
    n_head, n_head_kv, head_dim, rope_dims, rope_base = 4, 2, 64, 32, 1e7


def tiny_tensors(rng, c, draft=False):
    """Random tensors of a two-layer model (DeltaNet, then attention) by GGUF name; with `draft`,
    block n_layer is the draft head's attention block with its nextn tensors."""
    H, d = c.n_embd, c.ssm_head_dim
    qk, vw = c.ssm_head_k * d, c.ssm_head_v * d
    gam = lambda n: (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    t = {"token_embd.weight": rng.standard_normal((c.vocab, H)).astype(np.float16).view(np.uint16),
         "output_norm.weight": gam(H), "output.weight": q4(rng, c.vocab, H)}
    for l in range(c.n_layer + (1 if draft else 0)):
        b = lambda n: "blk.%d.%s.weight" % (l, n)
        t[b("attn_norm")], t[b("post_attention_norm")] = gam(H), gam(H)
        if l >= c.n_layer:
            t[b("nextn.enorm")], t[b("nextn.hnorm")], t[b("nextn.shared_head_norm")] = gam(H), gam(H), gam(H)
            t[b("nextn.eh_proj")] = q4(rng, H, 2 * H)
        if l >= c.n_layer or (l + 1) % c.attn_every == 0:
            t[b("attn_q")], t[b("attn_k")], t[b("attn_v")] = q4(rng, c.n_head * 2 * c.head_dim, H), q4(rng, c.n_head_kv * c.head_dim, H), q4(rng, c.n_head_kv * c.head_dim, H)
            t[b("attn_output")] = q4(rng, H, c.n_head * c.head_dim)
            t[b("attn_q_norm")] = np.ones(c.head_dim, np.float32)
            t[b("attn_k_norm")] = np.ones(c.head_dim, np.float32)
        else:
            t[b("attn_qkv")], t[b("attn_gate")] = q4(rng, 2 * qk + vw, H), q4(rng, vw, H)
            t[b("ssm_alpha")], t[b("ssm_beta")], t[b("ssm_out")] = q4(rng, c.ssm_head_v, H), q4(rng, c.ssm_head_v, H), q4(rng, H, vw)
            t[b("ssm_conv1d")] = (rng.standard_normal((2 * qk + vw, 4)) * 0.3).astype(np.float32)
            t[b("ssm_a")] = (-np.exp(rng.standard_normal(c.ssm_head_v))).astype(np.float32)
            t[b("ssm_dt")] = rng.standard_normal(c.ssm_head_v).astype(np.float32)
            t[b("ssm_norm")] = np.ones(d, np.float32)
        t[b("ffn_gate_inp")] = (rng.standard_normal((c.n_expert, H)) * 0.05).astype(np.float32)
        t[b("ffn_gate_inp_shexp")] = (rng.standard_normal(H) * 0.05).astype(np.float32)
        t[b("ffn_gate_exps")], t[b("ffn_up_exps")] = q4(rng, c.n_expert * c.ffn_expert, H), q4(rng, c.n_expert * c.ffn_expert, H)
        t[b("ffn_down_exps")] = q4(rng, c.n_expert * H, c.ffn_expert)
        t[b("ffn_gate_shexp")], t[b("ffn_up_shexp")], t[b("ffn_down_shexp")] = q4(rng, c.ffn_expert, H), q4(rng, c.ffn_expert, H), q4(rng, H, c.ffn_expert)
    return t


def test_model_loop_chunk_split_and_composition():
    """Pre-norm residual composition (attn every 2nd layer here): the loop in pieces equals the loop
    at once, and the hidden state equals the layers applied by hand."""
    rng = np.random.default_rng(13)

    c = TinyCfg
    H, d = c.n_embd, c.ssm_head_dim
    qk, vw = c.ssm_head_k * d, c.ssm_head_v * d
    t = tiny_tensors(rng, c)
    ids = rng.integers(0, c.vocab, size=6).astype(np.int32)
    m1 = O.OracleModel(c, t, max_cells=16, sections=(6, 5, 5, 0))
    lg1, hd1 = m1.extend(ids, threads=1)
    m2 = O.OracleModel(c, t, max_cells=16, sections=(6, 5, 5, 0))
    m2.extend(ids[:2], threads=1)
    lg2, hd2 = m2.extend(ids[2:], threads=1)
    assert np.array_equal(lg1, lg2) and np.array_equal(hd1, hd2) and m1.past == m2.past == 6
    # by hand, one token from an empty state: x + dn(norm x); + moe(norm .); then attention layer
    m3 = O.OracleModel(c, t, max_cells=16, sections=(6, 5, 5, 0))
    _, hd3 = m3.extend(ids[:1], threads=1)
    x = t["token_embd.weight"][ids[0]].view(np.float16).astype(np.float32)[None]
    for l in range(c.n_layer):
        lw = m3.layers[l]
        b = lambda n: t["blk.%d.%s.weight" % (l, n)]
        xn = O.rmsnorm(x, b("attn_norm"), EPS)
        y = np.empty_like(x)
        if (l + 1) % c.attn_every == 0:
            kc, vc = np.zeros((16, c.n_head_kv, c.head_dim), np.uint16), np.zeros((16, c.n_head_kv, c.head_dim), np.uint16)
            L.shv_ref_attn_layer(O.C.byref(m3.mcfg.attn), O.C.byref(lw.attn), O.F(xn), 1, 0, O.H(kc), O.H(vc), O.F(y), None, None, 1)
        else:
            conv, S = np.zeros((2 * qk + vw, 3), np.float32), np.zeros((c.ssm_head_v, d, d), np.float32)
            L.shv_ref_deltanet_layer(O.C.byref(m3.mcfg.dn), O.C.byref(lw.dn), O.F(xn), 1, O.F(conv), O.F(S), O.F(y),
                                     None, None, None, None, None, None, None, 0, 1)
        x = x + y
        xn = O.rmsnorm(x, b("post_attention_norm"), EPS)
        L.shv_ref_moe_block(O.C.byref(m3.mcfg.moe), O.C.byref(lw.moe), O.F(xn), 1, O.F(y), None, None, None, None, None, None, 1)
        x = x + y
    assert np.array_equal(x[0], hd3)



def test_extend_rows_is_extend_row_by_row():
    """Every row of the verification pass carries the logits and residual that Extend returns for
    the sequence cut after that row; the carried state afterwards is the same."""
    rng = np.random.default_rng(21)
    c = TinyCfg
    t = tiny_tensors(rng, c)
    ids = rng.integers(0, c.vocab, size=5).astype(np.int32)
    a = O.OracleModel(c, t, max_cells=16, sections=(6, 5, 5, 0))
    a.extend(ids[:2], threads=1)
    lg_rows, hd_rows = a.extend_rows(ids[2:], threads=1)
    b = O.OracleModel(c, t, max_cells=16, sections=(6, 5, 5, 0))
    b.extend(ids[:2], threads=1)
    for r in range(3):
        lg, hd = b.extend(ids[2 + r:3 + r], threads=1)
        assert np.array_equal(lg, lg_rows[r]) and np.array_equal(hd, hd_rows[r]), r
    assert a.past == b.past == 5
    assert np.array_equal(a.dn_s[0], b.dn_s[0]) and np.array_equal(a.kc[1], b.kc[1])
    # snapshot / restore brings the sequence back to where it was
    snap = a.snapshot()
    a.extend(ids[:1], threads=1)
    a.restore(snap)
    assert a.past == 5 and np.array_equal(a.dn_s[0], b.dn_s[0]) and np.array_equal(a.kc[1], b.kc[1])


def test_draft_head_wiring():
    """The draft head from its parts: concat(norm(embedding), norm(h)) through eh_proj, one attention
    block over the draft's own cache, the MoE, the head norm and the trunk's lm_head.  Swapping the
    two input norms or the halves of the concatenation changes the result (negative controls), and
    three rows at once equal one row then two."""
    rng = np.random.default_rng(22)
    c = TinyCfg
    t = tiny_tensors(rng, c, draft=True)
    H = c.n_embd
    om = O.OracleModel(c, t, max_cells=16, sections=(6, 5, 5, 0))
    hs = rng.standard_normal((3, H)).astype(np.float32)
    ids = rng.integers(0, c.vocab, size=3).astype(np.int32)
    d1 = O.OracleMTP(om, 16)
    lg, res = d1.rows(hs, ids, 0, threads=1)
    d2 = O.OracleMTP(om, 16)
    d2.rows(hs[:1], ids[:1], 0, threads=1)
    lg2, res2 = d2.rows(hs[1:], ids[1:], 1, threads=1)
    assert np.array_equal(lg, lg2) and np.array_equal(res[1:], res2)
    assert np.array_equal(d1.kc, d2.kc) and np.array_equal(d1.vc, d2.vc)

    b = lambda n: t["blk.%d.%s.weight" % (c.n_layer, n)]

    def by_hand(first_norm, second_norm, swap_halves):
        e = t["token_embd.weight"][ids[:1]].view(np.float16).astype(np.float32)
        parts = [O.rmsnorm(e, b(first_norm), EPS)[0], O.rmsnorm(hs[:1], b(second_norm), EPS)[0]]
        cat = np.concatenate(parts[::-1] if swap_halves else parts)
        x = O.gemv_q4k(b("nextn.eh_proj"), cat, H, 2 * H)[None]
        lw = d1.w.layer
        y = np.empty_like(x)
        kc, vc = np.zeros((16, c.n_head_kv, c.head_dim), np.uint16), np.zeros((16, c.n_head_kv, c.head_dim), np.uint16)
        xn = O.rmsnorm(x, b("attn_norm"), EPS)
        L.shv_ref_attn_layer(O.C.byref(om.mcfg.attn), O.C.byref(lw.attn), O.F(xn), 1, 0, O.H(kc), O.H(vc), O.F(y), None, None, 1)
        x = x + y
        xn = O.rmsnorm(x, b("post_attention_norm"), EPS)
        L.shv_ref_moe_block(O.C.byref(om.mcfg.moe), O.C.byref(lw.moe), O.F(xn), 1, O.F(y), None, None, None, None, None, None, 1)
        x = x + y
        logits = O.gemv_q4k(t["output.weight"], O.rmsnorm(x, b("nextn.shared_head_norm"), EPS)[0], c.vocab, H)
        return x[0], logits

    d3 = O.OracleMTP(om, 16)
    lg1, res1 = d3.rows(hs[:1], ids[:1], 0, threads=1)
    x, logits = by_hand("nextn.enorm", "nextn.hnorm", False)
    assert np.array_equal(x, res1[0]) and np.array_equal(logits, lg1)
    for args in (("nextn.hnorm", "nextn.enorm", False), ("nextn.enorm", "nextn.hnorm", True)):
        x_bad, _ = by_hand(*args)
        assert O.rel_l2(x_bad, res1[0]) > 1e-2


# ------------------------------------------------------------ block-sparse indexer -------------

def test_f2ui_keeps_the_order_of_floats():
    """llm/attn.go:672-682: flip the sign bit of a positive, invert a negative: an unsigned key that
    orders as the float does, -inf the smallest there is."""
    rng = np.random.default_rng(30)
    v = np.concatenate([rng.standard_normal(2000) * 10.0 ** rng.integers(-20, 20, 2000),
                        [0.0, 1e9, -1e9, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, -3.4e38]]).astype(np.float32)
    keys = np.array([L.shv_ref_f2ui(float(x)) for x in v], np.uint64)
    order = np.argsort(v, kind="stable")
    vs, ks = v[order], keys[order]
    assert all(ks[i] < ks[i + 1] for i in range(len(vs) - 1) if vs[i] < vs[i + 1])
    assert all(ks[i] == ks[i + 1] for i in range(len(vs) - 1) if vs[i] == vs[i + 1] and np.signbit(vs[i]) == np.signbit(vs[i + 1]))
    assert keys[list(v).index(-np.inf)] == keys.min()


def _topk(x, n):
    x = np.ascontiguousarray(x, np.float32)
    sel = np.empty(min(n, len(x)), np.int32)
    above = L.shv_ref_topk(O.F(x), len(x), n, O.I(sel))
    return sel, above


def test_radix_select_is_the_nth_largest_with_ties_filled_in_index_order():
    """llm/attn.go:588-670 (topK, topKThreshold): the threshold is the n-th largest value; every cell
    strictly above it is taken, then cells equal to it in ascending index until n are held.  Brute
    force by sorting, on rows without ties, rows that are mostly ties (a block's cells share one
    score) and rows that are mostly -inf (the causal mask)."""
    rng = np.random.default_rng(31)
    for trial in range(60):
        n_cells = int(rng.integers(1, 400))
        n = int(rng.integers(1, n_cells + 1))
        kind = trial % 3
        if kind == 0:
            x = rng.standard_normal(n_cells).astype(np.float32)
        elif kind == 1:
            x = np.repeat(rng.integers(-3, 4, (n_cells + 3) // 4).astype(np.float32), 4)[:n_cells]   # blocks of equal scores
        else:
            x = rng.standard_normal(n_cells).astype(np.float32)
            x[rng.random(n_cells) < 0.7] = -np.inf
        thr_key = L.shv_ref_topk_threshold(O.F(x), n_cells, n)
        nth = np.sort(x)[::-1][n - 1]
        assert thr_key == L.shv_ref_f2ui(float(nth))
        sel, above = _topk(x, n)
        assert len(sel) == n and len(set(sel)) == n
        want_above = np.flatnonzero(x > nth)
        assert above == len(want_above) and list(sel[:above]) == list(want_above)
        fill = np.flatnonzero(x == nth)[:n - above]
        assert list(sel[above:]) == list(fill)
    # the negative control: taking the ties from the top instead is another set
    x = np.array([1, 1, 1, 1, 5, 1, 1], np.float32)
    sel, above = _topk(x, 3)
    assert above == 1 and sorted(sel) == [0, 1, 4]


def qsa_cfg(top_k=8, ratio=4, idx_heads=2, idx_dim=32, **kw):
    c = attn_cfg(**kw)
    c.idx_heads, c.idx_dim, c.top_k, c.ratio = idx_heads, idx_dim, top_k, ratio
    return c


def qsa_setup(rng, cfg):
    aw, w = attn_setup(rng, cfg)
    H, D, IH = cfg.n_embd, cfg.idx_dim, cfg.idx_heads
    w["iq"] = (rng.standard_normal((IH * D, H)) * 0.05).astype(np.float32)
    w["ik"] = (rng.standard_normal((D, H)) * 0.05).astype(np.float32)
    w["iqn"] = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    w["ikn"] = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    aw.idx_q, aw.idx_k, aw.idx_q_norm, aw.idx_k_norm = O.F(w["iq"]), O.F(w["ik"]), O.F(w["iqn"]), O.F(w["ikn"])
    return aw, w


def run_qsa(cfg, aw, x, past, kc, vc, ic, n_kv):
    T = x.shape[0]
    width = min(cfg.top_k + cfg.ratio - 1, n_kv)
    nb = (n_kv + cfg.ratio - 1) // cfg.ratio
    out, pre = np.empty((T, cfg.n_embd), np.float32), np.empty((T, cfg.n_head * cfg.head_dim), np.float32)
    topk, above, score = np.empty((T, width), np.int32), np.empty(T, np.int32), np.empty((T, nb), np.float32)
    L.shv_ref_attn_layer_qsa(O.C.byref(cfg), O.C.byref(aw), O.F(x), T, past, O.H(kc), O.H(vc), O.H(ic), n_kv, O.F(out), None, O.F(pre),
                             O.I(topk), O.I(above), O.F(score), 1)
    return dict(out=out, pre=pre, topk=topk, above=above, score=score)


def _rope64(x, pos, rot, base):
    """NeoX rotation in float64: x [..., dim], one position for the whole array."""
    y = x.copy()
    half = rot // 2
    i = np.arange(half)
    th = pos * base ** (-2.0 * i / rot)
    c, s = np.cos(th), np.sin(th)
    y[..., :half] = x[..., :half] * c - x[..., half:rot] * s
    y[..., half:rot] = x[..., :half] * s + x[..., half:rot] * c
    return y


def _indexer64(cfg, w, xn, n_kv):
    """The selection re-derived in float64 for a prompt from position 0: visible sets per row and
    the margin between the last value taken and the first left out."""
    T, D, IH, R = xn.shape[0], cfg.idx_dim, cfg.idx_heads, cfg.ratio
    half = lambda a: a.astype(np.float16).astype(np.float64)
    raw = half((xn.astype(np.float64) @ w["ik"].astype(np.float64).T).astype(np.float32))     # the cache holds halves
    n_bid = T // R
    norm = lambda v, g: v / np.sqrt((v ** 2).mean(axis=-1, keepdims=True) + EPS) * g.astype(np.float64)
    keys = np.stack([_rope64(norm(raw[b * R:(b + 1) * R].mean(axis=0), w["ikn"]), b * R, cfg.rope_dims, 1e7) for b in range(n_bid)]) \
        if n_bid else np.zeros((0, D))
    dead = norm(raw[0], w["ikn"])                                           # a block that is not there: cell 0, position 0
    q = (xn.astype(np.float64) @ w["iq"].astype(np.float64).T).reshape(T, IH, D)
    q = np.stack([_rope64(norm(q[i], w["iqn"]), i, cfg.rope_dims, 1e7) for i in range(T)])
    width = min(cfg.top_k + R - 1, n_kv)
    sets, margins = [], []
    for i in range(T):
        sc = np.maximum(q[i] @ keys.T, 0).sum(axis=0) if n_bid else np.zeros(0)       # [n_bid]
        sd = np.maximum(q[i] @ dead, 0).sum()
        tail_start = (i + 1) // R * R
        v = np.full(i + 1, -np.inf)
        for j in range(i + 1):
            if j < n_bid * R:
                b = j // R
                v[j] = np.float32(np.float32(sc[b]) + np.float32(1e9 if b * R >= tail_start else 0))
            else:
                v[j] = np.float32(np.float32(sd) + np.float32(1e9))
        if i + 1 <= width:
            sets.append(set(range(i + 1)))
            margins.append(np.inf)
            continue
        order = np.sort(v)[::-1]
        nth = order[width - 1]
        take = list(np.flatnonzero(v > nth))
        take += list(np.flatnonzero(v == nth)[:width - len(take)])
        sets.append(set(int(t) for t in take))
        below = order[order < nth]
        above = order[order > nth]
        m = min((above.min() - nth) if len(above) else np.inf, (nth - below.max()) if len(below) else np.inf)
        margins.append(m)
    return sets, margins


def test_indexer_selection_against_independent_float64():
    """indexerAt (llm/attn.go:231-421) re-derived in numpy float64 — raw keys through a binary16
    cache, whole blocks pooled, normed and turned at their first cell's position, rectified
    per-head scores, the 1e9 tail, the causal mask, the top (top_k + ratio - 1) cells with ties
    filled in index order — must name the same visible cells row for row wherever the value at
    the cut is clear of its neighbours."""
    cfg = qsa_cfg(top_k=8, ratio=4)
    rng = np.random.default_rng(32)
    aw, w = qsa_setup(rng, cfg)
    T, n_kv = 45, 64
    x = rng.standard_normal((T, cfg.n_embd)).astype(np.float32)
    kc = np.zeros((n_kv, cfg.n_head_kv, cfg.head_dim), np.uint16)
    vc, ic = np.zeros_like(kc), np.zeros((n_kv, cfg.idx_dim), np.uint16)
    got = run_qsa(cfg, aw, x, 0, kc, vc, ic, n_kv)
    sets, margins = _indexer64(cfg, w, x, n_kv)
    checked = 0
    for i in range(T):
        mine = set(int(c) for c in got["topk"][i] if c <= i)
        if margins[i] > 1e-4:
            assert mine == sets[i], (i, sorted(mine ^ sets[i]))
            checked += 1
        # what every row must hold whatever the scores: its own incomplete tail
        assert set(range((i + 1) // 4 * 4, i + 1)) <= mine
    assert checked >= T - 4
    # selections really cut: late rows see fewer cells than are visible
    assert len(set(int(c) for c in got["topk"][T - 1] if c <= T - 1)) == 11 < T
    # the lists are ascending within the strictly-above part and within the fill
    for i in range(T):
        a = got["above"][i]
        assert list(got["topk"][i][:a]) == sorted(got["topk"][i][:a])


def test_indexer_at_seven_tokens_in_a_larger_cache():
    """llm/attn.go:124-133, :221-230: 7 tokens in a 256-cell cache make one block of 4 and leave
    cells 4..6 unpooled; every block that does not exist pools cell 0, so their scores all equal
    the score of the spare block that collects the tail; the selection covers every visible cell
    and the layer is the dense one bit for bit."""
    cfg = qsa_cfg(top_k=16, ratio=4)
    rng = np.random.default_rng(33)
    aw, w = qsa_setup(rng, cfg)
    T, n_kv = 7, 256
    x = rng.standard_normal((T, cfg.n_embd)).astype(np.float32)
    mk = lambda: (np.zeros((n_kv, cfg.n_head_kv, cfg.head_dim), np.uint16), np.zeros((n_kv, cfg.n_head_kv, cfg.head_dim), np.uint16))
    kc, vc = mk()
    ic = np.zeros((n_kv, cfg.idx_dim), np.uint16)
    got = run_qsa(cfg, aw, x, 0, kc, vc, ic, n_kv)
    assert (got["score"][:, 1:] == got["score"][:, 1:2]).all()       # blocks 1..63 are all cell 0's key
    assert not (got["score"][:, 0] == got["score"][:, 1]).all()
    for i in range(T):
        assert set(range(i + 1)) <= set(int(c) for c in got["topk"][i])
    dense = attn_cfg()
    kd, vd = mk()
    out_d, pre_d = run_attn(dense, aw, x, 0, kd, vd)
    assert np.array_equal(got["out"], out_d) and np.array_equal(got["pre"], pre_d)


def test_indexer_over_a_cache_is_a_chunk_split():
    """Rows appended over a cache select what the same rows select in one pass from position 0,
    and the layer's output is the same bit for bit (19 + 13 + 1 = 33 rows)."""
    cfg = qsa_cfg(top_k=8, ratio=4)
    rng = np.random.default_rng(34)
    aw, w = qsa_setup(rng, cfg)
    T, n_kv = 33, 64
    x = rng.standard_normal((T, cfg.n_embd)).astype(np.float32)
    z = lambda: (np.zeros((n_kv, cfg.n_head_kv, cfg.head_dim), np.uint16), np.zeros((n_kv, cfg.n_head_kv, cfg.head_dim), np.uint16),
                 np.zeros((n_kv, cfg.idx_dim), np.uint16))
    whole = run_qsa(cfg, aw, x, 0, *z(), n_kv)
    kc, vc, ic = z()
    parts, past = [], 0
    for n in (19, 13, 1):
        parts.append(run_qsa(cfg, aw, x[past:past + n], past, kc, vc, ic, n_kv))
        past += n
    out = np.concatenate([p["out"] for p in parts])
    vis = lambda tk, i: set(int(c) for c in tk if c <= i)
    tk = np.concatenate([p["topk"] for p in parts])
    for i in range(T):
        assert vis(tk[i], i) == vis(whole["topk"][i], i), i
    assert np.array_equal(out, whole["out"])
    # and the selection matters: the dense layer gives other numbers on the late rows
    dense = attn_cfg()
    kd, vd, _ = z()
    out_d, _ = run_attn(dense, aw, x, 0, kd, vd)
    assert np.array_equal(out_d[:11], whole["out"][:11]) and O.rel_l2(out_d[20:], whole["out"][20:]) > 1e-3
