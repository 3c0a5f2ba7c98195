#!/usr/bin/env python3
"""Benchmark of the token loop on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one batch-1 greedy decode token of the synthetic Qwen3-Next-shape model (48 layers, 3
gated-DeltaNet + 1 gated-attention repeating, 512-expert top-10 Q4_K MoE on every layer, vocab
151 936): the prompt of 2048 random ids is prefilled first (untimed), W tokens are decoded untimed,
then exactly K tokens are timed between two synchronisations.  Everything the timed region reads is
resident in HBM before it starts.  Prints ONE JSON line.

Beside the headline it reports
  roofline      the dominant kernel of the step (the expert-gathered gate/up GEMV, 48 launches a
                token, which on one-row passes also makes the token's top-10 selection first):
                algorithmic bytes per launch over the kernel's own measured duration (timestamps on
                the kernel's dispatch, taken live), against 8 TB/s
  cpu_baseline  the CPU restatement of the reference's Go path (oracle/), timed on this host on a
                bounded sample of the same model: layers 0..3 (one DeltaNet x3 + attention period)
                plus the head, a few decode tokens, scaled by 12 periods to a 48-layer token
  gemv          the single Q4_K GEMV of BASELINE config 1 (4096x2048) over a rotating set of
                distinct weight matrices of more than 2 GiB in all (the Infinity Cache is 256 MB), and
                the 175 MB lm_head GEMV, in GB/s and as a fraction of 8 TB/s
  mtp           BASELINE config 5's second run: a one-block draft head at depth 2 and batched
                3-row verification passes.  What a 2-row and a 3-row pass cost in decode steps, what
                a draft costs, and the greedy speculative loop's rounds on this (random-init, so
                never-agreeing) draft head; beside it the same rounds fed the true continuation as
                drafts, which prices the mechanics when every draft is accepted
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK = 8.0e12  # bytes/s, MI355X
Q4K_ROW = lambda k: k // 256 * 144


def moe_up_bytes(cfg):
    """Algorithmic bytes of one moe.up launch at batch 1: gate and up rows of the routed experts
    and the shared one, the normalised activation in, the SwiGLU activations out."""
    experts = cfg.n_expert_used + 1
    w = experts * 2 * cfg.ffn_expert * Q4K_ROW(cfg.n_embd)
    return w + cfg.n_embd * 4 + experts * cfg.ffn_expert * 4 + cfg.n_expert_used * 4


def token_bytes(cfg, ctx_len):
    """Algorithmic bytes one decode token touches (each weight, state and cache byte once)."""
    H, E, U, F = cfg.n_embd, cfg.n_expert, cfg.n_expert_used, cfg.ffn_expert
    qk, vw = cfg.ssm_head_k * cfg.ssm_head_dim, cfg.ssm_head_v * cfg.ssm_head_dim
    dn_rows = 2 * qk + 2 * vw + 2 * cfg.ssm_head_v
    dn = dn_rows * Q4K_ROW(H) + H * Q4K_ROW(vw) + 2 * cfg.ssm_head_v * cfg.ssm_head_dim ** 2 * 4 + (2 * qk + vw) * 16
    at_rows = cfg.n_head * 2 * cfg.head_dim + 2 * cfg.n_head_kv * cfg.head_dim
    at = at_rows * Q4K_ROW(H) + H * Q4K_ROW(cfg.n_head * cfg.head_dim) + ctx_len * cfg.n_head_kv * cfg.head_dim * 2 * 2
    moe = E * H * 4 + H * 4 + (U + 1) * (2 * F * Q4K_ROW(H) + H * Q4K_ROW(F))
    n_attn = cfg.n_layer // cfg.attn_every
    head = cfg.vocab * Q4K_ROW(H) + H * 2
    return (cfg.n_layer - n_attn) * dn + n_attn * at + cfg.n_layer * moe + head


def first_period_tensors(m, cfg):
    """Host copies of the tensors of layers 0..attn_every-1 and of the head (what the CPU legs read)."""
    per = cfg.attn_every
    names = [t[0] for t in m.tensors()]
    keep = [n for n in names if not n.startswith("blk.") or int(n.split(".")[1]) < per]
    return {n: m.download(n) for n in keep}


def cpu_baseline(m, cfg, LA, A, tensors, n_tokens, cores):
    """Time the oracle's token loop on a 4-layer slice of the same weights, and hold the GPU's
    4-layer result against the oracle's on the same tokens."""
    import ctypes as C
    import oracle_lib as O
    per = cfg.attn_every
    sub = LA.Config(**{f: getattr(cfg, f) for f, _ in cfg._fields_})
    cells = (n_tokens + 2 + 127) // 128 * 128
    sub.n_layer, sub.nkv, sub.max_tokens, sub.slots, sub.speculative, sub.nextn, sub.head_rows = per, cells, 4, 1, 0, 0, 1
    om = O.OracleModel(sub, tensors, max_cells=cells)
    rng = np.random.default_rng(1)
    ids = rng.integers(0, cfg.vocab, size=n_tokens + 1).astype(np.int32)
    om.extend(ids[:1], threads=cores)  # touch everything once
    t0 = time.perf_counter()
    head_s = 0.0
    for i in range(n_tokens):
        _, hidden = om.extend(ids[1 + i:2 + i], threads=cores)
    dt = (time.perf_counter() - t0) / n_tokens
    # the head runs once per token, the 4-layer period 12 times: time the head alone to split them
    x = rng.standard_normal(cfg.n_embd).astype(np.float32)
    t0 = time.perf_counter()
    O.gemv_q4k(tensors["output.weight"], x, cfg.vocab, cfg.n_embd, threads=cores)
    head_s = time.perf_counter() - t0
    periods = cfg.n_layer // per
    per_token = (dt - head_s) * periods + head_s
    # the same tokens through the GPU path on a model of those four layers (the tensors copied on the
    # device from the 48-layer model): the residual stream after layer 3, outside every timed region
    m4 = LA.LLM(sub)
    try:
        src = {t[0]: t for t in m.tensors()}
        for t in m4.tensors():
            if not t[6]:
                A.check(A.load().shv_copy(m4.ctx, C.c_void_p(t[1]), C.c_void_p(src[t[0]][1]), t[2]))
        m4.stage()
        for i in range(n_tokens + 1):
            _, got = m4.extend(ids[i:i + 1], want_logits=False, want_hidden=True)
    finally:
        m4.close()
    err = O.rel_l2(got, hidden)
    if not err <= 1e-3:
        raise SystemExit("bench.py: the GPU's residual stream after layer %d differs from the oracle's by rel-L2 %.3e (> 1e-3)" % (per - 1, err))
    return {"value": round(1.0 / per_token, 3), "unit": "tok/s", "cores": cores, "host_cpus": os.cpu_count(), "kind": "port", "sample_seconds": round(dt * n_tokens, 2),
            "hidden_rel_l2_vs_gpu": float("%.3e" % err),
            "sample": "C restatement of the reference's Go CPU path (oracle/), layers 0-%d + lm_head of the same "
                      "weights, %d decode tokens at context <= %d; period time x%d + head time; rows of each matvec "
                      "split over %d threads (os.cpu_count() of this host: %s); the GPU path over the same four layers "
                      "and tokens leaves a residual stream within rel-L2 %.1e of the oracle's (checked here, bound 1e-3)"
                      % (per - 1, n_tokens, n_tokens + 1, periods, cores, os.cpu_count(), err)}


def gemv_rates(m, cfg, A, LA):
    """Config 1's GEMV over rotating weights, and the lm_head GEMV, timed by GPU events."""
    pkg = importlib.import_module("strix-halo-vulkan_amd")
    H = pkg.hip_api.load()
    import ctypes as C
    ctx = m.ctx
    out = {}

    def alloc(n):
        p = C.c_void_p()
        A.check(H.shv_alloc(ctx, n, C.byref(p)))
        return p.value

    n, k = 4096, cfg.n_embd
    mat_bytes = n * Q4K_ROW(k)
    # distinct 4096x2048 matrices: windows of the experts' gate banks, layer after layer, until
    # more than 2 GiB of weights rotate
    mats = []
    for t in m.tensors():
        if t[0].endswith("ffn_gate_exps.weight") and len(mats) * mat_bytes < (2 << 30):
            mats += [t[1] + i * mat_bytes for i in range(t[2] // mat_bytes)]
    copies = len(mats)
    dx, dy = alloc(k * 4), alloc(max(n, cfg.vocab) * 4)
    x = np.random.default_rng(2).standard_normal(k).astype(np.float32)
    A.check(H.shv_upload(ctx, dx, x.ctypes.data, x.nbytes))
    ops = [A.make_op(A.OP_GEMV_Q4K, A.gemv_args(w, dx, dy, n, k)) for w in mats]
    arr = (A.Op * len(ops))(*ops)
    ns = C.c_uint64()
    eager = os.environ.get("LLM_NO_PRERECORD", "")[:1] == "1"  # the profiler cannot follow a replay
    if eager:
        A.check(H.shv_dispatch_multi(ctx, arr, len(ops), 2, C.byref(ns), None))
        A.check(H.shv_dispatch_multi(ctx, arr, len(ops), 10, C.byref(ns), None))
    else:
        pre = C.c_void_p()
        A.check(H.shv_prerecord(ctx, arr, len(ops), C.byref(pre)))
        A.check(H.shv_prerecorded_submit(ctx, pre, 2, C.byref(ns)))
        A.check(H.shv_prerecorded_submit(ctx, pre, 10, C.byref(ns)))
        H.shv_prerecorded_destroy(ctx, pre)
    per = ns.value / (10 * copies) / 1e9
    alg = mat_bytes + k * 4 + n * 4
    out["config1_4096x2048"] = {"us": round(per * 1e6, 3), "GBps": round(alg / per / 1e9, 1),
                                "frac_hbm_peak": round(alg / per / HBM_PEAK, 4),
                                "distinct_matrices": int(copies), "rotating_MB": round(copies * mat_bytes / 1e6, 1)}
    if not eager:
        # The same GEMVs as four independent in-order streams (one context each, a quarter of the
        # matrices each, replayed together): launches of different streams overlap, so this is the
        # rate the kernel streams at when the 3.7 us of a dependent launch is not between every
        # two of them - the token loop, whose launches do depend on one another, sees the figure above.
        n_streams = 4
        extra, pres, dys = [], [], []
        try:
            for s in range(n_streams):
                c = ctx
                if s > 0:
                    cp = C.c_void_p()
                    A.check(H.shv_init(0, C.byref(cp)))
                    c = cp
                    extra.append(cp)
                dys_s = alloc(n * 4)
                dys.append(dys_s)
                sops = [A.make_op(A.OP_GEMV_Q4K, A.gemv_args(w, dx, dys_s, n, k)) for w in mats[s::n_streams]]
                sarr = (A.Op * len(sops))(*sops)
                pre = C.c_void_p()
                A.check(H.shv_prerecord(c, sarr, len(sops), C.byref(pre)))
                pres.append((c, pre))
            reps = 10
            for timed in (False, True):
                for c, _ in pres:
                    A.check(H.shv_sync(c))
                t0 = time.perf_counter()
                for _ in range(reps if timed else 2):
                    for c, pre in pres:
                        A.check(H.shv_prerecorded_launch(c, pre))
                for c, _ in pres:
                    A.check(H.shv_sync(c))
                dt = time.perf_counter() - t0
            per4 = dt / (reps * copies)
            out["config1_4096x2048"]["four_streams"] = {"us_per_gemv": round(per4 * 1e6, 3), "GBps": round(alg / per4 / 1e9, 1),
                                                        "frac_hbm_peak": round(alg / per4 / HBM_PEAK, 4)}
        finally:
            for c, pre in pres:
                H.shv_prerecorded_destroy(c, pre)
            for p in dys:
                H.shv_free(ctx, p)
            for c in extra:
                H.shv_destroy(c)
    # the vocabulary projection as the token step sees it: cold.  Between two runs of it, 128 of
    # the 4.7 MB matrices above (600 MB, more than twice the Infinity Cache) go through.
    head = next(t for t in m.tensors() if t[0] == "output.weight")
    hops = [A.make_op(A.OP_GEMV_Q4K, A.gemv_args(head[1], dx, dy, cfg.vocab, k))] + ops[:128]
    harr = (A.Op * len(hops))(*hops)
    per = (C.c_uint64 * len(hops))()
    tot, reps = 0, 10
    A.check(H.shv_dispatch_multi(ctx, harr, len(hops), 1, C.byref(ns), per))
    for _ in range(reps):
        A.check(H.shv_dispatch_multi(ctx, harr, len(hops), 1, C.byref(ns), per))
        tot += per[0]
    per_s = tot / reps / 1e9
    alg = head[2] + k * 4 + cfg.vocab * 4
    out["lm_head_151936x2048"] = {"us": round(per_s * 1e6, 2), "GBps": round(alg / per_s / 1e9, 1),
                                  "frac_hbm_peak": round(alg / per_s / HBM_PEAK, 4), "cold": True}
    # the DeltaNet input projection (12352x2048, 14.2 MB), one per DeltaNet layer: 36 distinct
    # matrices, 512 MB a round
    fused = [t for t in m.tensors() if t[0].endswith("ssm_in_fused.weight")]
    if fused:
        rows = fused[0][4]
        fops = [A.make_op(A.OP_GEMV_Q4K, A.gemv_args(t[1], dx, dy, rows, k)) for t in fused]
        farr = (A.Op * len(fops))(*fops)
        A.check(H.shv_dispatch_multi(ctx, farr, len(fops), 2, C.byref(ns), None))
        A.check(H.shv_dispatch_multi(ctx, farr, len(fops), 10, C.byref(ns), None))
        per_s = ns.value / (10 * len(fops)) / 1e9
        alg = fused[0][2] + k * 4 + rows * 4
        out["dn_in_proj_%dx%d" % (rows, k)] = {"us": round(per_s * 1e6, 2), "GBps": round(alg / per_s / 1e9, 1),
                                             "frac_hbm_peak": round(alg / per_s / HBM_PEAK, 4), "distinct_matrices": len(fops)}
    for p in (dx, dy):
        H.shv_free(ctx, p)
    return out


class _Borrowed:
    """hip_api.Context's buffer helpers over the model's own context (which the model destroys)."""

    def __init__(self, A, handle):
        self.c = A.Context.__new__(A.Context)
        self.c.L, self.c.h, self.c._bufs = A.load(), handle, []

    def __enter__(self):
        return self.c

    def __exit__(self, *exc):
        for b in self.c._bufs:
            if b.ptr:
                b.free()
        self.c._bufs = []


def _timed(c, ops, labels, reps=6):
    """Average ns per label over reps timed runs of the op list (each op has its own timestamps)."""
    c.dispatch_multi(ops)
    acc = {}
    for _ in range(reps):
        _, per = c.dispatch_multi(ops, per_op=True)
        for k, v in zip(labels, per):
            acc[k] = acc.get(k, 0.0) + v / reps
    return acc


def config_blocks(m, cfg, A, tensors, cores, want_cpu):
    """BASELINE configs 2, 3 (decode) and 4 as blocks of their own, each over all the layers of the
    model that hold such a block, one after the other, so that every launch finds its weights, state
    and cache cold as in the token loop.  GPU times are the kernels' own dispatch timestamps; the CPU
    times beside them are the oracle's block over layer 0's (DeltaNet, experts) or layer 3's
    (attention) tensors on this host."""
    import oracle_lib as O
    out = {}
    H, E, U, F = cfg.n_embd, cfg.n_expert, cfg.n_expert_used, cfg.ffn_expert
    tmap = {t[0]: t[1] for t in m.tensors()}
    blk = lambda l, n: tmap["blk.%d.%s.weight" % (l, n)]
    rng = np.random.default_rng(7)
    is_attn = lambda l: (l + 1) % cfg.attn_every == 0
    eps = cfg.rms_eps

    # ---- config 2: the MoE FFN step ----
    with _Borrowed(A, m.ctx) as c:
        res = {}
        for T in (1, 4, 16):
            h = rng.standard_normal((T, H)).astype(np.float32)
            d_h, xn, logits = c.upload(h), c.alloc(T * H * 4), c.alloc(T * (E + 1) * 4)
            topk, weights = c.alloc(cfg.n_layer * T * U * 4), c.alloc(T * (U + 1) * 4)
            act, o = c.alloc(T * (U + 1) * F * 4), c.alloc(T * H * 4)
            defer = 1 if T == 1 else 0   # a one-row pass makes its selection in the expert kernel
            ops, labels = [], []
            for l in range(cfg.n_layer):
                tk = topk.at(l * T * U * 4)
                ra = A.MoeRouterArgs(d_h.ptr, blk(l, "post_attention_norm"), blk(l, "ffn_gate_inp"), blk(l, "ffn_gate_inp_shexp"),
                                     xn.ptr, logits.ptr, tk, weights.ptr, T, H, E, U, eps, H, defer)
                ua = A.MoeUpArgs(xn.ptr, tk, blk(l, "ffn_gate_exps"), blk(l, "ffn_up_exps"), blk(l, "ffn_gate_shexp"),
                                 blk(l, "ffn_up_shexp"), act.ptr, T, H, U, F, logits.ptr if defer else None,
                                 weights.ptr if defer else None, E, 0, 0, 0, 0, None, 0)
                da = A.MoeDownArgs(act.ptr, tk, weights.ptr, blk(l, "ffn_down_exps"), blk(l, "ffn_down_shexp"), d_h.ptr, o.ptr,
                                   T, H, U, F, H, H, 0, 0, E, None, None)
                ops += [A.make_op(A.OP_MOE_ROUTER, ra), A.make_op(A.OP_MOE_UP, ua), A.make_op(A.OP_MOE_DOWN, da)]
                labels += ["router", "up", "down"]
            t = _timed(c, ops, labels)
            sel = topk.read(np.int32, cfg.n_layer * T * U).reshape(cfg.n_layer, T * U)
            distinct = float(np.mean([len(np.unique(r)) for r in sel]))
            per_expert = 2 * F * Q4K_ROW(H) + H * Q4K_ROW(F)
            alg = (distinct + 1) * per_expert + E * H * 4 + T * (2 * H + 2 * (U + 1) * F + H) * 4
            us = sum(t.values()) / cfg.n_layer / 1e3
            r = {"gpu_us": round(us, 2), "router_us": round(t["router"] / cfg.n_layer / 1e3, 2),
                 "up_us": round(t["up"] / cfg.n_layer / 1e3, 2), "down_us": round(t["down"] / cfg.n_layer / 1e3, 2),
                 "distinct_routed_experts": round(distinct, 2), "bytes": int(alg),
                 "GBps": round(alg / us / 1e3, 1), "frac_hbm_peak": round(alg / (us * 1e-6) / HBM_PEAK, 4)}
            if want_cpu:
                w = O.MoeW(*[O.F(tensors["blk.0.%s.weight" % n]) for n in ("ffn_gate_inp", "ffn_gate_inp_shexp")],
                           *[O.B(tensors["blk.0.%s.weight" % n]) for n in ("ffn_gate_exps", "ffn_up_exps", "ffn_down_exps",
                                                                            "ffn_gate_shexp", "ffn_up_shexp", "ffn_down_shexp")],
                           (O.C.c_int * 6)(0, 0, 0, 0, 0, 0))
                mc = O.MoeCfg(H, E, U, F, F)
                xn_h = O.rmsnorm(h, tensors["blk.0.post_attention_norm.weight"], eps)
                y = np.empty((T, H), np.float32)
                best = 1e9
                for _ in range(3):
                    t0 = time.perf_counter()
                    O.lib().shv_ref_moe_block(O.C.byref(mc), O.C.byref(w), O.F(xn_h), T, O.F(y), None, None, None, None, None, None, cores)
                    best = min(best, time.perf_counter() - t0)
                r["cpu_us"], r["cpu_cores"] = round(best * 1e6, 1), cores
            res["T%d" % T] = r
        out["config2_moe_ffn_step"] = res

    # ---- config 3: one gated-DeltaNet layer at decode, 1 and 8 sequences ----
    hk, hv, d, conv = cfg.ssm_head_k, cfg.ssm_head_v, cfg.ssm_head_dim, cfg.ssm_conv
    qk, vw = hk * d, hv * d
    cw, width = 2 * qk + vw, 2 * qk + 2 * vw + 2 * hv
    dn_layers = [l for l in range(cfg.n_layer) if not is_attn(l)]
    with _Borrowed(A, m.ctx) as c:
        res = {}
        ring_slots = 8
        for B in (1, 8):
            x = rng.standard_normal((B, H)).astype(np.float32)
            d_x, d_attn, d_o = c.upload(x), c.alloc(B * vw * 4), c.alloc(B * H * 4)
            d_pos = c.upload(np.full(B, 100, np.int32))
            d_slot = c.upload(np.arange(B, dtype=np.int32))
            d_row = c.alloc(width * 4)
            ops, labels, keep = [], [], []
            for l in dn_layers:
                ring = c.alloc(B * ring_slots * width * 4).zero()
                state = c.alloc(B * hv * d * d * 4).zero()
                p = A.gemv_args(blk(l, "ssm_in_fused"), d_x, ring, width, H, B, prologue=A.PRO_RMSNORM, gamma=blk(l, "attn_norm"),
                                eps=eps, pos=d_pos, slot=d_slot if B > 1 else None, seq_len=1, ring_slots=ring_slots, ring_stride=width)
                s = A.DnStepArgs(ring.ptr, blk(l, "ssm_conv1d"), blk(l, "ssm_a"), blk(l, "ssm_dt"), state.ptr, d_attn.ptr, d_pos.ptr,
                                 d_slot.ptr if B > 1 else None, B, 1, hk, hv, d, conv, ring_slots, width, eps, 0, None, 1, 0)
                o = A.gemv_args(blk(l, "ssm_out"), d_attn, d_o, H, vw, B, prologue=A.PRO_GATED_NORM, gamma=blk(l, "ssm_norm"),
                                residual=d_x, eps=eps, head_dim=d)
                if B == 1:
                    p.y_flat = d_row.ptr
                    o.z, o.z_stride = d_row.at(cw * 4), width
                else:
                    o.z, o.pos, o.slot, o.seq_len = ring.at(cw * 4), d_pos.ptr, d_slot.ptr, 1
                    o.ring_slots, o.ring_stride, o.z_ring = ring_slots, width, 1
                ops += [A.make_op(A.OP_GEMV_Q4K, p), A.make_op(A.OP_DN_STEP, s), A.make_op(A.OP_GEMV_Q4K, o)]
                labels += ["qkv", "step", "out"]
            t = _timed(c, ops, labels)
            n = len(dn_layers)
            alg = width * Q4K_ROW(H) + H * Q4K_ROW(vw) + B * (2 * hv * d * d * 4 + (H + width + conv * cw + vw + 2 * H) * 4)
            us = sum(t.values()) / n / 1e3
            r = {"gpu_us": round(us, 2), "qkv_us": round(t["qkv"] / n / 1e3, 2), "step_us": round(t["step"] / n / 1e3, 2),
                 "out_us": round(t["out"] / n / 1e3, 2), "bytes": int(alg), "GBps": round(alg / us / 1e3, 1),
                 "frac_hbm_peak": round(alg / (us * 1e-6) / HBM_PEAK, 4)}
            if want_cpu:
                g = lambda n_: tensors["blk.0.%s.weight" % n_]
                w = O.DnW(O.B(g("attn_qkv")), O.B(g("attn_gate")), O.B(g("ssm_alpha")), O.B(g("ssm_beta")), O.B(g("ssm_out")),
                          O.F(g("ssm_conv1d")), O.F(g("ssm_a")), O.F(g("ssm_dt")), O.F(g("ssm_norm")))
                dc = O.DnCfg(H, d, hk, hv, conv, eps, 0)
                xn_h = O.rmsnorm(x[:1], g("attn_norm"), eps)
                cs, ss = np.zeros((cw, conv - 1), np.float32), np.zeros((hv, d, d), np.float32)
                y, at = np.empty((1, H), np.float32), np.empty((1, vw), np.float32)
                best = 1e9
                for _ in range(3):
                    t0 = time.perf_counter()
                    O.lib().shv_ref_deltanet_layer(O.C.byref(dc), O.C.byref(w), O.F(xn_h), 1, O.F(cs), O.F(ss), O.F(y),
                                                   None, None, None, None, None, O.F(at), None, 0, cores)
                    best = min(best, time.perf_counter() - t0)
                # the CPU path takes its sequences one after the other
                r["cpu_us"], r["cpu_cores"] = round(best * 1e6 * B, 1), cores
            res["decode_B%d" % B] = r
        if want_cpu:
            # the prefill side on the CPU: 256 rows through the oracle's layer (it walks them one by one), per row
            g = lambda n_: tensors["blk.0.%s.weight" % n_]
            w = O.DnW(O.B(g("attn_qkv")), O.B(g("attn_gate")), O.B(g("ssm_alpha")), O.B(g("ssm_beta")), O.B(g("ssm_out")),
                      O.F(g("ssm_conv1d")), O.F(g("ssm_a")), O.F(g("ssm_dt")), O.F(g("ssm_norm")))
            dc = O.DnCfg(H, d, hk, hv, conv, eps, 0)
            n_s = 256
            xs = rng.standard_normal((n_s, H)).astype(np.float32)
            cs, ss = np.zeros((cw, conv - 1), np.float32), np.zeros((hv, d, d), np.float32)
            y, at = np.empty((n_s, H), np.float32), np.empty((n_s, vw), np.float32)
            t0 = time.perf_counter()
            O.lib().shv_ref_deltanet_layer(O.C.byref(dc), O.C.byref(w), O.F(xs), n_s, O.F(cs), O.F(ss), O.F(y),
                                           None, None, None, None, None, O.F(at), None, 0, cores)
            res["prefill_cpu"] = {"rows": n_s, "us_per_row": round((time.perf_counter() - t0) / n_s * 1e6, 1), "cpu_cores": cores}
        out["config3_deltanet_layer"] = res

    # ---- config 4: gated attention decode over a long fp16 cache ----
    NH, NKV, D, ROPE = cfg.n_head, cfg.n_head_kv, cfg.head_dim, cfg.rope_dims
    awidth = NH * 2 * D + 2 * NKV * D
    at_layers = [l for l in range(cfg.n_layer) if is_attn(l)]
    with _Borrowed(A, m.ctx) as c:
        res = {}
        max_cells = 131072
        n_slots = 3
        # one cache pair per attention layer would be 9.7 GB at three slots; four pairs in rotation
        # (3.2 GB, far more than every cache level) keep each launch's cells cold
        n_rot = 4
        caches = [(c.alloc(n_slots * max_cells * NKV * D * 2), c.alloc(n_slots * max_cells * NKV * D * 2)) for _ in range(n_rot)]
        fill = A.FillNormalArgs
        for kc, vc in caches:
            for buf in (kc, vc):
                f = fill(buf.ptr, n_slots * max_cells * NKV * D, 11, 0.0, 1.0, 1)
                A.check(c.L.shv_fill_normal(c.h, O.C.byref(f)))
        d_rope = c.upload(np.ones((max_cells, ROPE), np.float32) * np.float32(0.70710678))
        for cells in (4096, 32768, 131072):
            for S in (1, 3):
                x = rng.standard_normal((S, H)).astype(np.float32)
                d_x, d_qkv, d_ctx, d_o = c.upload(x), c.alloc(S * awidth * 4), c.alloc(S * NH * D * 4), c.alloc(S * H * 4)
                d_pos = c.upload(np.full(S, cells - 1, np.int32))
                d_slot = c.upload(np.arange(S, dtype=np.int32))
                n_splits = min(512, max(8, (cells + 31) // 32))
                d_part = c.alloc((S * 2 * NKV * n_splits * (NH // NKV) * (D + 2) + 8192) * 4)
                ops, labels = [], []
                for i, l in enumerate(at_layers):
                    kc, vc = caches[i % n_rot]
                    p = A.gemv_args(blk(l, "attn_qkv_fused"), d_x, d_qkv, awidth, H, S, prologue=A.PRO_RMSNORM, gamma=blk(l, "attn_norm"), eps=eps)
                    a = A.AttnDecodeArgs(d_qkv.ptr, blk(l, "attn_q_norm"), blk(l, "attn_k_norm"), d_rope.ptr, kc.ptr, vc.ptr, d_part.ptr,
                                         d_ctx.ptr, d_pos.ptr, d_slot.ptr if S > 1 else None, S, 1, NH, NKV, D, ROPE, max_cells, awidth, n_splits, eps)
                    o = A.gemv_args(blk(l, "attn_output"), d_ctx, d_o, H, NH * D, S, prologue=A.PRO_MUL_SIGMOID, z=d_qkv, head_dim=D,
                                    z_stride=awidth, residual=d_x)
                    ops += [A.make_op(A.OP_GEMV_Q4K, p), A.make_op(A.OP_ATTN_DECODE, a), A.make_op(A.OP_GEMV_Q4K, o)]
                    labels += ["qkv", "attn", "out"]
                t = _timed(c, ops, labels, reps=4)
                n = len(at_layers)
                cache_bytes = S * cells * NKV * D * 2 * 2
                alg = awidth * Q4K_ROW(H) + H * Q4K_ROW(NH * D) + cache_bytes + S * (2 * H + awidth + NH * D) * 4
                us = sum(t.values()) / n / 1e3
                r = {"gpu_us": round(us, 2), "qkv_us": round(t["qkv"] / n / 1e3, 2), "attn_us": round(t["attn"] / n / 1e3, 2),
                     "out_us": round(t["out"] / n / 1e3, 2), "bytes": int(alg), "GBps": round(alg / us / 1e3, 1),
                     "frac_hbm_peak": round(alg / (us * 1e-6) / HBM_PEAK, 4),
                     "cache_GBps": round(cache_bytes / (t["attn"] / n) , 1)}
                if want_cpu and S == 1:
                    g = lambda n_: tensors["blk.%d.%s.weight" % (cfg.attn_every - 1, n_)]
                    w = O.AttnW(O.B(g("attn_q")), O.B(g("attn_k")), O.B(g("attn_v")), O.B(g("attn_output")), O.F(g("attn_q_norm")), O.F(g("attn_k_norm")))
                    ac = O.AttnCfg(H, NH, NKV, D, ROPE, cfg.rope_base, (O.C.c_int * 4)(11, 11, 10, 0), eps)
                    kh = rng.standard_normal((cells, NKV, D)).astype(np.float16).view(np.uint16)
                    vh = kh.copy()
                    xn_h = O.rmsnorm(x[:1], g("attn_norm"), eps)
                    y = np.empty((1, H), np.float32)
                    t0 = time.perf_counter()
                    O.lib().shv_ref_attn_layer(O.C.byref(ac), O.C.byref(w), O.F(xn_h), 1, cells - 1, O.H(kh), O.H(vh), O.F(y), None, None, cores)
                    res_cpu = time.perf_counter() - t0
                    r["cpu_us"], r["cpu_cores"] = round(res_cpu * 1e6, 1), cores
                res["ctx%d_slots%d" % (cells, S)] = r
        out["config4_attention_decode"] = res
    return out


def mtp_run(m, cfg, prompt, plain, acc, rounds):
    """Pass costs in decode steps and the speculative loop at depth 2 (3-row verification)."""
    kernels = lambda st: sum(v for k, v in st if k != "total")
    step_ns = sum(v for k, v in acc.items() if k != "total")
    out = {"depth": 2, "draft_vocab": 65536}
    for rows in (2, 3):
        # op-by-op dispatch is noisy from pass to pass: the median of a dozen
        st = sorted(kernels(m.profile_rows(rows)) for _ in range(12))
        out["pass_%d_rows_in_steps" % rows] = round((st[5] + st[6]) / 2 / step_ns, 3)
    m.mtp_stage(max_tok=4, vocab_prefix=65536)
    m.spec_open(2)
    # The continuation fed as drafts in the second leg is the one the first leg emitted: the greedy
    # sequence under the verification pass's own numerics (a rejected round emits row 0's arg-max,
    # which does not depend on the drafts behind it).  The plain one-row loop's sequence is not used
    # for that: a pass of other shape rounds differently, and on a random-init model, whose best two
    # logits are nearly level, that flips an arg-max now and then, after which plain greedy's tokens
    # are another sequence's and every draft taken from it is refused.
    reference = plain
    for mode in ("draft_head", "true_continuation_as_drafts"):
        n_rounds = rounds if mode != "draft_head" else 3 * rounds + 4
        first = m.spec_start(prompt)       # prefills the trunk again and primes the draft over the prompt
        toks = [first]
        t0 = time.perf_counter()
        for _ in range(n_rounds):
            forced = reference[len(toks):len(toks) + 2] if mode != "draft_head" else []
            toks += list(m.spec_round(forced))
        dt = time.perf_counter() - t0
        st = m.spec_stats()
        same = lambda other: next((i for i, (x, y) in enumerate(zip(toks, other)) if x != y), min(len(toks), len(other)))
        out[mode] = {"rounds": st["rounds"], "tokens_per_round": round((st["tokens"] - 1) / st["rounds"], 3),
                     "accepted_at": st["accepted_at"][:2], "drafted_at": st["drafted_at"][:2],
                     "round_ms": round(dt / n_rounds * 1e3, 4), "tok_s": round((len(toks) - 1) / dt, 1),
                     "draft_gpu_ms_per_round": round(st["draft_ns"] / st["rounds"] / 1e6, 4),
                     "verify_gpu_ms_per_round": round(st["verify_ns"] / st["rounds"] / 1e6, 4),
                     "tokens_equal_to_plain_greedy": same(plain),
                     "tokens_emitted": len(toks)}
        if mode == "draft_head":
            reference = toks
        else:
            out[mode]["tokens_equal_to_the_first_leg"] = same(reference)
    return out


def batched_run(m, cfg, n_slots, rng, prompt_len=256, steps=48):
    """Several sequences advanced one token each per pass (Graph.DecodeRows): the projections
    read their weights once for all of them, on the matrix cores from five rows."""
    m.speculate(False)
    for s in range(n_slots):
        m.use_slot(s)
        m.reset()
        m.extend(rng.integers(0, cfg.vocab, size=prompt_len).astype(np.int32), want_logits=False)
    slots = np.arange(n_slots, dtype=np.int32)
    ids = rng.integers(0, cfg.vocab, size=n_slots).astype(np.int32)
    for _ in range(4):
        ids, _ = m.decode_rows(slots, ids)
    t0 = time.perf_counter()
    for _ in range(steps):
        ids, _ = m.decode_rows(slots, ids)   # each pass: upload ids, run, download the arg-maxes
    dt = time.perf_counter() - t0
    m.use_slot(0)
    return {"slots": n_slots, "context": prompt_len + 4 + steps, "ms_per_pass": round(dt / steps * 1e3, 4),
            "tok_s": round(n_slots * steps / dt, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=48)
    ap.add_argument("--cpu-tokens", type=int, default=384,
                    help="decode tokens of the CPU leg (four layers and the head each; about ten seconds of host work at the default)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-mtp", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-config blocks (configs 1-4 each on its own)")
    ap.add_argument("--mtp-rounds", type=int, default=64)
    ap.add_argument("--batch-slots", type=int, default=8,
                    help="sequences of the batched-decode leg (one token each per pass); 0 skips it")
    ap.add_argument("--prefill-rows", type=int, default=2048,
                    help="prompt rows per pass (up to 4096; the default sends the 2048-token prompt through as one "
                         "chunk); 1 (with --no-mtp) sends the prompt through the one-row decode "
                         "step itself, so that a kernel trace of the run holds decode launches only")
    ap.add_argument("--pmc-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy, the known-size kernel that "
                         "hardware-counter readings of HBM traffic are scaled by")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs the token loop on ONE GPU (one process, one stream); "
                 "--gpus %d is not supported (experts and heads would shard across GPUs; none of that is built)." % a.gpus)
    if a.steps < 1 or a.warmup < 1:
        sys.exit("bench.py: --steps and --warmup must be at least 1")
    pkg = importlib.import_module("strix-halo-vulkan_amd")
    LA, A = pkg.llm_api, pkg.hip_api
    big = 4096 if a.prefill_rows >= 64 else 0   # a 4096-row chunk is also timed op by op (config 3's prefill shape)
    nkv = a.prompt + a.warmup + a.steps + 3 * a.mtp_rounds + 64 + a.prefill_rows + big
    # prompt rows go through four at a time; the draft block and the state planes of rewindable
    # 3-row passes are staged for the speculative run and cost the plain decode step nothing
    if a.prefill_rows < 1 or (a.prefill_rows < 4 and not a.no_mtp):
        sys.exit("bench.py: --prefill-rows below 4 needs --no-mtp (the speculative leg stages 3-row passes)")
    if a.no_mtp:
        cfg = LA.Config(n_layer=a.layers, nkv=(nkv + 127) // 128 * 128, max_tokens=max(a.prefill_rows, big))
    else:
        cfg = LA.Config(n_layer=a.layers, nkv=(nkv + 127) // 128 * 128, max_tokens=max(a.prefill_rows, big),
                        head_rows=max(3, a.batch_slots), slots=max(1, a.batch_slots), speculative=1, spec_rows=3, nextn=1)
    m = LA.LLM(cfg)
    m.init_synthetic(20260101)
    m.stage()
    rng = np.random.default_rng(0)
    prompt = rng.integers(0, cfg.vocab, size=a.prompt).astype(np.int32)
    t0 = time.perf_counter()
    m.extend(prompt, want_logits=False)
    prefill_s = time.perf_counter() - t0
    ids_w, _ = m.generate(a.warmup + 1)   # W untimed decode steps
    t0 = time.perf_counter()              # generate() returns only after the stream has drained
    ids, gpu_ns = m.generate(a.steps + 1)  # exactly K replays of the recorded decode step
    wall = time.perf_counter() - t0
    ctx_len = m.past()
    tok_s = a.steps / wall

    # the dominant kernel, timed live from its own dispatch timestamps over a few real steps
    acc, n_prof = {}, 8
    for _ in range(n_prof):
        for k, v in m.profile_step():
            acc[k] = acc.get(k, 0.0) + v / n_prof
    up_ns = acc["moe.up"] / cfg.n_layer
    up_bytes = moe_up_bytes(cfg)
    # HBM bytes per launch from hardware counters, measured in separate rocprofv3 runs of this same
    # script and kept with the other profile summaries; only valid for the shape it was taken on
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "moe_up_hbm_traffic.json")
    if os.path.exists(tpath) and (cfg.n_embd, cfg.n_expert_used, cfg.ffn_expert) == (2048, 10, 512):
        traffic = json.load(open(tpath)).get("traffic_bytes_per_launch")
    # one-row passes route in the expert kernel itself unless LLM_MOE_ROUTE=kernel keeps the selection a launch of its own
    fused = os.environ.get("LLM_MOE_ROUTE", "rows") in ("rows", "fused")
    # the router's logits ride on the mixer's output projection unless LLM_ROUTER_FOLD=0; gate/up then also normalises its row
    folded = fused and os.environ.get("LLM_ROUTER_FOLD", "1") != "0"
    roof = {"bound": "hbm", "kernel": "moe_up_kernel<2048, 1%s> (%sexpert-gathered Q4_K gate/up GEMV + SwiGLU)" %
                      (", true" if folded else "", ("RMSNorm of the residual row, " if folded else "") +
                       ("softmax and top-10 of the token's 512 router logits, then the " if fused else "")),
            "routing": "in this launch" if fused else "a launch of its own",
            "router_logits": "rows of the mixer's output projection launch" if folded else "a launch of their own",
            "achieved": round(up_bytes / (up_ns / 1e9) / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": round(up_bytes / (up_ns / 1e9) / HBM_PEAK, 4), "traffic": traffic,
            "bytes_per_launch": up_bytes, "avg_launch_us": round(up_ns / 1e3, 3), "launches_per_step": cfg.n_layer}
    tb = token_bytes(cfg, ctx_len)
    rec = {
        "metric": "batch-1 decode tok/s (Q4_K MoE+DeltaNet)", "value": round(tok_s, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(wall / a.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE config 5: synthetic random-init Qwen3-Next-shape model, %d layers "
                               "(3 gated-DeltaNet + 1 gated-attention), 512 experts top-10 + shared, Q4_K weights "
                               "drawn N(0,0.02) and quantised on the device by the reference's quantiser, fp16 KV "
                               "cache, vocab 151936; prompt %d random ids then greedy decode at batch 1"
                               % (cfg.n_layer, a.prompt),
                   "context_at_end": ctx_len, "prefill": "%d rows a pass (%.1f tok/s by the host's clock, upload and first-use set-up included, untimed)" % (a.prefill_rows, a.prompt / prefill_s),
                   "weights_GB": round(m.weight_bytes() / 1e9, 2), "dispatches_per_step": m.dispatches()},
        "gpu_ms_per_step": round(gpu_ns / a.steps / 1e6, 4),
        "token_bytes": tb, "token_roofline_tok_s": round(HBM_PEAK / tb, 1), "frac_of_token_roofline": round(tok_s * tb / HBM_PEAK, 4),
        # each op's own duration in an op-by-op profiled step (events around every op), and their sum; the wall time
        # of such a step, which the events themselves stretch, is not reported
        "step_kernel_us": dict([("sum_of_ops", round(sum(v for k, v in acc.items() if k != "total") / 1e3, 1))] +
                               [(k, round(v / 1e3, 1)) for k, v in sorted(acc.items(), key=lambda kv: -kv[1]) if k != "total"]),
        "roofline": roof,
        "gemv": gemv_rates(m, cfg, A, LA),
    }
    # one prompt chunk timed op by op (on a second sequence slot's worth of cells past the decoded
    # tokens): where a many-row pass spends its time, and what the expert kernels reach once a
    # launch carries enough bytes
    if a.prefill_rows >= 16 and ctx_len + a.prefill_rows + 1 <= cfg.nkv:
        st = dict(m.profile_chunk(rng.integers(0, cfg.vocab, size=a.prefill_rows).astype(np.int32)))
        rows = a.prefill_rows
        per_tok_up = (cfg.n_expert_used + 1) * 2 * cfg.ffn_expert * Q4K_ROW(cfg.n_embd)
        per_tok_down = (cfg.n_expert_used + 1) * cfg.n_embd * Q4K_ROW(cfg.ffn_expert)
        chunk_us = sum(v for k, v in st.items() if k != "total") / 1e3
        rec["prefill_chunk"] = {
            "rows": rows, "us": round(chunk_us, 1), "tok_s": round(rows / chunk_us * 1e6, 1),
            "op_us": {k: round(v / 1e3, 1) for k, v in sorted(st.items(), key=lambda kv: -kv[1]) if k != "total"},
            # multiply-adds of the rows' (10 routed + shared) experts, two flops each
            "moe_up_TFLOPs": round(rows * per_tok_up / 0.5625 * 2 * cfg.n_layer / (st["moe.up"] / 1e9) / 1e12, 1),
            "moe_down_TFLOPs": round(rows * per_tok_down / 0.5625 * 2 * cfg.n_layer / (st["moe.down"] / 1e9) / 1e12, 1)}
        if rows < 128:
            # below 128 rows every row reads its own experts: rows x (10 routed + shared) x rows of the banks
            rec["prefill_chunk"]["moe_up_GBps"] = round(rows * per_tok_up * cfg.n_layer / (st["moe.up"] / 1e9) / 1e9, 1)
            rec["prefill_chunk"]["moe_down_GBps"] = round(rows * per_tok_down * cfg.n_layer / (st["moe.down"] / 1e9) / 1e9, 1)
        if big and m.past() + big + 1 <= cfg.nkv:
            # BASELINE config 3's prefill shape and config 4's long-pass side: one chunk of 4096 rows
            st4 = dict(m.profile_chunk(rng.integers(0, cfg.vocab, size=big).astype(np.int32)))
            us4 = sum(v for k, v in st4.items() if k != "total") / 1e3
            n_dn = cfg.n_layer - cfg.n_layer // cfg.attn_every
            dn_us = sum(st4.get(k, 0) for k in ("dn.hist", "dn.qkv", "dn.step", "dn.out")) / 1e3
            at_us = sum(st4.get(k, 0) for k in ("attn.qkv", "attn.attn", "attn.out")) / 1e3
            rec["prefill_chunk_4096"] = {
                "rows": big, "context_before": m.past() - big, "us": round(us4, 1), "tok_s": round(big / us4 * 1e6, 1),
                "op_us": {k: round(v / 1e3, 1) for k, v in sorted(st4.items(), key=lambda kv: -kv[1]) if k != "total"},
                "deltanet_layer_us": round(dn_us / n_dn, 1), "deltanet_step_us_per_layer": round(st4.get("dn.step", 0) / 1e3 / n_dn, 1),
                "attention_layer_us": round(at_us / (cfg.n_layer // cfg.attn_every), 1)}
    if a.pmc_copy:
        import ctypes as C
        H = A.load()
        n = 256 << 20
        src, dst = C.c_void_p(), C.c_void_p()
        A.check(H.shv_alloc(m.ctx, n, C.byref(src)))
        A.check(H.shv_alloc(m.ctx, n, C.byref(dst)))
        A.check(H.shv_zero(m.ctx, src, n))
        A.check(H.shv_copy(m.ctx, dst, src, n))
        A.check(H.shv_sync(m.ctx))
        rec["pmc_copy_bytes"] = n
    if not a.no_mtp:
        plain = [int(t) for t in ids_w] + [int(t) for t in ids[1:]]
        rounds = min(a.mtp_rounds, (len(plain) - 4) // 3)
        if rounds >= 1:
            rec["mtp"] = mtp_run(m, cfg, prompt, plain, acc, rounds)
            # the recorded 3-row verification pass against the recorded one-row step, both as the GPU's clock has them
            # (pass_N_rows_in_steps above are sums of per-kernel times of passes dispatched op by op)
            rec["mtp"]["verify_pass_in_steps"] = round(rec["mtp"]["true_continuation_as_drafts"]["verify_gpu_ms_per_round"] / rec["gpu_ms_per_step"], 3)
    if not a.no_mtp and a.batch_slots >= 2:
        rec["batched_decode"] = batched_run(m, cfg, a.batch_slots, rng)
        # fewer sequences a pass, on the same staged slots: what a lightly loaded server runs
        rec["batched_decode_few"] = {str(n): batched_run(m, cfg, n, rng, steps=24) for n in (2, 3, 4) if n < a.batch_slots}
    cores = min(os.cpu_count() or 1, 16)
    tensors = first_period_tensors(m, cfg) if not a.no_cpu else None
    if not a.no_configs:
        rec["configs"] = config_blocks(m, cfg, A, tensors, cores, not a.no_cpu)
        rec["configs"]["config1_gemv_4096x2048"] = dict(rec["gemv"]["config1_4096x2048"])
        if "prefill_chunk_4096" in rec:
            pc = rec["prefill_chunk_4096"]
            rec["configs"]["config3_deltanet_layer"]["prefill_4096_rows"] = {
                "gpu_us_per_layer": pc["deltanet_layer_us"], "gpu_us_per_row": round(pc["deltanet_layer_us"] / pc["rows"], 4),
                "step_us_per_layer": pc["deltanet_step_us_per_layer"], "recurrence": "closed form over chunks of 64 rows"}
            rec["configs"]["config4_attention_decode"]["prefill_4096_rows"] = {
                "gpu_us_per_layer": pc["attention_layer_us"], "context_before": pc["context_before"]}
        if not a.no_cpu:
            x = rng.standard_normal(cfg.n_embd).astype(np.float32)
            import oracle_lib as O
            wq = tensors["blk.0.ffn_gate_exps.weight"][:4096 * Q4K_ROW(cfg.n_embd)]
            best = 1e9
            for _ in range(5):
                t0 = time.perf_counter()
                O.gemv_q4k(wq, x, 4096, cfg.n_embd, threads=cores)
                best = min(best, time.perf_counter() - t0)
            rec["configs"]["config1_gemv_4096x2048"].update(cpu_us=round(best * 1e6, 1), cpu_cores=cores)
    if not a.no_cpu:
        rec["cpu_baseline"] = cpu_baseline(m, cfg, LA, A, tensors, a.cpu_tokens, cores)
    m.close()
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
