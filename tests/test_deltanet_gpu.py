"""Gated DeltaNet layer on the GPU (fused projection GEMV -> dn_step -> out projection with the
gated norm as its prologue) against the oracle's DeltaNetLayer (llm/deltanet.go:212-403)."""
import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu
A = shv.api
TOL = 1e-3
EPS = 1e-6


class DnCase:
    def __init__(self, ctx, seed, H=2048, hk=16, hv=32, d=128, conv=4):
        rng = np.random.default_rng(seed)
        self.ctx, self.H, self.hk, self.hv, self.d, self.conv = ctx, H, hk, hv, d, conv
        self.qk, self.vw = hk * d, hv * d
        self.cw = 2 * self.qk + self.vw
        self.width = self.cw + self.vw + 2 * hv  # fused projection rows: qkv | z | alpha | beta
        q = lambda rows, k: O.quantize_q4k((rng.standard_normal((rows, k)) * 0.02).astype(np.float32))
        self.qkv, self.z, self.alpha, self.beta = q(self.cw, H), q(self.vw, H), q(hv, H), q(hv, H)
        self.out = q(H, self.vw)
        self.conv1d = (rng.standard_normal((self.cw, conv)) * 0.3).astype(np.float32)
        self.a = (-np.exp(rng.standard_normal(hv))).astype(np.float32)
        self.dt_bias = rng.standard_normal(hv).astype(np.float32)
        self.norm = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        self.rng = rng
        self.fused = np.concatenate([self.qkv, self.z, self.alpha, self.beta], axis=0)

    def cfg(self):
        return O.DnCfg(self.H, self.d, self.hk, self.hv, self.conv, EPS, 0)

    def w(self):
        return O.DnW(O.B(self.qkv), O.B(self.z), O.B(self.alpha), O.B(self.beta), O.B(self.out),
                     O.F(self.conv1d), O.F(self.a), O.F(self.dt_bias), O.F(self.norm))

    def oracle(self, xn, conv_state, s_state):
        T = xn.shape[0]
        res = np.empty((T, self.H), np.float32)
        attn = np.empty((T, self.vw), np.float32)
        cfg, w = self.cfg(), self.w()
        O.lib().shv_ref_deltanet_layer(O.C.byref(cfg), O.C.byref(w), O.F(xn), T, O.F(conv_state),
                                       O.F(s_state), O.F(res), None, None, None, None, None,
                                       O.F(attn), None, 0, 8)
        return res, attn

    def upload(self):
        c = self.ctx
        self.d_fused, self.d_out = c.upload(self.fused), c.upload(self.out)
        self.d_conv, self.d_a, self.d_dt = c.upload(self.conv1d), c.upload(self.a), c.upload(self.dt_bias)
        self.d_norm = c.upload(self.norm)

    def step_ops(self, d_x, d_ring, d_state, d_attn, d_res, d_pos, d_slot, n_seq, seq_len, ring_slots, work=None):
        """work: a scratch buffer; with it a pass of more than 16 rows takes the chunked kernels."""
        n_tok = n_seq * seq_len
        return [
            A.make_op(A.OP_GEMV_Q4K, A.gemv_args(self.d_fused, d_x, d_ring, self.width, self.H, n_tok,
                                                 pos=d_pos, slot=d_slot, seq_len=seq_len,
                                                 ring_slots=ring_slots, ring_stride=self.width)),
            A.make_op(A.OP_DN_STEP, A.DnStepArgs(d_ring.ptr, self.d_conv.ptr, self.d_a.ptr, self.d_dt.ptr,
                                                 d_state.ptr, d_attn.ptr, d_pos.ptr,
                                                 A.ptr(d_slot), n_seq, seq_len, self.hk, self.hv,
                                                 self.d, self.conv, ring_slots, self.width, EPS, 0, None, 0, 0,
                                                 A.ptr(work), work.nbytes // 4 if work is not None else 0)),
            A.make_op(A.OP_GEMV_Q4K, A.gemv_args(self.d_out, d_attn, d_res, self.H, self.vw, n_tok,
                                                 prologue=A.PRO_GATED_NORM, gamma=self.d_norm,
                                                 z=d_ring.at(0), head_dim=self.d, eps=EPS)),
        ]


def test_decode_steps_from_a_fresh_state(ctx):
    """Seven tokens one at a time on the GPU against seven tokens in one oracle call."""
    case = DnCase(ctx, seed=1)
    case.upload()
    T = 7
    xn = case.rng.standard_normal((T, case.H)).astype(np.float32)
    conv_state = np.zeros((case.cw, 3), np.float32)
    s_state = np.zeros((case.hv, case.d, case.d), np.float32)
    want_res, want_attn = case.oracle(xn, conv_state, s_state)

    c = ctx
    slots = 4
    d_ring = c.alloc(slots * case.width * 4).zero()
    d_state = c.alloc(s_state.nbytes).zero()
    d_attn, d_res = c.alloc(case.vw * 4), c.alloc(case.H * 4)
    d_pos, d_x = c.alloc(4), c.alloc(case.H * 4)
    got_res, got_attn = [], []
    for t in range(T):
        d_pos.write(np.array([t], np.int32))
        d_x.write(xn[t])
        ops = case.step_ops(d_x, d_ring, d_state, d_attn, d_res, d_pos, None, 1, 1, slots)
        # the out projection reads z from the ring row of this position
        ga = A.gemv_args(case.d_out, d_attn, d_res, case.H, case.vw, 1, prologue=A.PRO_GATED_NORM,
                         gamma=case.d_norm, z=d_ring.at(((t % slots) * case.width + case.cw) * 4),
                         head_dim=case.d, eps=EPS)
        ops[2] = A.make_op(A.OP_GEMV_Q4K, ga)
        c.dispatch_multi(ops)
        got_res.append(d_res.read(np.float32, case.H))
        got_attn.append(d_attn.read(np.float32, case.vw))
    got_res, got_attn = np.array(got_res), np.array(got_attn)
    e_attn, e_res = O.rel_l2(got_attn, want_attn), O.rel_l2(got_res, want_res)
    e_state = O.rel_l2(d_state.read(np.float32, s_state.size), s_state)
    print(f"deltanet decode x{T}: attn {e_attn:.3e} result {e_res:.3e} state {e_state:.3e}")
    assert e_attn <= TOL and e_res <= TOL and e_state <= TOL
    for t in range(T):
        assert O.rel_l2(got_res[t], want_res[t]) <= TOL, t


@pytest.mark.parametrize("B,R", [(1, 1), (8, 1), (5, 6)])
def test_decode_step_with_random_state(ctx, B, R):
    """BASELINE config 3, decode mode: batch 1 and 8 sequences, each with its own state ~N(0,0.1)
    and its own three rows of conv history, at different positions; and five sequences of six rows
    each in one call (from four sequences on a wave holds four state rows instead of two)."""
    case = DnCase(ctx, seed=10 + B)
    case.upload()
    rng = case.rng
    slots = 4 if R == 1 else 12
    xn = rng.standard_normal((B, R, case.H)).astype(np.float32)
    s0 = (rng.standard_normal((B, case.hv, case.d, case.d)) * 0.1).astype(np.float32)
    hist = rng.standard_normal((B, 3, case.width)).astype(np.float32)  # rows at positions p-3..p-1
    pos = (3 + 5 * np.arange(B)).astype(np.int32)
    ring = np.zeros((B, slots, case.width), np.float32)
    for b in range(B):
        for i in range(3):
            ring[b, (pos[b] - 3 + i) % slots] = hist[b, i]
    c = ctx
    d_ring, d_state = c.upload(ring), c.upload(s0)
    d_attn, d_res = c.alloc(B * R * case.vw * 4), c.alloc(B * R * case.H * 4)
    d_pos, d_x = c.upload(pos), c.upload(xn.reshape(B * R, case.H))
    ops = case.step_ops(d_x, d_ring, d_state, d_attn, d_res, d_pos, None, B, R, slots)[:2]
    c.dispatch_multi(ops)
    got_attn = d_attn.read(np.float32, B * R * case.vw).reshape(B, R, case.vw)
    got_state = d_state.read(np.float32, s0.size).reshape(s0.shape)
    for b in range(B):
        conv_state = np.ascontiguousarray(hist[b, :, :case.cw].T)  # [cw][3], column 0 oldest
        s_state = s0[b].copy()
        _, want_attn = case.oracle(xn[b], conv_state, s_state)
        for r in range(R):
            assert O.rel_l2(got_attn[b, r], want_attn[r]) <= TOL, (b, r)
        assert O.rel_l2(got_state[b], s_state) <= TOL, b


@pytest.mark.parametrize("T,slots,pos0", [(3, 8, 0), (8, 16, 0), (9, 16, 0), (37, 48, 0), (64, 80, 0), (21, 32, 27)])
def test_rows_in_one_call_equal_single_steps(ctx, T, slots, pos0):
    """A multi-row pass over one sequence (a verify pass, a prompt chunk) walks its rows in order
    on one state: the CPU's answer row by row.  Up to eight rows go through the decode kernel, more
    through the one whose extra waves prepare the next group of eight while the rule runs on this
    one: whole and ragged groups, and a start in mid-sequence with the ring wrapping (history rows
    at pos0-3..pos0-1, the state of a sequence that has already run)."""
    case = DnCase(ctx, seed=21 + T)
    case.upload()
    rng = case.rng
    xn = rng.standard_normal((T, case.H)).astype(np.float32)
    hist = rng.standard_normal((3, case.width)).astype(np.float32) if pos0 else np.zeros((3, case.width), np.float32)
    s0 = (rng.standard_normal((case.hv, case.d, case.d)) * 0.1).astype(np.float32) if pos0 else np.zeros((case.hv, case.d, case.d), np.float32)
    conv_state = np.ascontiguousarray(hist[:, :case.cw].T)       # [cw][3], column 0 oldest
    s_state = s0.copy()
    _, want_attn = case.oracle(xn, conv_state, s_state)
    ring = np.zeros((slots, case.width), np.float32)
    for i in range(3):
        if pos0:
            ring[(pos0 - 3 + i) % slots] = hist[i]
    c = ctx
    d_ring, d_state = c.upload(ring), c.upload(s0)
    d_attn, d_res = c.alloc(T * case.vw * 4), c.alloc(T * case.H * 4)
    ops = case.step_ops(c.upload(xn), d_ring, d_state, d_attn, d_res, c.upload(np.array([pos0], np.int32)),
                        None, 1, T, slots)[:2]
    c.dispatch_multi(ops)
    got = d_attn.read(np.float32, T * case.vw).reshape(T, -1)
    for t in range(T):
        assert O.rel_l2(got[t], want_attn[t]) <= TOL, t
    assert O.rel_l2(d_state.read(np.float32, s_state.size), s_state) <= TOL


@pytest.mark.parametrize("T,pos0,n_seq", [(17, 0, 1), (64, 0, 1), (150, 0, 1), (257, 41, 1), (64, 27, 1), (100, 5, 3), (2048, 3, 1), (4096, 0, 1)])
def test_chunked_rows_equal_the_row_by_row_rule(ctx, T, pos0, n_seq):
    """With a workspace a pass of more than 16 rows goes 64 rows at a time on the matrix cores (the
    delta rule's closed form over a chunk).  Against the oracle's row-by-row rule (every row's
    output and the final state within 1e-3), and against this library's own row-by-row kernel on
    the same inputs, which it must match far closer than that: whole chunks, ragged ones, several
    chunks, a start in mid-sequence (history rows, a state that has already run), several sequences
    in one call, and passes of 2048 and 4096 rows.  With room in the workspace for a record per chunk
    and value head, what a chunk needs that does not depend on the state is formed for all chunks at
    once by a launch of its own, (I + A)^-1 whole among it, so that road's solve is one product
    where the other walks the block rows: the two chunked roads are held to the same bar against the
    row-by-row kernel, and to each other."""
    case = DnCase(ctx, seed=300 + T + n_seq)
    case.upload()
    rng = case.rng
    slots = T + 3
    xn = rng.standard_normal((n_seq, T, case.H)).astype(np.float32)
    started = pos0 > 0
    hist = rng.standard_normal((n_seq, 3, case.width)).astype(np.float32) if started else np.zeros((n_seq, 3, case.width), np.float32)
    s0 = (rng.standard_normal((n_seq, case.hv, case.d, case.d)) * 0.1).astype(np.float32) if started else np.zeros((n_seq, case.hv, case.d, case.d), np.float32)
    pos = (pos0 + 7 * np.arange(n_seq)).astype(np.int32) if started else np.zeros(n_seq, np.int32)
    ring = np.zeros((n_seq, slots, case.width), np.float32)
    for b in range(n_seq):
        for i in range(3):
            if started:
                ring[b, (pos[b] - 3 + i) % slots] = hist[b, i]
    c = ctx
    d_x, d_pos = c.upload(xn.reshape(n_seq * T, case.H)), c.upload(pos)
    results = []
    prep_floats = (n_seq * T * (case.cw + 2 * case.hv) + 3) & ~3
    rec_floats = n_seq * ((T + 63) // 64) * case.hv * 10880
    for chunked in ("records", "in the walk", None):
        d_ring, d_state = c.upload(ring), c.upload(s0)
        d_attn, d_res = c.alloc(n_seq * T * case.vw * 4), c.alloc(n_seq * T * case.H * 4)
        work = c.alloc((prep_floats + (rec_floats if chunked == "records" else 0)) * 4) if chunked else None
        ops = case.step_ops(d_x, d_ring, d_state, d_attn, d_res, d_pos, None, n_seq, T, slots, work=work)[:2]
        c.dispatch_multi(ops)
        results.append((d_attn.read(np.float32, n_seq * T * case.vw).reshape(n_seq, T, case.vw),
                        d_state.read(np.float32, s0.size).reshape(s0.shape)))
        for b in (d_ring, d_state, d_attn, d_res):
            b.free()
        if work is not None:
            work.free()
    (got_attn, got_state), (walk_attn, walk_state), (seq_attn, seq_state) = results
    e_w = max(O.rel_l2(walk_attn, seq_attn), O.rel_l2(walk_state, seq_state), O.rel_l2(got_attn, walk_attn), O.rel_l2(got_state, walk_state))
    print(f"deltanet chunked T={T} x{n_seq}: the walk that forms its chunks' operands itself, and the two walks against each other: {e_w:.3e}")
    assert e_w <= 2e-5
    e_a, e_s = O.rel_l2(got_attn, seq_attn), O.rel_l2(got_state, seq_state)
    print(f"deltanet chunked T={T} x{n_seq}: against the row-by-row kernel: rows {e_a:.3e} state {e_s:.3e}")
    assert e_a <= 2e-5 and e_s <= 2e-5
    for b in range(n_seq if T <= 300 else 0):
        conv_state = np.ascontiguousarray(hist[b, :, :case.cw].T)
        s_state = s0[b].copy()
        _, want_attn = case.oracle(xn[b], conv_state, s_state)
        worst = max(O.rel_l2(got_attn[b, t], want_attn[t]) for t in range(T))
        assert worst <= TOL, (b, worst)
        assert O.rel_l2(got_state[b], s_state) <= TOL, b
    if T > 300:
        # the long pass against the oracle too (a few seconds of CPU)
        conv_state = np.ascontiguousarray(hist[0, :, :case.cw].T)
        s_state = s0[0].copy()
        _, want_attn = case.oracle(xn[0], conv_state, s_state)
        assert O.rel_l2(got_attn[0], want_attn) <= TOL
        assert max(O.rel_l2(got_attn[0, t], want_attn[t]) for t in range(0, T, 97)) <= TOL
        assert O.rel_l2(got_state[0], s_state) <= TOL


def test_dn_step_refuses_unsupported_shapes(ctx):
    d = ctx.alloc(1 << 16)
    with pytest.raises(shv.pkg.ShvError):
        ctx.enqueue(A.OP_DN_STEP, A.DnStepArgs(d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, None, 1, 1,
                                               16, 32, 64, 4, 4, 12352, EPS, 0))
    with pytest.raises(shv.pkg.ShvError):
        ctx.enqueue(A.OP_DN_STEP, A.DnStepArgs(d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, None, 1, 4,
                                               16, 32, 128, 4, 4, 12352, EPS, 0))
