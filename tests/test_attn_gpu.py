"""Gated full-attention decode on the GPU (fused q|gate,k,v GEMV -> attn_decode -> output
projection with the sigmoid gate as prologue) against the oracle's AttnLayerAt restated over an
fp16 cache (llm/attn.go:135-219,444-586)."""
import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu
A = shv.api
TOL = 1e-3
EPS = 1e-6
H, NH, NKV, D, ROPE, BASE = 2048, 16, 2, 256, 64, 1e7
SECTIONS = (11, 11, 10, 0)


def rope_table(max_pos, rope_dims=ROPE, base=BASE):
    """cos/sin per position as the reference builds them: theta_i = pos * s^i with s =
    base^(-2/rope_dims), the power taken by repeated multiplication in float64
    (llm/attn.go:553-584), rounded to float32 once."""
    half = rope_dims // 2
    scale = float(base) ** (-2.0 / rope_dims)
    theta = np.arange(max_pos, dtype=np.float64)
    out = np.empty((max_pos, rope_dims), dtype=np.float32)
    for i in range(half):
        out[:, i] = np.cos(theta)
        out[:, half + i] = np.sin(theta)
        theta = theta * scale
    return out


class AttnCase:
    def __init__(self, ctx, seed):
        rng = np.random.default_rng(seed)
        self.ctx, self.rng = ctx, rng
        q = lambda rows, k: O.quantize_q4k((rng.standard_normal((rows, k)) * 0.02).astype(np.float32))
        self.q, self.k, self.v, self.o = q(NH * 2 * D, H), q(NKV * D, H), q(NKV * D, H), q(H, NH * D)
        self.q_norm = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
        self.k_norm = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
        self.fused = np.concatenate([self.q, self.k, self.v], axis=0)
        self.width = NH * 2 * D + 2 * NKV * D

    def cfg(self):
        return O.AttnCfg(H, NH, NKV, D, ROPE, BASE, (O.C.c_int * 4)(*SECTIONS), EPS)

    def w(self):
        return O.AttnW(O.B(self.q), O.B(self.k), O.B(self.v), O.B(self.o), O.F(self.q_norm), O.F(self.k_norm))

    def oracle(self, xn, past, kc, vc):
        T = xn.shape[0]
        out = np.empty((T, H), np.float32)
        pre = np.empty((T, NH * D), np.float32)
        cfg, w = self.cfg(), self.w()
        O.lib().shv_ref_attn_layer(O.C.byref(cfg), O.C.byref(w), O.F(xn), T, past, O.H(kc), O.H(vc),
                                   O.F(out), None, O.F(pre), 8)
        return out, pre

    def upload(self, max_cells):
        c = self.ctx
        self.d_fused, self.d_o = c.upload(self.fused), c.upload(self.o)
        self.d_qn, self.d_kn = c.upload(self.q_norm), c.upload(self.k_norm)
        self.d_rope = c.upload(rope_table(max_cells))

    def ops(self, d_x, d_qkv, d_kc, d_vc, d_part, d_ctx, d_out, d_pos, n_seq, seq_len, max_cells, n_splits):
        rows = n_seq * seq_len
        return [
            A.make_op(A.OP_GEMV_Q4K, A.gemv_args(self.d_fused, d_x, d_qkv, self.width, H, rows)),
            A.make_op(A.OP_ATTN_DECODE, A.AttnDecodeArgs(
                d_qkv.ptr, self.d_qn.ptr, self.d_kn.ptr, self.d_rope.ptr, d_kc.ptr, d_vc.ptr, d_part.ptr,
                d_ctx.ptr, d_pos.ptr, None, n_seq, seq_len, NH, NKV, D, ROPE, max_cells, self.width,
                n_splits, EPS)),
            A.make_op(A.OP_GEMV_Q4K, A.gemv_args(self.d_o, d_ctx, d_out, H, NH * D, rows,
                                                 prologue=A.PRO_MUL_SIGMOID, z=d_qkv, head_dim=D,
                                                 z_stride=self.width)),
        ]


def v_dev(vc):
    """the device's V layout, tiles of 32 cells transposed: [..., cell/32, kv head, dim, cell%32] from
    the reference's [..., cell, kv head, dim]"""
    lead, (cells, nkv, d) = vc.shape[:-3], vc.shape[-3:]
    t = vc.reshape(*lead, cells // 32, 32, nkv, d)
    return np.ascontiguousarray(np.moveaxis(t, -3, -1))


def v_host(vt):
    """back to [..., cell, kv head, dim]"""
    lead, (blocks, nkv, d, _) = vt.shape[:-4], vt.shape[-4:]
    return np.ascontiguousarray(np.moveaxis(vt, -1, -3)).reshape(*lead, blocks * 32, nkv, d)


def _part_floats(n_seq, n_splits, seq_len=1):
    return n_seq * (seq_len + (seq_len & 1)) * NKV * n_splits * (NH // NKV) * (D + 2)


def test_decode_steps_from_an_empty_cache(ctx):
    """Nine tokens one at a time against nine tokens in one oracle call (prefill == steps)."""
    case = AttnCase(ctx, seed=3)
    T, max_cells, n_splits = 9, 64, 4
    case.upload(max_cells)
    xn = case.rng.standard_normal((T, H)).astype(np.float32)
    kc = np.zeros((max_cells, NKV, D), np.uint16)
    vc = np.zeros_like(kc)
    want_out, want_pre = case.oracle(xn, 0, kc, vc)
    c = ctx
    d_kc, d_vc = c.alloc(kc.nbytes).zero(), c.alloc(vc.nbytes).zero()
    d_qkv, d_ctx, d_out = c.alloc(case.width * 4), c.alloc(NH * D * 4), c.alloc(H * 4)
    d_part, d_pos, d_x = c.alloc(_part_floats(1, n_splits) * 4), c.alloc(4), c.alloc(H * 4)
    for t in range(T):
        d_pos.write(np.array([t], np.int32))
        d_x.write(xn[t])
        c.dispatch_multi(case.ops(d_x, d_qkv, d_kc, d_vc, d_part, d_ctx, d_out, d_pos, 1, 1, max_cells, n_splits))
        e_pre = O.rel_l2(d_ctx.read(np.float32, NH * D), want_pre[t])
        e_out = O.rel_l2(d_out.read(np.float32, H), want_out[t])
        assert e_pre <= TOL and e_out <= TOL, (t, e_pre, e_out)
    # the cache the GPU wrote is the oracle's, half for half (norm, rope and rounding agree)
    got_k = d_kc.read(np.uint16, kc.size).reshape(kc.shape)[:T]
    got_v = v_host(d_vc.read(np.uint16, vc.size).reshape(max_cells // 32, NKV, D, 32))[:T]
    # float32 sums that differ in the last bits round to neighbouring halves now and then: never
    # more than one spacing of halves apart (or 1e-5 near zero), and only on a few percent of cells
    for got, want in ((got_k, kc[:T]), (got_v, vc[:T])):
        g, w = got.view(np.float16).astype(np.float32), want.view(np.float16).astype(np.float32)
        assert (np.abs(g - w) <= np.abs(w) * 2.0 ** -10 + 1e-5).all()
        assert np.count_nonzero(got != want) <= got.size // 20


@pytest.mark.parametrize("past,rows,n_splits", [(0, 2, 4), (0, 5, 4), (61, 4, 8), (300, 3, 16), (4000, 2, 64),
                                                # three and four rows write their cells inside the launch, the second pair's
                                                # blocks the first pair's too: new cells on either side of a slice's and of
                                                # a tile's boundary, in the first tile, deep in a long cache
                                                (127, 4, 8), (126, 3, 8), (31, 4, 4), (255, 3, 16), (0, 3, 4), (1, 4, 4), (2046, 4, 64)])
def test_rows_of_one_sequence_in_one_call(ctx, past, rows, n_splits):
    """A verification pass or a prompt chunk: `rows` consecutive rows appended in one call, each
    seeing the cells up to its own (the cache is walked once for two rows at a time), against the
    oracle's layer over the same rows; the new cells may straddle a slice boundary."""
    case = AttnCase(ctx, seed=5 + past)
    max_cells = ((past + rows + 63) // 64) * 64
    case.upload(max_cells)
    rng = case.rng
    kc = np.zeros((max_cells, NKV, D), np.uint16)
    vc = np.zeros_like(kc)
    kc[:past] = rng.standard_normal((past, NKV, D)).astype(np.float16).view(np.uint16)
    vc[:past] = rng.standard_normal((past, NKV, D)).astype(np.float16).view(np.uint16)
    xn = rng.standard_normal((rows, H)).astype(np.float32)
    c = ctx
    d_kc, d_vc = c.upload(kc), c.upload(v_dev(vc))
    want_out, want_pre = case.oracle(xn, past, kc, vc)
    d_qkv, d_ctx, d_out = c.alloc(rows * case.width * 4), c.alloc(rows * NH * D * 4), c.alloc(rows * H * 4)
    d_part = c.alloc(_part_floats(1, n_splits, rows) * 4)
    c.dispatch_multi(case.ops(c.upload(xn), d_qkv, d_kc, d_vc, d_part, d_ctx, d_out,
                              c.upload(np.array([past], np.int32)), 1, rows, max_cells, n_splits))
    got_pre = d_ctx.read(np.float32, rows * NH * D).reshape(rows, -1)
    got_out = d_out.read(np.float32, rows * H).reshape(rows, -1)
    for t in range(rows):
        assert O.rel_l2(got_pre[t], want_pre[t]) <= TOL and O.rel_l2(got_out[t], want_out[t]) <= TOL, t
    got_k = d_kc.read(np.uint16, kc.size).reshape(kc.shape)[past:past + rows]
    g, w = got_k.view(np.float16).astype(np.float32), kc[past:past + rows].view(np.float16).astype(np.float32)
    assert (np.abs(g - w) <= np.abs(w) * 2.0 ** -10 + 1e-5).all()


@pytest.mark.parametrize("past,rows,n_splits", [(1030, 64, 64), (1500, 48, 64), (2100, 32, 16), (4200, 16, 64), (700, 40, 6)])
def test_prompt_chunk_with_a_slice_left_empty(ctx, past, rows, n_splits):
    """A prompt chunk of 15 rows and more over a cache that holds more cells than its slices were
    cut for: slices start on whole tiles of V, so the last of a row pair's slices can start past the
    pair's cells and hold nothing.  The merge must take such a slice for empty whatever its record
    held before (here noise: the records of an earlier layer's pass in real use)."""
    case = AttnCase(ctx, seed=50 + past)
    max_cells = ((past + rows + 63) // 64) * 64
    case.upload(max_cells)
    rng = case.rng
    kc = np.zeros((max_cells, NKV, D), np.uint16)
    vc = np.zeros_like(kc)
    kc[:past] = rng.standard_normal((past, NKV, D)).astype(np.float16).view(np.uint16)
    vc[:past] = rng.standard_normal((past, NKV, D)).astype(np.float16).view(np.uint16)
    xn = rng.standard_normal((rows, H)).astype(np.float32)
    c = ctx
    d_kc, d_vc = c.upload(kc), c.upload(v_dev(vc))
    want_out, want_pre = case.oracle(xn, past, kc, vc)
    d_qkv, d_ctx, d_out = c.alloc(rows * case.width * 4), c.alloc(rows * NH * D * 4), c.alloc(rows * H * 4)
    d_part = c.upload((rng.standard_normal(_part_floats(1, n_splits, rows)) * 8).astype(np.float32))
    c.dispatch_multi(case.ops(c.upload(xn), d_qkv, d_kc, d_vc, d_part, d_ctx, d_out,
                              c.upload(np.array([past], np.int32)), 1, rows, max_cells, n_splits))
    got_pre = d_ctx.read(np.float32, rows * NH * D).reshape(rows, -1)
    got_out = d_out.read(np.float32, rows * H).reshape(rows, -1)
    for t in range(rows):
        assert O.rel_l2(got_pre[t], want_pre[t]) <= TOL and O.rel_l2(got_out[t], want_out[t]) <= TOL, t


@pytest.mark.parametrize("past,n_seq,n_splits", [(4096, 1, 16), (4096, 3, 16), (32768, 1, 64),
                                                 (32768, 3, 64), (131071, 1, 256), (131071, 3, 128),
                                                 (1000, 1, 7), (5, 1, 64)])
def test_decode_over_a_prefilled_cache(ctx, past, n_seq, n_splits):
    """BASELINE config 4: cache prefilled with N(0,1) halves; one decode row per slot."""
    case = AttnCase(ctx, seed=1000 + past + n_seq)
    rng = case.rng
    max_cells = (past + 32) // 32 * 32   # room for the new cell, a multiple of 32
    case.upload(max_cells)
    c = ctx
    xn = rng.standard_normal((n_seq, H)).astype(np.float32)
    kcs = rng.standard_normal((n_seq, max_cells, NKV, D), dtype=np.float32).astype(np.float16).view(np.uint16)
    vcs = rng.standard_normal((n_seq, max_cells, NKV, D), dtype=np.float32).astype(np.float16).view(np.uint16)
    d_kc, d_vc = c.upload(kcs), c.upload(v_dev(vcs))
    d_qkv, d_ctx, d_out = c.alloc(n_seq * case.width * 4), c.alloc(n_seq * NH * D * 4), c.alloc(n_seq * H * 4)
    d_part = c.alloc(_part_floats(n_seq, n_splits) * 4)
    d_pos = c.upload(np.full(n_seq, past, np.int32))
    c.dispatch_multi(case.ops(c.upload(xn), d_qkv, d_kc, d_vc, d_part, d_ctx, d_out, d_pos, n_seq, 1,
                              max_cells, n_splits))
    got_pre = d_ctx.read(np.float32, n_seq * NH * D).reshape(n_seq, -1)
    got_out = d_out.read(np.float32, n_seq * H).reshape(n_seq, -1)
    for s in range(n_seq):
        kc, vc = kcs[s].copy(), vcs[s].copy()
        want_out, want_pre = case.oracle(xn[s:s + 1], past, kc, vc)
        e_pre, e_out = O.rel_l2(got_pre[s], want_pre[0]), O.rel_l2(got_out[s], want_out[0])
        print(f"attn ctx={past + 1} slot {s}/{n_seq}: pregate {e_pre:.3e} out {e_out:.3e}")
        assert e_pre <= TOL and e_out <= TOL
    for b in (d_kc, d_vc):
        b.free()


def test_split_count_does_not_change_the_answer(ctx):
    """llm/gpu_attn_cache_test.go:395 (split vs unsplit within 1e-3); here 1e-5."""
    case = AttnCase(ctx, seed=5)
    past, max_cells = 3000, 3008 + 32 - 3008 % 32
    case.upload(max_cells)
    rng, c = case.rng, ctx
    xn = rng.standard_normal((1, H)).astype(np.float32)
    kc = rng.standard_normal((max_cells, NKV, D), dtype=np.float32).astype(np.float16).view(np.uint16)
    vc = rng.standard_normal((max_cells, NKV, D), dtype=np.float32).astype(np.float16).view(np.uint16)
    outs = []
    for n_splits in (3, 16, 100):
        d_kc, d_vc = c.upload(kc), c.upload(v_dev(vc))
        d_qkv, d_ctx, d_out = c.alloc(case.width * 4), c.alloc(NH * D * 4), c.alloc(H * 4)
        c.dispatch_multi(case.ops(c.upload(xn), d_qkv, d_kc, d_vc, c.alloc(_part_floats(1, n_splits) * 4),
                                  d_ctx, d_out, c.upload(np.array([past], np.int32)), 1, 1, max_cells, n_splits))
        outs.append(d_ctx.read(np.float32, NH * D))
    assert O.rel_l2(outs[1], outs[0]) <= 1e-5 and O.rel_l2(outs[2], outs[0]) <= 1e-5


def test_attn_refuses_unsupported_shapes(ctx):
    d = ctx.alloc(1 << 16)
    mk = lambda **kw: A.AttnDecodeArgs(**{**dict(qkv=d.ptr, q_norm=d.ptr, k_norm=d.ptr, rope=d.ptr, kcache=d.ptr,
                                                 vcache=d.ptr, partial=d.ptr, out=d.ptr, pos=d.ptr, slot=None,
                                                 n_seq=1, seq_len=1, n_head=16, n_head_kv=2, head_dim=256,
                                                 rope_dims=64, max_cells=64, qkv_stride=9216, n_splits=4,
                                                 eps=EPS), **kw})
    for bad in (dict(head_dim=128), dict(n_head=24), dict(n_splits=1000), dict(qkv_stride=100)):
        with pytest.raises(shv.pkg.ShvError):
            ctx.enqueue(A.OP_ATTN_DECODE, mk(**bad))
