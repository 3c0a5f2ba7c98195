"""The block-sparse indexer and the attention that honours its selection on the GPU (shv_qsa_index +
shv_attn_decode with a mask) against the oracle's AttnLayerAt with Ratio > 0 (llm/attn.go:221-443,
588-682).  Selected cells are demanded bit for bit wherever the value at the cut is clear of its
neighbours (the reference's own practice for top-k under rounding, llm/moe_test.go:59-66; its
selection test compares set for set, llm/qsa4k_test.go)."""
import numpy as np
import pytest

import oracle_lib as O
import shv
from test_attn_gpu import AttnCase, rope_table, v_dev, H, NH, NKV, D, ROPE, BASE, SECTIONS, EPS, TOL, _part_floats

pytestmark = pytest.mark.gpu
A = shv.api
IH, ID = 4, 128


class QsaCase(AttnCase):
    def __init__(self, ctx, seed, top_k, ratio):
        super().__init__(ctx, seed)
        rng = self.rng
        self.top_k, self.ratio = top_k, ratio
        self.gamma = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
        self.iq = (rng.standard_normal((IH * ID, H)) * 0.02).astype(np.float32)
        self.ik = (rng.standard_normal((ID, H)) * 0.02).astype(np.float32)
        self.iqn = (1 + 0.1 * rng.standard_normal(ID)).astype(np.float32)
        self.ikn = (1 + 0.1 * rng.standard_normal(ID)).astype(np.float32)

    def cfg(self):
        c = super().cfg()
        c.idx_heads, c.idx_dim, c.top_k, c.ratio = IH, ID, self.top_k, self.ratio
        return c

    def w(self):
        w = super().w()
        w.idx_q, w.idx_k, w.idx_q_norm, w.idx_k_norm = O.F(self.iq), O.F(self.ik), O.F(self.iqn), O.F(self.ikn)
        return w

    def sel_width(self, n_kv):
        return min(self.top_k + self.ratio - 1, n_kv)

    def oracle_qsa(self, x, past, kc, vc, ic, n_kv):
        T = x.shape[0]
        xn = O.rmsnorm(x, self.gamma, EPS)
        nb = n_kv // self.ratio
        out, pre = np.empty((T, H), np.float32), np.empty((T, NH * D), np.float32)
        topk, above, score = np.empty((T, self.sel_width(n_kv)), np.int32), np.empty(T, np.int32), np.empty((T, nb), np.float32)
        cfg, w = self.cfg(), self.w()
        O.lib().shv_ref_attn_layer_qsa(O.C.byref(cfg), O.C.byref(w), O.F(xn), T, past, O.H(kc), O.H(vc), O.H(ic), n_kv, O.F(out), None,
                                       O.F(pre), O.I(topk), O.I(above), O.F(score), 8)
        return dict(out=out, pre=pre, topk=topk, above=above, score=score)

    def cut_margin(self, score_row, p, N, n_kv):
        """How far the value at the selection's cut lies from the nearest other value among row p's
        visible cells (inf when every visible cell is taken)."""
        R, width = self.ratio, self.sel_width(n_kv)
        if p + 1 <= width:
            return np.inf
        n_bid, nb = N // R, n_kv // R
        dead = n_bid if n_bid < nb else nb - 1
        tail = (p + 1) // R * R
        v = np.empty(p + 1, np.float32)
        for j in range(p + 1):
            if j < n_bid * R:
                b = j // R
                v[j] = np.float32(score_row[b]) + np.float32(1e9 if b * R >= tail else 0)
            else:
                v[j] = np.float32(score_row[dead]) + np.float32(1e9)
        order = np.sort(v.astype(np.float64))[::-1]
        nth = order[width - 1]
        other = order[order != nth]
        return float(np.abs(other - nth).min()) if len(other) else np.inf


class QsaDevice:
    """The device side of one layer: caches, the indexer's tables and scratch for up to max_rows rows."""

    def __init__(self, case, max_cells, max_rows, n_splits=16):
        c = case.ctx
        self.case, self.max_cells, self.n_splits = case, max_cells, n_splits
        case.upload(max_cells)
        self.d_gamma = c.upload(case.gamma)
        self.d_w = c.upload(np.concatenate([case.iq, case.ik], axis=0))
        self.d_iqn, self.d_ikn = c.upload(case.iqn), c.upload(case.ikn)
        nb = max_cells // case.ratio
        self.rows_w = IH * ID + ID
        self.d_kc, self.d_vc = c.alloc(max_cells * NKV * D * 2).zero(), c.alloc(max_cells * NKV * D * 2).zero()
        self.d_ic = c.alloc(max_cells * ID * 2).zero()
        self.d_pooled = c.alloc((nb + 1) * ID * 4).zero()
        self.d_work, self.d_score = c.alloc(max_rows * self.rows_w * 4), c.alloc(max_rows * (nb + 1) * 4)
        self.stride = max_cells // 32
        self.d_mask = c.alloc(max_rows * self.stride * 4)
        self.d_qkv, self.d_ctx, self.d_out = c.alloc(max_rows * case.width * 4), c.alloc(max_rows * NH * D * 4), c.alloc(max_rows * H * 4)
        # slice records: short passes take up to n_splits slices a row pair, long ones two or four (the launcher's own rule)
        self.d_part = c.alloc((_part_floats(1, n_splits, min(max_rows, 64)) + _part_floats(1, 4, max_rows)) * 4)
        self.d_pos = c.alloc(4)

    def run(self, x, past, masked=True):
        case, c = self.case, self.case.ctx
        T = x.shape[0]
        self.d_pos.write(np.array([past], np.int32))
        d_x = c.upload(x)
        qa = A.QsaIndexArgs(d_x.ptr, self.d_gamma.ptr, self.d_w.ptr, self.d_iqn.ptr, self.d_ikn.ptr, case.d_rope.ptr, self.d_ic.ptr,
                            self.d_pooled.ptr, self.d_pos.ptr, None, self.d_work.ptr, self.d_score.ptr, self.d_mask.ptr, 1, T, H, IH, ID,
                            case.top_k, case.ratio, ROPE, self.max_cells, self.stride, EPS)
        aa = A.AttnDecodeArgs(self.d_qkv.ptr, case.d_qn.ptr, case.d_kn.ptr, case.d_rope.ptr, self.d_kc.ptr, self.d_vc.ptr, self.d_part.ptr,
                              self.d_ctx.ptr, self.d_pos.ptr, None, 1, T, NH, NKV, D, ROPE, self.max_cells, case.width, self.n_splits, EPS,
                              self.d_mask.ptr if masked else None, self.stride)
        ops = [A.make_op(A.OP_QSA_INDEX, qa),
               A.make_op(A.OP_GEMV_Q4K, A.gemv_args(case.d_fused, d_x, self.d_qkv, case.width, H, T, prologue=A.PRO_RMSNORM, gamma=self.d_gamma)),
               A.make_op(A.OP_ATTN_DECODE, aa),
               A.make_op(A.OP_GEMV_Q4K, A.gemv_args(case.d_o, self.d_ctx, self.d_out, H, NH * D, T, prologue=A.PRO_MUL_SIGMOID, z=self.d_qkv,
                                                    head_dim=D, z_stride=case.width))]
        c.dispatch_multi(ops)
        mask = self.d_mask.read(np.uint32, T * self.stride).reshape(T, self.stride)
        bits = np.unpackbits(mask.view(np.uint8), axis=1, bitorder="little")
        return dict(bits=bits, pre=self.d_ctx.read(np.float32, T * NH * D).reshape(T, NH * D),
                    out=self.d_out.read(np.float32, T * H).reshape(T, H))


def _compare(case, got, want, past, n_kv):
    """rows whose selection is the oracle's; a row may differ only where the value at the cut is a near-tie"""
    T = got["out"].shape[0]
    N = past + T
    same = []
    for i in range(T):
        p = past + i
        mine = set(np.flatnonzero(got["bits"][i]).tolist())
        theirs = set(int(c) for c in want["topk"][i] if c <= p)
        assert max(mine, default=0) <= p, "a cell past the row's own position is selected"
        if mine == theirs:
            same.append(i)
        else:
            m = case.cut_margin(want["score"][i], p, N, n_kv)
            assert m < 2e-4, (p, m, sorted(mine ^ theirs))
    return same


def test_prompt_in_passes_of_every_kind_matches_oracle(ctx):
    """236 rows over an empty cache as passes of 200 (eight row pairs a block, tiles through LDS),
    5 (row pairs, cells written first), 2 and 1 (the decode step's kernels, which append their own
    cells), 27 and 1: every pass's selection is the CPU's and so is what attention makes of it;
    late rows see 35 of their 200-odd cells."""
    case = QsaCase(ctx, seed=21, top_k=32, ratio=4)
    n_kv = 512
    dev = QsaDevice(case, n_kv, 200)
    rng = np.random.default_rng(22)
    kc, vc, ic = np.zeros((n_kv, NKV, D), np.uint16), np.zeros((n_kv, NKV, D), np.uint16), np.zeros((n_kv, ID), np.uint16)
    past, differ = 0, 0
    for T in (200, 5, 2, 1, 27, 1):
        x = rng.standard_normal((T, H)).astype(np.float32)
        want = case.oracle_qsa(x, past, kc, vc, ic, n_kv)
        got = dev.run(x, past)
        same = _compare(case, got, want, past, n_kv)
        differ += T - len(same)
        assert O.rel_l2(got["pre"][same], want["pre"][same]) <= TOL, (T, past)
        assert O.rel_l2(got["out"][same], want["out"][same]) <= TOL, (T, past)
        if past + T > 60:
            last = set(np.flatnonzero(got["bits"][T - 1]).tolist())
            assert len(last) == case.sel_width(n_kv) < past + T
        past += T
    print("qsa: %d of %d rows select differently (near-ties at the cut)" % (differ, past))
    assert differ <= past // 50
    # the indexer's own cache is the CPU's, half for half up to rounding of the projection
    got_ic = dev.d_ic.read(np.uint16, n_kv * ID).reshape(n_kv, ID)[:past].view(np.float16).astype(np.float32)
    assert O.rel_l2(got_ic, ic[:past].view(np.float16).astype(np.float32)) <= 1e-3


def test_selection_that_covers_everything_is_the_dense_layer(ctx):
    """While a row sees no more cells than the selection holds, the mask is every visible cell and
    the masked kernels give the unmasked kernels' numbers bit for bit."""
    case = QsaCase(ctx, seed=23, top_k=64, ratio=4)
    n_kv = 128
    rng = np.random.default_rng(24)
    x = rng.standard_normal((40, H)).astype(np.float32)
    outs = []
    for masked in (True, False):
        dev = QsaDevice(case, n_kv, 40)
        a = dev.run(x[:38], 0, masked)
        b = dev.run(x[38:39], 38, masked)
        outs.append((a, b))
    for i in range(38):
        assert set(np.flatnonzero(outs[0][0]["bits"][i]).tolist()) == set(range(i + 1))
    assert np.array_equal(outs[0][0]["out"], outs[1][0]["out"]) and np.array_equal(outs[0][1]["out"], outs[1][1]["out"])


def test_decode_over_a_long_cache_reads_what_the_indexer_names(ctx):
    """One row at position 3000 of a cache filled by the indexer itself: 67 cells of 3001 are read,
    the CPU's 67, and the output is the CPU's; most tiles of the cache hold no selected cell and are
    never loaded (the slices that skip them leave empty records for the merge)."""
    case = QsaCase(ctx, seed=25, top_k=64, ratio=4)
    n_kv, past = 4096, 3000
    rng = np.random.default_rng(26)
    dev = QsaDevice(case, n_kv, 3000, n_splits=128)
    # K and V of the earlier cells: random halves straight into both caches; the indexer's keys and
    # pooled blocks through the indexer itself (a pass of 3000 rows), whose attention is not looked at
    kc = (rng.standard_normal((n_kv, NKV, D))).astype(np.float16).view(np.uint16)
    vc = (rng.standard_normal((n_kv, NKV, D))).astype(np.float16).view(np.uint16)
    x_old = rng.standard_normal((past, H)).astype(np.float32)
    ic = np.zeros((n_kv, ID), np.uint16)
    xn_old = O.rmsnorm(x_old, case.gamma, EPS)
    raw = np.empty((past, ID), np.float32)
    for i in range(past):
        O.lib().shv_ref_matvec(O.F(raw[i]), O.F(case.ik), O.F(xn_old[i]), ID, H)
    ic[:past] = raw.astype(np.float16).view(np.uint16)
    dev.run(x_old, 0)
    dev.d_kc.write(kc)
    dev.d_vc.write(v_dev(vc))
    # the device's own keys differ from the CPU's in the last bit now and then: the CPU gets the device's cache
    ic_dev = dev.d_ic.read(np.uint16, n_kv * ID).reshape(n_kv, ID)
    assert O.rel_l2(ic_dev[:past].view(np.float16).astype(np.float32), ic[:past].view(np.float16).astype(np.float32)) <= 1e-3
    ic[:past] = ic_dev[:past]
    x = rng.standard_normal((1, H)).astype(np.float32)
    want = case.oracle_qsa(x, past, kc.copy(), vc.copy(), ic, n_kv)
    got = dev.run(x, past)
    same = _compare(case, got, want, past, n_kv)
    assert same == [0], "the row's selection sits on a near-tie; pick another seed"
    assert int(got["bits"][0].sum()) == 67
    assert O.rel_l2(got["pre"], want["pre"]) <= TOL and O.rel_l2(got["out"], want["out"]) <= TOL
    # and it matters: the dense layer over the same cache gives other numbers
    dense = dev.run(x, past, masked=False)
    assert O.rel_l2(dense["pre"], want["pre"]) > 1e-2


# ---- through the op surface: AttnGPU with Ratio > 0 inside the token loop ------------------------

LA = shv.pkg.llm_api


def test_token_loop_with_an_indexer_matches_the_cpu_loop(tmp_path):
    """A four-layer model (three DeltaNet layers and one full-attention layer with an indexer of
    four heads, top 16, ratio 4): a prompt of 70 in passes of 64 and 6, then greedy steps through
    the recorded one-row pass, against the CPU loop over the same tensors.  Past 19 cells the
    attention layer reads a selection; the logits stay the CPU's and the ids equal.  The same
    model staged without the indexer's cut (top_k as large as the cache) gives other logits: the
    selection is really applied."""
    kw = dict(n_layer=4, n_expert=16, n_expert_used=4, vocab=4096, nkv=256, max_tokens=64, idx_heads=4, idx_dim=128, idx_top_k=16, idx_ratio=4)
    cfg = LA.Config(**kw)
    m = LA.LLM(cfg)
    try:
        m.init_synthetic(99)
        m.stage()
        names = [t[0] for t in m.tensors()]
        assert "blk.3.indexer.q_proj.weight" in names and "blk.3.indexer.k_norm.weight" in names and "blk.0.indexer.q_proj.weight" not in names
        tensors = {t[0]: m.download(t[0]) for t in m.tensors()}
        om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
        rng = np.random.default_rng(5)
        prompt = rng.integers(0, cfg.vocab, size=70).astype(np.int32)
        lg_gpu, hd_gpu = m.extend(prompt, want_hidden=True)
        lg_cpu, hd_cpu = om.extend(prompt)
        assert O.rel_l2(hd_gpu, hd_cpu) <= 1e-3 and O.rel_l2(lg_gpu, lg_cpu) <= 1e-3
        lg = lg_cpu
        for i in range(6):
            tok = int(O.lib().shv_ref_argmax(O.F(lg), cfg.vocab))
            assert int(np.argmax(lg_gpu)) == tok
            lg, _ = om.extend(np.array([tok], np.int32))
            lg_gpu, _ = m.extend(np.array([tok], np.int32))
            assert O.rel_l2(lg_gpu, lg) <= 1e-3, i
        # the device loop (arg-max in the launch, positions on the device) walks the same ids
        m.reset()
        m.extend(prompt)
        ids_gpu, _ = m.generate(6)
        om2 = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
        lg, _ = om2.extend(prompt)
        want = []
        for i in range(6):
            want.append(int(O.lib().shv_ref_argmax(O.F(lg), cfg.vocab)))
            lg, _ = om2.extend(np.array([want[-1]], np.int32))
        assert list(ids_gpu) == want
        # the checkpoint carries the indexer: its shape in the metadata (llm/model.go:385-405), its
        # projections under their own names, and what is read back decodes bit for bit
        path = tmp_path / "qsa.gguf"
        m.save_gguf(path)
        m.reset()
        lg_a, _ = m.extend(prompt)
    finally:
        m.close()
    back = LA.LLM(LA.Config(nkv=256, max_tokens=64), gguf=path)
    try:
        assert (back.cfg.idx_heads, back.cfg.idx_dim, back.cfg.idx_top_k, back.cfg.idx_ratio) == (4, 128, 16, 4)
        back.stage()
        lg_b, _ = back.extend(prompt)
        assert np.array_equal(lg_a, lg_b)
    finally:
        back.close()
    # without the cut
    wide = LA.LLM(LA.Config(**dict(kw, idx_top_k=256)))
    try:
        wide.init_synthetic(99)
        wide.stage()
        lg_wide, _ = wide.extend(prompt)
        assert O.rel_l2(lg_wide, lg_cpu) > 1e-3
    finally:
        wide.close()
