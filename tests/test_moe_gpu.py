"""MoE FFN step on the GPU against the oracle's MoEBlock (llm/moe.go:215-409)."""
import numpy as np
import pytest

import oracle_lib as O
import shv
from test_dequant_gpu import random_tensor

pytestmark = pytest.mark.gpu
A = shv.api
TOL = 1e-3
EPS = 1e-6


class MoeCase:
    """Seeded synthetic block: router f32 ~N(0,0.02), experts ~N(0,0.02) -> Q4_K by the
    reference quantiser, gamma ~ 1+N(0,0.1), tokens ~N(0,1)."""

    BANKS = ("gate_exps", "up_exps", "down_exps", "gate_sh", "up_sh", "down_sh")
    types = (0,) * 6    # every bank Q4_K unless a case says otherwise

    def __init__(self, ctx, seed, H=2048, E=32, used=4, ffn=512, T=1, tie_router=False, types=None):
        """types: {bank: tensor type name} for banks held in another type than Q4_K (random blocks
        of that type with small scales)."""
        rng = np.random.default_rng(seed)
        self.ctx, self.H, self.E, self.used, self.ffn, self.T = ctx, H, E, used, ffn, T
        self.router = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
        if tie_router:
            self.router[:] = self.router[0]
        self.shared_gate = (rng.standard_normal(H) * 0.02).astype(np.float32)
        q = lambda rows, k: O.quantize_q4k((rng.standard_normal((rows, k)) * 0.02).astype(np.float32))
        self.gate_exps, self.up_exps = q(E * ffn, H), q(E * ffn, H)
        self.down_exps = q(E * H, ffn)
        self.gate_sh, self.up_sh, self.down_sh = q(ffn, H), q(ffn, H), q(H, ffn)
        self.types = [0] * 6
        for i, bank in enumerate(self.BANKS):
            if types and bank in types:
                name = types[bank]
                self.types[i] = O.GGML_TYPES[name]
                n = getattr(self, bank).size // O.q4k_row_bytes(256) * 256
                if name in ("F16", "BF16"):
                    v = (rng.standard_normal(n) * 0.02).astype(np.float32)
                    raw = v.astype(np.float16).view(np.uint8) if name == "F16" else (v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
                else:
                    raw = random_tensor(name, n, seed=seed + i, scale={"Q8_0": 3e-4, "IQ4_NL": 3e-4}.get(name, 1e-4 if name.endswith("_K") else 2e-3))
                setattr(self, bank, np.ascontiguousarray(raw))
        self.gamma = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
        self.h = rng.standard_normal((T, H)).astype(np.float32)
        self.res = rng.standard_normal((T, H)).astype(np.float32)

    def oracle(self):
        xn = O.rmsnorm(self.h, self.gamma, EPS)
        cfg = O.MoeCfg(self.H, self.E, self.used, self.ffn, self.ffn)
        w = O.MoeW(O.F(self.router), O.F(self.shared_gate), O.B(self.gate_exps), O.B(self.up_exps),
                   O.B(self.down_exps), O.B(self.gate_sh), O.B(self.up_sh), O.B(self.down_sh), (O.C.c_int * 6)(*self.types))
        T = self.T
        r = dict(out=np.empty((T, self.H), np.float32), logits=np.empty((T, self.E), np.float32),
                 topk=np.empty((T, self.used), np.int32), weights=np.empty((T, self.used), np.float32),
                 swiglu=np.empty((T, self.used, self.ffn), np.float32),
                 moe_out=np.empty((T, self.H), np.float32), sig=np.empty(T, np.float32))
        O.lib().shv_ref_moe_block(O.C.byref(cfg), O.C.byref(w), O.F(xn), T, O.F(r["out"]),
                                  O.F(r["logits"]), O.I(r["topk"]), O.F(r["weights"]),
                                  O.F(r["swiglu"]), O.F(r["moe_out"]), O.F(r["sig"]), 8)
        r["xn"] = xn
        return r

    def gpu(self, residual=False, defer=False, grouped=False, packed=False, group_ready=None):
        """grouped: hand the expert kernels the workspaces that let a pass of many rows go grouped by
        expert on the matrix cores.  packed: act goes from the gate/up kernel to the down kernel
        as matrix-core operands instead of floats."""
        c, T, H, E, used, ffn = self.ctx, self.T, self.H, self.E, self.used, self.ffn
        d = {k: c.upload(getattr(self, k)) for k in
             ("router", "shared_gate", "gate_exps", "up_exps", "down_exps", "gate_sh", "up_sh",
              "down_sh", "gamma", "h", "res")}
        xn, logits = c.alloc(T * H * 4), c.alloc(T * (E + 1) * 4)
        topk, weights = c.alloc(T * used * 4), c.alloc(T * (used + 1) * 4)
        act, out = c.alloc(T * (used + 1) * ffn * 4), c.alloc(T * H * 4)
        ra = A.MoeRouterArgs(d["h"].ptr, d["gamma"].ptr, d["router"].ptr, d["shared_gate"].ptr, xn.ptr,
                             logits.ptr, topk.ptr, weights.ptr, T, H, E, used, EPS, H, 1 if defer else 0)
        ua = A.MoeUpArgs(xn.ptr, topk.ptr, d["gate_exps"].ptr, d["up_exps"].ptr, d["gate_sh"].ptr,
                         d["up_sh"].ptr, act.ptr, T, H, used, ffn, logits.ptr if defer else None,
                         weights.ptr if defer else None, E, self.types[0], self.types[1], self.types[3], self.types[4],
                         None)
        da = A.MoeDownArgs(act.ptr, topk.ptr, weights.ptr, d["down_exps"].ptr, d["down_sh"].ptr,
                           d["res"].ptr if residual else None, out.ptr, T, H, used, ffn, H, H, self.types[2], self.types[5],
                           E, None, None)
        if grouped:
            # "down": only the down projection gets the workspaces (lists poisoned, so that walking
            # them instead of making them would show)
            group, pairs = c.upload(np.full(2 * E + 1 + T * used, 1 << 20, np.int32)), c.alloc(T * (used + 1) * H * 4)
            da.group = group.ptr
            if grouped != "down":
                ua.group = group.ptr
            da.pairs = pairs.ptr
        if packed:
            ua.act_packed = da.act_packed = 1
        if packed or group_ready is not None:
            da.group_ready = 1 if group_ready is None else group_ready
        ops = [A.make_op(A.OP_MOE_ROUTER, ra), A.make_op(A.OP_MOE_UP, ua), A.make_op(A.OP_MOE_DOWN, da)]
        c.dispatch_multi(ops)
        return dict(group=group.read(np.int32, 2 * E + 1 + T * used) if grouped else None,
                    xn=xn.read(np.float32, T * H).reshape(T, H),
                    logits=logits.read(np.float32, T * (E + 1)).reshape(T, E + 1),
                    topk=topk.read(np.int32, T * used).reshape(T, used),
                    weights=weights.read(np.float32, T * (used + 1)).reshape(T, used + 1),
                    act=act.read(np.float32, T * (used + 1) * ffn).reshape(T, used + 1, ffn),
                    out=out.read(np.float32, T * H).reshape(T, H), ops=ops)


def _margin(probs_row, used):
    s = np.sort(probs_row.astype(np.float64))[::-1][:used + 1]
    return float(np.min((s[:-1] - s[1:]) / s[:-1]))


def _check(case, residual=False, defer=False):
    want, got = case.oracle(), case.gpu(residual, defer)
    assert O.rel_l2(got["xn"], want["xn"]) <= 1e-5
    assert O.rel_l2(got["logits"][:, :case.E], want["logits"]) <= 1e-4
    # top-k ids are demanded bit-exact; the inputs must not sit on a near-tie for that to be a
    # statement about the kernel rather than about rounding (llm/moe_test.go:59-66)
    for t in range(case.T):
        lg = want["logits"][t].astype(np.float64)
        p = np.exp(lg - lg.max())
        assert _margin(p / p.sum(), case.used) > 1e-4, "seed sits on a near-tie; pick another"
    assert np.array_equal(got["topk"], want["topk"])
    assert O.rel_l2(got["weights"][:, :case.used], want["weights"]) <= 1e-5
    assert O.rel_l2(got["weights"][:, case.used], want["sig"]) <= 1e-5
    assert O.rel_l2(got["act"][:, :case.used], want["swiglu"]) <= TOL
    ref = want["out"] + (case.res if residual else 0)
    err = O.rel_l2(got["out"], ref)
    print(f"moe T={case.T} E={case.E} used={case.used}: out rel-L2 {err:.3e}")
    assert err <= TOL
    return got


@pytest.mark.parametrize("defer", [False, True])
@pytest.mark.parametrize("T", [1, 4, 9, 16])
def test_moe_block_matches_oracle(ctx, T, defer):
    """defer: the selection is made by the expert kernel from the router's logits instead of by
    the router's last block; both must give the reference's selection."""
    _check(MoeCase(ctx, seed=100 + T, E=64, used=10, T=T), defer=defer)


@pytest.mark.parametrize("types", [
    dict(gate_exps="Q8_0", up_exps="Q8_0", down_exps="Q8_0", gate_sh="Q8_0", up_sh="Q8_0", down_sh="Q8_0"),
    dict(down_exps="Q5_K", down_sh="Q6_K"),
    dict(gate_exps="Q5_K", up_exps="Q6_K", gate_sh="Q5_1", up_sh="Q4_1"),
    dict(gate_exps="IQ4_NL", down_exps="IQ4_NL", up_sh="Q5_0", down_sh="Q5_1"),
    dict(up_exps="F16", down_exps="BF16", gate_sh="Q4_K"),        # routed slots on the other arms, the shared expert on the Q4_K kernels
    dict(gate_sh="Q8_0", up_sh="Q8_0", down_sh="Q8_0"),           # and the other way round: what a converter's 8-bit shared expert gives
], ids=lambda d: "+".join(sorted(set(d.values()))) + "-" + str(len(d)))
@pytest.mark.parametrize("T", [1, 5, 17])
def test_moe_block_over_banks_in_other_types(ctx, types, T):
    """Banks read as the checkpoint holds them (llm/gpu_moe.go:673-688, llm_moe_gemv.comp's arms beside
    Q4_K), routed and shared ones of different types in one block, against the CPU block walking
    the same banks through Dequantize (llm/moe.go:289-409)."""
    _check(MoeCase(ctx, seed=300 + T, E=32, used=6, T=T, types=types), residual=True)
    with pytest.raises(A.ShvError, match="take the selection from the router"):
        MoeCase(ctx, seed=1, E=16, used=2, T=1, types=dict(gate_exps="Q8_0")).gpu(defer=True)
    bad = MoeCase(ctx, seed=1, E=16, used=2, T=1)
    bad.types[2] = 10
    with pytest.raises(A.ShvError, match="moe_down: rows of 512 elements of ggml type 10"):
        bad.gpu()


@pytest.mark.parametrize("T,E,used", [(160, 64, 10), (300, 64, 10), (130, 128, 8), (517, 128, 8), (1030, 512, 2)])
def test_lists_by_expert_hold_every_pair_once(ctx, T, E, used):
    """The workspace the grouped kernels walk (llm/moe.go:289-409 batches a chunk's tokens per expert): starts that
    add up, under every expert exactly the (token, slot) pairs that chose it, in any order, and the experts' launch
    order by list length, longer first, equal lengths by index.  Passes below 2048 pairs over fewer than 128 experts
    are listed by one block, the others by sixteen in two launches: both roads are here."""
    case = MoeCase(ctx, seed=T, E=E, used=used, T=T)
    got = case.gpu(residual=True, grouped=True)
    g, topk = got["group"], got["topk"]
    starts, lists, order = g[:E + 1], g[E + 1:E + 1 + T * used], g[E + 1 + T * used:]
    counts = np.bincount(topk.ravel(), minlength=E)
    assert starts[0] == 0 and np.array_equal(np.diff(starts), counts)
    for e in range(E):
        want = sorted(t * (used + 1) + s for t, s in zip(*np.nonzero(topk == e)))
        assert sorted(lists[starts[e]:starts[e + 1]]) == want, e
    assert list(order) == sorted(range(E), key=lambda e: (-counts[e], e))


@pytest.mark.parametrize("T,E,used,seed", [(160, 64, 10, 165), (131, 16, 4, 137), (128, 64, 1, 264)])
def test_many_rows_grouped_by_expert_match_oracle(ctx, T, E, used, seed):
    """Passes of 128 rows and more, given workspaces, run the experts grouped on the matrix cores:
    whole and ragged token tiles, experts wanted by several tiles of 16 tokens and by none, with
    the residual (seeds chosen clear of near-ties in the routing).  The grouped products also
    agree with the per-(token, slot) kernels' to rounding."""
    case = MoeCase(ctx, seed=seed, E=E, used=used, T=T)
    want = case.oracle()
    for t in range(T):
        p = np.exp(want["logits"][t].astype(np.float64) - want["logits"][t].max())
        if _margin(p / p.sum(), used) <= 1e-4:
            pytest.skip("seed sits on a near-tie; pick another")
    got = case.gpu(residual=True, grouped=True)
    ref = case.gpu(residual=True)
    assert np.array_equal(got["topk"], want["topk"]) and np.array_equal(ref["topk"], want["topk"])
    assert O.rel_l2(got["act"][:, :used], want["swiglu"]) <= TOL
    assert O.rel_l2(got["out"], want["out"] + case.res) <= TOL
    assert O.rel_l2(got["act"], ref["act"]) <= 1e-5
    assert O.rel_l2(got["out"], ref["out"]) <= 1e-5
    assert not np.array_equal(got["out"], ref["out"]), "the workspaces were given: the grouped kernels should have run"
    # act handed over as operands: the same products, the down projection's rows staged by its loads
    pk = case.gpu(residual=True, grouped=True, packed=True)
    assert np.array_equal(pk["topk"], want["topk"])
    assert O.rel_l2(pk["out"], want["out"] + case.res) <= TOL
    assert O.rel_l2(pk["out"], got["out"]) <= 1e-5
    assert not np.array_equal(pk["act"], got["act"]), "act should hold operands, not floats"
    with pytest.raises(A.ShvError, match="did not leave act as operands"):
        case.gpu(residual=True, grouped=True, packed=True, group_ready=0)


@pytest.mark.parametrize("types", [dict(down_exps="Q8_0", down_sh="Q8_0"), dict(down_sh="Q6_K"), dict(gate_sh="Q8_0")],
                         ids=["down-q8_0", "shared-down-q6_k", "shared-gate-q8_0"])
def test_flags_that_do_not_fit_the_road_taken_are_refused(ctx, types):
    """A 128-row pass whose gate/up banks are Q4_K and whose down banks are not (or the other way
    round): one projection would go grouped and the other not.  group_ready / act_packed that claim
    a hand-over which did not happen are refused instead of believed, and with honest flags the
    block is the CPU's."""
    case = MoeCase(ctx, seed=411, E=32, used=4, T=128, types=types)
    want = case.oracle()
    if "gate_sh" in types:
        # gate/up did not go grouped and left floats; the grouped down launch would read them as operands
        with pytest.raises(A.ShvError, match="did not leave act as operands"):
            case.gpu(residual=True, grouped=True, packed=True)
    else:
        # gate/up went grouped and packed act; the down launch goes another road, which reads floats
        with pytest.raises(A.ShvError, match="left act as matrix-core operands"):
            case.gpu(residual=True, grouped=True, packed=True)
    got = case.gpu(residual=True, grouped=True)
    ok = [t for t in range(case.T) if np.array_equal(got["topk"][t], want["topk"][t])]
    assert len(ok) >= case.T - 2
    assert O.rel_l2(got["out"][ok], (want["out"] + case.res)[ok]) <= TOL


def test_lists_claimed_ready_but_never_made_are_rebuilt(ctx):
    """group_ready on a down projection whose gate/up launch did not go grouped (it was handed no
    workspace): the lists in `group` are nobody's, and the down projection makes its own instead
    of walking them."""
    case = MoeCase(ctx, seed=421, E=16, used=4, T=128)
    want = case.oracle()
    got = case.gpu(residual=True, grouped="down", group_ready=1)
    ok = [t for t in range(case.T) if np.array_equal(got["topk"][t], want["topk"][t])]
    assert len(ok) >= case.T - 2
    assert O.rel_l2(got["out"][ok], (want["out"] + case.res)[ok]) <= TOL


def test_moe_block_with_residual_and_few_experts(ctx):
    _check(MoeCase(ctx, seed=7, E=16, used=4, T=2), residual=True)


def test_route_ties_go_to_the_lower_index(ctx):
    """Equal logits must select experts 0..used-1 in order (sort.SliceStable, llm/moe.go:249-252)
    with equal weights 1/used."""
    case = MoeCase(ctx, seed=9, E=64, used=10, T=3, tie_router=True)
    for defer in (False, True):
        got = case.gpu(defer=defer)
        assert np.array_equal(got["topk"], np.tile(np.arange(10, dtype=np.int32), (3, 1)))
        assert np.allclose(got["weights"][:, :10], 0.1, rtol=1e-6)
    want = case.oracle()
    assert np.array_equal(want["topk"], got["topk"])


def test_weights_sum_to_one_and_slots_descend(ctx):
    case = MoeCase(ctx, seed=11, E=64, used=10, T=16)
    got = case.gpu()
    assert np.allclose(got["weights"][:, :10].sum(axis=1), 1.0, atol=1e-5)
    assert (np.diff(got["weights"][:, :10], axis=1) <= 0).all()
    for t in range(16):
        assert len(set(got["topk"][t])) == 10


def test_moe_refuses_unsupported_shapes(ctx):
    d = ctx.alloc(1 << 16)
    with pytest.raises(shv.pkg.ShvError):
        ctx.enqueue(A.OP_MOE_ROUTER, A.MoeRouterArgs(d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr,
                                                     d.ptr, 1, 2048, 1024, 10, EPS, 2048, 0))
    with pytest.raises(shv.pkg.ShvError):
        ctx.enqueue(A.OP_MOE_DOWN, A.MoeDownArgs(d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, None, d.ptr, 1,
                                                 2048, 10, 640, 2048, 2048))


@pytest.fixture(scope="module")
def full_bank(ctx):
    """BASELINE shape: 512 experts, top-10, ffn 512, H 2048.  The 906 MB bank is drawn and quantised
    on the device (the device quantiser is bit-exact with the reference's) and downloaded once, so
    that the oracle runs on the same bytes."""
    H, E, used, ffn = 2048, 512, 10, 512
    c = ctx
    rng = np.random.default_rng(77)

    def bank(rows, k, seed):
        f = c.alloc(rows * k * 4)
        c.enqueue(A.OP_FILL_NORMAL, A.FillNormalArgs(f.ptr, rows * k, seed, 0.0, 0.02))
        q = c.alloc(rows * (k // 256 * 144))
        c.enqueue(A.OP_QUANTIZE_Q4K, A.QuantizeQ4KArgs(f.ptr, q.ptr, rows, k))
        c.sync()
        f.free()
        return q

    case = MoeCase.__new__(MoeCase)
    case.ctx, case.H, case.E, case.used, case.ffn = c, H, E, used, ffn
    case.types = [0] * 6
    dev = dict(gate_exps=bank(E * ffn, H, 1), up_exps=bank(E * ffn, H, 2), down_exps=bank(E * H, ffn, 3))
    for k, b in dev.items():
        setattr(case, k, b.read(np.uint8, b.nbytes))
    for b in dev.values():
        b.free()
    case.router = (rng.standard_normal((E, H)) * 0.02).astype(np.float32)
    case.shared_gate = (rng.standard_normal(H) * 0.02).astype(np.float32)
    q = lambda rows, k: O.quantize_q4k((rng.standard_normal((rows, k)) * 0.02).astype(np.float32))
    case.gate_sh, case.up_sh, case.down_sh = q(ffn, H), q(ffn, H), q(H, ffn)
    case.gamma = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    return case


def _full_case(full_bank, T, seed):
    """The bank with T token rows of its own; a seed whose rows sit on a near-tie is stepped past."""
    import copy
    case = copy.copy(full_bank)
    case.T = T
    for s in range(seed, seed + 50):
        rng = np.random.default_rng(s)
        case.h = rng.standard_normal((T, case.H)).astype(np.float32)
        case.res = rng.standard_normal((T, case.H)).astype(np.float32)
        xn = case.h * (1.0 / np.sqrt((case.h.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + EPS)) * case.gamma
        lg = xn.astype(np.float64) @ case.router.astype(np.float64).T
        p = np.exp(lg - lg.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        if all(_margin(p[t], case.used) > 2e-4 for t in range(T)):
            return case
    raise AssertionError("no seed clear of near-ties")


@pytest.mark.parametrize("defer", [False, True])
@pytest.mark.parametrize("T", [1, 4, 16])
def test_moe_full_config_bank(ctx, full_bank, T, defer):
    """BASELINE config 2 at its three batch sizes over the full 512-expert bank, with the selection
    made by the routing launch (the block-wide routing kernel that every pass of several rows at
    this shape takes) and by the expert kernel from the logits."""
    _check(_full_case(full_bank, T, 1000 + T), residual=True, defer=defer)


@pytest.mark.parametrize("T", [128, 256, 333])
def test_long_pass_over_the_full_bank_matches_oracle(ctx, full_bank, T):
    """What a prompt chunk of BASELINE's model runs, held to the CPU block directly: from 128 rows
    the router's logits come from the matrix cores (float32 rows as two binary16 parts), the
    experts are grouped over all 512 lists, act goes to the down projection as operands and the
    pairs are folded in slot order.  Whole and ragged token tiles.  A row's selection may differ
    from the CPU's only where the CPU's own 10th and 11th probabilities are a near-tie
    (llm/moe_test.go:59-66); such rows are counted and left out of the sums."""
    import copy
    case = copy.copy(full_bank)
    case.T = T
    rng = np.random.default_rng(3000 + T)
    case.h = rng.standard_normal((T, case.H)).astype(np.float32)
    case.res = rng.standard_normal((T, case.H)).astype(np.float32)
    want = case.oracle()
    got = case.gpu(residual=True, grouped=True, packed=True)
    # the logits of the wide router against the CPU's sequential float32 matvec
    assert O.rel_l2(got["logits"][:, :case.E], want["logits"]) <= 1e-5
    assert O.rel_l2(got["xn"], want["xn"]) <= 1e-5
    clear, same = [], []
    for t in range(T):
        lg = want["logits"][t].astype(np.float64)
        p = np.exp(lg - lg.max())
        clear.append(_margin(p / p.sum(), case.used) > 1e-4)
        same.append(np.array_equal(got["topk"][t], want["topk"][t]))
    clear, same = np.array(clear), np.array(same)
    assert same[clear].all(), "a selection differs on a row that is clear of near-ties"
    print(f"long MoE pass T={T}: {int((~clear).sum())} near-tie rows, {int((~same).sum())} selections differ")
    assert (~same).sum() <= max(2, T // 50)
    assert O.rel_l2(got["weights"][same][:, :case.used], want["weights"][same]) <= 1e-5
    assert O.rel_l2(got["out"][same], (want["out"] + case.res)[same]) <= TOL
    # act holds operands on this road; the floats are checked on the same road without the hand-over
    flt = case.gpu(residual=True, grouped=True)
    assert np.array_equal(flt["topk"], got["topk"])
    assert O.rel_l2(flt["act"][same][:, :case.used], want["swiglu"][same]) <= TOL
    assert O.rel_l2(flt["out"], got["out"]) <= 1e-5


@pytest.mark.parametrize("T,E", [(200, 512), (2048, 130), (4100, 130), (4099, 512)])
def test_router_of_a_long_pass_alone(ctx, T, E):
    """shv_moe_router over passes long enough for the matrix cores (llm/moe.go:219-243: xn = rmsnorm(h) * gamma, logits
    = W xn in float32): xn and every logit against a float64 product of the same rows, with four waves a block below
    4096 rows and eight from there on, row counts that leave a ragged last group of 64 and router rows (E + the shared
    gate's) that leave a ragged last block."""
    rng = np.random.default_rng(T + E)
    H, used = 2048, 4
    h = rng.standard_normal((T, H)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    W = (rng.standard_normal((E, H)) * 0.05).astype(np.float32)
    sg = (rng.standard_normal(H) * 0.05).astype(np.float32)
    c = ctx
    d = {k: c.upload(v) for k, v in dict(h=h, gamma=gamma, W=W, sg=sg).items()}
    xn, logits = c.alloc(T * H * 4), c.alloc(T * (E + 1) * 4)
    topk, weights = c.alloc(T * used * 4), c.alloc(T * (used + 1) * 4)
    c.enqueue(A.OP_MOE_ROUTER, A.MoeRouterArgs(d["h"].ptr, d["gamma"].ptr, d["W"].ptr, d["sg"].ptr, xn.ptr, logits.ptr, topk.ptr, weights.ptr,
                                               T, H, E, used, EPS, H, 0))
    h64 = h.astype(np.float64)
    want_xn = h64 / np.sqrt((h64 * h64).mean(axis=1, keepdims=True) + EPS) * gamma
    got_xn = xn.read(np.float32, T * H).reshape(T, H)
    assert O.rel_l2(got_xn, want_xn) <= 1e-6
    got = logits.read(np.float32, T * (E + 1)).reshape(T, E + 1)
    want = want_xn @ np.vstack([W, sg]).astype(np.float64).T
    err = max(O.rel_l2(got[t], want[t]) for t in range(0, T, 37))
    assert O.rel_l2(got, want) <= 1e-5 and err <= 1e-5, err
    # the selection from those logits: each row's ids are its largest logits, in descending order
    ids = topk.read(np.int32, T * used).reshape(T, used)
    for t in (0, 63, 64, T // 2, T - 1):
        assert list(ids[t]) == list(np.argsort(-got[t, :E], kind="stable")[:used])


@pytest.mark.parametrize("defer", [False, True])
def test_route_with_many_equal_probabilities_at_512_experts(ctx, full_bank, defer):
    """More than 64 experts share the largest probability: the candidates do not fit the ranking
    table and the selection falls back to rounds of arg-max; ties still go to the lower index
    (sort.SliceStable, llm/moe.go:249-252)."""
    import copy
    case = copy.copy(full_bank)
    case.T = 2
    rng = np.random.default_rng(5)
    case.h = rng.standard_normal((2, case.H)).astype(np.float32)
    case.res = rng.standard_normal((2, case.H)).astype(np.float32)
    case.router = case.router.copy()
    tied = np.arange(37, 37 + 150)
    case.router[tied] = case.router[300]          # 151 equal logits ...
    case.router[[3, 490]] = 4.0 * case.router[300]  # ... and two rows that may or may not lie above them
    want, got = case.oracle(), case.gpu(residual=True, defer=defer)
    assert np.array_equal(got["topk"], want["topk"])
    assert O.rel_l2(got["weights"][:, :case.used], want["weights"]) <= 1e-5
    assert O.rel_l2(got["out"], want["out"] + case.res) <= TOL


def test_expert_kernel_routing_without_a_shared_gate(ctx, full_bank):
    """A router run without a shared gate leaves its logit unwritten; the expert kernel, told so,
    stores 0 for the shared expert's weight, as the routing launch does."""
    case = _full_case(full_bank, 1, 2000)
    c, T, H, E, used, ffn = ctx, 1, case.H, case.E, case.used, case.ffn
    d = {k: c.upload(getattr(case, k)) for k in ("router", "gate_exps", "up_exps", "gate_sh", "up_sh", "gamma", "h")}
    xn, logits = c.alloc(T * H * 4), c.upload(np.full(T * (E + 1), 77.0, np.float32))
    topk, weights = c.alloc(T * used * 4), c.upload(np.full(T * (used + 1), 5.0, np.float32))
    act = c.alloc(T * (used + 1) * ffn * 4)
    out = {}
    for defer in (0, 1):
        ra = A.MoeRouterArgs(d["h"].ptr, d["gamma"].ptr, d["router"].ptr, None, xn.ptr, logits.ptr, topk.ptr, weights.ptr,
                             T, H, E, used, EPS, H, defer)
        ua = A.MoeUpArgs(xn.ptr, topk.ptr, d["gate_exps"].ptr, d["up_exps"].ptr, d["gate_sh"].ptr, d["up_sh"].ptr, act.ptr,
                         T, H, used, ffn, logits.ptr if defer else None, weights.ptr if defer else None, E, 0, 0, 0, 0, None, 1)
        c.dispatch_multi([A.make_op(A.OP_MOE_ROUTER, ra), A.make_op(A.OP_MOE_UP, ua)])
        out[defer] = (topk.read(np.int32, used), weights.read(np.float32, used + 1))
    assert np.array_equal(out[0][0], out[1][0])
    assert out[0][1][used] == 0.0 and out[1][1][used] == 0.0
    assert np.allclose(out[0][1], out[1][1], rtol=1e-6)


# ---- the router's logits formed by the launch of the output projection that feeds the block ----

def _fold_case(ctx, case, seed, prologue):
    """A 2048 x 4096 Q4_K output projection W, its input v (with what the prologue needs) and the
    residual row x in front of the MoE block `case`: h = x + W pro(v) is the block's input."""
    rng = np.random.default_rng(seed)
    H, K = case.H, 4096
    w = O.quantize_q4k((rng.standard_normal((H, K)) * 0.02).astype(np.float32))
    v = rng.standard_normal(K).astype(np.float32)
    x = rng.standard_normal(H).astype(np.float32)
    z = rng.standard_normal(K).astype(np.float32)
    gn = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    if prologue == A.PRO_GATED_NORM:
        vh = v.reshape(-1, 128).astype(np.float64)
        pv = vh / np.sqrt((vh ** 2).mean(axis=1, keepdims=True) + EPS) * gn * (1 / (1 + np.exp(-z.reshape(-1, 128).astype(np.float64))))
        pv = pv.reshape(-1)
    elif prologue == A.PRO_MUL_SIGMOID:
        pv = v.astype(np.float64) / (1 + np.exp(-z.astype(np.float64)))
    else:
        pv = v.astype(np.float64)
    wf = O.dequant_q4k(w, K).astype(np.float64)
    h = (x.astype(np.float64) + wf @ pv).astype(np.float32)
    return dict(w=w, v=v, x=x, z=z, gn=gn, h=h)


@pytest.mark.parametrize("prologue", [A.PRO_NONE, A.PRO_GATED_NORM, A.PRO_MUL_SIGMOID], ids=["plain", "gated-norm", "sigmoid-gate"])
@pytest.mark.parametrize("E,used", [(512, 10), (16, 4)])
def test_router_rows_ride_on_the_output_projection(ctx, full_bank, prologue, E, used):
    """One row: the output projection's launch also forms R diag(gamma) h from the table
    shv_router_fold makes, and the gate/up kernel applies the RMSNorm's factor to those products,
    to the row it stages and to its own products.  Held to the CPU block on h = x + W pro(v)
    (float64), and to the launches it replaces (projection in place, router, gate/up, down)."""
    import copy
    if E == 512:
        case = copy.copy(full_bank)
        case.T = 1
    else:
        case = MoeCase(ctx, seed=77, E=E, used=used, T=1)
    H, K, ffn, c = case.H, 4096, case.ffn, ctx
    for seed in range(500, 540):
        f = _fold_case(ctx, case, seed, prologue)
        case.h = f["h"].reshape(1, H)
        case.res = np.zeros((1, H), np.float32)
        want = case.oracle()
        lg = want["logits"][0].astype(np.float64)
        p = np.exp(lg - lg.max())
        if _margin(p / p.sum(), used) > 2e-4:
            break
    else:
        raise AssertionError("no seed clear of near-ties")
    d = {k: c.upload(getattr(case, k)) for k in ("router", "shared_gate", "gate_exps", "up_exps", "down_exps", "gate_sh", "up_sh", "down_sh", "gamma")}
    dw, dv, dx, dz, dgn = (c.upload(f[k]) for k in ("w", "v", "x", "z", "gn"))
    table, scratch = c.alloc((E + 1) * (K + H) * 4), c.alloc(H * K * 4)
    c.enqueue(A.OP_ROUTER_FOLD, A.RouterFoldArgs(d["router"].ptr, d["shared_gate"].ptr, d["gamma"].ptr, dw.ptr, table.ptr, scratch.ptr, E, H, K))
    # the table against its definition in float64
    tb = table.read(np.float32, (E + 1) * (K + H)).reshape(E + 1, K + H)
    rg = np.vstack([case.router, case.shared_gate[None]]).astype(np.float64) * case.gamma.astype(np.float64)
    wf = O.dequant_q4k(f["w"], K).astype(np.float64)
    assert O.rel_l2(tb[:, K:], rg) <= 1e-7
    assert O.rel_l2(tb[:, :K], rg @ wf) <= 1e-7
    y, raw = c.alloc(H * 4), c.alloc((E + 1) * 4)
    topk, weights, act, out = c.alloc(used * 4), c.alloc((used + 1) * 4), c.alloc((used + 1) * ffn * 4), c.alloc(H * 4)
    g = A.gemv_args(dw, dv, y, H, K, 1, prologue, dgn if prologue == A.PRO_GATED_NORM else None, dz if prologue != A.PRO_NONE else None,
                    dx, EPS, 128 if prologue == A.PRO_GATED_NORM else 0)
    # the shared gate's product either as the table's last row (few experts here) or formed by the
    # gate/up kernel from the row it stages (what the token loop does: 512 rows fill 256 blocks evenly)
    sg_in_up = E == 512
    g.fold, g.fold_out, g.fold_rows = table.ptr, raw.ptr, E if sg_in_up else E + 1
    ua = A.MoeUpArgs(y.ptr, topk.ptr, d["gate_exps"].ptr, d["up_exps"].ptr, d["gate_sh"].ptr, d["up_sh"].ptr, act.ptr, 1, H, used, ffn,
                     raw.ptr, weights.ptr, E, 0, 0, 0, 0, None, 0, 0, d["gamma"].ptr, EPS, d["shared_gate"].ptr if sg_in_up else None)
    da = A.MoeDownArgs(act.ptr, topk.ptr, weights.ptr, d["down_exps"].ptr, d["down_sh"].ptr, y.ptr, out.ptr, 1, H, used, ffn, H, H, 0, 0, E, None, None)
    c.dispatch_multi([A.make_op(A.OP_GEMV_Q4K, g), A.make_op(A.OP_MOE_UP, ua), A.make_op(A.OP_MOE_DOWN, da)])
    got_h = y.read(np.float32, H)
    assert O.rel_l2(got_h, f["h"]) <= 1e-5
    scale = 1.0 / np.sqrt((f["h"].astype(np.float64) ** 2).mean() + EPS)
    got_lg = raw.read(np.float32, E + 1).astype(np.float64) * scale
    assert O.rel_l2(got_lg[:E], want["logits"][0]) <= 2e-5
    assert np.array_equal(topk.read(np.int32, used), want["topk"][0])
    wt = weights.read(np.float32, used + 1)
    assert O.rel_l2(wt[:used], want["weights"][0]) <= 1e-5
    assert abs(wt[used] - want["sig"][0]) <= 1e-5
    assert O.rel_l2(act.read(np.float32, (used + 1) * ffn).reshape(used + 1, ffn)[:used], want["swiglu"][0]) <= TOL
    got_out = out.read(np.float32, H)
    assert O.rel_l2(got_out, want["out"][0] + f["h"]) <= TOL
    # the launches it replaces, on the same inputs
    case.h = got_h.reshape(1, H)
    case.res = got_h.reshape(1, H)
    ref = case.gpu(residual=True, defer=True)
    assert np.array_equal(ref["topk"][0], topk.read(np.int32, used))
    assert O.rel_l2(got_out, ref["out"][0]) <= 1e-5
    # refusals: y aliasing the residual the fold reads; more than one row
    g.y = dx.ptr
    with pytest.raises(A.ShvError, match="different"):
        c.enqueue(A.OP_GEMV_Q4K, g)
    ua.n_tok = 5
    with pytest.raises(A.ShvError, match="four rows"):
        c.enqueue(A.OP_MOE_UP, ua)


@pytest.mark.parametrize("T", [2, 3, 4])
def test_router_rows_ride_on_a_projection_of_a_few_rows(ctx, T):
    """The same for two to four rows (a verification pass, a few sequences' steps): the rows-side-by-side
    projection kernel forms every row's products, the gate/up kernel normalises each row itself."""
    E, used = 64, 10
    case = MoeCase(ctx, seed=91, E=E, used=used, T=T)
    H, K, ffn, c = case.H, 4096, case.ffn, ctx
    rng = np.random.default_rng(600 + T)
    w = O.quantize_q4k((rng.standard_normal((H, K)) * 0.02).astype(np.float32))
    v = rng.standard_normal((T, K)).astype(np.float32)
    z = rng.standard_normal((T, K)).astype(np.float32)
    x = rng.standard_normal((T, H)).astype(np.float32)
    pv = v.astype(np.float64) / (1 + np.exp(-z.astype(np.float64)))
    h = (x.astype(np.float64) + pv @ O.dequant_q4k(w, K).astype(np.float64).T).astype(np.float32)
    case.h, case.res = h, np.zeros((T, H), np.float32)
    want = case.oracle()
    d = {k: c.upload(getattr(case, k)) for k in ("router", "shared_gate", "gate_exps", "up_exps", "down_exps", "gate_sh", "up_sh", "down_sh", "gamma")}
    dw, dv, dx, dz = c.upload(w), c.upload(v), c.upload(x), c.upload(z)
    table, scratch = c.alloc(E * (K + H) * 4), c.alloc(H * K * 4)
    c.enqueue(A.OP_ROUTER_FOLD, A.RouterFoldArgs(d["router"].ptr, None, d["gamma"].ptr, dw.ptr, table.ptr, scratch.ptr, E, H, K))
    y, raw = c.alloc(T * H * 4), c.alloc(T * (E + 1) * 4)
    topk, weights, act, out = c.alloc(T * used * 4), c.alloc(T * (used + 1) * 4), c.alloc(T * (used + 1) * ffn * 4), c.alloc(T * H * 4)
    g = A.gemv_args(dw, dv, y, H, K, T, A.PRO_MUL_SIGMOID, None, dz, dx, EPS, 0)
    g.fold, g.fold_out, g.fold_rows, g.fold_stride = table.ptr, raw.ptr, E, E + 1
    ua = A.MoeUpArgs(y.ptr, topk.ptr, d["gate_exps"].ptr, d["up_exps"].ptr, d["gate_sh"].ptr, d["up_sh"].ptr, act.ptr, T, H, used, ffn,
                     raw.ptr, weights.ptr, E, 0, 0, 0, 0, None, 0, 0, d["gamma"].ptr, EPS, d["shared_gate"].ptr)
    da = A.MoeDownArgs(act.ptr, topk.ptr, weights.ptr, d["down_exps"].ptr, d["down_sh"].ptr, y.ptr, out.ptr, T, H, used, ffn, H, H, 0, 0, E, None, None)
    c.dispatch_multi([A.make_op(A.OP_GEMV_Q4K, g), A.make_op(A.OP_MOE_UP, ua), A.make_op(A.OP_MOE_DOWN, da)])
    got_h = y.read(np.float32, T * H).reshape(T, H)
    assert O.rel_l2(got_h, h) <= 1e-5
    scale = 1.0 / np.sqrt((h.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + EPS)
    got_lg = raw.read(np.float32, T * (E + 1)).reshape(T, E + 1)[:, :E].astype(np.float64) * scale
    assert O.rel_l2(got_lg, want["logits"]) <= 2e-5
    tk = topk.read(np.int32, T * used).reshape(T, used)
    for t in range(T):
        lg = want["logits"][t].astype(np.float64)
        p = np.exp(lg - lg.max())
        assert _margin(p / p.sum(), used) > 1e-4, "seed sits on a near-tie; pick another"
    assert np.array_equal(tk, want["topk"])
    wt = weights.read(np.float32, T * (used + 1)).reshape(T, used + 1)
    assert O.rel_l2(wt[:, :used], want["weights"]) <= 1e-5 and O.rel_l2(wt[:, used], want["sig"]) <= 1e-5
    assert O.rel_l2(out.read(np.float32, T * H).reshape(T, H), want["out"] + h) <= TOL
