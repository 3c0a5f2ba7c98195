"""Multi-row passes, sequence slots, rewindable passes, the draft head and the speculative loop on
the GPU against the CPU oracle.  The reference's gates of this kind: TestGraphIsAChunkSplit
(llm/graph_cache_test.go:39), TestSpeculationRewindIsTheSequence and the keep-prefix tests of
llm/graph_spec_test.go, TestDecodeRowsIsTheSequences (llm/batch_test.go), and the losslessness
argument of llm/spec.go:49-56 (every emitted token is the trunk's own arg-max)."""
import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu
LA = shv.pkg.llm_api
ROWS = 4  # rows of the widest pass: draft depth 3 + 1


def cfg_rows(**kw):
    d = dict(n_layer=4, n_expert=16, n_expert_used=4, vocab=4096, nkv=128, max_tokens=ROWS, slots=3,
             head_rows=ROWS, speculative=1, spec_rows=ROWS, nextn=1)
    d.update(kw)
    return LA.Config(**d)


@pytest.fixture(scope="module")
def rig():
    cfg = cfg_rows()
    m = LA.LLM(cfg)
    m.init_synthetic(4321)
    m.stage()
    tensors = {t[0]: m.download(t[0]) for t in m.tensors()}
    yield m, cfg, tensors
    m.close()


def fresh(m, slot=0):
    m.speculate(False)
    m.speculate_first(False)
    m.use_slot(slot)
    m.reset()


def test_chunked_prompt_matches_the_cpu(rig):
    """11 prompt rows go through as 4+4+3; the last row's logits and residual are the CPU's."""
    m, cfg, tensors = rig
    rng = np.random.default_rng(11)
    prompt = rng.integers(0, cfg.vocab, size=11).astype(np.int32)
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    fresh(m)
    lg, hd = m.extend(prompt, want_hidden=True)
    lg_cpu, hd_cpu = om.extend(prompt)
    assert O.rel_l2(hd, hd_cpu) <= 1e-3 and O.rel_l2(lg, lg_cpu) <= 1e-3
    assert m.past() == 11
    # the same prompt in other pieces (5+6: passes of 4+1 and 4+2 rows, which run through other
    # kernels than 4+4+3 and add up in another order)
    fresh(m)
    m.extend(prompt[:5])
    lg2, _ = m.extend(prompt[5:])
    assert O.rel_l2(lg2, lg) <= 1e-4
    # the carried state agrees with the CPU's
    assert O.rel_l2(m.dn_state(0), om.dn_s[0]) <= 1e-3
    k, v = m.kv(3, 11)
    kf = lambda a: a.view(np.float16).astype(np.float32)
    assert O.rel_l2(kf(k), kf(om.kc[3][:11])) <= 2e-3 and O.rel_l2(kf(v), kf(om.vc[3][:11])) <= 2e-3


def test_long_pass_matches_the_cpu():
    """A long pass: 150 prompt rows go through as one pass of 136 and one of 14.  The 136 rows take
    every block whole: one matrix-core launch per projection, the DeltaNet recurrence in chunks of
    64 rows in closed form (64 + 64 + 8), the attention four row pairs a block over tiles shared
    through LDS, the experts grouped by expert on the matrix cores.  Last row, carried state and
    cache are the CPU's, and the same rows in passes of 64 agree to rounding."""
    rng = np.random.default_rng(150)
    out = {}
    for rows in (136, 64):
        cfg = cfg_rows(max_tokens=rows, nkv=256, slots=1, head_rows=1, speculative=0, nextn=0)
        prompt = rng.integers(0, cfg.vocab, size=150).astype(np.int32) if rows == 136 else prompt
        m = LA.LLM(cfg)
        m.init_synthetic(4321)
        m.stage()
        lg, hd = m.extend(prompt, want_hidden=True)
        assert m.past() == 150
        if rows == 136:
            tensors = {t[0]: m.download(t[0]) for t in m.tensors()}
        out[rows] = (lg, hd, m.dn_state(0), m.dn_state(2), m.kv(3, 150))
        nxt = m.generate(4)
        out[rows] += (nxt,)
        m.close()
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    lg_cpu, hd_cpu = om.extend(prompt)
    a, b = out[136], out[64]
    assert O.rel_l2(a[1], hd_cpu) <= 1e-3 and O.rel_l2(a[0], lg_cpu) <= 1e-3, (O.rel_l2(a[1], hd_cpu), O.rel_l2(a[0], lg_cpu))
    assert O.rel_l2(a[2], om.dn_s[0]) <= 1e-3 and O.rel_l2(a[3], om.dn_s[2]) <= 1e-3
    kf = lambda x: x.view(np.float16).astype(np.float32)
    assert O.rel_l2(kf(a[4][0]), kf(om.kc[3][:150])) <= 2e-3 and O.rel_l2(kf(a[4][1]), kf(om.vc[3][:150])) <= 2e-3
    assert O.rel_l2(a[1], b[1]) <= 1e-4 and O.rel_l2(a[0], b[0]) <= 1e-4 and O.rel_l2(a[2], b[2]) <= 1e-4
    assert int(np.argmax(a[0])) == int(np.argmax(lg_cpu))
    print("136-row pass vs CPU: hidden %.2e logits %.2e; vs 64-row passes: logits %.2e; next tokens %s / %s" %
          (O.rel_l2(a[1], hd_cpu), O.rel_l2(a[0], lg_cpu), O.rel_l2(a[0], b[0]), a[5], b[5]))


def test_long_passes_on_another_slot_and_with_a_one_row_group():
    """195 prompt rows as passes of 130 (DeltaNet chunks of 64 + 64 + 2) and 65 (a chunk of 64 and one of a
    single row), on sequence slot 1 and on slot 0: the same bits on both (the pass's ring takes its
    conv history from the slot's own ring and hands the last rows back to it), and the rows in passes
    of 64 to rounding."""
    rng = np.random.default_rng(195)
    prompt = None
    out = {}
    for rows in (130, 64):
        cfg = cfg_rows(max_tokens=rows, nkv=256, slots=2, head_rows=1, speculative=0, nextn=0)
        if prompt is None:
            prompt = rng.integers(0, cfg.vocab, size=195).astype(np.int32)
        m = LA.LLM(cfg)
        m.init_synthetic(4321)
        m.stage()
        got = []
        for slot in (1, 0):
            m.use_slot(slot)
            m.reset()
            lg, hd = m.extend(prompt, want_hidden=True)
            assert m.past() == 195
            got.append((lg, hd, m.generate(3)[0]))
        assert np.array_equal(got[0][0], got[1][0]) and np.array_equal(got[0][1], got[1][1])
        assert np.array_equal(got[0][2], got[1][2])
        out[rows] = got[0]
        m.close()
    assert O.rel_l2(out[130][0], out[64][0]) <= 1e-4 and O.rel_l2(out[130][1], out[64][1]) <= 1e-4
    assert np.array_equal(out[130][2], out[64][2])


def test_extend_rows_is_every_rows_logits(rig):
    m, cfg, tensors = rig
    rng = np.random.default_rng(12)
    prompt = rng.integers(0, cfg.vocab, size=6).astype(np.int32)
    rows = rng.integers(0, cfg.vocab, size=ROWS).astype(np.int32)
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    om.extend(prompt)
    lg_cpu, res_cpu = om.extend_rows(rows)
    fresh(m)
    m.extend(prompt)
    best, lg, res = m.extend_rows(rows, want_logits=True, want_res=True)
    assert m.past() == 6 + ROWS
    for r in range(ROWS):
        assert O.rel_l2(lg[r], lg_cpu[r]) <= 1e-3, r
        assert O.rel_l2(res[r], res_cpu[r]) <= 1e-3, r
        assert best[r] == int(O.lib().shv_ref_argmax(O.F(np.ascontiguousarray(lg[r])), cfg.vocab))
    with pytest.raises(shv.pkg.ShvError):
        m.extend_rows(np.zeros(ROWS + 1, np.int32))      # more rows than the head arena holds


@pytest.mark.parametrize("keep", [1, 2, 3, 4])
def test_keeping_a_prefix_is_the_shorter_sequence(rig, keep):
    """A rewindable 4-row pass, then Keep(k): the sequence, the DeltaNet state and what the next
    token sees are those of the prompt plus the first k rows alone."""
    m, cfg, tensors = rig
    rng = np.random.default_rng(13)
    prompt = rng.integers(0, cfg.vocab, size=7).astype(np.int32)
    rows = rng.integers(0, cfg.vocab, size=ROWS).astype(np.int32)
    probe = rng.integers(0, cfg.vocab, size=1).astype(np.int32)
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    om.extend(prompt)
    om.extend(rows[:keep])
    want_state = om.dn_s[0].copy()
    lg_cpu, _ = om.extend(probe)

    fresh(m)
    m.extend(prompt)
    plane0 = m.plane()
    m.speculate(True)
    m.speculate_first(True)
    m.extend_rows(rows)
    with pytest.raises(shv.pkg.ShvError):
        m.extend_rows(rows)                               # one pass in flight at most
    with pytest.raises(shv.pkg.ShvError):
        m.rewind()                                        # a keep-first pass is kept or committed
    m.keep(keep)
    assert m.past() == 7 + keep
    assert m.plane() == (plane0 + keep) % (ROWS + 1)
    assert O.rel_l2(m.dn_state_at(0, 0, m.plane()), want_state) <= 1e-3
    assert list(m.ids()) == list(prompt) + list(rows[:keep])
    lg = m.extend_rows(probe, want_logits=True)[1]
    m.commit()
    assert O.rel_l2(lg[0], lg_cpu) <= 1e-3
    # and the plain recorded decode step runs from the plane the passes left committed
    m.speculate(False)
    tok = np.array([int(np.argmax(lg_cpu))], np.int32)
    lg_next, _ = m.extend(tok)
    lg_next_cpu, _ = om.extend(tok)
    assert O.rel_l2(lg_next, lg_next_cpu) <= 1e-3


def test_rewind_discards_the_pass(rig):
    m, cfg, tensors = rig
    rng = np.random.default_rng(14)
    prompt = rng.integers(0, cfg.vocab, size=5).astype(np.int32)
    rows = rng.integers(0, cfg.vocab, size=3).astype(np.int32)
    probe = rng.integers(0, cfg.vocab, size=2).astype(np.int32)
    fresh(m)
    m.extend(prompt)
    before = m.dn_state_at(0, 0, m.plane()).copy()
    want, _ = m.extend(probe)            # the control: the probe straight after the prompt
    fresh(m)
    m.extend(prompt)
    m.speculate(True)
    m.extend_rows(rows)
    assert m.past() == 8
    with pytest.raises(shv.pkg.ShvError):
        m.keep(1)                         # prefixes are kept only under SpeculateFirst
    m.rewind()
    assert m.past() == 5
    assert np.array_equal(m.dn_state_at(0, 0, m.plane()), before)
    m.speculate(False)
    got, _ = m.extend(probe)
    assert np.array_equal(got, want)
    with pytest.raises(shv.pkg.ShvError):
        m.commit()                        # nothing in flight


def test_speculate_needs_the_planes():
    cfg = cfg_rows(speculative=0, nextn=0, slots=1)
    m = LA.LLM(cfg)
    m.init_synthetic(1)
    m.stage()
    with pytest.raises(shv.pkg.ShvError):
        m.speculate(True)
    m.close()


def test_decode_rows_advances_each_sequence(rig):
    """Three sequences of different lengths take one token each in one pass; every row's logits are
    those of its own sequence run alone on the CPU (llm/graph.go:1527-1666)."""
    m, cfg, tensors = rig
    rng = np.random.default_rng(15)
    prompts = [rng.integers(0, cfg.vocab, size=n).astype(np.int32) for n in (3, 9, 6)]
    toks = rng.integers(0, cfg.vocab, size=3).astype(np.int32)
    oms = [O.OracleModel(cfg, tensors, max_cells=cfg.nkv) for _ in prompts]
    for s, p in enumerate(prompts):
        fresh(m, s)
        m.extend(p)
        oms[s].extend(p)
    order = [2, 0, 1]
    best, lg = m.decode_rows(order, toks, want_logits=True)
    for r, s in enumerate(order):
        lg_cpu, _ = oms[s].extend(toks[r:r + 1])
        assert O.rel_l2(lg[r], lg_cpu) <= 1e-3, (r, s)
        assert best[r] == int(np.argmax(lg[r]))
    for s, p in enumerate(prompts):
        m.use_slot(s)
        assert m.past() == len(p) + 1
        assert m.ids()[-1] == toks[order.index(s)]
    # a second batched step over two of them, then one alone through the same entry point
    toks2 = rng.integers(0, cfg.vocab, size=2).astype(np.int32)
    _, lg2 = m.decode_rows([1, 2], toks2, want_logits=True)
    for r, s in enumerate([1, 2]):
        lg_cpu, _ = oms[s].extend(toks2[r:r + 1])
        assert O.rel_l2(lg2[r], lg_cpu) <= 1e-3
    _, lg3 = m.decode_rows([0], toks2[:1], want_logits=True)
    lg_cpu, _ = oms[0].extend(toks2[:1])
    assert O.rel_l2(lg3[0], lg_cpu) <= 1e-3
    with pytest.raises(shv.pkg.ShvError):
        m.decode_rows([0, 0], toks2)                      # a slot twice in one batch
    with pytest.raises(shv.pkg.ShvError):
        m.decode_rows([0, 3], toks2)                      # a slot that does not exist
    m.use_slot(0)


def test_draft_head_rows_match_the_cpu(rig):
    m, cfg, tensors = rig
    rng = np.random.default_rng(16)
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    dm = O.OracleMTP(om, cfg.nkv)
    fresh(m)
    m.extend(np.array([1, 2, 3], np.int32))               # the head borrows a staged graph
    m.mtp_stage(max_tok=ROWS)
    hs = rng.standard_normal((3, cfg.n_embd)).astype(np.float32)
    ids = rng.integers(0, cfg.vocab, size=3).astype(np.int32)
    lg, res = m.mtp_rows(hs, ids, 0)
    lg_cpu, res_cpu = dm.rows(hs, ids, 0)
    assert O.rel_l2(res, res_cpu) <= 1e-3 and O.rel_l2(lg, lg_cpu) <= 1e-3
    # a chained step: the draft's own residual behind the next row, over the cells just written
    one = rng.integers(0, cfg.vocab, size=1).astype(np.int32)
    lg2, res2 = m.mtp_rows(res[-1:], one, 3)
    lg2_cpu, res2_cpu = dm.rows(res_cpu[-1:], one, 3)
    assert O.rel_l2(res2, res2_cpu) <= 1e-3 and O.rel_l2(lg2, lg2_cpu) <= 1e-3
    assert m.mtp_past() == 4
    # rewinding is the whole of the draft's rollback: position 2 again sees cells 0..1 only
    m.mtp_rewind(2)
    lg3, _ = m.mtp_rows(hs[2:], ids[2:], 2)
    dm3 = O.OracleMTP(om, cfg.nkv)
    dm3.rows(hs[:2], ids[:2], 0)
    lg3_cpu, _ = dm3.rows(hs[2:], ids[2:], 2)
    assert O.rel_l2(lg3, lg3_cpu) <= 1e-3
    with pytest.raises(shv.pkg.ShvError):
        m.mtp_rows(hs[:1], ids[:1], 7)                    # a gap in the draft's cache


@pytest.mark.parametrize("mode", ["draft", "all-right", "first-right", "second-right"])
def test_speculative_loop_emits_the_greedy_sequence(rig, mode):
    """Whatever the drafts are — the draft head's own, all correct, or correct up to a point — the
    loop emits exactly the tokens of plain greedy decoding, and keeps as many rows as agree."""
    m, cfg, tensors = rig
    rng = np.random.default_rng(17)
    prompt = rng.integers(0, cfg.vocab, size=10).astype(np.int32)
    n_new = 24
    fresh(m)
    m.extend(prompt)
    plain, _ = m.generate(n_new + ROWS)
    plain = list(plain)

    fresh(m)
    m.mtp_stage(max_tok=ROWS)
    depth = ROWS - 1
    m.spec_open(depth)
    out = [m.spec_start(prompt)]
    assert out[0] == plain[0]
    rounds = 0
    while len(out) < n_new:
        nxt = plain[len(out):len(out) + depth]            # the true continuation after the pending token
        forced = {"draft": [], "all-right": nxt, "first-right": [nxt[0], (nxt[1] + 1) % cfg.vocab, nxt[2]],
                  "second-right": [nxt[0], nxt[1], (nxt[2] + 1) % cfg.vocab]}[mode]
        got = list(m.spec_round(forced))
        want_keep = {"all-right": depth + 1, "first-right": 2, "second-right": 3}.get(mode)
        if want_keep:
            assert len(got) == want_keep, (mode, got)
        out += got
        rounds += 1
    assert out[:n_new] == plain[:n_new], mode
    st = m.spec_stats()
    assert st["rounds"] == rounds and st["tokens"] == len(out)
    assert st["passes"][min(depth + 1, 4)] == rounds
    if mode == "all-right":
        assert st["accepted_at"][:3] == [rounds] * 3
    if mode == "first-right":
        assert st["accepted_at"][0] == rounds and st["accepted_at"][1] == 0
    # the trunk holds exactly the emitted tokens but the pending one
    assert m.past() == len(prompt) + len(out) - 1
    assert list(m.ids()) == list(prompt) + out[:-1]


def test_a_round_handed_over_whole_is_the_round_waited_for_call_by_call(rig, monkeypatch):
    """The greedy round launches its draft calls and the verification pass back to back and waits once (the drafts
    travel through the trunk's id ring on the device); LLM_SPEC_CHAIN=0 waits after every call and carries the drafts
    through the host, as the reference's loop does.  Same tokens round by round, same counters, same sequence left
    in the trunk, with the head's own drafts and with forced ones that end a round early."""
    m, cfg, tensors = rig
    rng = np.random.default_rng(23)
    prompt = rng.integers(0, cfg.vocab, size=9).astype(np.int32)
    depth = ROWS - 1
    runs = {}
    for chain in ("0", "1"):
        monkeypatch.setenv("LLM_SPEC_CHAIN", chain)
        fresh(m)
        m.mtp_stage(max_tok=ROWS)
        m.spec_open(depth)
        rounds = [[m.spec_start(prompt)]]
        for i in range(10):
            forced = [] if i % 3 else [int(rounds[-1][-1] + 1) % cfg.vocab]   # a wrong first draft: one token kept
            rounds.append(list(m.spec_round(forced)))
            if not i % 3:
                assert len(rounds[-1]) == 1
        st = m.spec_stats()
        runs[chain] = (rounds, {k: st[k] for k in ("rounds", "tokens", "drafted", "accepted", "passes", "drafted_at", "accepted_at")},
                       list(m.ids()), m.past())
    assert runs["0"] == runs["1"]
    assert runs["1"][1]["rounds"] == 10


def test_sampled_speculation(rig):
    """The loop under a sampler (Speculator.UseSampler; llm/spec.go:703-857 with llm/sample.go:183-250):
    drafts are draws from the draft sampler's distribution, rows go through Verify on the host.
    top-k 1 at any temperature is the arg-max, so that loop is the greedy loop token for token,
    round for round; at temperature 1 the run is a function of its seeds, and every token it emits is
    one the trunk's own cuts allow at its position."""
    m, cfg, tensors = rig
    rng = np.random.default_rng(23)
    prompt = rng.integers(0, cfg.vocab, size=9).astype(np.int32)
    n_new, depth = 20, ROWS - 1

    def run(sampler):
        fresh(m)
        m.mtp_stage(max_tok=ROWS)
        m.spec_open(depth)
        if sampler:
            m.spec_sampler(**sampler)
        out = [m.spec_start(prompt)]
        while len(out) < n_new:
            out += list(m.spec_round())
        st = m.spec_stats()
        assert st["tokens"] == len(out) and m.past() == len(prompt) + len(out) - 1
        assert list(m.ids()) == list(prompt) + out[:-1]
        return out, st

    greedy, st_g = run(None)
    wall, st_w = run(dict(temp=0.8, top_k=1, seed=3, draft_seed=4))
    assert wall == greedy and st_w["accepted_at"] == st_g["accepted_at"] and st_w["rounds"] == st_g["rounds"]
    cold, _ = run(dict(temp=0.0, top_k=40, top_p=0.9))
    assert cold == greedy

    warm = dict(temp=1.0, top_k=6, seed=11, draft_seed=12)
    a, _ = run(warm)
    b, _ = run(warm)
    c, _ = run(dict(warm, seed=13))
    assert a == b and a != c and a != greedy
    # each emitted token is among the trunk's most likely at its position (ten allowed for the six
    # kept: a pass of other shape rounds a little differently)
    for i in (0, 1, 5, 12, n_new - 1):
        fresh(m)
        lg, _ = m.extend(np.concatenate([prompt, np.array(a[:i], np.int32)]))
        assert a[i] in np.argsort(-lg)[:10], i
    # penalties reach the loop: a large presence penalty keeps a token from repeating inside the window
    pen, _ = run(dict(temp=1.0, top_k=6, presence_penalty=50.0, seed=11, draft_seed=12))
    assert len(set(pen)) == len(pen)
    for t in prompt:
        assert t not in pen


def test_checkpoint_restore_is_the_shorter_sequence(rig):
    """Graph.Checkpoint / Restore (llm/graph.go:1004-1062): after going on past a checkpoint and
    coming back, the sequence continues exactly as one that never went on; a slot that no longer
    starts with the checkpoint's tokens is refused, and so is a pass in flight."""
    m, cfg, tensors = rig
    rng = np.random.default_rng(77)
    head, tail, other = (rng.integers(0, cfg.vocab, size=n).astype(np.int32) for n in (7, 5, 6))
    fresh(m)
    for t in head:
        m.extend(np.array([t], np.int32), want_logits=False)
    c = m.checkpoint()
    for t in other:  # the conversation goes somewhere else ...
        m.extend(np.array([t], np.int32), want_logits=False)
    m.restore(c)     # ... and comes back
    assert m.past() == len(head)
    got = [m.extend(np.array([t], np.int32))[0] for t in tail]
    state = m.dn_state(0)
    fresh(m)
    for t in head:
        m.extend(np.array([t], np.int32), want_logits=False)
    want = [m.extend(np.array([t], np.int32))[0] for t in tail]
    for g, w in zip(got, want):
        assert np.array_equal(g, w)  # same kernels on the same bytes
    assert np.array_equal(state, m.dn_state(0))
    # against the CPU too
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    lg_cpu, _ = om.extend(np.concatenate([head, tail]))
    assert O.rel_l2(got[-1], lg_cpu) <= 1e-3
    # a second restore from the same checkpoint, after a chunked continuation
    m.extend(other)
    m.restore(c)
    lg, _ = m.extend(tail)
    assert O.rel_l2(lg, lg_cpu) <= 1e-3
    # refusals
    fresh(m)
    m.extend(other)
    with pytest.raises(shv.api.ShvError, match="no longer holds"):
        m.restore(c)
    fresh(m)
    with pytest.raises(shv.api.ShvError, match="nothing to checkpoint"):
        m.checkpoint()
    m.extend(head)
    m.speculate(True)
    m.extend_rows(tail[:2])
    with pytest.raises(shv.api.ShvError, match="in flight"):
        m.checkpoint()
    m.rewind()
    m.speculate(False)
    m.checkpoint_free(c)


def test_chunk_size_does_not_matter_over_4096_tokens():
    """BASELINE's prefill shape: 4096 tokens through a period of three DeltaNet layers and one
    attention layer at the full widths, as one pass of 4096, in chunks of 2048 (either way every
    block whole: whole-pass projections, the recurrence in closed form 64 rows at a time, attention
    tiles shared by four row pairs, experts grouped on the matrix cores), of 64, of 16, and (the
    first 192) token by token.
    Every chunk size runs other kernels (matrix cores from 3 or 5 rows, operands staged once from
    17, the row-by-row recurrence up to 16 rows and the chunked one above, pairs of attention rows)
    over the same arithmetic, so the carried state and the last row must agree to rounding."""
    cfg = dict(n_layer=4, vocab=8192, nkv=4224, slots=1)
    rng = np.random.default_rng(4096)
    prompt = rng.integers(0, 8192, size=4096).astype(np.int32)
    out = {}
    for rows in (4096, 2048, 64, 16):
        m = LA.LLM(LA.Config(max_tokens=rows, **cfg))
        m.init_synthetic(99)
        m.stage()
        lg, hd = m.extend(prompt, want_hidden=True)
        out[rows] = (lg, hd, m.dn_state(0), m.dn_state(2), m.kv(3, 4096))
        if rows == 16:
            m.reset()
            m.extend(prompt[:192], want_logits=False)
            short16 = (m.dn_state(1), m.kv(3, 192))
            m.reset()
            for t in prompt[:192]:
                m.extend(np.array([t], np.int32), want_logits=False)
            short1 = (m.dn_state(1), m.kv(3, 192))
        m.close()
    a, b = out[64], out[2048]
    assert O.rel_l2(a[1], b[1]) <= 1e-3 and O.rel_l2(a[0], b[0]) <= 1e-3, (O.rel_l2(a[1], b[1]), O.rel_l2(a[0], b[0]))
    assert O.rel_l2(a[2], b[2]) <= 1e-3 and O.rel_l2(a[3], b[3]) <= 1e-3
    print("64 vs 2048 rows a chunk over 4096 tokens: hidden %.2e logits %.2e state %.2e" %
          (O.rel_l2(a[1], b[1]), O.rel_l2(a[0], b[0]), O.rel_l2(a[2], b[2])))
    a, b = out[64], out[4096]
    assert O.rel_l2(a[1], b[1]) <= 1e-3 and O.rel_l2(a[0], b[0]) <= 1e-3, (O.rel_l2(a[1], b[1]), O.rel_l2(a[0], b[0]))
    assert O.rel_l2(a[2], b[2]) <= 1e-3 and O.rel_l2(a[3], b[3]) <= 1e-3
    print("64 vs 4096 rows a chunk over 4096 tokens: hidden %.2e logits %.2e state %.2e" %
          (O.rel_l2(a[1], b[1]), O.rel_l2(a[0], b[0]), O.rel_l2(a[2], b[2])))
    a, b = out[64], out[16]
    assert O.rel_l2(a[1], b[1]) <= 1e-3 and O.rel_l2(a[0], b[0]) <= 1e-3, (O.rel_l2(a[1], b[1]), O.rel_l2(a[0], b[0]))
    assert O.rel_l2(a[2], b[2]) <= 1e-3 and O.rel_l2(a[3], b[3]) <= 1e-3
    f16 = lambda bits: bits.view(np.float16).astype(np.float32)
    for ka, kb in zip(a[4], b[4]):  # the cache: halves, the last bit of a few percent of them flips
        assert O.rel_l2(f16(ka), f16(kb)) <= 1e-3 and np.mean(ka != kb) <= 0.1
    assert O.rel_l2(short16[0], short1[0]) <= 1e-3
    for ka, kb in zip(short16[1], short1[1]):
        assert O.rel_l2(f16(ka), f16(kb)) <= 1e-3 and np.mean(ka != kb) <= 0.1
    print("64 vs 16 rows a chunk over 4096 tokens: hidden %.2e logits %.2e state %.2e" %
          (O.rel_l2(a[1], b[1]), O.rel_l2(a[0], b[0]), O.rel_l2(a[2], b[2])))


def test_chunk_size_does_not_matter_to_a_second_attention_layer():
    """What a chunk's rows leave an attention layer with is only seen by the layers after it: two
    attention layers in a row, 2560 tokens as one chunk and in chunks of 512 down to 16 rows.  The second
    layer's keys are made of every row the first one put out, so they hold the first layer's
    attention to account at every row and cache length, where the last row's logits hold one."""
    cfg = dict(n_layer=2, attn_every=1, vocab=8192, nkv=2688, slots=1)
    prompt = np.random.default_rng(2560).integers(0, 8192, size=2560).astype(np.int32)
    out = {}
    sizes = (2560, 512, 256, 128, 100, 64, 48, 32, 16)
    for rows in sizes:
        m = LA.LLM(LA.Config(max_tokens=rows, **cfg))
        m.init_synthetic(7)
        m.stage()
        _, hd = m.extend(prompt, want_hidden=True)
        k, v = m.kv(1, 2560)
        out[rows] = (hd, k.view(np.float16).astype(np.float32).reshape(2560, -1), v.view(np.float16).astype(np.float32).reshape(2560, -1))
        m.close()
    for rows in sizes[:-1]:
        a, b = out[rows], out[16]
        assert O.rel_l2(a[0], b[0]) <= 1e-4, (rows, O.rel_l2(a[0], b[0]))
        for x, y in ((a[1], b[1]), (a[2], b[2])):
            # halves: a cell here and there rounds the other way, none is off by more than that
            e = np.linalg.norm(x - y, axis=1) / np.linalg.norm(y, axis=1)
            assert e.max() <= 2e-3, (rows, int(e.argmax()), float(e.max()))


def test_sequences_of_very_different_lengths_decode_together():
    """Eight sequences of 5 to 5000 tokens advanced together for twenty steps against each of them advanced alone on
    the same tokens, over two periods of layers (so that what a batched pass leaves an attention layer with is read by
    the layers after it), at the full widths; then a three-row pass at 5020 cells against three steps."""
    S, steps = 8, 20
    cfg = LA.Config(n_layer=8, nkv=6144, max_tokens=256, head_rows=S, slots=S, vocab=32768)
    m = LA.LLM(cfg)
    m.init_synthetic(20260101)
    m.stage()
    try:
        rng = np.random.default_rng(3)
        lens = [5, 100, 700, 1023, 1500, 2049, 3000, 5000]
        prompts = [rng.integers(0, cfg.vocab, size=n).astype(np.int32) for n in lens]

        def prefill():
            for s in range(S):
                m.use_slot(s)
                m.reset()
                m.extend(prompts[s], want_logits=False)

        prefill()
        slots = np.arange(S, dtype=np.int32)
        ids = rng.integers(0, cfg.vocab, size=S).astype(np.int32)
        fed, batched = [], []
        for _ in range(steps):
            fed.append(ids.copy())
            ids, lg = m.decode_rows(slots, ids, want_logits=True)
            batched.append(lg.copy())
        prefill()
        for s in range(S):
            m.use_slot(s)
            for t in range(steps):
                lg, _ = m.extend(np.array([fed[t][s]], np.int32))
                assert O.rel_l2(batched[t][s], lg) <= 1e-3, (lens[s], t)
        three = rng.integers(0, cfg.vocab, size=3).astype(np.int32)
        m.use_slot(7)
        _, lg3, _ = m.extend_rows(three, want_logits=True)
        m.use_slot(6)
        m.reset()
        m.extend(np.concatenate([prompts[7], np.array([fed[t][7] for t in range(steps)], np.int32)]), want_logits=False)
        for i in range(3):
            lg, _ = m.extend(three[i:i + 1])
            assert O.rel_l2(lg3[i], lg) <= 1e-3, i
    finally:
        m.close()
