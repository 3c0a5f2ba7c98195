"""The whole token loop on the GPU (llm::Graph: recorded decode step, device-side greedy loop)
against the CPU oracle's loop on a reduced model with the same weights.  The reference's gates of
this kind are TestGraphIsAChunkSplit (llm/graph_cache_test.go:39), TestPrerecordedDecodeIsThe
RecordedDecode and the greedy-text acceptance of cmd/llm/generate.go:11-13."""
import os

import numpy as np
import pytest

import oracle_lib as O
import shv

pytestmark = pytest.mark.gpu
LA = shv.pkg.llm_api


def small_cfg(**kw):
    d = dict(n_layer=4, n_expert=16, n_expert_used=4, vocab=4096, nkv=128)
    d.update(kw)
    return LA.Config(**d)


@pytest.fixture(scope="module")
def small():
    cfg = small_cfg()
    m = LA.LLM(cfg)
    m.init_synthetic(1234)
    m.stage()
    tensors = {t[0]: m.download(t[0]) for t in m.tensors()}
    yield m, cfg, tensors
    m.close()


def test_greedy_loop_matches_the_cpu_loop(small):
    """Prompt of 12 random ids, then 12 greedy tokens: ids bit-exact, logits within 1e-3 rel-L2.
    A flip is only a failure if the CPU's own margin between its best two logits is not tiny."""
    m, cfg, tensors = small
    rng = np.random.default_rng(5)
    prompt = rng.integers(0, cfg.vocab, size=12).astype(np.int32)
    n_new = 12
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    m.reset()
    lg_gpu, hd_gpu = m.extend(prompt, want_hidden=True)
    lg_cpu, hd_cpu = om.extend(prompt)
    assert O.rel_l2(hd_gpu, hd_cpu) <= 1e-3
    assert O.rel_l2(lg_gpu, lg_cpu) <= 1e-3
    ids_gpu, _ = m.generate(n_new)
    ids_cpu, margins = [], []
    lg = lg_cpu
    for i in range(n_new):
        tok = int(O.lib().shv_ref_argmax(O.F(lg), cfg.vocab))
        top2 = np.sort(lg)[-2:]
        margins.append(float(top2[1] - top2[0]))
        ids_cpu.append(tok)
        if i + 1 < n_new:
            lg, _ = om.extend(np.array([tok], np.int32))
    print("greedy ids gpu", list(ids_gpu), "cpu", ids_cpu, "min margin %.3e" % min(margins))
    for i in range(n_new):
        if ids_gpu[i] != ids_cpu[i]:
            assert margins[i] < 1e-4, f"token {i}: gpu {ids_gpu[i]} cpu {ids_cpu[i]} at margin {margins[i]:.3e}"
            break  # after a rounding flip the two sequences are different sequences
    else:
        assert list(ids_gpu) == ids_cpu
    # carried state agrees too: DeltaNet S of layer 0 and the attention cache of layer 3
    assert m.past() == om.past == len(prompt) + n_new - 1
    assert O.rel_l2(m.dn_state(0), om.dn_s[0]) <= 1e-3
    k, v = m.kv(3, om.past)
    kf = lambda a: a.view(np.float16).astype(np.float32)
    assert O.rel_l2(kf(k), kf(om.kc[3][:om.past])) <= 2e-3
    assert O.rel_l2(kf(v), kf(om.vc[3][:om.past])) <= 2e-3


def test_device_loop_is_the_host_loop(small):
    """Generate (replays feeding the arg-max back on the device) must give the tokens of the
    reference-style loop: Extend one id, read logits back, Argmax on the host, repeat."""
    m, cfg, _ = small
    rng = np.random.default_rng(6)
    prompt = rng.integers(0, cfg.vocab, size=9).astype(np.int32)
    m.reset()
    lg, _ = m.extend(prompt)
    host_ids = []
    for _ in range(10):
        tok = int(np.argmax(lg))
        host_ids.append(tok)
        lg, _ = m.extend(np.array([tok], np.int32))
    m.reset()
    m.extend(prompt)
    dev_ids, ns = m.generate(10)
    assert list(dev_ids) == host_ids and ns > 0


def test_prompt_in_pieces_is_the_whole_prompt(small):
    """Chunk-split identity (llm/graph_cache_test.go:39): 5+6 tokens == 11 tokens, bit for bit
    here, because every row goes through the same recorded step."""
    m, cfg, _ = small
    rng = np.random.default_rng(7)
    prompt = rng.integers(0, cfg.vocab, size=11).astype(np.int32)
    m.reset()
    whole, _ = m.extend(prompt)
    m.reset()
    m.extend(prompt[:5])
    parts, _ = m.extend(prompt[5:])
    assert np.array_equal(whole, parts)
    assert m.past() == 11


def test_reset_restarts_the_sequence(small):
    m, cfg, _ = small
    ids = np.array([1, 2, 3, 4], np.int32)
    m.reset()
    a, _ = m.extend(ids)
    m.extend(ids)
    m.reset()
    b, _ = m.extend(ids)
    assert np.array_equal(a, b)


def test_graph_refusals(small):
    m, cfg, _ = small
    m.reset()
    with pytest.raises(shv.pkg.ShvError):
        m.extend(np.array([cfg.vocab], np.int32))          # outside the vocabulary
    with pytest.raises(shv.pkg.ShvError):
        m.extend(np.zeros(cfg.nkv + 5, np.int32))           # more than the cache holds
    with pytest.raises(shv.pkg.ShvError):
        m.generate(3)                                       # before any prompt
    bad = LA.LLM(small_cfg(n_layer=4, n_expert=2, n_expert_used=1, vocab=256, head_dim=128, n_head=32))
    with pytest.raises(shv.pkg.ShvError):
        bad.stage()                                         # a shape the kernels do not cover
    bad.close()


def test_profile_step_labels(small):
    m, cfg, _ = small
    m.reset()
    m.extend(np.array([5, 6, 7], np.int32))
    st = dict(m.profile_step())
    for k in ("embed", "dn.qkv", "dn.step", "dn.out", "attn.qkv", "attn.attn", "attn.out",
              "moe.up", "moe.down", "head", "total"):
        assert k in st and st[k] > 0, k
    # the vocabulary projection's launch names the next token itself (LLM_HEAD_ARGMAX=0: a launch of its own)
    own_argmax = os.environ.get("LLM_HEAD_ARGMAX", "1") == "0"
    assert ("argmax" in st) == own_argmax
    # the router's logits come with the launch of the mixer's output projection on a one-row pass
    # (LLM_ROUTER_FOLD=0 keeps the router's own launch): five ops a layer, not six
    folded = os.environ.get("LLM_ROUTER_FOLD", "1") != "0"
    assert ("moe.router" in st) == (not folded)
    assert m.dispatches() == 1 + 4 * (5 if folded else 6) + (2 if own_argmax else 1)


def _oracle_rows_with_gaps(om, tensors, cfg, ids, threads=16):
    """The oracle's pass over rows `ids` (its block functions in the order of its own token loop,
    oracle/shv_oracle.c shv_ref_model_extend_rows), which also returns, per row, the smallest gap
    over all layers between the 10th and the 11th router logit: where that gap is of the size of
    float32 rounding, which expert is selected is not a statement about the kernels."""
    C, L, mc = O.C, O.lib(), om.mcfg
    T, H, E, U = len(ids), cfg.n_embd, cfg.n_expert, cfg.n_expert_used
    x = tensors["token_embd.weight"].view(np.float16).reshape(cfg.vocab, H)[ids].astype(np.float32)
    gaps = np.full(T, np.inf)
    y, lg = np.empty((T, H), np.float32), np.empty((T, E), np.float32)
    for l in range(cfg.n_layer):
        lw = om.layers[l]
        xn = O.rmsnorm(x, tensors["blk.%d.attn_norm.weight" % l], cfg.rms_eps)
        if (l + 1) % cfg.attn_every == 0:
            L.shv_ref_attn_layer(C.byref(mc.attn), C.byref(lw.attn), O.F(xn), T, om.state.past, O.H(om.kc[l]), O.H(om.vc[l]),
                                 O.F(y), None, None, threads)
        else:
            L.shv_ref_deltanet_layer(C.byref(mc.dn), C.byref(lw.dn), O.F(xn), T, O.F(om.dn_conv[l]), O.F(om.dn_s[l]), O.F(y),
                                     None, None, None, None, None, None, None, 0, threads)
        x = x + y
        xn = O.rmsnorm(x, tensors["blk.%d.post_attention_norm.weight" % l], cfg.rms_eps)
        L.shv_ref_moe_block(C.byref(mc.moe), C.byref(lw.moe), O.F(xn), T, O.F(y), O.F(lg), None, None, None, None, None, threads)
        x = x + y
        top = np.sort(lg.astype(np.float64), axis=1)[:, ::-1]
        gaps = np.minimum(gaps, top[:, U - 1] - top[:, U])
    om.state.past += T
    xn = O.rmsnorm(x[-1:], tensors["output_norm.weight"], cfg.rms_eps)
    logits = O.gemv_q4k(tensors["output.weight"], xn[0], cfg.vocab, H, threads=threads)
    return x, logits, gaps


@pytest.mark.timeout(900)
def test_full_size_model_matches_the_cpu_loop():
    """The benchmark's own model (48 layers, 512 experts top-10, vocab 151 936) rather than a reduced
    one: a prompt of 6 ids through the multi-row pass, then 4 greedy tokens through the recorded
    one-row step, against the oracle over the very same tensors (downloaded, 46 GB on the host).
    Every row's residual stream within 1e-3 rel-L2, logits too; ids equal unless the oracle's own
    best two logits sit closer than twice the two paths' largest logit difference.  With 288 top-10 selections among 512 nearly level logits
    a pass, now and then one sits on a near-tie (a gap of 1e-5 where the logits themselves agree to
    1e-5): such a row may take the other expert, as the reference's own routing tests exclude
    near-ties (llm/moe_test.go:59-66); it is left out of the comparison, and most rows must remain."""
    cfg = LA.Config(nkv=128, max_tokens=8, head_rows=6, speculative=1, spec_rows=3, nextn=1)
    assert (cfg.n_layer, cfg.n_expert, cfg.n_expert_used, cfg.vocab) == (48, 512, 10, 151936)
    GAP = 4e-4   # router logits are O(1) and agree to about 2e-4 by the last layers: twice that
    m = LA.LLM(cfg)
    try:
        m.init_synthetic(20260101)
        m.stage()
        tensors = {t[0]: m.download(t[0]) for t in m.tensors()}
        om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
        check = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
        greedy_done, lost = False, 0
        for seed in (17, 18, 19, 20, 21):   # until a prompt without a flipped row lets the greedy steps be compared
            m.reset()
            om.reset()
            check.reset()
            rng = np.random.default_rng(seed)
            prompt = rng.integers(0, cfg.vocab, size=6).astype(np.int32)
            rows_cpu, lg_cpu, gaps = _oracle_rows_with_gaps(om, tensors, cfg, prompt)
            # the walk above is the oracle's own loop: same hidden state, bit for bit
            _, hd_loop = check.extend(prompt, threads=16)
            assert np.array_equal(hd_loop, rows_cpu[-1])
            _, lg_rows, rows_gpu = m.extend_rows(prompt, want_logits=True, want_res=True)
            errs = [O.rel_l2(rows_gpu[t], rows_cpu[t]) for t in range(len(prompt))]
            print("full size: prompt rows rel-L2", ["%.2e" % e for e in errs], "gaps", ["%.1e" % g for g in gaps], flush=True)
            # a row past a near-tie (its own, or an earlier row's, whose state it reads) may hold
            # another expert's output; every other row must agree
            so_far = np.minimum.accumulate(gaps)
            within = [e <= 1e-3 for e in errs]
            assert all(w or g < GAP for w, g in zip(within, so_far)), (errs, list(so_far))
            if sum(within) < 4:
                # the near-tie sits in one of the first rows and every later row reads its state: this prompt says
                # nothing further; at most two prompts of the five may go that way
                lost += 1
                print("full size: seed %d: a router gap of %.1e in row %d; next prompt" % (seed, so_far[within.index(False)], within.index(False)), flush=True)
                assert lost <= 2
                continue
            compared = 0
            if all(within):
                assert O.rel_l2(lg_rows[-1], lg_cpu) <= 1e-3
                lg, lg_gpu = lg_cpu, lg_rows[-1]
                for i in range(4):
                    tok_cpu = int(O.lib().shv_ref_argmax(O.F(lg), cfg.vocab))
                    tok_gpu = int(np.argmax(lg_gpu))
                    top2 = np.sort(lg)[-2:]
                    margin = float(top2[1] - top2[0])
                    if tok_gpu != tok_cpu:
                        # only logits closer than twice their own disagreement can swap places
                        assert margin < 2 * float(np.max(np.abs(lg_gpu - lg))), f"token {i}: gpu {tok_gpu} cpu {tok_cpu} at margin {margin:.3e}"
                        break
                    hd_cpu, lg, gap = _oracle_rows_with_gaps(om, tensors, cfg, np.array([tok_cpu], np.int32))
                    # the recorded one-row step (the decode path proper), fed the same id
                    lg_gpu, hd_gpu = m.extend(np.array([tok_cpu], np.int32), want_hidden=True)
                    e_h, e_l = O.rel_l2(hd_gpu, hd_cpu[0]), O.rel_l2(lg_gpu, lg)
                    print("full size: token %d id %d margin %.3e gap %.1e hidden rel-L2 %.3e logits rel-L2 %.3e"
                          % (i, tok_cpu, margin, gap[0], e_h, e_l), flush=True)
                    if e_h > 1e-3 or e_l > 1e-3:
                        assert min(gap[0], so_far[-1]) < GAP, (e_h, e_l, gap[0])
                        break
                    compared += 1
                if compared == 4:
                    # carried state of the last DeltaNet layer and the last attention layer's cache
                    assert O.rel_l2(m.dn_state(46), om.dn_s[46]) <= 1e-3
                    k, v = m.kv(47, om.past)
                    kf = lambda a: a.view(np.float16).astype(np.float32)
                    assert O.rel_l2(kf(k), kf(om.kc[47][:om.past])) <= 2e-3
                    assert O.rel_l2(kf(v), kf(om.vc[47][:om.past])) <= 2e-3
            excluded = len(prompt) - sum(within)
            print("full size: seed %d: %d of %d prompt rows within 1e-3 (%d excluded behind a router gap below %.0e), %d greedy steps compared"
                  % (seed, sum(within), len(prompt), excluded, GAP, compared), flush=True)
            assert excluded <= 2
            if compared >= 2:
                greedy_done = True
                break
        assert greedy_done, "no prompt of five left the greedy steps comparable"
        _full_size_speculative_round(m, cfg, tensors, prompt)
    finally:
        m.close()


def _full_size_speculative_round(m, cfg, tensors, prompt):
    """BASELINE config 5's second run at full size (llm/spec.go:703-857; llm/graph_spec_test.go): one-layer
    draft head, depth 2, three-row rewindable verification passes.  The loop's tokens are plain
    greedy decoding's (a token may differ only where plain decoding's own two best logits lie
    closer than the two pass shapes' rounding), and the verified rows' logits are the CPU's."""
    depth, n_new = 2, 10
    m.speculate(False)
    m.reset()
    m.extend(prompt)
    plain = [int(t) for t in m.generate(n_new + depth + 1)[0]]
    # the verification pass itself against the CPU: the pending token and two drafts as three
    # rewindable rows, every row's logits.  A row at or behind a router near-tie of the oracle's own
    # (in the pass or in what was fed before it, as in the prompt pass above) may hold another
    # expert's output and says nothing; the pass is then taken one token further on, and one of
    # four such passes must agree in every row.
    GAP = 4e-4
    om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv)
    gamma = tensors["output_norm.weight"]
    clean = False
    for start in range(4):
        before = np.concatenate([prompt, np.array(plain[:start], np.int32)])
        rows = np.array(plain[start:start + depth + 1], np.int32)
        om.reset()
        _, _, gaps_before = _oracle_rows_with_gaps(om, tensors, cfg, before)
        x_cpu, _, gaps = _oracle_rows_with_gaps(om, tensors, cfg, rows)
        lg_cpu = [O.gemv_q4k(tensors["output.weight"], O.rmsnorm(x_cpu[t:t + 1], gamma, cfg.rms_eps)[0], cfg.vocab, cfg.n_embd, threads=16)
                  for t in range(depth + 1)]
        m.speculate(False)
        m.reset()
        m.extend(before)
        m.speculate(True)
        _, lg_rows, _ = m.extend_rows(rows, want_logits=True, want_res=True)
        m.rewind()
        errs = [O.rel_l2(lg_rows[t], lg_cpu[t]) for t in range(depth + 1)]
        print("full size: verification pass after %d tokens: rows' logits rel-L2" % start, ["%.2e" % e for e in errs],
              "gaps", ["%.1e" % g for g in gaps], flush=True)
        so_far = np.minimum.accumulate(np.concatenate([gaps_before, gaps]))[-(depth + 1):]
        assert all(e <= 1e-3 or g < GAP for e, g in zip(errs, so_far)), (errs, list(so_far))
        if max(errs) <= 1e-3:
            clean = True
            break
    assert clean, "every verification pass of four sat behind a router near-tie"
    m.speculate(False)
    # the loop: true continuations as drafts in even rounds, the draft head's own in odd ones
    m.reset()
    m.mtp_stage(max_tok=depth + 1)
    m.spec_open(depth)
    out = [m.spec_start(prompt)]
    rounds = 0
    while len(out) < n_new:
        forced = plain[len(out):len(out) + depth] if rounds % 2 == 0 else []
        out += [int(t) for t in m.spec_round(forced)]
        rounds += 1
    st = m.spec_stats()
    print("full size: speculative loop %d rounds, %d tokens, accepted %s" % (rounds, len(out), st["accepted_at"][:depth]), flush=True)
    same = [a == b for a, b in zip(out[:n_new], plain[:n_new])]
    if not all(same):
        i = same.index(False)
        # plain decoding's own margin at the first token that differs
        m.speculate(False)
        m.reset()
        lg, _ = m.extend(np.concatenate([prompt, np.array(plain[:i], np.int32)]))
        top2 = np.sort(lg)[-2:]
        assert float(top2[1] - top2[0]) < 1e-3 * float(np.abs(lg).max()), (i, out[:n_new], plain[:n_new])
        print("full size: token %d differs at a margin of %.2e" % (i, float(top2[1] - top2[0])), flush=True)
