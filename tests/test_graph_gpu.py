"""The whole token loop on the GPU (llm::Graph: recorded decode step, device-side greedy loop)
against the CPU oracle's loop on a reduced model with the same weights.  The reference's gates of
this kind are TestGraphIsAChunkSplit (llm/graph_cache_test.go:39), TestPrerecordedDecodeIsThe
RecordedDecode and the greedy-text acceptance of cmd/llm/generate.go:11-13."""
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
    for k in ("embed", "dn.qkv", "dn.step", "dn.out", "attn.qkv", "attn.attn", "attn.out", "moe.router",
              "moe.up", "moe.down", "head", "argmax", "total"):
        assert k in st and st[k] > 0, k
    assert m.dispatches() == 1 + 4 * 6 + 2
