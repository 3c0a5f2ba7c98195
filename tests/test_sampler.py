"""The host sampler (host/sample.hpp) held to the properties the reference's own tests hold its
sampler to (llm/sample_test.go): first-maximum arg-max, top-n and the one-pass top-k against a
stable sort, temperature zero is greedy, top-k is a wall, the empirical distribution is the
softmax, penalties and their window, min-p, speculative sampling's Verify leaves the distribution
unchanged and keeps the draft with probability sum(min(p, q)), Verify without a draft distribution
is Sample draw for draw.  Random streams are this library's own, not Go's: every check here is a
property of the arithmetic, none of a particular stream."""
import numpy as np
import pytest

import shv

S = shv.pkg.sample_api


def test_argmax_keeps_the_first_of_equal_maxima():
    """llm/sample_test.go:17-39"""
    rng = np.random.default_rng(7)
    for _ in range(200):
        v = rng.integers(0, 20, size=1 + rng.integers(0, 500)).astype(np.float32)   # coarse, so ties happen
        assert S.argmax(v) == int(np.argmax(v))
    assert S.argmax(np.array([np.nan, 1.0, np.nan, 1.0], np.float32)) == 1           # NaN never wins a `>`
    assert S.argmax(np.full(5, -np.inf, np.float32)) == 0


def test_top_n_is_the_n_largest_in_order():
    """llm/sample_test.go:41-65"""
    rng = np.random.default_rng(11)
    for _ in range(300):
        v = rng.standard_normal(1 + rng.integers(0, 300)).astype(np.float32)
        k = 1 + int(rng.integers(0, len(v)))
        got = S.top_n(v, k)
        assert len(got) == k
        assert np.array_equal(v[got], np.sort(v)[::-1][:k])
    assert len(S.top_n(np.zeros(3, np.float32), 10)) == 3


def test_top_k_of_is_the_stable_sort():
    """llm/sample_test.go:180-213: same ids in the same order as sorting the whole row, ties to the lower id."""
    rng = np.random.default_rng(3)
    for trial in range(40):
        n = 1000 + int(rng.integers(0, 5000))
        row = rng.standard_normal(n).astype(np.float32)
        if trial % 2 == 1:
            row = rng.integers(0, 50, size=n).astype(np.float32)   # ties everywhere
        order = np.argsort(-row, kind="stable")
        for k in (1, 20, 40, 256):
            assert np.array_equal(S.top_k_of(row, k), order[:k]), (trial, k)


def test_temperature_zero_is_greedy():
    """llm/sample_test.go:67-86"""
    v = np.random.default_rng(13).standard_normal(1000).astype(np.float32)
    for s in (S.Sampler(0, 0, 0, 1), S.Sampler(0, 40, 0.9, 2)):
        assert s.greedy() and s.sample(v) == S.argmax(v)
        assert s.draft_sampler(1) is None


def test_top_k_is_a_wall():
    """llm/sample_test.go:88-109"""
    v = np.random.default_rng(17).standard_normal(500).astype(np.float32)
    allowed = set(S.top_n(v, 5).tolist())
    counts = S.Sampler(1.0, 5, 0, 3).sample_many(v, 2000)
    assert set(np.nonzero(counts)[0].tolist()) <= allowed and counts.sum() == 2000
    assert len(np.nonzero(counts)[0]) == 5


def test_distribution_is_the_softmax():
    """llm/sample_test.go:111-137, tightened to four standard errors over 200 000 draws."""
    v = np.array([2, 1, 0, -1, 0.5, 1.5, -2, 0.25], np.float32)
    want = np.exp(v.astype(np.float64))
    want /= want.sum()
    draws = 200000
    got = S.Sampler(1.0, 0, 0, 5).sample_many(v, draws) / draws
    assert (np.abs(got - want) <= 4 * np.sqrt(want * (1 - want) / draws) + 1e-4).all()
    ids, p = S.Sampler(1.0, 0, 0, 5).dist(v)
    assert np.array_equal(ids, np.argsort(-v, kind="stable")) and np.allclose(p, want[ids], rtol=1e-6)
    # temperature sharpens: p_i proportional to exp(v_i / T)
    ids, p = S.Sampler(0.5, 0, 0, 5).dist(v)
    w2 = np.exp(2 * v.astype(np.float64))
    assert np.allclose(p, (w2 / w2.sum())[ids], rtol=1e-5)


def test_top_p_keeps_the_smallest_prefix_that_reaches_p():
    v = np.log(np.array([0.5, 0.25, 0.15, 0.1], np.float32))
    ids, p = S.Sampler(1.0, 0, 0.7, 1).dist(v)
    assert ids.tolist() == [0, 1] and np.allclose(p, [2 / 3, 1 / 3], rtol=1e-5)
    ids, p = S.Sampler(1.0, 0, 0.75, 1).dist(v)       # 0.75 is reached exactly at the second id
    assert ids.tolist() == [0, 1]
    ids, p = S.Sampler(1.0, 0, 0.76, 1).dist(v)
    assert ids.tolist() == [0, 1, 2] and abs(p.sum() - 1) < 1e-6
    assert len(S.Sampler(1.0, 0, 1.0, 1).dist(v)[0]) == 4      # one and zero are off
    assert len(S.Sampler(1.0, 3, 0.0, 1).dist(v)[0]) == 3


def test_penalties_and_their_window():
    """llm/sample_test.go:139-164"""
    v = np.array([0, 2.0, 1.5, -1], np.float32)
    s = S.Sampler(0, 0, 0, 1, presence_penalty=1)
    s.accept(1)
    assert s.sample(v) == 2                     # 2.0 - 1 < 1.5
    assert v[1] == 2.0                          # the row comes back untouched
    s.accept(*([3] * 64))
    assert s.sample(v) == 1                     # token 1 has slid out of the window
    r = S.Sampler(0, 0, 0, 1, repeat_penalty=2)
    r.accept(1)
    assert r.sample(v) == 2                     # 2.0 / 2 = 1.0 < 1.5
    n = S.Sampler(0, 0, 0, 1, repeat_penalty=2)
    n.accept(3, 3, 9, -1)                       # a negative logit is multiplied, ids off the row ignored, once per id
    w = np.array([0, -0.1, -0.3, -0.12], np.float32)
    assert n.sample(w) == 0 and w[3] == np.float32(-0.12)
    plain = S.Sampler(0, 0, 0, 1)
    plain.accept(1)                             # no penalty configured: nothing is recorded, nothing applied
    assert plain.sample(v) == 1


def test_min_p():
    """llm/sample_test.go:166-178"""
    v = np.array([0, 0, 3], np.float32)          # probabilities ~0.045, 0.045, 0.91
    counts = S.Sampler(1, 0, 0, 5, min_p=0.1).sample_many(v, 500)
    assert counts.tolist() == [0, 0, 500]
    ids, p = S.Sampler(1, 0, 0, 5, min_p=0.04).dist(v)
    assert len(ids) == 3 and abs(p.sum() - 1) < 1e-6


@pytest.mark.parametrize("n,top_k,top_p,temp", [(400, 20, 0.95, 1.0), (200, 0, 0.0, 0.7)])
def test_verify_is_the_distribution(n, top_k, top_p, temp):
    """llm/sample_test.go:229-301: under top-k/top-p cuts and with none (the map path past 64 ids),
    with a draft whose support differs."""
    r = np.random.default_rng(3)
    pl = (r.standard_normal(n) * 2).astype(np.float32)
    ql = (pl + r.standard_normal(n) * 0.8).astype(np.float32)     # the draft: the trunk's row, noised
    s = S.Sampler(temp, top_k, top_p, 7)
    ds = s.draft_sampler(9)
    p_ids, p_p = s.dist(pl)
    ds.propose(ql)
    q_ids, q_p = ds.last_dist()
    q_of = dict(zip(q_ids.tolist(), q_p.tolist()))
    keep = sum(min(float(pp), q_of.get(int(i), 0.0)) for i, pp in zip(p_ids, p_p))
    draws = 200000
    counts, kept = s.speculate_many(ds, pl, ql, draws)
    assert counts.sum() == draws
    assert set(np.nonzero(counts)[0].tolist()) <= set(p_ids.tolist())      # nothing the cuts remove
    want = np.zeros(n)
    want[p_ids] = p_p
    got = counts / draws
    assert (np.abs(got - want) <= 4 * np.sqrt(want * (1 - want) / draws) + 1e-4).all()
    assert abs(kept / draws - keep) <= 0.01
    p_of = dict(zip(p_ids.tolist(), p_p.tolist()))
    print("kept %.3f (sum min(p,q) %.3f) against an argmax draft's %.3f" % (kept / draws, keep, p_of.get(int(q_ids[0]), 0.0)))


def test_verify_without_a_draft_distribution_is_sample():
    """llm/sample_test.go:303-315"""
    r = np.random.default_rng(4)
    a, b = S.Sampler(1, 20, 0.95, 11), S.Sampler(1, 20, 0.95, 11)
    for _ in range(500):
        row = (r.standard_normal(1000) * 3).astype(np.float32)
        assert a.sample(row) == b.verify(row, 5, None)


def test_verify_of_a_token_outside_the_draft_distribution_is_a_plain_draw():
    """llm/sample.go:196-199: q(draft) = 0 means there is no proposal to weigh."""
    r = np.random.default_rng(5)
    pl = r.standard_normal(50).astype(np.float32)
    s, ds = S.Sampler(1, 5, 0, 1), S.Sampler(1, 5, 0, 2)
    ds.propose(pl)
    q_ids, _ = ds.last_dist()
    outside = next(i for i in range(50) if i not in set(q_ids.tolist()))
    allowed = set(s.dist(pl)[0].tolist())
    for _ in range(200):
        assert s.verify(pl, outside, ds) in allowed


def test_empty_rows_and_counts_are_answered_not_read():
    empty = np.zeros(0, np.float32)
    s = S.Sampler(1, 5, 0.9, 1)
    assert s.sample(empty) == -1 and s.propose(empty) == -1 and s.verify(empty, 3, None) == -1
    assert len(s.dist(empty)[0]) == 0
    v = np.arange(5, dtype=np.float32)
    assert len(S.top_n(v, 0)) == 0 and len(S.top_k_of(v, 0)) == 0


def test_seeds_name_streams():
    v = np.random.default_rng(1).standard_normal(100).astype(np.float32)
    a = [S.Sampler(1, 0, 0, 42).sample(v) for _ in range(1)]
    s1, s2, s3 = S.Sampler(1, 0, 0, 42), S.Sampler(1, 0, 0, 42), S.Sampler(1, 0, 0, 43)
    x1, x2, x3 = ([s.sample(v) for _ in range(64)] for s in (s1, s2, s3))
    assert x1 == x2 and x1 != x3 and a[0] == x1[0]
