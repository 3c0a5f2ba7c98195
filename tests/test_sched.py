"""The scheduler's policy without a device (backend/llm_sched.go:201-898).

The scheduler object is opened with no graph: next() says which pass the policy would run and
finish() books a device time the test names, so every rule is checked on a clock the test owns.
Each case is built so that the rule it names decides the outcome: drop the rule and the order,
the slot or the chunk length changes.  The reference holds no unit test of the policy alone (its
backend/llm_sched_test.go runs whole conversations on a served model); the expectations below
are read off the rules in its file comment (:13-59) and the code they cite.
"""
import numpy as np
import pytest

import shv
from shv import pkg

api = pkg.llm_api
I, B = api.INTERACTIVE, api.BACKGROUND
NONE, CHUNK, STEPS = 0, 1, 2


@pytest.fixture
def sched():
    made = []

    def make(**kw):
        s = api.Sched(None, **kw)
        made.append(s)
        return s

    yield make
    for s in made:
        s.close()


def ids(n, base=0):
    return np.arange(base, base + n, dtype=np.int32)


def prefill(s, job, prompt, ms=1.0):
    """Queues the job's prompt past what its slot saves and runs chunks until it is through; returns the chunk plans."""
    j = s.job(job)
    u = s.run(job, prompt[j.reused:], j.reused == 0)
    plans = []
    while s.unit(u)[0] == 0:
        p = s.next()
        assert p.kind == CHUNK and p.unit == u
        plans.append((p.pos, p.n, bool(p.fresh), bool(p.restore), bool(p.take)))
        s.finish(ms)
    return plans


def test_interactive_goes_first_and_keeps_the_device_between_its_units(sched):
    # backend/llm_sched.go:15-19 (rule 1), :873-898
    s = sched(slots=3, reserve=0, preempt_chunk=64)
    a, b = s.acquire(B, ids(8)), s.acquire(B, ids(8, 100))
    prefill(s, a, ids(8)), prefill(s, b, ids(8, 100))
    ua, ub = s.step(a, 1), s.step(b, 2)
    v = s.acquire(I, ids(40, 500))
    assert s.job(v).slot == 2
    uv = s.run(v, ids(40, 500), True)
    p = s.next()
    assert (p.kind, p.unit, p.n) == (CHUNK, uv, 40), "the interactive prefill runs before two older background steps"
    s.finish(5.0)
    # the interactive request is sampling: nothing of its own is queued, and still no background unit starts
    p = s.next(now_ms=100.0)
    assert p.kind == NONE and p.wait_ms <= 0
    assert s.counts()["pending"] == 2
    us = s.step(v, 7)
    p = s.next(now_ms=100.0)
    assert (p.kind, p.unit, bool(p.step)) == (CHUNK, us, True), "a background row does not ride in an interactive pass"
    s.finish(1.0, now_ms=101.0)
    s.release(v, now_ms=101.0)
    p = s.next(now_ms=200.0)
    assert p.kind == STEPS and sorted(p.units[:p.n_units]) == sorted([ua, ub])
    s.finish(2.0, now_ms=202.0)
    assert s.unit(ua)[0] == 1 and s.unit(ub)[0] == 1


def test_without_the_class_the_same_arrival_shares_the_device(sched):
    # the control of backend/llm_sched_test.go:147-162: a third background request does not hold the others back
    s = sched(slots=3, reserve=0)
    a, b = s.acquire(B, ids(8)), s.acquire(B, ids(8, 100))
    prefill(s, a, ids(8)), prefill(s, b, ids(8, 100))
    s.step(a, 1), s.step(b, 2)
    v = s.acquire(B, ids(4, 500))
    assert s.job(v).served_ms == pytest.approx(1.0), "a newcomer starts level with the least served of its class"
    s.run(v, ids(4, 500), True)
    kinds = []
    for _ in range(2):
        p = s.next(now_ms=1000.0)
        kinds.append(p.kind)
        s.finish(1.0, now_ms=1000.0)
    assert sorted(kinds) == [CHUNK, STEPS]


def test_least_device_time_first_then_the_oldest(sched):
    # backend/llm_sched.go:20-22 (rule 2), :887-888
    s = sched(slots=2, reserve=0, preempt_chunk=64, no_batch_decode=True)
    a, b = s.acquire(B, ids(256)), s.acquire(B, ids(4, 1000))
    ua = s.run(a, ids(256), True)
    ub = s.run(b, ids(4, 1000), True)
    p = s.next()
    assert p.unit == ua, "equal device time: the older arrival"
    s.finish(10.0)  # a now has 10 ms, b none
    p = s.next()
    assert p.unit == ub
    s.finish(1.0)
    order = []
    tok = 0
    while s.unit(ua)[0] == 0:
        if s.counts()["pending"] < 2:
            s.step(b, tok)
            tok += 1
        p = s.next()
        order.append("a" if p.unit == ua else "b")
        s.finish(10.0 if p.unit == ua else 1.0)
    # b decodes at 1 ms a step until it has had as much as a, then a's next 10 ms chunk, and so on:
    # counting units instead of time would alternate a b a b
    assert "".join(order).startswith("bbbbbbbbbabbbbbbbbbba"), "".join(order)
    assert s.job(a).served_ms == pytest.approx(40.0)


def test_a_background_prefill_runs_in_preempt_chunks_cut_at_the_mark(sched):
    # backend/llm_sched.go:23-27 (rule 3), :557-576, :589
    s = sched(slots=2, reserve=0, batch=128, preempt_chunk=64)
    a = s.acquire(B, ids(300), mark=100)
    plans = prefill(s, a, ids(300))
    assert [(pos, n) for pos, n, *_ in plans] == [(0, 64), (64, 36), (100, 64), (164, 64), (228, 64), (292, 8)]
    assert [take for *_, take in plans] == [False, True, False, False, False, False]
    assert plans[0][2] and not any(p[2] for p in plans[1:]), "only the first chunk starts the sequence over"
    held, ck = s.held(0)
    assert len(held) == 300 and ck == 100
    # the interactive class is cut only by the batch and the mark
    v = s.acquire(I, ids(300, 5000), mark=100)
    plans = prefill(s, v, ids(300, 5000))
    assert [(pos, n, take) for pos, n, _, _, take in plans] == [(0, 100, True), (100, 128, False), (228, 72, False)]


def test_slots_are_reserved_for_the_interactive_class(sched):
    # backend/llm_sched.go:29-31, :325-340; waiters: interactive first, then the oldest (:309-319)
    s = sched(slots=3, reserve=1)
    a, b, c = (s.acquire(B, ids(4, 10 * k)) for k in range(3))
    assert [s.job(x).slot for x in (a, b, c)] == [0, 1, -1], "two background requests may not take the third slot"
    assert s.counts()["waiting"] == 1
    v = s.acquire(I, ids(4, 900))
    assert s.job(v).slot == 2
    w = s.acquire(I, ids(4, 950))
    assert s.job(w).slot == -1
    s.release(a, now_ms=1.0)
    assert s.job(w).slot == 0 and s.job(c).slot == -1, "the interactive waiter takes the freed slot before the older background one"
    s.release(v, now_ms=2.0)
    # b is the only background holder now, so c may have the free slot
    assert s.job(c).slot == 2
    # with no more slots than the reserve the rule is off, or background would never run
    one = sched(slots=1, reserve=1)
    assert one.job(one.acquire(B, ids(4))).slot == 0


def test_a_later_waiter_never_overtakes_the_best_one(sched):
    # grant stops at the first waiter it cannot serve (backend/llm_sched.go:294-307)
    s = sched(slots=2, reserve=1)
    a = s.acquire(B, ids(4))
    v = s.acquire(I, ids(4, 50))
    w = s.acquire(I, ids(4, 60))   # waits: no slot
    c = s.acquire(B, ids(4, 70))   # waits behind it
    assert [s.job(x).slot for x in (a, v, w, c)] == [0, 1, -1, -1]
    s.release(a, now_ms=1.0)
    assert s.job(w).slot == 0 and s.job(c).slot == -1


def test_the_slot_that_saves_the_most_of_the_prompt(sched):
    # backend/llm_sched.go:127-138, :341-352, :374-383
    s = sched(slots=3, reserve=0)
    sys_a, sys_b = ids(50, 1000), ids(50, 2000)
    turn1 = np.concatenate([sys_a, ids(10, 3000)])
    other = np.concatenate([sys_b, ids(10, 4000)])
    a = s.acquire(B, turn1, mark=50)
    b = s.acquire(B, other, mark=50)
    assert (s.job(a).slot, s.job(b).slot) == (0, 1)
    prefill(s, a, turn1), prefill(s, b, other)
    for t in (7, 8, 9):  # the generated tokens are part of what the slot holds
        s.step(a, 6000 + t)
        assert s.next().kind == CHUNK
        s.finish(1.0)
    s.release(b, now_ms=1.0)
    s.release(a, now_ms=2.0)  # slot 0 is the most recently used, slot 2 never
    held0 = s.held(0)[0]
    assert len(held0) == 63
    # the conversation's next turn continues what slot 0 holds, although slot 2 is the oldest
    turn2 = np.concatenate([held0, ids(5, 7000)])
    j = s.acquire(B, turn2, mark=50)
    info = s.job(j)
    assert (info.slot, info.reused, info.restored) == (0, 63, 0)
    plans = prefill(s, j, turn2)
    assert plans == [(63, 5, False, False, False)]
    s.release(j, now_ms=3.0)
    # a prompt that IS what the slot holds cannot continue it, because the logits of a finished pass
    # are not kept: what it saves is the checkpoint below
    j = s.acquire(B, s.held(0)[0])
    assert (s.job(j).reused, s.job(j).restored) == (50, 1)
    s.release(j, now_ms=3.5)
    # another command on the same system prompt: the held turn does not match, the checkpoint does
    cmd = np.concatenate([sys_a, ids(7, 8000)])
    j = s.acquire(I, cmd, mark=50)
    info = s.job(j)
    assert (info.slot, info.reused, info.restored) == (0, 50, 1)
    plans = prefill(s, j, cmd)
    assert plans == [(50, 7, False, True, False)]
    assert s.counts()["restores"] == 1
    assert np.array_equal(s.held(0)[0], cmd) and s.held(0)[1] == 50
    s.release(j, now_ms=4.0)
    # nothing saved anywhere: the slot with less checkpointed goes first (slot 2 has none), not the least recently used
    j = s.acquire(B, ids(6, 9000))
    assert s.job(j).slot == 2
    # and between two equally checkpointed slots the least recently used: slot 1 (released at 1) before slot 0 (at 4)
    k = s.acquire(B, ids(6, 9100))
    assert s.job(k).slot == 1


def test_a_checkpoint_counts_only_while_the_slot_still_holds_its_tokens(sched):
    # backend/llm_sched.go:110-113, :133
    s = sched(slots=1, reserve=0)
    sysp = ids(20, 100)
    first = np.concatenate([sysp, ids(4, 500)])
    a = s.acquire(I, first, mark=20)
    prefill(s, a, first)
    s.release(a)
    assert s.held(0)[1] == 20
    # an unrelated request starts the slot over without a mark: the old checkpoint's cells are gone
    b = s.acquire(I, ids(30, 9000))
    prefill(s, b, ids(30, 9000))
    s.release(b)
    c = s.acquire(I, np.concatenate([sysp, ids(3, 600)]), mark=20)
    assert (s.job(c).reused, s.job(c).restored) == (0, 0)
    s.release(c)
    # with no checkpoint to fall back on, a prompt that is exactly what the slot holds saves nothing,
    # and one token more saves all of it
    assert s.job(s.acquire(I, ids(30, 9000))).reused == 0
    two = sched(slots=1, reserve=0)
    prefill(two, two.acquire(I, ids(30, 9000)), ids(30, 9000))
    two.release(1)
    assert two.job(two.acquire(I, ids(31, 9000))).reused == 30


def test_pending_decode_steps_of_one_class_share_a_pass(sched):
    # backend/llm_sched.go:33-41, :757-789, :845-870
    s = sched(slots=3, reserve=0, coalesce_ms=5.0)
    jobs = [s.acquire(B, ids(4, 10 * k)) for k in range(3)]
    for k, j in enumerate(jobs):
        prefill(s, j, ids(4, 10 * k))
    served0 = [s.job(j).served_ms for j in jobs]
    us = [s.step(j, 40 + k) for k, j in enumerate(jobs)]
    p = s.next(now_ms=10.0)
    assert p.kind == STEPS and p.n_units == 3
    assert sorted(p.slots[:3]) == [0, 1, 2]
    s.finish(3.0, now_ms=13.0)
    for k, j in enumerate(jobs):
        assert s.job(j).served_ms - served0[k] == pytest.approx(1.0), "each row a share of the pass"
        assert s.unit(us[k])[2] == pytest.approx(3.0), "and its whole latency"
        assert s.held(s.job(j).slot)[0][-1] == 40 + k
    assert (s.counts()["batches"], s.counts()["batch_rows"]) == (1, 3)
    # two of the three have sampled and are back; the batch waits for the third until 5 ms after the last step
    s.step(jobs[0], 50), s.step(jobs[1], 51)
    p = s.next(now_ms=14.0)
    assert p.kind == NONE and p.wait_ms == pytest.approx(4.0)
    u3 = s.step(jobs[2], 52)
    p = s.next(now_ms=14.5)
    assert p.kind == STEPS and p.n_units == 3 and u3 in p.units[:3]
    s.finish(3.0, now_ms=17.5)
    s.step(jobs[0], 60), s.step(jobs[1], 61)
    p = s.next(now_ms=22.5)
    assert p.kind == STEPS and p.n_units == 2, "past the wait the two run without the third"
    s.finish(2.0, now_ms=24.5)
    # a request that is still prefilling is no peer: its class's lone step does not wait for it
    s.release(jobs[2], now_ms=25.0)
    late = s.acquire(B, ids(200, 7000))
    s.run(late, ids(200, 7000), True)
    s.release(jobs[1], now_ms=25.0)
    u = s.step(jobs[0], 70)
    seen = []
    while s.unit(u)[0] == 0:
        p = s.next(now_ms=25.0)
        assert p.kind == CHUNK and p.wait_ms <= 0
        seen.append(p.unit)
        s.finish(1.0, now_ms=25.0)
    assert u in seen


def test_no_batch_decode_runs_every_step_alone(sched):
    s = sched(slots=2, reserve=0, no_batch_decode=True)
    a, b = s.acquire(B, ids(4)), s.acquire(B, ids(4, 100))
    prefill(s, a, ids(4)), prefill(s, b, ids(4, 100))
    s.step(a, 1), s.step(b, 2)
    for _ in range(2):
        p = s.next()
        assert p.kind == CHUNK and p.step and p.n == 1
        s.finish(1.0)
    assert s.counts()["batches"] == 0


def test_a_failed_pass_forgets_what_the_slot_held(sched):
    # backend/llm_sched.go:714-717, :853-855
    s = sched(slots=2, reserve=0)
    a = s.acquire(B, ids(40), mark=10)
    prefill(s, a, ids(40))
    assert s.held(0)[1] == 10
    u = s.step(a, 3)
    assert s.next().kind == CHUNK
    s.finish(1.0, ok=False)
    assert s.unit(u)[0] == 2
    held, ck = s.held(0)
    assert len(held) == 0 and ck == 0
    s.release(a)
    j = s.acquire(B, np.concatenate([ids(40), ids(3, 900)]))
    assert s.job(j).reused == 0


def test_release_and_withdraw_take_queued_units_out(sched):
    # backend/llm_sched.go:483-495
    s = sched(slots=2, reserve=0)
    a, b = s.acquire(B, ids(4)), s.acquire(B, ids(4, 100))
    ua = s.run(a, ids(4), True)
    ub = s.run(b, ids(4, 100), True)
    s.withdraw(ua)
    assert s.unit(ua)[0] == 2
    p = s.next()
    assert p.unit == ub
    with pytest.raises(shv.pkg.hip_api.ShvError):
        s.release(b)  # its unit is on the device
    with pytest.raises(shv.pkg.hip_api.ShvError):
        s.next()  # one pass at a time
    s.finish(1.0)
    s.release(b)
    s.release(a)
    assert s.counts()["pending"] == 0 and s.next().kind == NONE


def test_bad_arguments_are_refused(sched):
    s = sched(slots=2)
    with pytest.raises(shv.pkg.hip_api.ShvError):
        s.acquire(5, ids(4))
    with pytest.raises(shv.pkg.hip_api.ShvError):
        s.acquire(B, ids(4), mark=9)
    with pytest.raises(shv.pkg.hip_api.ShvError):
        s.pump()  # no graph
    with pytest.raises(shv.pkg.hip_api.ShvError):
        s.finish(1.0)  # no pass is out
    with pytest.raises(shv.pkg.hip_api.ShvError):
        api.Sched(None, slots=0)


ROUND = 3


def test_a_decode_runs_as_a_round_only_while_its_draft_is_caught_up_and_it_decodes_alone(sched):
    # backend/llm_sched.go:936-953: asked to, draft caught up, room for two tokens, no other conversation of its class decoding
    s = sched(slots=2, reserve=0, spec_depth=2)
    a = s.acquire(I, ids(8))
    p = prefill_plans = None
    u = s.run(a, ids(8), True)
    p = s.next()
    assert p.kind == CHUNK and p.prime and not p.tracked   # a fresh text chunk primes the slot's draft
    s.finish(1.0)
    assert s.tracked(0)
    # a plain step() never speculates; a decode() with room for one token does not either
    u1 = s.step(a, 1)
    p = s.next()
    assert p.kind == CHUNK and p.step and p.tracked and not p.prime   # owed to the draft, which stays caught up
    s.finish(1.0)
    assert s.tracked(0)
    u2 = s.decode(a, 2, room=1)
    assert s.next().kind == CHUNK
    s.finish(1.0)
    # room for two: a round; it keeps its input and all but the last token it drew
    u3 = s.decode(a, 3, room=8)
    p = s.next()
    assert p.kind == ROUND and p.unit == u3 and p.slot == 0 and p.pos == 10
    s.finish_round(2.0, [40, 41, 42])
    assert s.unit(u3)[0] == 1 and s.unit_tokens(u3).tolist() == [40, 41, 42]
    assert s.held(0)[0].tolist() == list(range(8)) + [1, 2, 3, 40, 41]
    assert s.round_counts() == dict(rounds=1, round_tokens=3)
    # a second conversation of the class starts decoding: both go as plain rows of one pass instead
    b = s.acquire(I, ids(8, 100))
    prefill(s, b, ids(8, 100))
    ub, ua = s.decode(b, 7, room=8), s.decode(a, 42, room=8)
    p = s.next()
    assert p.kind == STEPS and p.n_units == 2
    s.finish(1.0)
    assert s.unit_tokens(ua).size == 0 and s.tracked(0) and s.tracked(1)
    # alone again once the other is released
    s.release(b)
    ua = s.decode(a, 50, room=8)
    assert s.next().kind == ROUND
    s.finish_round(2.0, [60])
    assert s.held(0)[0].tolist()[-2:] == [42, 50]


def test_a_failed_round_costs_the_slot_its_sequence(sched):
    s = sched(slots=1, reserve=0, spec_depth=1)
    a = s.acquire(I, ids(8))
    prefill(s, a, ids(8))
    u = s.decode(a, 1, room=4)
    assert s.next().kind == ROUND
    s.finish_round(1.0, [], ok=False)
    assert s.unit(u)[0] == 2 and s.held(0)[0].size == 0 and not s.tracked(0)


def test_a_checkpoint_keeps_the_draft_only_when_a_priming_chunk_took_it(sched):
    # backend/llm_sched.go:625-637,696-703: a restore keeps the draft's cells below the mark when the checkpoint holds the
    # residual to resume from, which a chunk that primed the draft leaves; otherwise the draft is behind for good
    s = sched(slots=1, reserve=0, spec_depth=2)
    sysp = ids(50)
    a = s.acquire(I, np.concatenate([sysp, ids(10, 100)]), mark=50)
    plans = prefill(s, a, np.concatenate([sysp, ids(10, 100)]))
    assert plans[0][:2] == (0, 50) and plans[0][4]
    assert s.tracked(0)
    s.release(a)
    b = s.acquire(I, np.concatenate([sysp, ids(12, 200)]), mark=50)
    assert s.job(b).restored and s.job(b).reused == 50
    u = s.run(b, ids(12, 200), False)
    p = s.next()
    assert p.kind == CHUNK and p.restore and p.tracked and p.prime
    s.finish(1.0)
    assert s.tracked(0)
    s.release(b)
    # without a draft (spec_depth 0) nothing primes and no decode is a round
    t = sched(slots=1, reserve=0)
    c = t.acquire(I, ids(8))
    prefill(t, c, ids(8))
    assert not t.tracked(0)
    t.decode(c, 1, room=8)
    assert t.next().kind == CHUNK
