"""The scheduler's decisions on the CPU, and the engine above the torch stand-in kernels."""
import random

import pytest
import torch

from return_amd.cache import CacheManager, KVCapacityError, PagedKVSpec
from return_amd.engine.scheduler import Request, Scheduler
from return_amd.sampling import SamplingParams, UniformStream, ends_with_stop


def make(page=4, max_token=64, max_reside=4, budget=16, chunk=8, max_position=1000, window=None):
    layers = {0: PagedKVSpec(1, 8)}
    if window:
        layers[1] = PagedKVSpec(1, 8, window)
    cm = CacheManager(layers, page, max_token, max_reside, torch.float32, "cpu")
    return cm, Scheduler(cm, max_reside, budget, chunk, max_position)


def drive(cm, sched, pick=lambda r: 7, max_steps=10000):
    """Run to the end with a fake model: every sampled token is pick(request). Returns the step log."""
    log = []
    for _ in range(max_steps):
        if not sched.has_work():
            return log
        plan = sched.schedule()
        assert plan.entries or plan.failed, "scheduler idles with work left"
        if plan.entries:
            cm.begin_step([(e.request.id, len(e.tokens)) for e in plan.entries])
            cm.end_step()
            cm.check_invariants()
        log.append([(e.request.id, len(e.tokens), e.sample) for e in plan.entries])
        sched.finish_step(plan, {e.request.id: (pick(e.request), -1.0) for e in plan.entries if e.sample})
    raise AssertionError("did not finish")


def test_prompt_is_cut_under_the_budget_and_decodes_come_first():
    cm, s = make(budget=10, chunk=6)
    a = Request("a", list(range(20)), SamplingParams(max_new_tokens=3))
    b = Request("b", list(range(3)), SamplingParams(max_new_tokens=4))
    s.add(a); s.add(b)
    log = drive(cm, s)
    assert log[0] == [("a", 6, False), ("b", 3, True)]                 # chunk 6, then b's whole prompt
    assert log[1] == [("b", 1, True), ("a", 6, False)]                 # b decodes first, a goes on
    assert all(sum(n for _, n, _ in step) <= 10 for step in log)
    assert a.output == [7, 7, 7] and b.output == [7] * 4
    assert a.finish_reason == b.finish_reason == "length"
    assert a.num_computed == 20 + 2 and not cm.live                    # the last token is never fed


def test_portion_is_cut_to_what_the_budget_leaves():
    cm, s = make(budget=5, chunk=100, max_reside=2)
    s.add(Request("a", list(range(3)), SamplingParams(max_new_tokens=2)))
    s.add(Request("b", list(range(9)), SamplingParams(max_new_tokens=1)))
    log = drive(cm, s)
    assert log[0] == [("a", 3, True), ("b", 2, False)]
    assert log[1] == [("a", 1, True), ("b", 4, False)]
    assert log[2] == [("b", 3, True)]


def test_stop_sequences_and_length():
    assert ends_with_stop([1, 2, 3], [[2, 3]]) and not ends_with_stop([1, 2, 3], [[1, 2], []])
    cm, s = make()
    seq = iter([5, 9, 4, 1, 1])
    r = Request("r", [1, 2], SamplingParams(max_new_tokens=10, stop_ids=[[9, 4], [8]]))
    s.add(r)
    drive(cm, s, pick=lambda _: next(seq))
    assert r.output == [5, 9, 4] and r.finish_reason == "stop"         # rollout/engine.py:49-57


def test_requests_wait_when_pages_are_short_and_run_when_they_return():
    cm, s = make(page=4, max_token=32, max_reside=4, budget=64, chunk=64)      # 8 pages
    reqs = [Request(i, list(range(10)), SamplingParams(max_new_tokens=7)) for i in range(3)]   # 16 tokens = 4 pages each
    for r in reqs:
        s.add(r)
    log = drive(cm, s)
    assert [x[0] for x in log[0]] == [0, 1]                            # the third does not fit beside two
    first_seen = next(i for i, step in enumerate(log) if any(x[0] == 2 for x in step))
    done_01 = max(i for i, step in enumerate(log) if any(x[0] in (0, 1) for x in step))
    assert first_seen > done_01                                        # it ran only after pages came back
    assert all(len(r.output) == 7 for r in reqs) and not cm.live
    assert all(g.pages.in_use() == 0 for g in cm.groups)


def test_a_request_that_can_never_fit_fails_at_once_and_others_go_on():
    cm, s = make(page=4, max_token=32, max_reside=4)
    big = Request("big", list(range(30)), SamplingParams(max_new_tokens=8))       # 37 tokens > 32
    ok = Request("ok", list(range(5)), SamplingParams(max_new_tokens=2))
    s.add(big); s.add(ok)
    drive(cm, s)
    assert big.status == "failed" and isinstance(big.error, KVCapacityError) and big.finish_reason == "error"
    assert ok.output == [7, 7]


def test_position_limit():
    cm, s = make(max_position=12)
    long = Request("l", list(range(12)))
    r = Request("r", list(range(8)), SamplingParams(max_new_tokens=50))
    s.add(long); s.add(r)
    drive(cm, s)
    assert long.status == "failed" and "max_position" in str(long.error)
    assert len(r.output) == 5 and r.finish_reason == "length"          # 8 + 5 - 1 tokens reach position 11


def test_running_requests_never_run_out_of_pages():
    """Random workloads on a small pool: begin_step must never raise, every request ends."""
    for seed in range(5):
        rng = random.Random(seed)
        cm, s = make(page=4, max_token=80, max_reside=3, budget=12, chunk=5, window=6 if seed % 2 else None)
        reqs = [Request(i, [1] * rng.randint(1, 30), SamplingParams(max_new_tokens=rng.randint(1, 20)))
                for i in range(12)]
        for r in reqs:
            s.add(r)
        log = drive(cm, s)
        assert all(r.finish_reason == "length" and len(r.output) == r.params.max_new_tokens for r in reqs)
        assert max(len(step) for step in log) <= 3
        assert not cm.live


def test_budget_must_cover_the_decoding_requests():
    cm = CacheManager({0: PagedKVSpec(1, 8)}, 4, 64, 8, torch.float32, "cpu")
    with pytest.raises(ValueError, match="max_step_tokens"):
        Scheduler(cm, 8, 4, 4, 100)


def test_uniform_streams_do_not_depend_on_the_batch():
    a, b = UniformStream(3, 11), UniformStream(3, 11)
    xs = [a.next() for _ in range(5)]
    assert xs == [b.at(i) for i in range(5)] and all(0 <= x < 1 for x in xs)
    assert UniformStream(3, 12).at(0) != xs[0] and UniformStream(4, 11).at(0) != xs[0]
    assert abs(sum(UniformStream(0, 0).at(i) for i in range(4000)) / 4000 - 0.5) < 0.03


def test_sampling_params_checks():
    with pytest.raises(ValueError):
        SamplingParams(top_p=1.5)
    with pytest.raises(ValueError):
        SamplingParams(max_new_tokens=0)
    with pytest.raises(ValueError):
        Request("e", [])
    p = SamplingParams()                                               # the reference's defaults, rollout/engine.py:17-21
    assert (p.temperature, p.top_p, p.top_k, p.max_new_tokens, p.stop_ids) == (1.0, 1.0, 0, 32, [])


def test_kept_sessions_hold_pages_until_somebody_needs_them():
    """A kept session holds its pages and slot, resumes from them, and is given up for a waiting
    request only if that lets the request in; random turns never lose or double a page."""
    cm, s = make(page=4, max_token=48, max_reside=3, budget=32, chunk=32)      # twelve pages, three slots
    a = Request("a", list(range(10)), SamplingParams(max_new_tokens=3), keep=True)
    s.add(a)
    drive(cm, s)
    assert list(s.resident) == ["a"] and s.resident["a"] == list(range(10)) + [7, 7]
    assert cm.held_pages("a") == [3] and cm.free_pages() == [9]
    # a running request that has set aside most of the pool: the waiting one cannot get in even
    # without "a", so "a" stays
    b = Request("b", list(range(12)), SamplingParams(max_new_tokens=12))        # 23 tokens: six pages
    c = Request("c", list(range(20)), SamplingParams(max_new_tokens=9))         # 28 tokens: seven pages
    s.add(b); s.add(c)
    plan = s.schedule()
    assert [e.request.id for e in plan.entries] == ["b"] and list(s.resident) == ["a"] and c.status == "waiting"
    cm.begin_step([("b", 12)]); cm.end_step()
    s.finish_step(plan, {"b": (7, -1.0)})
    drive(cm, s)                                     # b ends, then c fits beside "a" (3 + 7 pages of 12)
    assert c.finish_reason == "length" and list(s.resident) == ["a"]
    # the next turn of "a": only the new tokens are planned
    a2 = Request("a", list(range(10)) + [7, 7, 7, 1, 2], SamplingParams(max_new_tokens=2), keep=True)
    s.add(a2)
    plan = s.schedule()
    assert [(e.request.id, e.tokens) for e in plan.entries] == [("a", [7, 1, 2])] and a2.resumed == 12
    cm.begin_step([("a", 3)]); cm.end_step()
    s.finish_step(plan, {"a": (9, -1.0)})
    drive(cm, s, pick=lambda r: 9)
    assert s.resident["a"] == list(range(10)) + [7, 7, 7, 1, 2, 9]
    # a request that needs the whole pool pushes "a" out
    d = Request("d", list(range(40)), SamplingParams(max_new_tokens=8))
    s.add(d)
    drive(cm, s)
    assert d.finish_reason == "length" and not s.resident and not cm.live
    # random turns of five sessions in three slots
    rnd = random.Random(3)
    convs = {k: [rnd.randrange(50) for _ in range(rnd.randint(1, 9))] for k in "vwxyz"}
    for _ in range(60):
        ks = rnd.sample(sorted(convs), rnd.randint(1, 4))
        reqs = [Request(k, convs[k], SamplingParams(max_new_tokens=rnd.randint(1, 4)), keep=rnd.random() < 0.7) for k in ks]
        for r in reqs:
            s.add(r)
        drive(cm, s, pick=lambda r: len(r.output) + 1)
        for r in reqs:
            assert r.finish_reason == "length" and r.resumed < len(r.prompt_ids)
            convs[r.id] = (r.prompt_ids + r.output + [rnd.randrange(50)])[-30:] if rnd.random() < 0.2 else \
                r.prompt_ids + r.output + [rnd.randrange(50)]
            if len(convs[r.id]) > 30:
                convs[r.id] = [rnd.randrange(50) for _ in range(rnd.randint(1, 9))]
        assert set(cm.live) == set(s.resident) and len(s.resident) <= 3
        if rnd.random() < 0.2 and s.resident:
            assert s.release(rnd.choice(list(s.resident)))
    for rid in list(s.resident):
        s.release(rid)
    assert not cm.live and cm.free_pages() == [12]
