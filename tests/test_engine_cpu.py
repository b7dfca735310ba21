"""The engine's host side (cache, step function, scheduler, entry point) on the CPU, with the
torch stand-in kernels of tests/torch_ops.py in place of the HIP library: every way of cutting
the work gives the plain implementation's logits, and generation does not depend on the knobs."""
import pytest
import torch

from return_amd import SamplingParams
from return_amd.config import EngineConfig
from return_amd.engine import Engine, ModelRunner, StepEntry
from tests import trace_tools as tt
from tests.conftest import TINY_A, TINY_B
from tests.plain import qwen3_plain as plain
from tests.torch_ops import TorchOps


def runner_for(folder, max_token, page=16, max_reside=4, **kw):
    ec = EngineConfig(dtype="float32", check_invariants=True, page_size=page, max_token=max_token, max_reside=max_reside,
                      max_step_tokens=max(max_token, max_reside), prefill_chunk=max_token, device="cpu", **kw)
    return ModelRunner(folder, engine_config=ec, ops=TorchOps())


@pytest.mark.parametrize("which", ["a", "b"])
@pytest.mark.parametrize("cut", ["whole", "tail_decoded", "portions", "mixed"])
def test_every_cut_matches_plain(which, cut, folder_a, folder_b):
    folder, raw = (folder_a, TINY_A) if which == "a" else (folder_b, TINY_B)
    reqs = {rid: tt.random_tokens(raw["vocab_size"], n, seed=ord(rid))
            for rid, n in {"a": 5, "b": 17, "c": 33, "d": 70, "e": 64, "g": 1}.items()}
    cfg, w = plain.read_folder(folder)
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in reqs.items()}
    steps = {"whole": tt.whole, "tail_decoded": tt.tail_decoded, "portions": tt.portions, "mixed": tt.mixed}[cut](reqs)
    runner = runner_for(folder, tt.peak_tokens(steps))
    got = tt.run_in_process(runner, steps)
    for rid, toks in reqs.items():
        for p in range(len(toks)):
            torch.testing.assert_close(got[(rid, p)], want[rid][p], atol=2e-5, rtol=1e-4)
    assert all(g.pages.in_use() == 0 for g in runner.cache.groups)


def test_generation_does_not_depend_on_the_knobs(folder_b):
    cfg, w = plain.read_folder(folder_b)
    prompts = [tt.random_tokens(TINY_B["vocab_size"], n, seed=n) for n in (1, 8, 31, 64, 100)]
    want = [plain.greedy_generate(cfg, w, p, 6) for p in prompts]
    for max_reside, chunk, max_token, page in ((4, 24, 1024, 32), (1, 1000, 256, 16), (5, 7, 416, 8)):
        ec = EngineConfig(dtype="float32", check_invariants=True, page_size=page, max_token=max_token, max_reside=max_reside,
                          max_step_tokens=64, prefill_chunk=chunk, device="cpu")
        eng = Engine(runner=ModelRunner(folder_b, engine_config=ec, ops=TorchOps()))
        got = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=6))
        assert [r.output_ids for r in got] == want
        assert all(r.finish_reason == "length" and r.num_tokens == 6 for r in got)
        for r, p in zip(got, prompts):                 # logprob is of the raw logits (rollout/model.py:64-67)
            lp = plain.chosen_logprob(plain.logits(cfg, w, p)[-1], r.output_ids[0])
            assert abs(r.output_logprobs[0] - lp) < 1e-4
        eng.runner.cache.check_invariants()
        assert not eng.runner.cache.live


def test_temperature_sampling_is_reproducible_and_batch_independent(folder_a):
    prompts = [tt.random_tokens(TINY_A["vocab_size"], n, seed=n) for n in (5, 17, 33)]
    sp = [SamplingParams(temperature=0.7, max_new_tokens=10, seed=100 + i) for i in range(3)]
    def run(max_reside):
        ec = EngineConfig(dtype="float32", check_invariants=True, page_size=16, max_token=512, max_reside=max_reside,
                          max_step_tokens=64, prefill_chunk=24, device="cpu", seed=7)
        return [r.output_ids for r in Engine(runner=ModelRunner(folder_a, engine_config=ec, ops=TorchOps()))
                .generate(prompts, sp)]
    together, alone = run(3), run(1)
    assert together == alone == run(3)
    assert len({tuple(x) for x in together}) == 3


def test_stop_sequence_through_the_entry_point(folder_a):
    cfg, w = plain.read_folder(folder_a)
    prompt = tt.random_tokens(TINY_A["vocab_size"], 9, seed=4)
    free = plain.greedy_generate(cfg, w, prompt, 8)
    eng = Engine(runner=runner_for(folder_a, 256))
    r = eng.generate([prompt], SamplingParams(temperature=0.0, max_new_tokens=8, stop_ids=[free[2:4]]))[0]
    want = plain.greedy_generate(cfg, w, prompt, 8, stop_ids=[free[2:4]])
    assert r.output_ids == want and len(want) < 8 and r.finish_reason == "stop"


def test_a_bad_prompt_is_refused_before_any_is_queued(folder_a):
    eng = Engine(runner=runner_for(folder_a, 256))
    sp = SamplingParams(temperature=0.0, max_new_tokens=2)
    for bad, why in (([], "empty prompt"), ([1, TINY_A["vocab_size"]], "outside the vocabulary")):
        with pytest.raises(ValueError, match=why):
            eng.generate([[1, 2, 3], bad, [4, 5]], sp)
        assert not eng.scheduler.has_work() and not eng.runner.cache.live     # the good ones were not left behind
    assert [r.num_tokens for r in eng.generate([[1, 2, 3], [4, 5]], sp)] == [2, 2]
    # what can never fit gives an error result of its own, the others run
    out = eng.generate([[1] * 256, [4, 5]], sp)
    assert out[0].finish_reason == "error" and "max_position" in out[0].error and out[1].num_tokens == 2


def test_step_checks(folder_a):
    from return_amd.engine import StepEntry
    runner = runner_for(folder_a, 64)
    runner.add_request("a")
    with pytest.raises(ValueError, match="vocabulary"):
        runner.step([StepEntry("a", [TINY_A["vocab_size"]], [0])])
    with pytest.raises(ValueError, match="not among"):
        runner.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(ValueError, match="no tokens"):
        runner.step([StepEntry("a", [], [])])
    assert runner.step([StepEntry("a", [1, 2, 3], [])]) is None          # nothing wanted, cache still filled
    assert runner.cache.seq_len("a") == 3
    with pytest.raises(ValueError, match="max_position"):
        runner.step([StepEntry("a", [1] * 300, [])])


def test_prepared_matrices_follow_the_tensor_not_its_address():
    """Runtime.matrix keeps one prepared copy per stored tensor (tied weights stay one copy); a
    tensor that is freed and another of the same shape at the same address must not get it."""
    from return_amd.parts.runtime import Runtime
    from tests.torch_ops import TorchOps
    rt = Runtime("cpu", "bfloat16", ops=TorchOps("cpu"))     # float32 stored, bfloat16 prepared: a copy
    t = torch.full((64, 80), 1.0)
    assert rt.matrix(t) is rt.matrix(t) and rt.matrix(t).dtype == torch.bfloat16
    seen = set()
    for i in range(200):
        t = torch.full((64, 80), float(i))
        seen.add(t.data_ptr())
        assert float(rt.matrix(t)[3, 5]) == float(i)
        del t
    rt.forget_casts()
    assert not rt._cast


def test_steps_launched_ahead_give_the_same_generation(folder_a):
    """With lookahead the next decode step is launched before this one's tokens are read. Requests
    of different lengths, one that ends on a stop sequence (found out one step late: the step
    already under way computed a token for it, which is dropped), more requests than may be live
    at once, temperature sampling: outputs, logprobs and finish reasons equal the run without it."""
    cfg, w = plain.read_folder(folder_a)
    V = TINY_A["vocab_size"]
    prompts = [tt.random_tokens(V, n, seed=30 + n) for n in (9, 3, 40, 17, 5, 64)]
    free = plain.greedy_generate(cfg, w, prompts[0], 12)
    params = [SamplingParams(temperature=0.0, max_new_tokens=12, stop_ids=[free[4:6]]),
              SamplingParams(temperature=0.0, max_new_tokens=1),
              SamplingParams(temperature=0.8, top_k=20, max_new_tokens=9, seed=5),
              SamplingParams(temperature=0.0, max_new_tokens=2),
              SamplingParams(temperature=1.1, top_p=0.8, max_new_tokens=15, seed=6),
              SamplingParams(temperature=0.0, max_new_tokens=7)]

    def run(lookahead, max_reside):
        ec = EngineConfig(dtype="float32", check_invariants=True, page_size=16, max_token=1024, max_reside=max_reside, max_step_tokens=64,
                          prefill_chunk=32, device="cpu", seed=3, lookahead=lookahead)
        eng = Engine(runner=ModelRunner(folder_a, engine_config=ec, ops=TorchOps()))
        out = eng.generate(prompts, params)
        eng.runner.cache.check_invariants()
        assert not eng.runner.cache.live and eng._in_flight is None
        assert all(g.pages.in_use() == 0 for g in eng.runner.cache.groups)
        return [(r.output_ids, r.finish_reason, [round(x, 5) for x in r.output_logprobs]) for r in out], eng

    plain_run, _ = run(False, 6)
    ahead_run, eng = run(True, 6)
    assert ahead_run == plain_run
    assert plain_run[0][1] == "stop" and len(plain_run[0][0]) < 12
    # requests wait for a slot: steps are decided ahead only now and then (other batches: logprobs to rounding)
    waited = run(True, 2)[0]
    assert [(o, why) for o, why, _ in waited] == [(o, why) for o, why, _ in plain_run]
    assert all(abs(x - y) < 1e-3 for (_, _, a), (_, _, b) in zip(waited, plain_run) for x, y in zip(a, b))
    assert eng.decode_tokens == sum(len(o) - 1 for o, _, _ in plain_run)    # a dropped token is not counted


def test_schedule_ahead_decides_on_the_state_the_step_under_way_will_leave(folder_a):
    from return_amd.engine.scheduler import Request, Scheduler
    runner = runner_for(folder_a, 512, max_reside=3)
    sch = Scheduler(runner.cache, 3, 64, 32, runner.max_position)
    a = Request("a", [1, 2, 3], SamplingParams(max_new_tokens=3))
    b = Request("b", list(range(40)), SamplingParams(max_new_tokens=2))
    sch.add(a); sch.add(b)

    def run(plan):                                           # the runner's side of a step
        runner.cache.begin_step([(e.request.id, len(e.tokens)) for e in plan.entries]); runner.cache.end_step()

    plan = sch.schedule()                                    # a's prompt whole, b's first portion
    assert [(e.request.id, len(e.tokens), e.sample) for e in plan.entries] == [("a", 3, True), ("b", 32, False)]
    run(plan)
    ahead = sch.schedule_ahead(plan)                         # a decodes a token nobody knows yet, b's prompt ends
    assert [(e.request.id, e.tokens if e.request is a else len(e.tokens), e.sample) for e in ahead.entries] == \
        [("a", [None], True), ("b", 8, True)]
    assert a.num_computed == 0 and not a.output              # nothing is booked by looking ahead
    sch.finish_step(plan, {"a": (7, 0.0)})
    run(ahead)
    sch.add(Request("c", [9, 9], SamplingParams(max_new_tokens=2)))
    ahead2 = sch.schedule_ahead(ahead)                       # both decode, the newcomer is let in
    assert [(e.request.id, e.tokens) for e in ahead2.entries] == [("a", [None]), ("b", [None]), ("c", [9, 9])]
    sch.finish_step(ahead, {"a": (8, 0.0), "b": (5, 0.0)})
    run(ahead2)
    ahead3 = sch.schedule_ahead(ahead2)                      # a's and b's tokens of ahead2 are their last: only c goes on
    assert [(e.request.id, e.tokens) for e in ahead3.entries] == [("c", [None])]
    done = sch.finish_step(ahead2, {"a": (1, 0.0), "b": (2, 0.0), "c": (3, 0.0)})
    assert {r.id for r in done} == {"a", "b"} and a.output == [7, 8, 1] and b.output == [5, 2]
    run(ahead3)
    assert sch.schedule_ahead(ahead3) is None                # c's token of ahead3 is its last: nothing is left to run
    sch.finish_step(ahead3, {"c": (4, 0.0)})
    assert not sch.has_work() and not runner.cache.live


def engine_for(folder, lookahead=True, **kw):
    ec = EngineConfig(dtype="float32", check_invariants=True, page_size=16, max_token=kw.pop("max_token", 1024), max_reside=kw.pop("max_reside", 4),
                      max_step_tokens=64, prefill_chunk=24, device="cpu", lookahead=lookahead, **kw)
    return Engine(runner=ModelRunner(folder, engine_config=ec, ops=TorchOps()))


@pytest.mark.parametrize("lookahead", [False, True])
def test_a_kept_session_goes_on_where_it_stopped(folder_a, lookahead):
    """Two turns of two sessions: the second turn's prompt repeats the first turn and its answer and
    goes on; only the rest is computed, and the answers are the plain implementation's on the
    whole prompts. One session ends its first turn on a stop sequence, which with steps launched
    ahead is found out after its last token was already fed."""
    cfg, w = plain.read_folder(folder_a)
    V = TINY_A["vocab_size"]
    p1 = {"s": tt.random_tokens(V, 21, seed=1), "t": tt.random_tokens(V, 40, seed=2)}
    free = plain.greedy_generate(cfg, w, p1["t"], 9)
    sp = {"s": SamplingParams(temperature=0.0, max_new_tokens=6),
          "t": SamplingParams(temperature=0.0, max_new_tokens=9, stop_ids=[free[3:5]])}
    eng = engine_for(folder_a, lookahead)
    out1 = dict(zip("st", eng.generate([p1["s"], p1["t"]], [sp["s"], sp["t"]], session_ids=["s", "t"], keep=True)))
    assert out1["s"].output_ids == plain.greedy_generate(cfg, w, p1["s"], 6)
    stopped = plain.greedy_generate(cfg, w, p1["t"], 9, stop_ids=[free[3:5]])
    assert out1["t"].output_ids == stopped and out1["t"].finish_reason == "stop" and len(stopped) < 9
    assert set(eng.runner.cache.live) == {"s", "t"} and eng.stats()["resident"] == 2
    eng.runner.cache.check_invariants()
    p2 = {k: p1[k] + out1[k].output_ids + tt.random_tokens(V, 7, seed=ord(k)) for k in "st"}
    before = eng.prefill_tokens
    out2 = dict(zip("st", eng.generate([p2["s"], p2["t"]], SamplingParams(temperature=0.0, max_new_tokens=5),
                                       session_ids=["s", "t"])))
    for k in "st":
        assert out2[k].output_ids == plain.greedy_generate(cfg, w, p2[k], 5)
    assert out2["s"].cached_tokens == len(p1["s"]) + 5                 # the sixth token was sampled, never fed
    assert out2["t"].cached_tokens == len(p1["t"]) + len(stopped) - (0 if lookahead else 1)
    assert eng.prefill_tokens - before == sum(len(p2[k]) - out2[k].cached_tokens for k in "st")
    assert not eng.runner.cache.live and eng.stats()["resident"] == 0    # the second turn did not keep
    assert all(g.pages.in_use() == 0 for g in eng.runner.cache.groups)


def test_kept_sessions_that_do_not_fit_or_do_not_match(folder_a):
    cfg, w = plain.read_folder(folder_a)
    V = TINY_A["vocab_size"]
    sp = SamplingParams(temperature=0.0, max_new_tokens=4)
    prompts = {k: tt.random_tokens(V, 30, seed=10 + i) for i, k in enumerate("abc")}
    eng = engine_for(folder_a, max_reside=2, max_token=160)            # ten pages, two slots
    outs = {}
    for k in "ab":
        outs[k] = eng.generate([prompts[k]], sp, session_ids=[k], keep=True)[0]
    assert list(eng.scheduler.resident) == ["a", "b"]
    with pytest.raises(ValueError, match="each differently"):
        eng.generate([prompts["a"], prompts["b"]], sp, session_ids=["a", "a"])
    # a third session needs a slot: the one used longest ago is given up
    outs["c"] = eng.generate([prompts["c"]], sp, session_ids=["c"], keep=True)[0]
    assert list(eng.scheduler.resident) == ["b", "c"] and set(eng.runner.cache.live) == {"b", "c"}
    # "a" comes back and starts afresh; "b" has to go for it, "c" goes on from its cache afterwards
    nxt = {k: prompts[k] + outs[k].output_ids + [5, 6] for k in "abc"}
    ra = eng.generate([nxt["a"]], sp, session_ids=["a"], keep=True)[0]
    assert ra.cached_tokens == 0 and ra.output_ids == plain.greedy_generate(cfg, w, nxt["a"], 4)
    assert list(eng.scheduler.resident) == ["c", "a"]
    rc = eng.generate([nxt["c"]], sp, session_ids=["c"], keep=True)[0]
    assert rc.cached_tokens == 33 and rc.output_ids == plain.greedy_generate(cfg, w, nxt["c"], 4)
    # a prompt that does not repeat what the cache holds: the cache is dropped, the answer is right
    other = tt.random_tokens(V, 35, seed=77)
    rc = eng.generate([other], sp, session_ids=["c"], keep=True)[0]
    assert rc.cached_tokens == 0 and rc.output_ids == plain.greedy_generate(cfg, w, other, 4)
    # a request that needs more pages than are free pushes kept sessions out, but only if that helps
    big = tt.random_tokens(V, 120, seed=5)
    rb = eng.generate([big], sp)[0]
    assert rb.output_ids == plain.greedy_generate(cfg, w, big, 4) and eng.stats()["resident"] < 2
    eng.runner.cache.check_invariants()
    # release: known ids give their pages back, unknown ones are reported
    for rid in list(eng.scheduler.resident):
        assert eng.release(rid)
    assert not eng.release("nobody") and not eng.runner.cache.live
    assert all(g.pages.in_use() == 0 for g in eng.runner.cache.groups)
    # released while under way: given back at the end although it asked to be kept
    r = eng.submit(prompts["a"], sp, request_id="z", keep=True)
    eng.step()
    assert eng.release("z")
    with pytest.raises(ValueError, match="already under way"):
        eng.submit(prompts["b"], sp, request_id="z")
    while eng.scheduler.has_work() or eng._in_flight is not None:
        eng.step()
    assert r.finish_reason == "length" and not eng.runner.cache.live


@pytest.mark.parametrize("seed", range(6))
def test_launching_ahead_never_changes_what_is_generated(folder_a, seed):
    """Random prompts, lengths, stop sequences and knobs: with every step launched before the one
    before it is collected (prompt portions beside decoded tokens included) the outputs and finish
    reasons equal the plain implementation's, and nothing is left in the cache."""
    import random
    rnd = random.Random(seed)
    cfg, w = plain.read_folder(folder_a)
    V = TINY_A["vocab_size"]
    n = rnd.randint(3, 9)
    prompts = [tt.random_tokens(V, rnd.randint(1, 90), seed=seed * 100 + i) for i in range(n)]
    news = [rnd.randint(1, 12) for _ in range(n)]
    stops = []
    for p, k in zip(prompts, news):
        free = plain.greedy_generate(cfg, w, p, k)
        stops.append([free[j:j + 2]] if k >= 4 and rnd.random() < 0.5 and (j := rnd.randint(0, k - 2)) >= 0 else [])
    want = [plain.greedy_generate(cfg, w, p, k, stop_ids=s) for p, k, s in zip(prompts, news, stops)]
    params = [SamplingParams(temperature=0.0, max_new_tokens=k, stop_ids=s) for k, s in zip(news, stops)]
    max_reside = rnd.randint(1, 5)
    eng = engine_for(folder_a, True, max_reside=max_reside, max_token=rnd.choice([256, 512, 2048]))
    eng.config.prefill_chunk = eng.scheduler.prefill_chunk = rnd.choice([5, 24, 64])
    launches = []
    inner = eng._launch_or_run
    eng._launch_or_run = lambda plan, previous=None: (launches.append(previous is not None), inner(plan, previous))[1]
    out = eng.generate(prompts, params)
    assert [r.output_ids for r in out] == want
    assert [r.finish_reason for r in out] == ["stop" if s and o[-2:] == s[0] else "length" for o, s in zip(want, stops)]
    assert any(launches) and eng._in_flight is None           # steps were launched ahead
    eng.runner.cache.check_invariants()
    assert not eng.runner.cache.live and all(g.pages.in_use() == 0 for g in eng.runner.cache.groups)


def test_a_prompt_of_one_token_beside_tokens_that_are_still_on_the_device(folder_a):
    """A newcomer whose prompt is a single token joins a step whose other tokens are not known
    yet: one token each, but not a step that takes all its tokens from the step before."""
    cfg, w = plain.read_folder(folder_a)
    V = TINY_A["vocab_size"]
    eng = engine_for(folder_a, True, max_reside=4)
    sp = SamplingParams(temperature=0.0, max_new_tokens=8)
    first = [eng.submit(tt.random_tokens(V, n, seed=n), sp) for n in (7, 20)]
    for _ in range(3):
        eng.step()
    late = [eng.submit([5], sp), eng.submit([9], SamplingParams(temperature=0.0, max_new_tokens=1))]
    while eng.scheduler.has_work() or eng._in_flight is not None:
        eng.step()
    for r in first + late:
        assert r.output == plain.greedy_generate(cfg, w, r.prompt_ids, r.max_new)
    assert not eng.runner.cache.live


def test_a_step_that_cannot_start_fails_its_requests_and_frees_them(folder_a, monkeypatch):
    eng = engine_for(folder_a, True, max_reside=4)
    sp = SamplingParams(temperature=0.0, max_new_tokens=5)
    a = eng.submit([1, 2, 3], sp)
    eng.step()

    def broken(*args, **kw):
        raise RuntimeError("the device said no")
    monkeypatch.setattr(eng.runner, "decode_launch", broken)
    monkeypatch.setattr(eng.runner, "step_launch", broken)
    b = eng.submit([4, 5], sp)
    with pytest.raises(RuntimeError, match="said no"):
        while eng.scheduler.has_work() or eng._in_flight is not None:
            eng.step()
    assert a.finish_reason == b.finish_reason == "error" and "said no" in str(a.error)
    monkeypatch.undo()
    out = eng.generate([[7, 8, 9]], sp)[0]                 # the step that was under way is collected, then life goes on
    assert out.num_tokens == 5 and not eng.runner.cache.live
    eng.runner.cache.check_invariants()


def test_duty_and_decode_streak(folder_a):
    """The reference's counters (rollout/engine.py:84-125, 361-364, 403): the share of the run that went
    into steps of each kind, and the mean run of decode-only steps between steps that brought prompts."""
    V = TINY_A["vocab_size"]
    eng = engine_for(folder_a, max_reside=2, max_token=512, lookahead=False)
    assert eng.stats()["decode_streak"] is None and eng.stats()["decode_duty"] == 0.0
    sp = SamplingParams(temperature=0.0, max_new_tokens=5)
    # two at once: one prompt step, then four steps that only decode; then the same again
    for turn in range(2):
        eng.generate([tt.random_tokens(V, 9, seed=turn), tt.random_tokens(V, 20, seed=7 + turn)], sp)
    st = eng.stats()
    assert st["steps"] == 10 and eng._decode_streak == 4        # the run under way is not counted yet
    assert st["decode_streak"] == 4.0                           # one closed run of four
    eng.generate([tt.random_tokens(V, 3, seed=5)], SamplingParams(temperature=0.0, max_new_tokens=2))
    st = eng.stats()
    assert st["decode_streak"] == 4.0 and eng._decode_streak == 1
    assert 0 < st["decode_duty"] < 1 and 0 < st["prefill_duty"] < 1
    assert st["decode_duty"] + st["prefill_duty"] <= 1.0 + 1e-9
    assert abs(st["decode_duty"] * st["run_seconds"] - eng.decode_seconds) < 1e-6


def test_norms_are_finished_inside_the_products_in_steps_of_few_rows(folder_b):
    """A step of up to 16 rows leaves every norm between two products to those products (the kernel
    set's linear_add_norm, and ScaledRows into linear / linear_silu_mul); a step of more rows, the first
    norm of the first layer and the last norm (on the wanted rows only) run as norms of their own. The
    logits are the plain implementation's either way."""
    from return_amd.parts.runtime import ScaledRows
    cfg, w = plain.read_folder(folder_b)
    L = cfg["num_hidden_layers"]
    toks = tt.random_tokens(TINY_B["vocab_size"], 40, seed=3)
    want = plain.logits(cfg, w, toks)
    for defer in (True, False):
        runner = runner_for(folder_b, 128, defer_norms=defer)
        ops = runner.rt.ops
        calls = {"add_norm": 0, "scaled_in": 0, "norm": 0}
        for name, key in (("linear_add_norm", "add_norm"), ("add_rmsnorm", "norm")):
            def counted(*a, _f=getattr(ops, name), _k=key, **k):
                calls[_k] += 1
                return _f(*a, **k)
            setattr(ops, name, counted)
        for name in ("linear", "linear_silu_mul"):
            def counted(x, *a, _f=getattr(ops, name), **k):
                calls["scaled_in"] += isinstance(x, ScaledRows)
                return _f(x, *a, **k)
            setattr(ops, name, counted)
        if not defer:
            ops.can_defer_norm = lambda *a: False
        runner.add_request("r")
        got = [runner.step([StepEntry("r", toks[:24], list(range(24)))])]          # 24 rows: norms of their own
        assert calls == {"add_norm": 0, "scaled_in": 0, "norm": 2 * L + 1}
        calls.update(add_norm=0, scaled_in=0, norm=0)
        got.append(runner.step([StepEntry("r", toks[24:], list(range(16)))]))     # 16 rows
        if defer:
            # every layer's two norms but the very first are left to the products; the last norm stands alone
            # (the stand-in's gated product calls its plain one, so each of the L gated products counts twice)
            assert calls == {"add_norm": 2 * L - 1, "scaled_in": 2 * L - 1 + L, "norm": 2}
        else:
            assert calls == {"add_norm": 0, "scaled_in": 0, "norm": 2 * L + 1}
        torch.testing.assert_close(torch.cat(got).cpu(), want, atol=2e-4, rtol=2e-4)


def test_the_engine_checks_the_cache_after_every_step_when_asked(folder_a):
    """EngineConfig.check_invariants: a page that is both held and free (put there by hand) is found
    at the end of the very next step; without the option the step goes through."""
    toks = tt.random_tokens(TINY_A["vocab_size"], 20, seed=1)
    for on in (True, False):
        runner = runner_for(folder_a, 256)
        runner.engine_config.check_invariants = on
        assert runner.engine_config.check_invariants == on
        runner.add_request("r")
        runner.step([StepEntry("r", toks[:10], [])])
        held = runner.cache.live["r"].pages[0][0]
        runner.cache.groups[0].pages._free.append(held)
        if on:
            with pytest.raises(AssertionError, match="both free and held|twice"):
                runner.step([StepEntry("r", toks[10:12], [])])
        else:
            runner.step([StepEntry("r", toks[10:12], [])])
