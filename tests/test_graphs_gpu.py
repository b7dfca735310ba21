"""Decode steps replayed from captured HIP graphs give what the eager path gives, on every
replay, with eager work and synchronisations between the replays."""
import pytest
import torch

from return_amd.config import EngineConfig
from return_amd.engine import ModelRunner, StepEntry
from tests import trace_tools as tt
from tests.conftest import TINY_B

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_graph_replays_match_eager(folder_b, dtype):
    V = TINY_B["vocab_size"]
    prompts = {rid: tt.random_tokens(V, n, seed=n) for rid, n in {"a": 40, "b": 7, "c": 130}.items()}

    def make(use_graphs):
        ec = EngineConfig(dtype=dtype, page_size=16, max_token=4096, max_reside=4, max_step_tokens=512,
                          prefill_chunk=512, use_graphs=use_graphs)
        r = ModelRunner(folder_b, engine_config=ec)
        for rid, toks in prompts.items():
            r.add_request(rid)
            r.step([StepEntry(rid, toks, [])])
        return r

    eager, graph = make(False), make(True)
    ids = list(prompts)
    toks_e = toks_g = [3, 5, 7]
    temps, ks, ps = [0.0, 0.8, 0.0], [0, 5, 0], [1.0, 0.9, 1.0]
    for step in range(140):                     # crosses pages and the 256-token context bucket
        us = [0.1 * ((step * 7 + i) % 10) for i in range(3)]
        te, le, logits_e = eager.decode_and_sample(ids, toks_e, temps, ks, ps, us)
        tg, lg, logits_g = graph.decode_and_sample(ids, toks_g, temps, ks, ps, us)
        assert torch.equal(logits_e, logits_g), f"replay {step} differs from the eager step"
        assert te == tg and le == lg
        toks_e = toks_g = te
        if step % 9 == 0:                       # eager work of the program's own between replays
            graph.add_request("x")
            graph.step([StepEntry("x", tt.random_tokens(V, 20, seed=step), [19])])
            graph.free_request("x")
            torch.cuda.synchronize()
    assert len(graph._graphs) >= 2              # more than one context bucket was captured
    # a different batch size gets a graph of its own
    graph.free_request("b"); eager.free_request("b")
    te, _, logits_e = eager.decode_and_sample(["a", "c"], [1, 2], [0.0, 0.0], [0, 0], [1.0, 1.0], [0.0, 0.0])
    tg, _, logits_g = graph.decode_and_sample(["a", "c"], [1, 2], [0.0, 0.0], [0, 0], [1.0, 1.0], [0.0, 0.0])
    assert te == tg and torch.equal(logits_e, logits_g)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32", "bfloat16, splits merged in the workgroup"])
def test_batch_filled_up_to_a_graph_size(folder_b, dtype):
    """Eleven requests run from the graph of sixteen: the five added rows write and read the
    spare page only; logits, tokens and every page that a request holds equal the eager run.
    (Products by rule: a measured plan may form products of 11 and of 16 rows in different ways,
    which differ in rounding.) Once more with the decode attention that merges a request's splits
    inside one workgroup, where the added rows are workgroups with a single key."""
    V = TINY_B["vocab_size"]
    lens = [5, 17, 33, 64, 2, 90, 16, 47, 1, 129, 31]
    dtype, _, merged = dtype.partition(",")

    def make(use_graphs):
        ec = EngineConfig(dtype=dtype, page_size=16, max_token=4096, max_reside=16, max_step_tokens=512,
                          prefill_chunk=512, use_graphs=use_graphs, tune_products=False)
        r = ModelRunner(folder_b, engine_config=ec)
        if merged:
            r.rt.ops.decode_merge_round = 1          # every count of requests is a whole round
        for i, n in enumerate(lens):
            r.add_request(i)
            r.step([StepEntry(i, tt.random_tokens(V, n, seed=100 + n), [])])
        return r

    eager, graph = make(False), make(True)
    assert graph.graph_batch_size(11) == 16 and graph.graph_batch_size(8) == 8 and graph.graph_batch_size(16) == 16
    ids = list(range(len(lens)))
    toks = [3 + i for i in ids]
    zeros, ones = [0.0] * len(ids), [1.0] * len(ids)
    for step in range(20):
        te, le, logits_e = eager.decode_and_sample(ids, toks, zeros, [0] * len(ids), ones, zeros)
        tg, lg, logits_g = graph.decode_and_sample(ids, toks, zeros, [0] * len(ids), ones, zeros)
        assert logits_g.shape == logits_e.shape and torch.equal(logits_e, logits_g), f"step {step}"
        assert te == tg and le == lg
        toks = te
        if step == 9:                               # the batch shrinks: ten requests, the same graph size
            for r in (eager, graph):
                r.free_request(ids[-1])
            ids, toks = ids[:-1], toks[:-1]
            zeros, ones = zeros[:-1], ones[:-1]
    assert {k[0] for k in graph._graphs} == {16}
    for ge, gg in zip(eager.cache.groups, graph.cache.groups):
        assert torch.equal(ge.pool[:, :, :ge.num_pages], gg.pool[:, :, :gg.num_pages])
    graph.cache.check_invariants()


def test_generation_with_graphs(folder_b):
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    prompts = [tt.random_tokens(TINY_B["vocab_size"], n, seed=n) for n in (1, 8, 31, 64, 100)]
    outs = []
    for use_graphs in (False, True):
        eng = Engine(folder_b, check_invariants=True, dtype="float32", page_size=32, max_token=4096, max_reside=5,
                     max_step_tokens=64, prefill_chunk=24, use_graphs=use_graphs)
        outs.append([r.output_ids for r in eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=20))])
    assert outs[0] == outs[1]


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("use_graphs", [False, True])
def test_steps_launched_ahead_on_the_device(folder_b, dtype, use_graphs):
    """The next decode step is launched before this one's tokens are read and takes them over on
    the device: outputs, logprobs and finish reasons equal the run that waits for every step.
    Lengths differ, one request ends on a stop sequence that is found out a step late, eleven
    requests make the graph of sixteen rows shrink to that of eight and below."""
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    V = TINY_B["vocab_size"]
    prompts = [tt.random_tokens(V, n, seed=50 + n) for n in (9, 3, 40, 17, 5, 64, 2, 33, 12, 7, 21)]
    news = [12, 1, 9, 2, 15, 7, 30, 4, 11, 26, 5]

    def run(lookahead, stops):
        # products by rule: a request that is found finished a step late makes a batch of one row more,
        # and a measured plan may form products of 8 and of 9 rows in ways that round differently
        eng = Engine(folder_b, check_invariants=True, dtype=dtype, page_size=16, max_token=4096, max_reside=11, max_step_tokens=128,
                     prefill_chunk=64, use_graphs=use_graphs, lookahead=lookahead, seed=4, tune_products=False)
        params = [SamplingParams(temperature=0.0 if i % 3 else 0.9, top_k=0 if i % 2 else 30, max_new_tokens=n,
                                 seed=i, stop_ids=stops if i == 6 else [])
                  for i, n in enumerate(news)]
        out = eng.generate(prompts, params)
        eng.runner.cache.check_invariants()
        assert not eng.runner.cache.live and all(g.pages.in_use() == 0 for g in eng.runner.cache.groups)
        return [(r.output_ids, r.finish_reason, r.output_logprobs) for r in out]

    free = run(False, [])
    stop = [free[6][0][9:11]]                     # two tokens that request 6 will write
    want, got = run(False, stop), run(True, stop)
    assert got == want
    assert want[6][1] == "stop" and len(want[6][0]) < 30
    assert [len(o) for o, _, _ in want][:6] == news[:6]
