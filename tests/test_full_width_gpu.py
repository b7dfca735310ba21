"""The engine at the layer sizes of Qwen3-8B (width 4096, 32 query heads on 8 kv heads of 128,
intermediate 12288; two layers and a shorter vocabulary keep it quick): the products, attention
kernels and graph paths that serving at that shape takes, under every way of cutting the work,
against the plain implementation. The tiny configurations never reach these kernels' fast paths
(x resident in LDS, the library's products, head size 128 with four query heads a kv head)."""
import pytest
import torch

from tests import trace_tools as tt
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

WIDE = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=32003, hidden_size=4096,
    num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
    intermediate_size=12288, max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=1e6,
    tie_word_embeddings=False)
LENGTHS = {"a": 5, "b": 17, "c": 700, "d": 100, "e": 64, "f": 150, "g": 1, "h": 47}
# float32: the bounds of the tiny configurations' replay. bfloat16: every product's result, the cache
# and the attention's probabilities are rounded to 8 bits of mantissa, which leaves noise of about
# 1.2 % of a row's norm (bounded below at 2 %, the reference's own bound); the logits' standard
# deviation here is 1.3, so one logit is off by 0.016 (one sigma), and the largest of the 35 million
# compared ones by six sigma.
TOL = {"float32": dict(atol=2e-4, rtol=2e-4), "bfloat16": dict(atol=1e-1, rtol=5e-2)}


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    from tests.conftest import make_folder
    folder = make_folder(tmp_path_factory, "wide", WIDE, dict(seed=5, std=0.02, embedding_std=0.02, norm_jitter=0.01))
    reqs = {rid: tt.random_tokens(WIDE["vocab_size"], n, seed=ord(rid)) for rid, n in LENGTHS.items()}
    cfg, w = plain.read_folder(folder)
    want = {rid: plain.logits(cfg, w, toks) for rid, toks in reqs.items()}
    return folder, reqs, want


def runner_for(folder, dtype, max_tokens, **kw):
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner
    # products by rule: what the measurement at load picks may differ from run to run, and with it
    # the rounding; the comparison below should be the same one every time
    ec = EngineConfig(dtype=dtype, page_size=16, max_token=max_tokens, max_reside=4,
                      max_step_tokens=max(max_tokens, 4), prefill_chunk=max_tokens, tune_products=False, **kw)
    return ModelRunner(folder, engine_config=ec)


def compare(got, want, reqs, dtype):
    worst, worst_rel = 0.0, 0.0
    for rid, toks in reqs.items():
        for p in range(len(toks)):
            a, b = got[(rid, p)], want[rid][p]
            worst = max(worst, (a - b).abs().max().item())
            worst_rel = max(worst_rel, ((a - b).norm() / b.norm()).item())
            try:
                torch.testing.assert_close(a, b, **TOL[dtype])
            except AssertionError as e:
                raise AssertionError(f"request {rid} position {p} (first wrong place): {e}") from None
    return worst, worst_rel


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail_decoded", "portions", "mixed"])
def test_full_width_replay(wide, dtype, cut):
    folder, reqs, want = wide
    steps = {"whole": tt.whole, "tail_decoded": tt.tail_decoded, "portions": tt.portions,
             "mixed": tt.mixed}[cut](reqs)
    runner = runner_for(folder, dtype, tt.peak_tokens(steps))
    got = tt.run_in_process(runner, steps)
    worst, rel = compare(got, want, reqs, dtype)
    print(f"full width {dtype} {cut}: largest difference {worst:.2e}, largest relative L2 {rel:.2e}")
    # the reference's own bound on a bf16 kernel against 32-bit: relative L2 of 2e-2 (rollout/utils/test_prefill_fwd_bwd.py:117)
    assert rel < (2e-2 if dtype == "bfloat16" else 1e-4)
    assert not runner.cache.live


def test_full_width_generation_through_graphs(wide):
    """Greedy generation in bfloat16 through the entry point, graphs and steps launched ahead on,
    four requests at once: every generated token is the 32-bit plain implementation's first or
    second choice at its place given the same prefix, and its logprob agrees."""
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    folder, reqs, _ = wide
    cfg, w = plain.read_folder(folder)
    prompts = [reqs[r] for r in ("b", "d", "e", "h")]
    eng = Engine(folder, dtype="bfloat16", page_size=16, max_token=2048, max_reside=4, max_step_tokens=256,
                 prefill_chunk=96, tune_products=False)
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12))
    for p, r in zip(prompts, out):
        assert r.num_tokens == 12
        rows = plain.logits(cfg, w, list(p) + r.output_ids[:-1])[len(p) - 1:]
        for i, tok in enumerate(r.output_ids):
            top2 = rows[i].topk(2)
            assert tok in top2.indices.tolist(), f"token {i}: {tok} is not among the plain top two {top2.indices.tolist()}"
            if tok != int(top2.indices[0]):           # a near tie that bfloat16 may decide the other way
                assert float(top2.values[0] - top2.values[1]) < 0.1
            assert abs(r.output_logprobs[i] - plain.chosen_logprob(rows[i], tok)) < 0.1


def test_full_width_graph_replays_equal_the_eager_steps(wide):
    """Twelve requests decode from the graph of sixteen at full width, where the products of a step
    are the library's: every replay gives the bits of the eager step, with eager work of the
    program's own (another request's prompt) and synchronisations between the replays."""
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner, StepEntry
    folder, _, _ = wide
    V = WIDE["vocab_size"]
    lens = [5, 17, 300, 64, 2, 90, 16, 47, 1, 129, 31, 200]

    def make(use_graphs):
        ec = EngineConfig(dtype="bfloat16", page_size=16, max_token=8192, max_reside=16, max_step_tokens=1024,
                          prefill_chunk=1024, use_graphs=use_graphs, tune_products=False)
        r = ModelRunner(folder, engine_config=ec)
        for i, n in enumerate(lens):
            r.add_request(i)
            r.step([StepEntry(i, tt.random_tokens(V, n, seed=300 + n), [])])
        return r

    eager, graph = make(False), make(True)
    ids = list(range(len(lens)))
    toks = [3 + i for i in ids]
    zeros, ones = [0.0] * len(ids), [1.0] * len(ids)
    for step in range(24):
        te, le, logits_e = eager.decode_and_sample(ids, toks, zeros, [0] * len(ids), ones, zeros)
        tg, lg, logits_g = graph.decode_and_sample(ids, toks, zeros, [0] * len(ids), ones, zeros)
        assert torch.equal(logits_e, logits_g), f"replay {step} differs from the eager step"
        assert te == tg and le == lg
        toks = te
        if step % 5 == 0:
            graph.add_request("x")
            graph.step([StepEntry("x", tt.random_tokens(V, 40, seed=step), [39])])
            graph.free_request("x")
            torch.cuda.synchronize()
    assert {k[0] for k in graph._graphs} == {16}


# ------------------------------------------------------------------ the engine as it is by default
class Spy:
    """Counts, per row count, the norms that a product finished (NormSink -> linear_add_norm) and the
    products that came as shares (Slabs -> _split_product) while a runner worked."""

    def __init__(self, ops):
        self.norm_rows, self.slab_rows, self.steps = [], [], []
        add_norm, split = ops.linear_add_norm, ops._split_product

        def spy_add_norm(x, w, h, wn, eps):
            self.norm_rows.append(h.shape[0])
            return add_norm(x, w, h, wn, eps)

        def spy_split(x, w, pieces):
            self.slab_rows.append(x.shape[0])
            return split(x, w, pieces)
        ops.linear_add_norm, ops._split_product = spy_add_norm, spy_split


def default_runner(folder, max_tokens, max_reside=4):
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner
    # tune_products and defer_norms as EngineConfig has them: on
    ec = EngineConfig(dtype="bfloat16", page_size=16, max_token=max_tokens, max_reside=max_reside,
                      max_step_tokens=max(max_tokens, 4), prefill_chunk=max_tokens)
    assert ec.tune_products and ec.defer_norms
    return ModelRunner(folder, engine_config=ec)


def shapes_of(runner):
    a, f = runner.model.blocks[0].mixer, runner.model.blocks[0].feed_forward
    return a.w_qkv, a.w_o, f.w_gate_up, f.w_down


@pytest.mark.parametrize("cut", ["whole", "tail_decoded", "portions", "mixed"])
def test_full_width_replay_of_the_default_engine(wide, cut):
    """The configuration that Engine(...) has by default and that bench.py times: the ways to form the
    products measured at load, the norms between products finished inside them where that was measured
    (or ruled) faster. In bfloat16 only: in float32 nothing is measured and no norm is deferred, so the
    default engine is the one of test_full_width_replay. The same four cuts and bounds; and the test
    looks at what ran: the measurement covered this model's shapes, norms were finished inside products
    at every row count at which the kernel set says it does that, and products came as shares at every
    row count at which its plan says so."""
    folder, reqs, want = wide
    steps = {"whole": tt.whole, "tail_decoded": tt.tail_decoded, "portions": tt.portions,
             "mixed": tt.mixed}[cut](reqs)
    runner = default_runner(folder, tt.peak_tokens(steps))
    ops = runner.rt.ops
    w_qkv, w_o, w_gu, w_down = shapes_of(runner)
    # the measurement ran on this model's four products and two pairs
    measured = {(k[1], k[2], k[3], k[4]) for k in ops._measured}
    for key in ((6144, 4096, False, torch.bfloat16), (4096, 4096, False, "residual"),
                (12288, 4096, True, torch.bfloat16), (4096, 12288, False, "residual")):
        assert key in measured, f"product {key} was not measured"
    pairs = {k[1:] for k in ops._defer}
    assert ((4096, 4096), (24576, 4096), True) in pairs and ((4096, 12288), (6144, 4096), False) in pairs
    spy = Spy(ops)
    got = tt.run_in_process(runner, steps)
    worst, rel = compare(got, want, reqs, "bfloat16")
    print(f"full width, default engine, {cut}: largest difference {worst:.2e}, largest relative L2 {rel:.2e}")
    assert rel < 2e-2
    assert not runner.cache.live
    # what the kernel set says it does at the row counts of this trace is what ran
    rows = sorted({sum(len(e["tokens"]) for e in s["entries"]) for s in steps})
    norm_at = {m for m in rows if ops.can_defer_norm(m, w_o, w_gu, True) or ops.can_defer_norm(m, w_down, w_qkv, False)}
    slabs_at = {m for m in rows if any(ops.route_linear(m, w.shape[0], w.shape[1], "residual").startswith("split")
                                       for w in (w_o, w_down))}
    assert set(spy.norm_rows) == norm_at and set(spy.slab_rows) == slabs_at
    assert norm_at, "no row count of this trace has a norm finished inside a product"
    if cut != "tail_decoded" or slabs_at:
        assert slabs_at, "no row count of this trace has a product in shares"


@pytest.mark.parametrize("inside", ["within_a_block", "between_blocks"])
@pytest.mark.parametrize("cut", ["portions", "mixed"])
def test_full_width_replay_with_one_norm_inside_its_products_and_the_next_not(wide, monkeypatch, inside, cut):
    """What the measurement at load may find: the norm between attention and feed-forward finished inside
    o and gate-up while the norm between two blocks is a kernel of its own, or the other way round, in one
    step (and one graph); at every row count up to 16 that the traces bring."""
    folder, reqs, want = wide
    steps = {"portions": tt.portions, "mixed": tt.mixed}[cut](reqs)
    runner = runner_for(folder, "bfloat16", tt.peak_tokens(steps))
    ops = runner.rt.ops
    w_qkv, w_o, w_gu, w_down = shapes_of(runner)
    within = (tuple(w_o.shape), tuple(w_gu.shape), True)
    between = (tuple(w_down.shape), tuple(w_qkv.shape), False)
    plan = {}
    for r in ops.ROW_STEPS:
        plan[(r,) + within] = inside == "within_a_block"
        plan[(r,) + between] = inside == "between_blocks"
    monkeypatch.setattr(ops, "_defer", plan)
    calls = []
    add_norm = ops.linear_add_norm
    monkeypatch.setattr(ops, "linear_add_norm", lambda x, w, h, wn, eps: (calls.append(tuple(w.shape)), add_norm(x, w, h, wn, eps))[1])
    got = tt.run_in_process(runner, steps)
    worst, rel = compare(got, want, reqs, "bfloat16")
    assert rel < 2e-2
    # only the one pair's first product ever finished a norm
    assert set(calls) == {tuple(w_o.shape) if inside == "within_a_block" else tuple(w_down.shape)}


def test_full_width_generation_of_a_whole_round_of_requests(wide):
    """Greedy generation of 32 requests in bfloat16 through the entry point as it is by default (products
    measured, norms deferred, graphs, steps launched ahead): 32 requests on 8 kv heads are one whole round
    of (request, kv head) pairs over the CUs, so the decode attention merges a request's splits inside one
    workgroup by its own rule. Every token is the 32-bit plain implementation's first choice at its place,
    or its second where the two are nearly tied; logprobs agree."""
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    folder, _, _ = wide
    cfg, w = plain.read_folder(folder)
    n_req, new = 32, 8
    prompts = [tt.random_tokens(WIDE["vocab_size"], 3 + (7 * i) % 90, seed=500 + i) for i in range(n_req)]
    eng = Engine(folder, dtype="bfloat16", page_size=16, max_token=8192, max_reside=n_req, max_step_tokens=2048,
                 prefill_chunk=512, check_invariants=True)
    ops = eng.runner.rt.ops
    assert ops.cu_count % 8 or (n_req * 8) % ops.cu_count == 0, "32 requests are no whole round on this chip"
    seen = []
    splits = ops._decode_splits
    ops._decode_splits = lambda *a, **k: (seen.append(splits(*a, **k)) or seen[-1])
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=new))
    assert any(merge for _, _, merge in seen), "no decode step merged inside the workgroup"
    assert any(k[0] == n_req for k in eng.runner._graphs), "no graph of 32 rows was captured"
    for p, r in zip(prompts, out):
        assert r.num_tokens == new
        rows = plain.logits(cfg, w, list(p) + r.output_ids[:-1])[len(p) - 1:]
        for i, tok in enumerate(r.output_ids):
            top2 = rows[i].topk(2)
            assert tok in top2.indices.tolist(), f"token {i}: {tok} is not among the plain top two {top2.indices.tolist()}"
            if tok != int(top2.indices[0]):
                assert float(top2.values[0] - top2.values[1]) < 0.1
            assert abs(r.output_logprobs[i] - plain.chosen_logprob(rows[i], tok)) < 0.1
