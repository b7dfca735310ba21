"""Generation through the entry points on the GPU: greedy equals the plain implementation,
temperature sampling is reproducible, the command line answers in the reference's fields."""
import json
import os
import subprocess
import sys

import pytest
import torch

from return_amd import SamplingParams
from tests import trace_tools as tt
from tests.conftest import TINY_A, TINY_B
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_greedy_matches_plain_fp32(folder_a, folder_b):
    from return_amd.engine import Engine
    for folder, raw, lens, page in ((folder_a, TINY_A, (5, 17, 33), 16), (folder_b, TINY_B, (1, 8, 31, 64, 100), 32)):
        cfg, w = plain.read_folder(folder)
        prompts = [tt.random_tokens(raw["vocab_size"], n, seed=n) for n in lens]
        want = [plain.greedy_generate(cfg, w, p, 16) for p in prompts]
        eng = Engine(folder, dtype="float32", page_size=page, max_token=2048, max_reside=4,
                     max_step_tokens=64, prefill_chunk=24)
        got = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=16))
        assert [r.output_ids for r in got] == want
        for r, p in zip(got, prompts):
            seq = p + r.output_ids
            lg = plain.logits(cfg, w, seq[:-1])
            for i, (tok, lp) in enumerate(zip(r.output_ids, r.output_logprobs)):
                assert abs(lp - plain.chosen_logprob(lg[len(p) - 1 + i], tok)) < 2e-4
        assert not eng.runner.cache.live


def test_bf16_generation_follows_plain_within_rounding(folder_b):
    """bfloat16 may flip near-ties; every sampled token must still be one the plain model finds
    nearly as likely as its own choice, and the logprobs must agree within bf16 rounding."""
    from return_amd.engine import Engine
    cfg, w = plain.read_folder(folder_b)
    prompts = [tt.random_tokens(TINY_B["vocab_size"], n, seed=n) for n in (8, 31, 64)]
    eng = Engine(folder_b, check_invariants=True, dtype="bfloat16", page_size=16, max_token=2048, max_reside=4)
    got = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12))
    for r, p in zip(got, prompts):
        seq = p + r.output_ids
        lg = plain.logits(cfg, w, seq[:-1])
        for i, (tok, lp) in enumerate(zip(r.output_ids, r.output_logprobs)):
            row = lg[len(p) - 1 + i].double().log_softmax(-1)
            assert float(row.max() - row[tok]) < 0.05, "sampled a token the plain model finds unlikely"
            assert abs(lp - float(row[tok])) < 0.05


def test_temperature_sampling_reproducible(folder_b):
    from return_amd.engine import Engine
    prompts = [tt.random_tokens(TINY_B["vocab_size"], n, seed=n) for n in (1, 8, 31, 64, 100)]
    sp = [SamplingParams(temperature=0.7, max_new_tokens=20, seed=50 + i) for i in range(5)]
    def run(max_reside, chunk):
        eng = Engine(folder_b, check_invariants=True, dtype="float32", page_size=32, max_token=4096, max_reside=max_reside,
                     max_step_tokens=64, prefill_chunk=chunk, seed=11)
        return [r.output_ids for r in eng.generate(prompts, sp)]
    a, b = run(5, 24), run(2, 1000)
    assert a == b and all(len(x) == 20 for x in a)


def test_top_k_top_p_through_the_engine(folder_a):
    from return_amd.engine import Engine
    cfg, w = plain.read_folder(folder_a)
    prompt = tt.random_tokens(TINY_A["vocab_size"], 12, seed=2)
    eng = Engine(folder_a, check_invariants=True, dtype="float32", page_size=16, max_token=1024, max_reside=4)
    greedy = eng.generate([prompt], SamplingParams(temperature=0.0, max_new_tokens=6))[0].output_ids
    k1 = eng.generate([prompt], SamplingParams(temperature=1.5, top_k=1, max_new_tokens=6))[0].output_ids
    p0 = eng.generate([prompt], SamplingParams(temperature=1.5, top_p=0.0, max_new_tokens=6))[0].output_ids
    assert greedy == k1 == p0 == plain.greedy_generate(cfg, w, prompt, 6)
    # with top_k=3 every token is among the plain model's three most likely
    r = eng.generate([prompt], SamplingParams(temperature=2.0, top_k=3, max_new_tokens=10, seed=5))[0]
    seq = prompt + r.output_ids
    lg = plain.logits(cfg, w, seq[:-1])
    for i, tok in enumerate(r.output_ids):
        assert tok in lg[len(prompt) - 1 + i].topk(3).indices.tolist()


def test_command_line(folder_a, tmp_path):
    cfg, w = plain.read_folder(folder_a)
    reqs = [{"session_id": "s0", "prompt_ids": tt.random_tokens(256, 9, seed=1), "max_new_tokens": 5, "temperature": 0.0},
            {"session_id": "s1", "prompt_ids": tt.random_tokens(256, 20, seed=2), "max_new_tokens": 3, "temperature": 0.0,
             "stop_ids": [[999]], "top_k": 0, "top_p": 1.0}]
    f = tmp_path / "reqs.jsonl"
    f.write_text("\n".join(json.dumps(r) for r in reqs))
    out = subprocess.run([sys.executable, "-m", "return_amd.cli", "generate", "--model", folder_a, "--dtype", "float32",
                          "--max-reside", "4", "--max-token", "1024", "--requests", str(f)],
                         cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    lines = [json.loads(l) for l in out.stdout.strip().splitlines()]
    assert [l["session_id"] for l in lines] == ["s0", "s1"]
    for l, r in zip(lines, reqs):
        assert set(l) == {"session_id", "output_ids", "output_logprobs", "num_tokens", "finish_reason"}
        assert l["output_ids"] == plain.greedy_generate(cfg, w, r["prompt_ids"], r["max_new_tokens"])
        assert l["finish_reason"] == "length" and l["num_tokens"] == r["max_new_tokens"]
    bad = subprocess.run([sys.executable, "-m", "return_amd.cli", "generate", "--model", folder_a, "--requests", "-"],
                         cwd=ROOT, input=json.dumps({"prompt_ids": [1], "swap": [3], "swap_at": 0}), capture_output=True,
                         text=True, timeout=300)
    assert bad.returncode != 0 and "paragraph" in bad.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_kept_sessions_on_the_gpu(folder_b, dtype):
    """Three turns of three sessions through the graphs: every turn repeats the conversation so far
    and adds to it; only the addition is computed. In 32-bit the answers are the plain
    implementation's on the whole prompts; in bfloat16 every token is the plain implementation's
    choice at its place, or its second choice where the two are nearly tied."""
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    cfg, w = plain.read_folder(folder_b)
    V = TINY_B["vocab_size"]
    sp = SamplingParams(temperature=0.0, max_new_tokens=7)
    eng = Engine(folder_b, check_invariants=True, dtype=dtype, page_size=16, max_token=2048, max_reside=4, max_step_tokens=64, prefill_chunk=32)
    convs = {k: tt.random_tokens(V, n, seed=n) for k, n in (("a", 5), ("b", 33), ("c", 70))}
    for turn in range(3):
        ids = list(convs)
        out = eng.generate([convs[k] for k in ids], sp, session_ids=ids, keep=turn < 2)
        for k, r in zip(ids, out):
            if dtype == "float32":
                assert r.output_ids == plain.greedy_generate(cfg, w, convs[k], 7)
            else:
                rows = plain.logits(cfg, w, convs[k] + r.output_ids[:-1])[len(convs[k]) - 1:]
                for row, tok in zip(rows, r.output_ids):
                    top = row.topk(2)
                    assert tok == int(top.indices[0]) or \
                        (tok == int(top.indices[1]) and float(top.values[0] - top.values[1]) < 0.05)
            assert (r.cached_tokens > 0) == (turn > 0) and r.cached_tokens < len(convs[k])
            convs[k] = convs[k] + r.output_ids + tt.random_tokens(V, 3 + turn, seed=turn * 10 + len(convs[k]))
        eng.runner.cache.check_invariants()
    assert not eng.runner.cache.live and all(g.pages.in_use() == 0 for g in eng.runner.cache.groups)


@pytest.mark.parametrize("lookahead", [True, False])
def test_kept_sessions_that_end_on_a_stop_sequence_found_a_step_late(folder_b, lookahead):
    """Kept sessions, stop sequences, graphs and steps launched ahead together, over three turns: with
    steps launched ahead a stop sequence is found when the next step, which feeds the last token back,
    is already under way, so the kept cache holds one token more than without; the next turn repeats
    the conversation and must find every one of them right. 32-bit: the answers are the plain
    implementation's, cut after the stop sequence."""
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    cfg, w = plain.read_folder(folder_b)
    V = TINY_B["vocab_size"]
    eng = Engine(folder_b, check_invariants=True, dtype="float32", page_size=16, max_token=2048, max_reside=4, max_step_tokens=64,
                 prefill_chunk=32, use_graphs=True, lookahead=lookahead, tune_products=False)
    convs = {k: tt.random_tokens(V, n, seed=90 + n) for k, n in (("a", 6), ("b", 31), ("c", 70), ("d", 16))}
    stop_after = {"a": 3, "b": 9, "c": 1, "d": None}           # d runs to its length
    for turn in range(3):
        ids = list(convs)
        free = {k: plain.greedy_generate(cfg, w, convs[k], 12) for k in ids}
        params, want = [], {}
        for k in ids:
            n = stop_after[k]
            if n is None:
                params.append(SamplingParams(temperature=0.0, max_new_tokens=12))
                want[k] = (free[k], "length")
                continue
            stop = free[k][n:n + 2]
            first = next(i for i in range(1, 12) if free[k][i - 1:i + 1] == stop)      # (it may come earlier by chance)
            params.append(SamplingParams(temperature=0.0, max_new_tokens=12, stop_ids=[stop]))
            want[k] = (free[k][:first + 1], "stop")
        out = eng.generate([convs[k] for k in ids], params, session_ids=ids, keep=turn < 2)
        for k, r in zip(ids, out):
            assert (r.output_ids, r.finish_reason) == want[k], (turn, k)
            assert (r.cached_tokens > 0) == (turn > 0) and r.cached_tokens < len(convs[k])
            if turn > 0:
                assert r.cached_tokens >= held[k] - 1           # all but at most the last token fed back
            convs[k] = convs[k] + r.output_ids + tt.random_tokens(V, 2 + turn, seed=turn * 7 + len(convs[k]))
        held = {k: eng.runner.cache.seq_len(k) for k in ids} if turn < 2 else {}
        eng.runner.cache.check_invariants()
    assert eng.runner._graphs
    assert not eng.runner.cache.live and all(g.pages.in_use() == 0 for g in eng.runner.cache.groups)


def test_command_line_turns_of_a_session(folder_a, tmp_path):
    """A session_id that comes again is the session's next turn: its cache was kept for it."""
    cfg, w = plain.read_folder(folder_a)
    first = tt.random_tokens(256, 19, seed=3)
    a1 = plain.greedy_generate(cfg, w, first, 4)
    second = first + a1 + [7, 8, 9]
    reqs = [{"session_id": "s", "prompt_ids": first, "max_new_tokens": 4, "temperature": 0.0},
            {"session_id": "u", "prompt_ids": [5, 6], "max_new_tokens": 2, "temperature": 0.0},
            {"session_id": "s", "prompt_ids": second, "max_new_tokens": 3, "temperature": 0.0}]
    out = subprocess.run([sys.executable, "-m", "return_amd.cli", "generate", "--model", folder_a, "--dtype", "float32",
                          "--max-reside", "4", "--max-token", "1024", "--requests", "-", "--stats"], cwd=ROOT,
                         input="\n".join(json.dumps(r) for r in reqs), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    lines = [json.loads(l) for l in out.stdout.strip().splitlines()]
    assert [l["session_id"] for l in lines] == ["s", "u", "s"]
    assert lines[0]["output_ids"] == a1 and lines[2]["output_ids"] == plain.greedy_generate(cfg, w, second, 3)
    assert lines[2]["cached_tokens"] == len(first) + 3 and "cached_tokens" not in lines[1]
    stats = json.loads(out.stderr.strip().splitlines()[-1])
    assert stats["resident"] == 0 and stats["kv_used"] == [0]


def test_a_cache_that_cannot_fit_is_refused_before_it_is_allocated(folder_a):
    from return_amd.engine import Engine
    with pytest.raises(ValueError, match=r"max_token=1073741824 takes .* GiB.*would fit"):
        Engine(folder_a, dtype="float32", page_size=16, max_token=2 ** 30, max_reside=2)


def test_the_library_is_the_one_that_runs():
    """The HIP library is loaded in this process; there is nothing else behind the kernels."""
    from return_amd.kernels.hip_ops import HipOps
    HipOps("cuda:0")
    with open("/proc/self/maps") as f:
        assert "libreturn_amd.so" in f.read()
