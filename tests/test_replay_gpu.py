"""Replay on the GPU: the same requests whole, with a decoded tail, in portions of changing
size and mixed with page reuse, in 32-bit and in bfloat16, against the plain implementation."""
import pytest
import torch

from tests import trace_tools as tt
from tests.conftest import TINY_A, TINY_A_PAGE, TINY_B, TINY_B_PAGE, TINY_C
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

LENGTHS = {"a": 5, "b": 17, "c": 33, "d": 100, "e": 64, "f": 150, "g": 1, "h": 47}
# float32: ten times the largest difference that these traces have shown (1.9e-6). bfloat16: three times
# the largest (0.014 on logits whose largest is 1.35), and per row the reference's own bound on a bf16 kernel against 32-bit, a relative L2 of 2e-2
# (rollout/utils/test_prefill_fwd_bwd.py:117)
TOL = {"float32": dict(atol=2e-5, rtol=1e-4), "bfloat16": dict(atol=4e-2, rtol=5e-2)}
REL_L2 = {"float32": 1e-4, "bfloat16": 2e-2}


def requests_for(vocab, max_pos):
    return {rid: tt.random_tokens(vocab, min(n, max_pos), seed=ord(rid)) for rid, n in LENGTHS.items()}


def oracle(folder, requests):
    cfg, w = plain.read_folder(folder)
    return {rid: plain.logits(cfg, w, toks) for rid, toks in requests.items()}


def make_runner(folder, dtype, max_tokens, page=16):
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner
    ec = EngineConfig(dtype=dtype, page_size=page, max_token=max_tokens, max_reside=4,
                      max_step_tokens=max(max_tokens, 4), prefill_chunk=max_tokens)
    return ModelRunner(folder, engine_config=ec)


def compare(got, want, requests, dtype):
    worst = 0.0
    for rid, toks in requests.items():
        for p in range(len(toks)):
            assert (rid, p) in got, f"no logits for request {rid} position {p}"
            a, b = got[(rid, p)], want[rid][p]
            err = (a - b).abs().max().item()
            worst = max(worst, err)
            try:
                torch.testing.assert_close(a, b, **TOL[dtype])
            except AssertionError as e:
                raise AssertionError(f"request {rid} position {p} (first wrong place): {e}") from None
            rel = ((a - b).norm() / b.norm()).item()
            assert rel < REL_L2[dtype], f"request {rid} position {p} (first wrong place): relative L2 {rel:.3e}"
            if dtype == "float32":
                assert int(a.argmax()) == int(b.argmax()), f"request {rid} position {p}: argmax differs"
    return worst


@pytest.fixture(scope="module", params=["a", "b", "c"])
def model(request, folder_a, folder_b, folder_c):
    folder = {"a": folder_a, "b": folder_b, "c": folder_c}[request.param]
    raw = {"a": TINY_A, "b": TINY_B, "c": TINY_C}[request.param]
    reqs = requests_for(raw["vocab_size"], raw["max_position_embeddings"])
    # every configuration at its own page size
    page = {"a": TINY_A_PAGE, "b": TINY_B_PAGE, "c": 16}[request.param]
    return folder, raw, reqs, oracle(folder, reqs), page


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail_decoded", "portions", "mixed"])
def test_replay_matches_plain(model, dtype, cut):
    folder, raw, reqs, want, page = model
    steps = {"whole": tt.whole, "tail_decoded": tt.tail_decoded, "portions": tt.portions,
             "mixed": tt.mixed}[cut](reqs)
    # the pool holds exactly the trace's peak, so pages of ended requests are used again
    runner = make_runner(folder, dtype, tt.peak_tokens(steps, max(64, page)), page)
    got = tt.run_in_process(runner, steps)
    worst = compare(got, want, reqs, dtype)
    print(f"replay {dtype} {cut} page {page}: largest difference {worst:.2e}")
    assert not runner.cache.live
    assert all(g.pages.in_use() == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("cut", ["tail_decoded", "mixed"])
def test_decode_attention_that_merges_inside_the_workgroup(model, cut):
    """The decode attention merges a request's splits inside one workgroup when the (request, kv
    head) pairs make whole rounds over the CUs, which tiny models never do: here every count is a
    whole round, so that each decoded token of the traces takes that path (requests of every length
    from one token on, beside each other, on pages used again)."""
    folder, raw, reqs, want, page = model
    steps = {"tail_decoded": tt.tail_decoded, "mixed": tt.mixed}[cut](reqs)
    runner = make_runner(folder, "bfloat16", tt.peak_tokens(steps, max(64, page)), page)
    ops = runner.rt.ops
    ops.decode_merge_round = 1
    seen = []
    splits = ops._decode_splits
    ops._decode_splits = lambda *a, **k: (seen.append(splits(*a, **k)) or seen[-1])
    compare(tt.run_in_process(runner, steps), want, reqs, "bfloat16")
    assert any(merge for _, _, merge in seen), "no step took the merging path"


@pytest.mark.parametrize("page", [8, 32, 64])
def test_other_page_sizes(folder_b, page):
    reqs = requests_for(TINY_B["vocab_size"], TINY_B["max_position_embeddings"])
    want = oracle(folder_b, reqs)
    steps = tt.mixed(reqs, seed=page)
    runner = make_runner(folder_b, "float32", tt.peak_tokens(steps, page) + page * 2, page)
    compare(tt.run_in_process(runner, steps), want, reqs, "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(folder_a, tmp_path, dtype):
    """The program itself, as a child process: stdin steps, done lines, .f32 files."""
    reqs = requests_for(TINY_A["vocab_size"], TINY_A["max_position_embeddings"])
    reqs = {k: reqs[k] for k in ("a", "b", "c", "d", "e")}
    want = oracle(folder_a, reqs)
    steps = tt.mixed(reqs, seed=3)
    got = tt.run_program(folder_a, dtype, steps, str(tmp_path / "out"), tt.peak_tokens(steps),
                         TINY_A["vocab_size"])
    compare(got, want, reqs, dtype)
    if dtype == "bfloat16":                      # a second replay gives the same bits
        again = tt.run_program(folder_a, dtype, steps, str(tmp_path / "out2"), tt.peak_tokens(steps),
                               TINY_A["vocab_size"])
        assert got.keys() == again.keys() and all(torch.equal(got[k], again[k]) for k in got)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program_at_the_page_size_of_tiny_b(folder_b, tmp_path, dtype):
    """Tiny B at its own geometry (pages of 32 rows) and with exactly as many request slots as the
    trace has live requests at a time, both given on the command line."""
    reqs = requests_for(TINY_B["vocab_size"], TINY_B["max_position_embeddings"])
    want = oracle(folder_b, reqs)
    steps = tt.mixed(reqs, seed=5)
    got = tt.run_program(folder_b, dtype, steps, str(tmp_path / "out"), tt.peak_tokens(steps),
                         TINY_B["vocab_size"], extra=("--page-size", "32", "--max-live", "4"))
    compare(got, want, reqs, dtype)


def test_trace_run_program_refuses_a_page_size_it_cannot_count_in(folder_a, tmp_path):
    import subprocess
    import sys
    p = subprocess.run([sys.executable, tt.os.path.join(tt.ROOT, "bin", "trace_run"), "--model", folder_a, "--dtype",
                        "float32", "--out", str(tmp_path), "--max-tokens", "64", "--page-size", "24"],
                       stdin=subprocess.DEVNULL, capture_output=True, text=True)
    assert p.returncode == 2 and "--page-size 24" in p.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folder_b, dtype):
    """300 tokens one by one after a short prompt."""
    toks = tt.random_tokens(TINY_B["vocab_size"], 320, seed=77)
    reqs = {"long": toks}
    want = oracle(folder_b, reqs)
    steps = tt.tail_decoded(reqs, tail=300)
    runner = make_runner(folder_b, dtype, 320)
    compare(tt.run_in_process(runner, steps), want, reqs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["a", "b"])
def test_first_tokens_of_a_sequence(folder_a, folder_b, which, dtype):
    """The first places of a sequence, where attention has one key, then two, and the first page
    is not yet full: one request decoded from its very first token, one that starts with two
    tokens and goes on one by one, one that starts with three; all live together."""
    folder, raw = (folder_a, TINY_A) if which == "a" else (folder_b, TINY_B)
    reqs = {rid: tt.random_tokens(raw["vocab_size"], 40, seed=ord(rid)) for rid in "xyz"}
    want = oracle(folder, reqs)
    first = {"x": 1, "y": 2, "z": 3}
    steps = [{"step": 0, "end": [], "entries": [
        {"id": rid, "tokens": reqs[rid][:k], "want": list(range(k))} for rid, k in first.items()]}]
    for i in range(1, 40):
        entries = [{"id": rid, "tokens": [reqs[rid][k + i - 1]], "want": [0]}
                   for rid, k in first.items() if k + i - 1 < 40]
        steps.append({"step": i, "entries": entries, "end": [e["id"] for e in entries if first[e["id"]] + i == 40]})
    runner = make_runner(folder, dtype, tt.peak_tokens(steps))
    compare(tt.run_in_process(runner, steps), want, reqs, dtype)
    assert not runner.cache.live


ODD = [
    # head size, heads, kv heads, width, intermediate, vocabulary, layers, page, tied
    (240, 6, 3, 100, 100, 331, 2, 4, True),       # width no multiple of 8: the plain product; a page of 4
    (16, 60, 3, 96, 328, 1000, 2, 8, True),       # 20 query heads to a kv head: two waves of the decode kernel
    (80, 7, 1, 100, 48, 1000, 1, 32, False),      # 7 heads on one kv head, head size 80
    (256, 5, 5, 136, 100, 97, 2, 48, False),      # the largest head size, a page of 48
    (40, 6, 2, 96, 72, 331, 2, 16, True),         # a head size that is no multiple of 16: the plain attention, in bfloat16 too
    (320, 2, 1, 64, 48, 97, 1, 8, False),         # a head size beyond the MFMA kernels' 256
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("D,Hq,Hkv,H,I,V,L,page,tied", ODD)
def test_odd_configurations(tmp_path, dtype, D, Hq, Hkv, H, I, V, L, page, tied):
    """Sizes at the edges of what the kernels take, or beyond (then the plain kernels must step in):
    a mixed trace with page reuse against the plain implementation."""
    import return_amd.models  # noqa: F401
    from return_amd.config import lookup_architecture
    from return_amd.weights import write_model_folder
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=V, hidden_size=H,
               num_hidden_layers=L, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D,
               intermediate_size=I, max_position_embeddings=256, rms_norm_eps=3e-4, rope_theta=5e4,
               tie_word_embeddings=tied)
    cls, _ = lookup_architecture("Qwen3ForCausalLM")
    folder = str(tmp_path / "model")
    write_model_folder(folder, cls.from_dict(raw), dtype="bfloat16", seed=D, std=0.05, embedding_std=0.05,
                       norm_jitter=0.03)
    reqs = {rid: tt.random_tokens(V, n, seed=ord(rid)) for rid, n in
            {"a": 5, "b": 70, "c": 33, "d": 130, "e": 64, "f": 2, "g": 1}.items()}
    want = oracle(folder, reqs)
    steps = tt.mixed(reqs, seed=D)
    runner = make_runner(folder, dtype, tt.peak_tokens(steps, page) + 2 * page, page)
    compare(tt.run_in_process(runner, steps), want, reqs, dtype)
    assert not runner.cache.live
