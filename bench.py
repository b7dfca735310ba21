#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Qwen3-8B shape, random weights.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole batch through the engine's own step function and
sampler (greedy), as generation runs it. Prints ONE JSON line. For --gpus > 1 it says that
this engine runs on one GPU and exits with 2.

What the reference's benches measure (definitions only, no numbers are published):
decode tok/s = bs*steps/wall after warm-up (rollout/utils/bench_sym.py:24-62), prefill
tok/s = ctx/mean(dt) (rollout/utils/bench_prefill.py:22-49).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

# the headline configuration: Qwen3-8B shape
QWEN3_8B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=151936, hidden_size=4096,
    num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
    intermediate_size=12288, max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1e6,
    tie_word_embeddings=False)
FULL_LAYERS = 36
CONTEXT = 2048          # every request's prefix when decoding starts
MAX_CONTEXT = 8192      # the cache holds this many tokens per request
PAGE = 16
PREFILL_TOKENS = 2048


def build_runner(layers, dtype, max_reside, seed=0, use_graphs=True, raw=None, std=0.02, **engine_options):
    """A runner with random weights made on the GPU. raw: config.json keys (default: the 8B shape
    with ``layers`` layers); engine_options override the engine configuration of the headline run."""
    import torch
    import return_amd.models  # noqa: F401
    from return_amd.config import EngineConfig, Qwen3Config
    from return_amd.engine import ModelRunner
    from return_amd.config import lookup_architecture
    from return_amd.weights import random_weights

    raw = dict(QWEN3_8B, num_hidden_layers=layers) if raw is None else raw
    cfg = Qwen3Config.from_dict(raw)
    _, build_spec = lookup_architecture(cfg.architecture)
    weights = random_weights(build_spec(cfg), seed=seed, std=std, dtype=dtype, device="cuda:0",
                             generator_device="cuda:0")
    options = dict(dtype=dtype, page_size=PAGE, max_token=max_reside * MAX_CONTEXT,
                   max_reside=max_reside, max_step_tokens=max(PREFILL_TOKENS, max_reside),
                   prefill_chunk=PREFILL_TOKENS, use_graphs=use_graphs)
    options.update(engine_options)
    runner = ModelRunner(config=cfg, weights=weights, engine_config=EngineConfig(**options))
    del weights
    torch.cuda.empty_cache()
    return cfg, runner


def weight_bytes(cfg, elt):
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    per_layer = ((cfg.q_width + 2 * cfg.kv_width) * H + H * cfg.q_width + 3 * H * I) * elt + 2 * H * 4 \
        + 2 * cfg.head_dim * 4
    return cfg.num_hidden_layers * per_layer + V * H * elt + H * 4


def kv_bytes_per_token(cfg, elt):
    return 2 * cfg.kv_width * elt * cfg.num_hidden_layers


def prefill_flops(cfg, T):
    H, I = cfg.hidden_size, cfg.intermediate_size
    linear = ((cfg.q_width + 2 * cfg.kv_width) * H + H * cfg.q_width + 3 * H * I) * cfg.num_hidden_layers
    attn = cfg.num_hidden_layers * 2 * T * T * cfg.num_attention_heads * cfg.head_dim   # causal QK^T + PV
    return 2 * T * linear + attn + 2 * cfg.vocab_size * H


def seat_requests(runner, batch, context, seed=1):
    """Live requests that already hold ``context`` tokens: pages are taken through the cache
    manager and filled with random keys and values (their content does not change the work)."""
    import torch
    ids = [f"r{i}" for i in range(batch)]
    for rid in ids:
        runner.add_request(rid)
        runner.cache.begin_step([(rid, context)])
        runner.cache.end_step()
    g = torch.Generator(device="cuda:0").manual_seed(seed)
    for grp in runner.cache.groups:
        grp.pool.normal_(0.0, 0.5, generator=g)
    return ids


def decode_steps(runner, ids, steps, warmup, vocab):
    """warmup untimed steps, then exactly ``steps`` timed; returns seconds. As the engine decodes:
    every step is launched before the one before it is collected, its tokens taken over on the device."""
    import torch
    n = len(ids)
    toks = [(7 * i + 3) % vocab for i in range(n)]
    zeros, ones, rows = [0.0] * n, [1.0] * n, list(range(n))

    launched = 0

    def launch():
        nonlocal launched
        first = launched == 0
        launched += 1
        return runner.decode_launch(ids, toks if first else None, zeros, [0] * n, ones, zeros,
                                    feed_rows=None if first else rows)

    def run(count):
        """count steps, each launched before the one before it is collected; all collected at the end"""
        ticket = None
        for _ in range(count):
            ahead = launch()
            if ticket is not None:
                runner.decode_collect(ticket)
            ticket = ahead
        if ticket is not None:
            runner.decode_collect(ticket)

    run(warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(steps)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def measured_peaks(runner, dtype):
    """What this machine reaches, measured in this run: GB/s of a plain read-only kernel over 2 GiB that
    nothing else touches, and TFLOP/s of one library product of the prefill's largest shape
    (2,048 x 4,096 times 12,288 x 4,096, random operands, the compute dtype)."""
    import torch
    ops = runner.rt.ops
    out = {}
    buf = torch.empty(2 << 30, dtype=torch.uint8, device="cuda:0")
    buf.random_(0, 256)
    best = None
    for _ in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ops.stream_read(buf)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    out["read_GBs"] = round(buf.numel() / best / 1e9, 1)
    del buf
    td = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    a = torch.randn(2048, 4096, device="cuda:0").to(td)
    b = torch.randn(12288, 4096, device="cuda:0").to(td)
    reps, best = 8, None
    for _ in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            torch.matmul(a, b.t())
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / reps
        best = dt if best is None else min(best, dt)
    out["product_TFLOPs"] = round(2.0 * 2048 * 4096 * 12288 / best / 1e12, 1)
    torch.cuda.empty_cache()
    return out


PROFILE_KERNELS = True      # --no-kernels: no profiler pass of bench.py's own (for runs under another profiler)


def kernel_split(run, steps):
    """Device time of `steps` calls of run() by kernel, from a profiler pass of its own (outside every
    timed region; what rollout/utils/prof_graph.py:64-101 does for the reference's decode): the ten
    kernels that take the most time, in microseconds per call, the rest as "other", and the sum."""
    import re
    import torch
    from torch.profiler import ProfilerActivity, profile
    if not PROFILE_KERNELS:
        return {"skipped": "--no-kernels"}
    try:
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            for _ in range(steps):
                run()
            torch.cuda.synchronize()
            # (the tracer hands over its last records late: without a pause the step's last kernels are missing)
            torch.zeros(1, device="cuda:0").add_(1)
            torch.cuda.synchronize()
            time.sleep(0.2)
        per = {}
        for e in prof.key_averages():
            us = getattr(e, "self_device_time_total", 0) or getattr(e, "self_cuda_time_total", 0)
            if us > 0 and not e.key.startswith("Memcpy") and not e.key.startswith("Memset"):
                name = re.sub(r"^void ", "", e.key)
                # (the hand-written products keep their template arguments: they say which form ran)
                name = re.sub(r"\(.*", "", name) if name.startswith("gemm_") else re.sub(r"[<(].*", "", name)
                tile = re.search(r"_(MT\d+x\d+x\d+)_", e.key)
                if e.key.startswith(("Cijk_", "Custom_Cijk_")) and tile:     # the library's products differ by their tile
                    name = "library product " + tile.group(1)
                name = name if len(name) <= 48 else name[:45] + "..."
                calls, total = per.get(name, (0, 0.0))
                per[name] = (calls + e.count, total + us)
        if not per:
            return {"error": "the profiler saw no kernels"}
        top = sorted(per.items(), key=lambda kv: -kv[1][1])
        out = {name: {"us": round(us / steps, 1), "calls": round(calls / steps, 1)} for name, (calls, us) in top[:10]}
        rest = sum(us for _, (_, us) in top[10:])
        if rest > 0:
            out["other"] = {"us": round(rest / steps, 1), "calls": round(sum(c for _, (c, _) in top[10:]) / steps, 1)}
        out["sum_us"] = round(sum(us for _, us in per.values()) / steps, 1)
        return out
    except Exception as error:          # a measurement beside the bench: its failure is reported, not raised
        return {"error": f"{type(error).__name__}: {error}"[:200]}


def release(runner, ids):
    for rid in ids:
        runner.free_request(rid)


def hbm_roofline(cfg, elt, batch, mean_ctx, ms, peaks=None):
    """Bytes a decode step has to read (every weight once, the cache of `batch` live requests of mean_ctx
    tokens) over its time, against the published read rate and the one measured in this run."""
    step_bytes = weight_bytes(cfg, elt) + batch * mean_ctx * kv_bytes_per_token(cfg, elt)
    got = step_bytes / (ms * 1e-3) / 1e9
    r = {"bound": "hbm", "achieved": round(got, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
         "frac": round(got / PEAK_HBM_GBS, 4)}
    if peaks:
        r["measured_peak"] = peaks["read_GBs"]
        r["frac_of_measured"] = round(got / peaks["read_GBs"], 4)
    return r


def prefill_record(cfg, dtype, tokens, secs, count=1, peaks=None, flops=None):
    """tok/s of `count` prompts of `tokens` tokens in `secs`, with the fraction of the published matrix rate
    and of the library product's rate measured in this run."""
    f = count * prefill_flops(cfg, tokens) if flops is None else flops
    r = {"value": round(count * tokens / secs, 1), "tokens": count * tokens, "ms": round(secs * 1e3, 3),
         "frac": round(f / secs / PEAK_FLOPS[dtype], 4)}
    if peaks:
        r["measured_peak_TFLOPs"] = peaks["product_TFLOPs"]
        r["frac_of_measured"] = round(f / secs / (peaks["product_TFLOPs"] * 1e12), 4)
    return r


def decode_point(runner, cfg, elt, batch, ctx, steps, warmup, peaks=None, kernels=False):
    """Seats `batch` requests at ctx tokens, times `steps` decode steps after `warmup`, gives the requests
    back. tok/s, ms a step and the roofline; with kernels the step's time by kernel from a pass of its own."""
    ids = seat_requests(runner, batch, ctx)
    secs = decode_steps(runner, ids, steps, warmup, cfg.vocab_size)
    ms = secs / steps * 1e3
    out = {"tok_s": round(batch * steps / secs, 1), "ms_per_step": round(ms, 4)}
    out.update(hbm_roofline(cfg, elt, batch, ctx + warmup + (steps + 1) / 2.0, ms, peaks))
    if kernels:
        def one_step():
            t = runner.decode_launch(ids, None, [0.0] * batch, [0] * batch, [1.0] * batch, [0.0] * batch,
                                     feed_rows=list(range(batch)))
            runner.decode_collect(t)
        out["kernels"] = kernel_split(one_step, 4)
    release(runner, ids)
    return out


# the two other shapes of the benchmark, each with its own workload
QWEN3_4B = dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, tie_word_embeddings=True)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=64,
                 intermediate_size=25600)


def shape_of(cfg, **more):
    d = {"hidden": cfg.hidden_size, "layers": cfg.num_hidden_layers, "heads": cfg.num_attention_heads,
         "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size,
         "vocab": cfg.vocab_size, "page_size": PAGE, "parallelism": "single GPU"}
    d.update(more)
    return d


def continuous_4b(args):
    """Continuous batching on the Qwen3-4B shape: 128 requests, prompts of 64 to 4,096 tokens and
    32 to 512 new tokens each (uniform), prompts in portions of 512 beside the decoded tokens (up to
    --step-tokens tokens a step), as Engine.generate runs them. value: generated tokens a second over
    the whole run."""
    import random
    import torch
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    n = args.batch if args.batch != 8 else 128
    # A step's token budget: every decoding request's token and up to four portions of 512 prompt tokens. What
    # a step costs whatever it brings (the weights read once, the decode attention of every live request) is
    # shared by more prompt tokens then: one portion a step gives 3,840 generated tok/s, four 4,660, sixteen 4,860.
    budget = args.step_tokens or 2048 + n
    cfg, runner = build_runner(0, args.dtype, n, raw=QWEN3_4B, use_graphs=not args.no_graphs,
                               tune_products=not args.no_tune, defer_norms=not args.no_defer_norms,
                               max_token=n * 4608, max_step_tokens=budget, prefill_chunk=512)
    elt = 2 if args.dtype == "bfloat16" else 4
    peaks = measured_peaks(runner, args.dtype)
    eng = Engine(runner=runner)
    rnd = random.Random(0)
    prompts = [[rnd.randrange(cfg.vocab_size) for _ in range(rnd.randint(64, 4096))] for _ in range(n)]
    params = [SamplingParams(temperature=0.0, max_new_tokens=rnd.randint(32, 512)) for _ in range(n)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reqs = [eng.submit(p, sp) for p, sp in zip(prompts, params)]
    # the steps one by one, as Engine.generate runs them; beside each what it had to read, so that the run's
    # last stretch, in which every prompt is done and the steps only decode, gets a roofline of its own
    log = []                                    # (seconds since t0, brought a prompt portion, requests, cached tokens)
    while eng.scheduler.has_work() or eng._in_flight is not None:
        before = eng.prefill_tokens
        live = [runner.cache.seq_len(rid) for rid in runner.cache.live]
        eng.step()
        log.append((time.perf_counter() - t0, eng.prefill_tokens != before, len(live), sum(live)))
    torch.cuda.synchronize()
    secs = time.perf_counter() - t0
    out = [eng.result_of(r) for r in reqs]
    if any(r.num_tokens != p.max_new_tokens for r, p in zip(out, params)):
        raise RuntimeError("a request ended early")
    runner.cache.check_invariants()
    made, read = sum(r.num_tokens for r in out), sum(map(len, prompts))
    flops = 2.0 * (read + made) * (weight_bytes(cfg, 1) - cfg.vocab_size * cfg.hidden_size)
    first = len(log)
    while first > 0 and not log[first - 1][1]:
        first -= 1
    tail = log[first:-1] if len(log) - first > 2 else []       # (the very last call only collects)
    tail_record = None
    if tail:
        t_tail = tail[-1][0] - (log[first - 1][0] if first else 0.0)
        ms = t_tail / len(tail) * 1e3
        mean_batch = sum(x[2] for x in tail) / len(tail)
        mean_ctx = sum(x[3] for x in tail) / max(1.0, sum(x[2] for x in tail))
        tail_record = dict(hbm_roofline(cfg, elt, mean_batch, mean_ctx, ms, peaks), steps=len(tail),
                           ms_per_step=round(ms, 4), mean_batch=round(mean_batch, 1), mean_context=round(mean_ctx, 1))
    # a decode step of 64 requests at 2,048 tokens on this shape, with its time by kernel (outside the timed run)
    decode64 = decode_point(runner, cfg, elt, 64, 2048, 16, 4, peaks, kernels=True)
    return {"metric": "generated tok/s, continuous batching (Qwen3-4B shape, random weights)",
            "value": round(made / secs, 1), "unit": "tok/s", "n_gpus": 1, "steps": eng.steps, "warmup": 0,
            "ms_per_step": round(secs / eng.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": shape_of(cfg, model="Qwen3-4B shape", global_batch=n, prompt_tokens=read, new_tokens=made,
                               prefill_chunk=512, step_tokens=budget, max_context=4608, hip_graphs=not args.no_graphs,
                               weights="random N(0,0.02)"),
            "seconds": round(secs, 3), "measured": peaks,
            # the whole run as matrix work: prompt and generated tokens through every projection
            "prefill": dict(prefill_record(cfg, args.dtype, read, secs, peaks=peaks, flops=flops), new_tokens=made),
            "roofline": tail_record,            # of the steps after the last prompt portion, which only decode
            "decode_b64_ctx2048": decode64}


def long_32b(args):
    """Long contexts on the Qwen3-32B shape: 16 prompts of 8,192 tokens (one portion each), then
    decoding at batch 16, then one prompt of 32,768 tokens in portions of 8,192. value: decoded
    tokens a second."""
    import random
    import torch
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    elt = 2 if args.dtype == "bfloat16" else 4
    n, ctx, new, long_ctx = 16, 8192, max(2, args.steps), 32768
    cfg, runner = build_runner(0, args.dtype, n, raw=QWEN3_32B, std=0.01, use_graphs=not args.no_graphs,
                               tune_products=not args.no_tune, defer_norms=not args.no_defer_norms,
                               max_token=n * (ctx + 512) + long_ctx, max_step_tokens=ctx, prefill_chunk=ctx)
    peaks = measured_peaks(runner, args.dtype)
    eng = Engine(runner=runner)
    rnd = random.Random(1)
    prompts = [[rnd.randrange(cfg.vocab_size) for _ in range(ctx)] for _ in range(n)]
    sp = SamplingParams(temperature=0.0, max_new_tokens=new)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reqs = [eng.submit(p, sp) for p in prompts]
    while any(not r.output for r in reqs):
        eng.step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    d0, n0 = eng.decode_tokens, eng.steps
    while eng.scheduler.has_work():
        eng.step()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    runner.cache.check_invariants()
    steps, made = eng.steps - n0, eng.decode_tokens - d0
    ms_step = (t2 - t1) / steps * 1e3
    long_prompt = [rnd.randrange(cfg.vocab_size) for _ in range(long_ctx)]
    best = None
    for _ in range(2):
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        eng.generate([long_prompt], SamplingParams(temperature=0.0, max_new_tokens=1))
        torch.cuda.synchronize()
        dt = time.perf_counter() - t3
        best = dt if best is None else min(best, dt)

    # the same decode step again with its time by kernel (a pass of its own, outside the timed run)
    again = decode_point(runner, cfg, elt, n, ctx, 8, 2, peaks, kernels=True)
    return {"metric": "decode tok/s at batch 16, 8,192-token prompts (Qwen3-32B shape, random weights)",
            "value": round(made / (t2 - t1), 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 0,
            "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": shape_of(cfg, model="Qwen3-32B shape", global_batch=n, seq_len=ctx, new_tokens=new,
                               long_prompt=long_ctx, prefill_chunk=ctx, hip_graphs=not args.no_graphs,
                               weights="random N(0,0.01)"),
            "measured": peaks, "roofline": hbm_roofline(cfg, elt, n, ctx + new / 2.0, ms_step, peaks),
            "prefill": prefill_record(cfg, args.dtype, ctx, t1 - t0, n, peaks),
            "prefill_long": prefill_record(cfg, args.dtype, long_ctx, best, 1, peaks),
            "kernels": again.pop("kernels")}


def contexts_8b(args):
    """The 8B shape at further context lengths: decode at batch 1, 8, 16, 32 and 64 over contexts of 8,192
    and 32,768 tokens (batch 64 at 32,768 would need 309 GB of cache and is left out), each with the
    fraction of the read roofline, published and measured in this run; prompts of 16,384 and 32,768
    tokens in one portion and of 32,768 in portions of 8,192; and what sampling with top_p = 0.9 costs at
    64 rows of this vocabulary beside greedy sampling. value: decode tok/s at batch 8 over 8,192 tokens."""
    import torch
    from return_amd.engine import StepEntry
    elt = 2 if args.dtype == "bfloat16" else 4
    points = {}
    cfg = runner = peaks = kernels = None
    k, w = max(8, min(args.steps, 32)), min(args.warmup, 4)
    for ctx, batches in ((8192, (1, 8, 16, 32, 64)), (32768, (1, 8, 16, 32))):
        del runner
        torch.cuda.empty_cache()
        cfg, runner = build_runner(args.layers, args.dtype, max_reside=max(batches), use_graphs=not args.no_graphs,
                                   tune_products=not args.no_tune, max_token=max(batches) * (ctx + 256))
        peaks = peaks or measured_peaks(runner, args.dtype)
        for b in batches:
            pt = decode_point(runner, cfg, elt, b, ctx, k, w, peaks, kernels=(ctx == 8192 and b == 8))
            kernels = pt.pop("kernels", kernels)
            points[f"decode_b{b}_ctx{ctx}"] = pt
    # ---- sampling at 64 rows of the full vocabulary: greedy, temperature 1 alone, with top_p 0.9, with top_k 50;
    # on flat rows (N(0, 3): thresholds are searched over the whole row) and on rows shaped like a language
    # model's (a bulk of N(0, 1.5), 500 tokens at 10 to 20 and one at 24: thresholds from the list of the largest)
    gen = torch.Generator(device="cuda:0").manual_seed(5)
    flat = torch.randn(64, cfg.vocab_size, device="cuda:0", generator=gen) * 3.0
    peaked = torch.randn(64, cfg.vocab_size, device="cuda:0", generator=gen) * 1.5
    for r in range(64):
        idx = torch.randperm(cfg.vocab_size, device="cuda:0", generator=gen)[:500]
        peaked[r, idx] = 10.0 + 10.0 * torch.rand(500, device="cuda:0", generator=gen)
        peaked[r, idx[0]] = 24.0
    sampling = {}
    for prefix, logits in (("", flat), ("peaked_", peaked)):
        for name, temp, top_p in (("greedy", 0.0, 1.0), ("temperature_1", 1.0, 1.0), ("top_p_0.9", 1.0, 0.9),
                                  ("top_k_50", 1.0, 1.0)):
            best = None
            for _ in range(5):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                runner.sample(logits, [temp] * 64, [50 if name == "top_k_50" else 0] * 64, [top_p] * 64, [0.37] * 64)
                dt = time.perf_counter() - t0
                best = dt if best is None else min(best, dt)
            sampling[prefix + name + "_us"] = round(best * 1e6, 1)
    del flat, peaked
    # ---- long prompts: 16,384 and 32,768 tokens in one portion each, 32,768 in portions of 8,192
    del runner
    torch.cuda.empty_cache()
    longest = 32768
    cfg, runner = build_runner(args.layers, args.dtype, max_reside=2, use_graphs=False, tune_products=not args.no_tune,
                               max_token=longest + 256, max_step_tokens=longest, prefill_chunk=longest)
    prefills = {}
    for n, portion in ((16384, 16384), (longest, longest), (longest, 8192)):
        prompt = [(13 * i + 5) % cfg.vocab_size for i in range(n)]
        times = []
        for _ in range(3):
            runner.add_request("p")
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for at in range(0, n, portion):
                last = at + portion >= n
                out = runner.step([StepEntry("p", prompt[at:at + portion], [portion - 1] if last else [])])
            out.sum().item()
            times.append(time.perf_counter() - t0)
            runner.free_request("p")
        name = f"prefill_{n}" + ("" if portion == n else f"_in_portions_of_{portion}")
        prefills[name] = prefill_record(cfg, args.dtype, n, min(times[1:]), 1, peaks)
    head = points["decode_b8_ctx8192"]
    line = {"metric": "decode tok/s at batch 8 over 8,192-token contexts (Qwen3-8B shape, random weights)",
            "value": head["tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": k, "warmup": w,
            "ms_per_step": head["ms_per_step"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic",
            "config": shape_of(cfg, model="Qwen3-8B shape", global_batch=8, seq_len=8192, hip_graphs=not args.no_graphs,
                               weights="random N(0,0.02)"),
            "measured": peaks, "roofline": {x: head[x] for x in head if x not in ("tok_s", "ms_per_step")},
            "kernels": kernels, "points": points, "sampling_64_rows": sampling}
    line.update(prefills)
    return line


def decode_shape(args, raw, name, std):
    """Decode at batch 1, 8 and 64 over 2,048-token prefixes on another shape of the family, as the headline
    run does on the 8B shape: tok/s, ms a step and the read roofline (published and measured in this run) per
    point, the time by kernel at batch 8. value: decode tok/s at batch 8."""
    elt = 2 if args.dtype == "bfloat16" else 4
    cfg, runner = build_runner(0, args.dtype, 64, raw=raw, std=std, use_graphs=not args.no_graphs,
                               tune_products=not args.no_tune, defer_norms=not args.no_defer_norms)
    peaks = measured_peaks(runner, args.dtype)
    k, w = max(8, min(args.steps, 32)), min(args.warmup, 4)
    points = {f"decode_b{b}": decode_point(runner, cfg, elt, b, CONTEXT, k, w, peaks, kernels=(b == 8))
              for b in (1, 8, 64)}
    head = points["decode_b8"]
    kernels = head.pop("kernels")
    return {"metric": f"decode tok/s ({name} shape, random weights)", "value": head["tok_s"], "unit": "tok/s",
            "n_gpus": 1, "steps": k, "warmup": w, "ms_per_step": head["ms_per_step"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic",
            "config": shape_of(cfg, model=f"{name} shape", global_batch=8, seq_len=CONTEXT, max_context=MAX_CONTEXT,
                               hip_graphs=not args.no_graphs, weights=f"random N(0,{std})"),
            "measured": peaks, "roofline": {x: head[x] for x in head if x not in ("tok_s", "ms_per_step")},
            "kernels": kernels, "points": points}


def products_8b(args):
    """The products of a 2,048-token prefill on the Qwen3-8B shape, one by one: the library's product
    (what the engine uses at these row counts) beside the hand-written tiled MFMA product that stands in
    where the library cannot be used. Weights of a shape are taken in turn, operands are random."""
    import torch
    from return_amd.kernels.hip_ops import HipOps
    ops = HipOps("cuda:0")
    torch.manual_seed(0)
    rows = 2048
    out = {}
    for name, N, K in (("qkv", 6144, 4096), ("o", 4096, 4096), ("gate_up", 24576, 4096), ("down", 4096, 12288)):
        ws = [(torch.randn(N, K, device="cuda:0") * 0.02).to(torch.bfloat16) for _ in range(4)]
        x = torch.randn(rows, K, device="cuda:0").to(torch.bfloat16)
        flops = 2.0 * rows * N * K
        got = {}
        for how in ("library", "mfma"):
            secs = ops._time_over(lambda w, how=how: ops._linear_by(how, x, w, torch.bfloat16), ws, 8)
            got[how] = {"us": round(secs * 1e6, 1), "TFLOPs": round(flops / secs / 1e12, 1)}
        out[name] = got
        del ws
    return {"metric": "products of a 2,048-token prefill, library and hand-written (Qwen3-8B shape)", "unit": "TFLOP/s",
            "n_gpus": 1, "dtype": "bf16", "data": "synthetic", "rows": rows, "products": out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="decode_8b",
                    choices=["decode_8b", "continuous_4b", "long_32b", "contexts_8b", "products_8b", "decode_4b",
                             "decode_32b"],
                    help="decode_8b: the headline run; the others: the 4B and 32B shapes with their own "
                         "workloads (one JSON line each, other fields)")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=FULL_LAYERS)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--no-graphs", action="store_true", help="launch every kernel from the host instead of replaying HIP graphs")
    ap.add_argument("--page-size", type=int, default=PAGE, help=f"tokens per cache page (the benchmark's is {PAGE})")
    ap.add_argument("--no-defer-norms", action="store_true",
                    help="run every RMSNorm as a kernel of its own instead of inside the products around it")
    ap.add_argument("--step-tokens", type=int, default=0,
                    help="continuous_4b: token budget of a step (default: 2,048 prompt tokens beside one token of every request)")
    ap.add_argument("--no-kernels", action="store_true",
                    help="leave out the profiler passes that split a step's time by kernel (for runs under rocprofv3)")
    ap.add_argument("--no-tune", action="store_true",
                    help="choose the kernel of every projection by rule instead of measuring at load "
                         "(keeps the measuring launches out of a profile)")
    args = ap.parse_args()
    global PROFILE_KERNELS
    PROFILE_KERNELS = not args.no_kernels
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible")
        return 1
    if args.workload != "decode_8b":
        print(json.dumps({"continuous_4b": continuous_4b, "long_32b": long_32b,
                          "contexts_8b": contexts_8b, "products_8b": products_8b,
                          "decode_4b": lambda a: decode_shape(a, QWEN3_4B, "Qwen3-4B", 0.02),
                          "decode_32b": lambda a: decode_shape(a, QWEN3_32B, "Qwen3-32B", 0.01)}[args.workload](args)))
        return 0
    elt = 2 if args.dtype == "bfloat16" else 4
    cfg, runner = build_runner(args.layers, args.dtype, max_reside=max(64, args.batch),
                               use_graphs=not args.no_graphs, tune_products=not args.no_tune,
                               defer_norms=not args.no_defer_norms, page_size=args.page_size)
    V = cfg.vocab_size

    def roofline(batch, ms, new_before, steps):
        """The step's roofline at the mean length of the live requests over the timed steps."""
        return hbm_roofline(cfg, elt, batch, CONTEXT + new_before + (steps + 1) / 2.0, ms, peaks)

    peaks = None if args.no_points else measured_peaks(runner, args.dtype)

    # ---- headline: decode at the given batch
    ids = seat_requests(runner, args.batch, CONTEXT)
    secs = decode_steps(runner, ids, args.steps, args.warmup, V)
    ms_step = secs / args.steps * 1e3
    value = args.batch * args.steps / secs
    headline = roofline(args.batch, ms_step, args.warmup, args.steps)
    kernels = None
    if not args.no_points:              # where the step's time goes, from a pass of its own after the timed one
        def one_step():
            n = args.batch
            t = runner.decode_launch(ids, None, [0.0] * n, [0] * n, [1.0] * n, [0.0] * n, feed_rows=list(range(n)))
            runner.decode_collect(t)
        kernels = kernel_split(one_step, 4)
    release(runner, ids)

    points, point_rooflines, prefill, prefill_kernels = {}, {}, None, None
    if not args.no_points:
        for b in (1, 16, 32, 64):
            if b == args.batch:
                continue
            k = max(8, min(args.steps, 32))
            pt = decode_point(runner, cfg, elt, b, CONTEXT, k, min(args.warmup, 4), peaks)
            points[f"decode_b{b}"] = pt.pop("tok_s")
            point_rooflines[f"decode_b{b}"] = pt
        # ---- prefill of one 2,048-token prompt, logits at the last place
        from return_amd.engine import StepEntry
        prompt = [(13 * i + 5) % V for i in range(PREFILL_TOKENS)]
        times = []

        def one_prefill():
            runner.add_request("p")
            out = runner.step([StepEntry("p", prompt, [PREFILL_TOKENS - 1])])
            out.sum().item()
            runner.free_request("p")
        for it in range(4):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            one_prefill()
            times.append(time.perf_counter() - t0)
        prefill = prefill_record(cfg, args.dtype, PREFILL_TOKENS, min(times[1:]), 1, peaks)
        prefill_kernels = kernel_split(one_prefill, 2)

    line = {
        "metric": "decode tok/s (Qwen3-8B shape, random weights)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": "Qwen3-8B shape", "layers": args.layers, "layers_full": FULL_LAYERS,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate_size, "vocab": V, "global_batch": args.batch,
                   "seq_len": CONTEXT, "max_context": MAX_CONTEXT, "page_size": args.page_size,
                   "new_tokens": args.warmup + args.steps, "parallelism": "single GPU",
                   "hip_graphs": not args.no_graphs, "tuned_products": not args.no_tune,
                   "norms_in_products": not args.no_defer_norms, "weights": "random N(0,0.02)"},
        "roofline": headline,
    }
    if peaks:
        line["measured"] = peaks
    if kernels:
        line["kernels"] = kernels
    if prefill_kernels:
        line["prefill_kernels"] = prefill_kernels
    plan = getattr(runner.rt.ops, "product_plan", None)
    if plan:            # where the measurement at load replaced the rule: rows x N x K -> way
        line["product_plan"] = {f"{rows}x{n}x{k}{'g' if gated else ''}": how
                                for (rows, n, k, gated, _), how in sorted(plan.items(), key=str)}
    if prefill:
        line["prefill"] = prefill
    if points:
        points[f"decode_b{args.batch}"] = round(value, 1)
        line["points"] = points
        line["point_rooflines"] = point_rooflines
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
