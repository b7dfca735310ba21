"""Traces for the replay tests: the same requests cut in different ways."""
from __future__ import annotations

import json
import os
import random
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def random_tokens(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def whole(requests):
    """Each request alone and whole, logits wanted everywhere."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def tail_decoded(requests, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}],
                      "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=(7, 2, 24, 3, 64, 2, 5, 33, 16, 1, 2)):
    """Portions of changing size, down to two tokens (and one)."""
    steps = []
    k = 0
    for rid, toks in requests.items():
        at = 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append({"step": len(steps),
                          "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                          "end": [rid] if at + n == len(toks) else []})
            at += n
    return steps


def mixed(requests, seed=0, max_live=4, decode_tail=12, sizes=(19, 2, 40, 7, 3, 64, 11)):
    """Up to max_live requests at a time; prompt portions of some beside single tokens of others;
    a request's last decode_tail tokens come one per step; some requests sit a step out."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}            # rid -> (tokens, position)
    steps = []
    k = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, ended = [], []
        for rid in list(live):
            toks, at = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                    # left out of this step, goes on later
            left = len(toks) - at
            if left <= decode_tail:
                n = 1
            else:
                n = min(sizes[k % len(sizes)], left - decode_tail)
                k += 1
            entries.append({"id": rid, "tokens": toks[at:at + n], "want": list(range(n))})
            live[rid][1] = at + n
            if at + n == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def peak_tokens(steps, round_to=64):
    """Most tokens live requests hold at any time, each rounded up (what --max-tokens must cover)."""
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def run_in_process(runner, steps):
    """Drive a ModelRunner with a trace; returns {(request, position): logits row (cpu fp32)}."""
    from return_amd.engine.runner import StepEntry
    got, pos = {}, {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if not runner.is_live(e["id"]):
                runner.add_request(e["id"])
                pos[e["id"]] = 0
            entries.append(StepEntry(e["id"], e["tokens"], e["want"], e.get("columns")))
        logits = runner.step(entries)
        if logits is not None:
            logits = logits.float().cpu()
        row = 0
        for e in s["entries"]:
            for w in e["want"]:
                got[(e["id"], pos[e["id"]] + w)] = logits[row]
                row += 1
            pos[e["id"]] += len(e["tokens"])
        for rid in s["end"]:
            runner.free_request(rid)
            pos.pop(rid, None)
        runner.cache.check_invariants()
    return got


def run_program(model_dir, dtype, steps, out_dir, max_tokens, vocab, env=None, extra=()):
    """Drive bin/trace_run as a child process; same result shape as run_in_process."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens), *extra]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    got, pos = {}, {}
    for s in steps:
        p.stdin.write(json.dumps(s) + "\n")
        p.stdin.flush()
        while True:
            line = p.stdout.readline()
            if not line:
                raise RuntimeError(f"trace_run ended early (exit {p.poll()})")
            if line.strip() == f"done {s['step']}":
                break
        path = os.path.join(out_dir, f"{s['step']}.f32")
        n_want = sum(len(e["want"]) for e in s["entries"])
        if n_want:
            arr = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n_want, vocab).copy())
        row = 0
        for e in s["entries"]:
            pos.setdefault(e["id"], 0)
            for w in e["want"]:
                got[(e["id"], pos[e["id"]] + w)] = arr[row]
                row += 1
            pos[e["id"]] += len(e["tokens"])
        for rid in s["end"]:
            pos.pop(rid, None)
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    return got
