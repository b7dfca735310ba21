"""Trace replay: feeds given token ids through the model step by step and writes logits.

In the spirit of the reference's teacher-forced recomputation (opd/replay.py:12-22,
opd/forward.py: forward of given ids over given context; rollout/utils/
kernel_gap_test.py:74-116 recomputes logprobs of recorded tokens): nothing is
sampled. It drives the ModelRunner that generation uses, with its cache manager and
kernels, and has no forward pass, cache or loader of its own.

Input, one JSON object per line on standard input:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step with wanted places it writes <out>/<step>.f32: little-endian float32
[wanted, vocab], in the order of the entries and of their ``want``. After every step
it prints "done <step>". Requests named in ``end`` give back what they hold.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

MAX_LIVE = 8            # default of --max-live: traces keep up to four requests live, with room to spare
PAGE_SIZE = 16          # default of --page-size
ROUND_TO = 64           # a request's token count is rounded up to this for --max-tokens (or to a larger page)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=PAGE_SIZE,
                    help=f"tokens per cache page (default {PAGE_SIZE}): a divisor or a multiple of {ROUND_TO}; with "
                         f"pages beyond {ROUND_TO} a request's count in --max-tokens is rounded up to whole pages")
    ap.add_argument("--max-live", type=int, default=MAX_LIVE,
                    help=f"most requests that are live at a time (default {MAX_LIVE})")
    args = ap.parse_args(argv)
    page = args.page_size
    if page < 1 or (ROUND_TO % page and page % ROUND_TO):
        ap.error(f"--page-size {page}: must divide {ROUND_TO} or be a multiple of it")
    if args.max_live < 1:
        ap.error(f"--max-live {args.max_live}: at least one request")

    from ..config.engine import EngineConfig
    from .runner import ModelRunner, StepEntry

    os.makedirs(args.out, exist_ok=True)
    unit = max(page, ROUND_TO)                  # whole pages, so the pool is exactly max-tokens
    pool = -(-args.max_tokens // unit) * unit
    # products by rule, not by the measurement at load, whose choices may differ from run to run:
    # two replays of a trace give the same bits
    ec = EngineConfig(dtype=args.dtype, page_size=page, max_token=pool, max_reside=args.max_live,
                      max_step_tokens=max(pool, args.max_live), prefill_chunk=pool, tune_products=False)
    runner = ModelRunner(args.model, engine_config=ec)

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            if not runner.is_live(e["id"]):
                runner.add_request(e["id"])
            # ("columns", name -> one integer per token, only for a model whose parts read such columns)
            entries.append(StepEntry(e["id"], e["tokens"], e.get("want", []), e.get("columns")))
        logits = runner.step(entries) if entries else None
        if logits is not None and logits.shape[0] > 0:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            arr.tofile(os.path.join(args.out, f"{step}.f32"))
        for rid in rec.get("end", []):
            if runner.is_live(rid):
                runner.free_request(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
