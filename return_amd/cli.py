"""Command line of the engine.

    python -m return_amd.cli generate --model DIR [--max-reside N] [--max-token N] ...
    python -m return_amd.cli random-model --config config.json --out DIR [--seed S] ...
    python -m return_amd.cli replay --model DIR --dtype ... --out DIR --max-tokens N   (= bin/trace_run)

Option names follow the reference's server (rollout/server.py:87-98): --model, --max-reside
(most live requests), --max-token (tokens the cache holds). Requests carry the fields of its
GenRequest (rollout/server.py:25-42): session_id, prompt_ids, stop_ids, max_new_tokens,
temperature, top_p, top_k; unknown fields are refused as there (extra="forbid"), and so are
the paragraph fields (split_ids, subs, swap, ephem_at, swap_at), which this engine does not
have. Answers carry output_ids, output_logprobs, num_tokens, finish_reason
(rollout/engine_actor.py:73-78). Token ids in and out; nothing is tokenised.
"""
from __future__ import annotations

import argparse
import json
import sys

REQUEST_FIELDS = {"session_id", "prompt_ids", "stop_ids", "max_new_tokens", "temperature", "top_p",
                  "top_k", "seed"}
PARAGRAPH_FIELDS = {"split_ids", "subs", "swap", "ephem_at", "swap_at"}


def parse_request(raw: dict, number: int):
    from .sampling import SamplingParams
    unknown = set(raw) - REQUEST_FIELDS
    para = sorted(k for k in unknown & PARAGRAPH_FIELDS if raw[k] not in (None, [], ()))
    if para:
        raise ValueError(f"request {number}: paragraph fields are not supported: {', '.join(para)}")
    unknown -= PARAGRAPH_FIELDS
    if unknown:
        raise ValueError(f"request {number}: unknown field(s) {', '.join(sorted(unknown))}")
    if "prompt_ids" not in raw:
        raise ValueError(f"request {number}: prompt_ids is required")
    params = SamplingParams(
        temperature=float(raw.get("temperature", 1.0)), top_p=float(raw.get("top_p", 1.0)),
        top_k=int(raw.get("top_k", 0)), max_new_tokens=int(raw.get("max_new_tokens", 1024)),
        stop_ids=raw.get("stop_ids", []), seed=raw.get("seed"))
    return raw.get("session_id", str(number)), list(raw["prompt_ids"]), params


def cmd_generate(args) -> int:
    from .engine import Engine
    raws = []
    if args.prompt_ids:
        raws.append({"session_id": "0", "prompt_ids": [int(t) for t in args.prompt_ids.split(",")],
                     "max_new_tokens": args.max_new_tokens, "temperature": args.temperature,
                     "top_p": args.top_p, "top_k": args.top_k,
                     "stop_ids": json.loads(args.stop_ids) if args.stop_ids else []})
    if args.requests:
        src = sys.stdin if args.requests == "-" else open(args.requests)
        raws += [json.loads(line) for line in src if line.strip()]
    if not raws:
        print("generate: give --prompt-ids or --requests", file=sys.stderr)
        return 2
    parsed = [parse_request(r, i) for i, r in enumerate(raws)]
    engine = Engine(args.model, max_token=args.max_token, max_reside=args.max_reside, dtype=args.dtype,
                    page_size=args.page_size, seed=args.seed, max_step_tokens=args.max_step_tokens,
                    prefill_chunk=args.prefill_chunk, use_graphs=not args.no_graphs,
                    tune_products=not args.no_tune, defer_norms=not args.no_defer_norms,
                    check_invariants=args.check_invariants)
    # Requests are run together until a session_id comes again: that request is a later turn of the
    # session (the reference keeps a session's cache for its next request, rollout/engine.py:286-306,
    # which sends the whole conversation again, 266-274). A session's cache is kept while more of
    # its turns follow.
    start = 0
    while start < len(parsed):
        end, seen = start, set()
        while end < len(parsed) and parsed[end][0] not in seen:
            seen.add(parsed[end][0])
            end += 1
        later = {sid for sid, _, _ in parsed[end:]}
        turn = parsed[start:end]
        results = [None] * len(turn)
        for keep in (True, False):                 # one call for the sessions that go on, one for the others
            idx = [i for i, (sid, _, _) in enumerate(turn) if (sid in later) == keep]
            if idx:
                got = engine.generate([turn[i][1] for i in idx], [turn[i][2] for i in idx],
                                      session_ids=[turn[i][0] for i in idx], keep=keep)
                for i, r in zip(idx, got):
                    results[i] = r
        for (sid, _, _), r in zip(turn, results):
            out = {"session_id": sid, "output_ids": r.output_ids, "output_logprobs": r.output_logprobs,
                   "num_tokens": r.num_tokens, "finish_reason": r.finish_reason}
            if r.cached_tokens:
                out["cached_tokens"] = r.cached_tokens
            if r.error:
                out["error"] = r.error
            print(json.dumps(out), flush=True)
        start = end
    if args.stats:
        print(json.dumps(engine.stats()), file=sys.stderr)
    return 0


def cmd_random_model(args) -> int:
    import return_amd.models  # noqa: F401
    from .config import load_config
    from .weights import write_model_folder
    cfg = load_config(args.config)
    write_model_folder(args.out, cfg, seed=args.seed, std=args.std, embedding_std=args.embedding_std,
                       norm_jitter=args.norm_jitter, dtype=args.dtype)
    print(args.out)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="return_amd")
    sub = ap.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate for requests given as token ids")
    g.add_argument("--model", required=True)
    g.add_argument("--max-reside", type=int, default=128)
    g.add_argument("--max-token", type=int, default=1048576)
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    g.add_argument("--page-size", type=int, default=16)
    g.add_argument("--max-step-tokens", type=int, default=8192)
    g.add_argument("--prefill-chunk", type=int, default=8192)
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--no-graphs", action="store_true",
                   help="launch every kernel of a decode step from the host instead of replaying HIP graphs")
    g.add_argument("--no-defer-norms", action="store_true",
                   help="run every RMSNorm as a kernel of its own instead of inside the products around it")
    g.add_argument("--no-tune", action="store_true",
                   help="choose the kernel of every projection by rule instead of measuring at load")
    g.add_argument("--check-invariants", action="store_true",
                   help="debugging: check after every step that no cache page or slot is lost or held twice")
    g.add_argument("--requests", help="file of JSON lines (or - for standard input), one request each")
    g.add_argument("--prompt-ids", help="one prompt as comma-separated token ids")
    g.add_argument("--max-new-tokens", type=int, default=32)
    g.add_argument("--temperature", type=float, default=1.0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--stop-ids", help='JSON list of stop sequences, e.g. "[[5, 6], [9]]"')
    g.add_argument("--stats", action="store_true")
    g.set_defaults(fn=cmd_generate)

    r = sub.add_parser("random-model", help="write a model folder with random weights")
    r.add_argument("--config", required=True, help="config.json of the architecture")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--std", type=float, default=0.02)
    r.add_argument("--embedding-std", type=float, default=None)
    r.add_argument("--norm-jitter", type=float, default=0.01)
    r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    r.set_defaults(fn=cmd_random_model)

    p = sub.add_parser("replay", help="feed given token ids step by step and write logits (bin/trace_run)",
                       add_help=False)
    p.set_defaults(fn=None)

    args, rest = ap.parse_known_args(argv)
    if args.command == "replay":
        from .engine.replay import main as replay_main
        return replay_main(rest)
    if rest:
        ap.error(f"unrecognized arguments: {' '.join(rest)}")
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
