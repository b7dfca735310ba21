"""Engine: requests in, generated tokens out.

The reference's Python entry point is ``await Engine.submit(Request(...))``
(rollout/engine.py:341-344) with a loop that admits, prefills and decodes
(350-409), and a response of output_ids, output_logprobs, num_tokens and
finish_reason ("length" or "stop", rollout/engine_actor.py:66-78). This engine is
synchronous: submit() queues a request, step() runs one scheduler step, generate()
drives a list of prompts to the end. Token ids in, token ids out; like the
reference's server it never tokenises.
"""
from __future__ import annotations

import dataclasses
import time
from typing import Dict, List, Optional, Sequence, Union

from ..config.engine import EngineConfig
from ..sampling.params import SamplingParams, UniformStream
from .runner import ModelRunner, StepEntry
from .scheduler import Request, Scheduler


@dataclasses.dataclass
class GenerationResult:
    """Fields of the reference's response (rollout/engine_actor.py:73-78)."""
    output_ids: List[int]
    output_logprobs: List[float]
    num_tokens: int
    finish_reason: str                      # "length" | "stop" | "error"
    error: Optional[str] = None
    cached_tokens: int = 0                  # tokens of the prompt that a kept session still held


class Engine:
    def __init__(self, model: Optional[str] = None, *, runner: Optional[ModelRunner] = None,
                 max_token: Optional[int] = None, max_reside: Optional[int] = None,
                 engine_config: Optional[EngineConfig] = None, **options):
        """model: a folder with config.json and model.safetensors.

        max_token (tokens the cache holds) and max_reside (most live requests) carry the
        reference's names (rollout/server.py:90-91); other options are EngineConfig fields.
        """
        if runner is None:
            ec = engine_config or EngineConfig(**options)
            if max_token is not None:
                ec.max_token = int(max_token)
            if max_reside is not None:
                ec.max_reside = int(max_reside)
            ec.max_step_tokens = max(ec.max_step_tokens, ec.max_reside)
            runner = ModelRunner(model, engine_config=ec)
        self.runner = runner
        ec = runner.engine_config
        self.config = ec
        self.scheduler = Scheduler(runner.cache, ec.max_reside, ec.max_step_tokens, ec.prefill_chunk,
                                   runner.max_position)
        self._submitted = 0
        self._in_flight = None              # (ticket, plan) of a step that was launched and not yet collected
        # running totals as in rollout/engine.py:84-125
        self.prefill_tokens = 0
        self.decode_tokens = 0
        self.step_seconds = 0.0
        self.decode_seconds = 0.0
        self.prefill_seconds = 0.0
        self.steps = 0
        self._t_start = time.perf_counter()
        self._decode_streak = 0             # steps that only decoded since the last step with a prompt portion
        self._streak_total = 0
        self._streak_count = 0

    # ------------------------------------------------------------------ requests
    def submit(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None,
               request_id=None, keep: bool = False, token_columns=None) -> Request:
        """Queue a request. request_id names its session (the reference's session_id,
        rollout/server.py:25-42); with keep, what the cache holds when it ends stays under that id,
        and a later request with the same id whose prompt repeats those tokens and goes on computes
        only the rest (rollout/engine.py:266-274, 286-306). release() gives a kept session back.
        token_columns: name -> one integer per prompt token, for a model whose parts read further
        integers per token beside the position (see Request)."""
        params = params or SamplingParams()
        self.check_prompt(prompt_ids)
        n = self._submitted
        self._submitted += 1
        unknown = set(token_columns or ()) - set(self.runner.builder.token_columns)
        if unknown:
            raise ValueError(f"token column(s) {sorted(unknown)}: the model reads {list(self.runner.builder.token_columns)}")
        r = Request(request_id if request_id is not None else n, prompt_ids, params, keep=keep,
                    token_columns=token_columns)
        r.stream = UniformStream(self.config.seed, params.seed if params.seed is not None else n)
        self.scheduler.add(r)
        return r

    def release(self, request_id) -> bool:
        """Give back what a kept session holds (the reference's /release, rollout/engine.py:276-284);
        a session still under way is given back when it ends. Returns whether the id was known."""
        return self.scheduler.release(request_id)

    def check_prompt(self, prompt_ids: Sequence[int], name="the request") -> None:
        """Raises ValueError for a prompt that can never run: empty, or a token outside the vocabulary."""
        if len(prompt_ids) == 0:
            raise ValueError(f"{name} has an empty prompt")
        for t in prompt_ids:
            if not 0 <= int(t) < self.runner.vocab_size:
                raise ValueError(f"{name}: prompt token {t} outside the vocabulary of {self.runner.vocab_size}")

    # ------------------------------------------------------------------ one step
    def _launch(self, plan, previous=None):
        """Start a plan; returns the ticket to collect its sampled tokens with. previous: the plan
        under way whose sampled tokens, still on the device, are the tokens of this plan's entries
        that hold None (their rows among previous's sampled entries are looked up by request)."""
        sampled = [e.request for e in plan.entries if e.sample]
        options = ([r.params.temperature for r in sampled], [r.params.top_k for r in sampled],
                   [r.params.top_p for r in sampled], [r.stream.next() for r in sampled])
        row_of = {}
        if previous is not None:
            row_of = {e.request.id: i for i, e in enumerate(x for x in previous.entries if x.sample)}
        unknown = [e.tokens[0] is None for e in plan.entries]
        if all(e.sample and len(e.tokens) == 1 for e in plan.entries) and (all(unknown) or not any(unknown)):
            # one token each (decoded tokens, or prompts of one token), all known or all still on the
            # device: one call that runs the model and the sampler (from a graph if enabled)
            ids = [e.request.id for e in plan.entries]
            columns = [e.request.columns_at(e.start, 1) for e in plan.entries]
            columns = columns if any(columns) else None
            if all(unknown):
                return self.runner.decode_launch(ids, None, *options, feed_rows=[row_of[i] for i in ids],
                                                 columns=columns)
            return self.runner.decode_launch(ids, [e.tokens[0] for e in plan.entries], *options, columns=columns)
        entries = [StepEntry(e.request.id, e.tokens, [len(e.tokens) - 1] if e.sample else [],
                             e.request.columns_at(e.start, len(e.tokens))) for e in plan.entries]
        feed = [(i, row_of[e.request.id]) for i, e in enumerate(plan.entries) if e.tokens[0] is None]
        return self.runner.step_launch(entries, *options, feed=feed)

    def _book(self, plan, sampled, t0):
        only_decode = all(len(e.tokens) == 1 and e.request.output for e in plan.entries if not e.request.finished)
        for e in plan.entries:
            if e.request.finished:
                continue
            if len(e.tokens) == 1 and e.request.output:
                self.decode_tokens += 1
            else:
                self.prefill_tokens += len(e.tokens)
        ended = self.scheduler.finish_step(plan, sampled)
        dt = time.perf_counter() - t0
        self.step_seconds += dt
        if only_decode:
            self.decode_seconds += dt               # steps that only decode
            self._decode_streak += 1
        else:
            self.prefill_seconds += dt              # steps that bring prompt portions (decoded tokens beside them)
            if self._decode_streak > 0:             # a run of decode steps ends (rollout/engine.py:361-364)
                self._streak_total += self._decode_streak
                self._streak_count += 1
                self._decode_streak = 0
        self.steps += 1
        return ended

    def _collect(self, ticket, plan, t0):
        sampled_entries = [e for e in plan.entries if e.sample]
        sampled = {}
        if sampled_entries:
            toks, logps = self.runner.decode_collect(ticket)
            sampled = {e.request.id: (t, lp) for e, t, lp in zip(sampled_entries, toks, logps)}
        return self._book(plan, sampled, t0)

    def step(self) -> List[Request]:
        """One scheduler step; returns the requests that ended in it (finished or failed).

        A step is launched and collected in two halves: while it runs, the step after it is
        decided (Scheduler.schedule_ahead) and launched, its tokens taken over on the device, so
        that the device does not wait for the host between steps.
        """
        t0 = time.perf_counter()
        ended: List[Request] = []
        if self._in_flight is None:
            plan = self.scheduler.schedule()
            ended += plan.failed
            if not plan.entries:
                return ended
            ticket = self._launch_or_run(plan)
            if not self.config.lookahead:
                return ended + self._collect(ticket, plan, t0)
            self._in_flight = (ticket, plan)
        ticket, plan = self._in_flight
        ahead = self.scheduler.schedule_ahead(plan) if self.config.lookahead else None
        following = None
        if ahead is not None:
            ended += ahead.failed
            if ahead.entries:
                following = (self._launch_or_run(ahead, previous=plan), ahead)
        ended += self._collect(ticket, plan, t0)
        self._in_flight = following
        return ended

    def _launch_or_run(self, plan, previous=None):
        """_launch, or for a plan in which nothing is sampled (prompt portions only) the plain step.
        If the step cannot be started, its requests fail with the error (what they hold goes back,
        as in the reference's _fail, rollout/engine.py:317-324) and the error is raised."""
        try:
            if any(e.sample for e in plan.entries):
                return self._launch(plan, previous)
            self.runner.step([StepEntry(e.request.id, e.tokens, [], e.request.columns_at(e.start, len(e.tokens)))
                              for e in plan.entries])
            return None
        except Exception as error:
            for e in plan.entries:
                if not e.request.finished:
                    self.scheduler.abort(e.request, error)
            raise

    # ------------------------------------------------------------------ whole jobs
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 session_ids: Optional[Sequence] = None, keep: bool = False,
                 token_columns: Optional[Sequence] = None) -> List[GenerationResult]:
        """Generate for every prompt (lists of token ids); results come in the prompts' order.
        session_ids name the requests (distinct within one call); with keep their caches stay
        for a later call that goes on with the same sessions. token_columns: per prompt, what
        submit() takes under that name (or None)."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but {len(params)} sampling parameter sets")
        if session_ids is not None and (len(session_ids) != len(prompts) or len(set(session_ids)) != len(prompts)):
            raise ValueError("session_ids must name every prompt, each differently")
        for i, p in enumerate(prompts):               # all of them before any is queued
            self.check_prompt(p, f"prompt {i}")
        if token_columns is not None and len(token_columns) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but token columns for {len(token_columns)}")
        requests = [self.submit(p, sp, request_id=None if session_ids is None else session_ids[i], keep=keep,
                                token_columns=None if token_columns is None else token_columns[i])
                    for i, (p, sp) in enumerate(zip(prompts, params))]
        while self.scheduler.has_work() or self._in_flight is not None:
            before = (self.steps, len(self.scheduler.waiting), len(self.scheduler.running))
            self.step()
            if before == (self.steps, len(self.scheduler.waiting), len(self.scheduler.running)):
                raise RuntimeError("scheduler made no progress")     # cannot happen; guards the loop
        return [self.result_of(r) for r in requests]

    @staticmethod
    def result_of(r: Request) -> GenerationResult:
        return GenerationResult(list(r.output), list(r.output_logprobs), len(r.output),
                                r.finish_reason or "error", str(r.error) if r.error else None, r.resumed)

    def stats(self) -> dict:
        cache = self.runner.cache
        run = time.perf_counter() - self._t_start
        return {"steps": self.steps, "prefill_tokens": self.prefill_tokens,
                "decode_tokens": self.decode_tokens, "step_seconds": self.step_seconds,
                # the reference's decode_tps / prefill_tps (rollout/engine.py:104-110): tokens over the
                # time of the steps of that kind (decoded tokens of mixed steps count as decoded)
                "decode_tps": self.decode_tokens / self.decode_seconds if self.decode_seconds > 0 else None,
                "prefill_tps": self.prefill_tokens / self.prefill_seconds if self.prefill_seconds > 0 else None,
                # share of the time since the engine was made that went into steps of each kind, and the
                # mean number of decode-only steps between two steps that brought prompt portions
                # (decode_duty, prefill_duty, decode_streak of rollout/engine.py:113-125)
                "run_seconds": run,
                "decode_duty": self.decode_seconds / run if run > 0 else 0.0,
                "prefill_duty": self.prefill_seconds / run if run > 0 else 0.0,
                "decode_streak": self._streak_total / self._streak_count if self._streak_count else None,
                "running": len(self.scheduler.running), "waiting": len(self.scheduler.waiting),
                "resident": len(self.scheduler.resident),
                "kv_used": [g.pages.in_use() for g in cache.groups],
                "kv_total": [g.num_pages for g in cache.groups]}
