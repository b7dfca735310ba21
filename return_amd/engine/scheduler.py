"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.

What it keeps of the reference (rollout/engine.py): a queue of pending requests
and a set of running ones (76-79); admission only while request slots are free and
the pages the newcomer needs fit beside what running requests still need
(_admit, 199-247); a request that can never fit fails at once with KVCapacityError
(219-221); a request ends at max_new_tokens or on a stop sequence (49-57).
What differs: the reference prefills all newly admitted prompts completely before
it decodes again (358-385); here every step mixes one token of each decoding
request with prompt portions, under max_step_tokens. And where the reference lets
decoding requests wait for pages and fails one if none can go on (326-339), here
pages for a request's whole life (prompt + max_new_tokens - 1 tokens) are set
aside when it is admitted, so a running request never runs out: when pages are
short, new requests wait in the queue, in order, until running ones finish.
"""
from __future__ import annotations

import collections
import dataclasses
from typing import Deque, Dict, List, Optional, Sequence, Tuple

from ..cache.manager import CacheManager
from ..cache.pages import KVCapacityError
from ..sampling.params import SamplingParams, UniformStream, ends_with_stop


class Request:
    """One generation request (the reference's Request, rollout/engine.py:13-62, without paragraphs)."""

    def __init__(self, request_id, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None,
                 keep: bool = False, token_columns: Optional[Dict[str, Sequence[int]]] = None):
        """token_columns: name -> one integer per prompt token, for models whose parts read further
        integers per token beside the position (positions along a second axis, say). Tokens beyond
        what a column lists (the generated ones) go on counting from its last value."""
        if len(prompt_ids) == 0:
            raise ValueError(f"request {request_id!r} has an empty prompt")
        self.token_columns = {k: [int(x) for x in v] for k, v in (token_columns or {}).items()}
        for name, col in self.token_columns.items():
            if not 0 < len(col) <= len(prompt_ids):
                raise ValueError(f"request {request_id!r}: token column {name!r} lists {len(col)} values for "
                                 f"{len(prompt_ids)} prompt tokens")
        self.id = request_id
        self.keep = bool(keep)              # what the cache holds stays under this id when the request ends
        self.resumed = 0                    # tokens of the prompt that were found in the cache at admission
        self.prompt_ids = [int(t) for t in prompt_ids]
        self.params = params or SamplingParams()
        self.output: List[int] = []
        self.output_logprobs: List[float] = []
        self.num_computed = 0               # tokens of prompt + output already in the cache
        self.status = "waiting"             # waiting | running | finished | failed
        self.finish_reason: Optional[str] = None
        self.error: Optional[BaseException] = None
        self.max_new = self.params.max_new_tokens   # may be lowered to fit max_position
        self.stream: Optional[UniformStream] = None

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.output)

    @property
    def finished(self) -> bool:
        return self.status in ("finished", "failed")

    def columns_at(self, start: int, n: int) -> Optional[Dict[str, List[int]]]:
        """The request's token columns for its tokens start .. start + n - 1, or None if it brings none."""
        if not self.token_columns:
            return None
        out = {}
        for name, col in self.token_columns.items():
            k = len(col)
            out[name] = [col[i] if i < k else col[-1] + (i - k + 1) for i in range(start, start + n)]
        return out


@dataclasses.dataclass
class PlannedEntry:
    request: Request
    tokens: List[int]
    sample: bool            # the portion reaches the request's last token: its logits are sampled
    start: int = 0          # place of the first of these tokens in the request's sequence


@dataclasses.dataclass
class StepPlan:
    entries: List[PlannedEntry]
    failed: List[Request]

    @property
    def n_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)


class Scheduler:
    def __init__(self, cache: CacheManager, max_reside: int, max_step_tokens: int,
                 prefill_chunk: int, max_position: int):
        if max_step_tokens < max_reside:
            raise ValueError(
                f"max_step_tokens {max_step_tokens} must be at least max_reside {max_reside}: "
                f"every decoding request brings one token to every step")
        self.cache = cache
        self.max_reside = int(max_reside)
        self.max_step_tokens = int(max_step_tokens)
        self.prefill_chunk = int(prefill_chunk)
        self.max_position = int(max_position)
        self.max_portion = min(self.prefill_chunk, self.max_step_tokens)
        self.waiting: Deque[Request] = collections.deque()
        self.running: List[Request] = []
        self._life_pages: Dict[object, List[int]] = {}     # request id -> pages of each group set aside
        # Sessions that ended with keep: id -> the tokens their cache holds, oldest first. The
        # reference keeps every session until it is released (rollout/engine.py:286-306 and 276-284);
        # here a kept session is also given up, oldest first, when a waiting request needs its
        # pages or its slot.
        self.resident: "collections.OrderedDict[object, List[int]]" = collections.OrderedDict()

    # ------------------------------------------------------------------ queue
    def add(self, request: Request) -> None:
        if any(r.id == request.id for r in self.running) or any(r.id == request.id for r in self.waiting):
            raise ValueError(f"request {request.id!r} is already under way")
        request.status = "waiting"
        self.waiting.append(request)

    def release(self, request_id) -> bool:
        """Give back what a kept session holds; one still under way is given back when it ends.
        Returns whether the id was known."""
        if request_id in self.resident:
            del self.resident[request_id]
            self.cache.free_request(request_id)
            return True
        known = False
        for r in list(self.running) + list(self.waiting):
            if r.id == request_id:
                r.keep = False
                known = True
        return known

    def _give_up_oldest(self, spare) -> bool:
        """Frees the kept session that was used longest ago, but not ``spare``."""
        for rid in self.resident:
            if rid != spare:
                del self.resident[rid]
                self.cache.free_request(rid)
                return True
        return False

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ accounting
    def _unclaimed(self) -> List[int]:
        """Free pages of each group minus what running requests may still take."""
        free = self.cache.free_pages()
        for r in self.running:
            held = self.cache.held_pages(r.id)
            for g, life in enumerate(self._life_pages[r.id]):
                free[g] -= max(0, life - held[g])
        return free

    def _try_admit(self, r: Request) -> Optional[bool]:
        """True: admitted. False: must wait. None: failed for good (r.error is set)."""
        n_prompt = len(r.prompt_ids)
        if n_prompt >= self.max_position:
            return self._fail(r, ValueError(
                f"prompt of {n_prompt} tokens leaves no room below max_position_embeddings "
                f"{self.max_position}"))
        r.max_new = min(r.params.max_new_tokens, self.max_position - n_prompt + 1)
        life = self.cache.max_pages(n_prompt + r.max_new - 1, self.max_portion)
        for g, need in enumerate(life):
            if need > self.cache.groups[g].num_pages:
                return self._fail(r, KVCapacityError(
                    f"request needs {need} pages of cache group {g}, the pool has "
                    f"{self.cache.groups[g].num_pages}"))
        # A kept session goes on where it stopped if the prompt repeats what its cache holds and
        # brings at least one token more (the reference strips the cached prefix unchecked,
        # rollout/engine.py:266-274); otherwise what it holds is given back and it starts afresh.
        held = self.resident.get(r.id)
        if held is not None and not (len(held) < n_prompt and r.prompt_ids[:len(held)] == held):
            del self.resident[r.id]
            self.cache.free_request(r.id)
            held = None
        have = self.cache.held_pages(r.id) if held is not None else [0] * len(life)
        others = [rid for rid in self.resident if rid != r.id]
        if held is None and len(self.running) >= self.max_reside:
            return False
        # kept sessions are given up only if that lets the request in
        could = self._unclaimed()
        for rid in others:
            for g, h in enumerate(self.cache.held_pages(rid)):
                could[g] += h
        if any(need - h > c for need, h, c in zip(life, have, could)):
            return False
        while True:
            slots_ok = held is not None or (len(self.running) + len(self.resident) < self.max_reside
                                            and self.cache.free_slots() >= 1)
            pages_ok = all(need - h <= free for need, h, free in zip(life, have, self._unclaimed()))
            if slots_ok and pages_ok:
                break
            if not self._give_up_oldest(spare=r.id):
                return False
        if held is not None:
            del self.resident[r.id]
            r.num_computed = r.resumed = len(held)
        else:
            self.cache.add_request(r.id)
        self._life_pages[r.id] = life
        r.status = "running"
        self.running.append(r)
        return True

    def _fail(self, r: Request, error: BaseException):
        r.status, r.error, r.finish_reason = "failed", error, "error"
        return None

    # ------------------------------------------------------------------ one step
    def schedule(self) -> StepPlan:
        """Decide the next step: one token of every decoding request, then prompt portions."""
        return self._plan({})

    def schedule_ahead(self, plan: StepPlan) -> Optional[StepPlan]:
        """The step after ``plan``, decided while plan is still under way and its sampled tokens
        are not known: the same decisions as schedule(), taken on the state that plan will leave.
        A request that samples in plan decodes next; its token is None here (it is still on the
        device) unless that token is its last (max_new_tokens), then it is left out. A request
        that ends on a stop sequence in plan is found out only later: finish_step then skips its
        entry in the step returned here (the token computed for it is dropped, its pages go back
        with the request). What plan's finished requests hold is given back only when plan is
        booked, so a newcomer may be let in one step later than without looking ahead.
        None: there is nothing to run."""
        under_way = {e.request.id: e for e in plan.entries if not e.request.finished}
        ahead = self._plan(under_way)
        return ahead if ahead.entries or ahead.failed else None

    def _plan(self, under_way: Dict[object, PlannedEntry]) -> StepPlan:
        """under_way: entries of a step that runs but is not booked yet, by request."""
        budget = self.max_step_tokens
        entries: List[PlannedEntry] = []
        failed: List[Request] = []

        def state(r: Request):
            e = under_way.get(r.id)
            computed = r.num_computed + (len(e.tokens) if e is not None else 0)
            outputs = len(r.output) + (1 if e is not None and e.sample else 0)
            return computed, outputs, e

        def portion(r: Request, computed: int):
            nonlocal budget
            n_prompt = len(r.prompt_ids)
            n = min(n_prompt - computed, self.prefill_chunk, budget)
            if n <= 0:
                return
            entries.append(PlannedEntry(r, r.prompt_ids[computed:computed + n], sample=(computed + n == n_prompt),
                                        start=computed))
            budget -= n

        for r in self.running:                      # decoding requests first
            computed, outputs, e = state(r)
            if computed < len(r.prompt_ids) or budget <= 0:
                continue
            if e is not None and e.sample:
                if outputs >= r.max_new:            # the step under way brings its last token
                    continue
                entries.append(PlannedEntry(r, [None], sample=True, start=computed))
            else:
                entries.append(PlannedEntry(r, [r.output[-1]], sample=True, start=computed))
            budget -= 1
        for r in self.running:                      # prompts under way
            computed, _, _ = state(r)
            if computed < len(r.prompt_ids):
                portion(r, computed)
        while self.waiting and budget > 0:          # newcomers, in order
            r = self.waiting[0]
            ok = self._try_admit(r)
            if ok is None:
                self.waiting.popleft()
                failed.append(r)
                continue
            if not ok:
                break
            self.waiting.popleft()
            portion(r, r.num_computed)
        return StepPlan(entries, failed)

    def finish_step(self, plan: StepPlan, sampled: Dict[object, Tuple[int, float]]) -> List[Request]:
        """Book the step: tokens are in the cache, sampled tokens join the outputs. Returns who finished."""
        done = []
        for e in plan.entries:
            r = e.request
            if r.finished:                  # ended while this step, decided ahead, was already under way
                continue
            r.num_computed += len(e.tokens)
            if not e.sample:
                continue
            tok, logp = sampled[r.id]
            r.output.append(int(tok))
            r.output_logprobs.append(float(logp))
            if ends_with_stop(r.output, r.params.stop_ids):
                r.finish_reason = "stop"
            elif len(r.output) >= r.max_new:
                r.finish_reason = "length"
            if r.finish_reason:
                r.status = "finished"
                done.append(r)
        for r in done:
            self.running.remove(r)
            self._life_pages.pop(r.id, None)
            if r.keep:
                # what the cache holds by now: the prompt and the tokens fed back so far (the last one
                # too, if the step after this one was launched before this one's tokens were read)
                self.resident[r.id] = (r.prompt_ids + r.output)[:self.cache.seq_len(r.id)]
            else:
                self.cache.free_request(r.id)
        return done

    def abort(self, r: Request, error: BaseException) -> None:
        """Take a running or waiting request out and give back what it holds."""
        if r in self.running:
            self.running.remove(r)
            self._life_pages.pop(r.id, None)
            self.cache.free_request(r.id)
        elif r in self.waiting:
            self.waiting.remove(r)
        self._fail(r, error)
