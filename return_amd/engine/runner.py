"""The model runner: a model, its cache and the ONE step function.

The reference has two entry points, prefill(reqs) for packed prompt pieces and
decode(reqs) for one token per request (rollout/model.py:184-294, 318-343); they
build the same tables and call the same forward. Here both are one step(): every
entry brings a request's next tokens, one or many, cut anywhere, and the logits
come back at the places asked for. Keys and values of the new tokens are written
first and attention then reads everything from the cache, as the reference does
(rollout/monkey_patch/qwen3.py:40-45), so whole prompts, portions and single
tokens take the same path.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.manager import CacheManager
from ..config.base import ModelConfig, load_config, lookup_architecture
from ..config.engine import EngineConfig
from ..models.decoder import Decoder
from ..parts.runtime import Runtime
from ..weights.loader import load_weights
from .batch import StepBatch, StepBuilder


class StepEntry:
    """One request's share of a step: its next tokens and the places (among them) whose logits are wanted.
    columns: name -> one integer per token, for the token columns that parts of the model read beside
    the position (Decoder.step_needs()["token_columns"]); a column that is not given is the position."""
    __slots__ = ("request_id", "tokens", "want", "columns")

    def __init__(self, request_id, tokens: Sequence[int], want: Sequence[int] = (), columns: Optional[dict] = None):
        self.request_id = request_id
        self.tokens = list(tokens)
        self.want = list(want)
        self.columns = columns


class ModelRunner:
    def __init__(self, model_dir: Optional[str] = None, *, config: Optional[ModelConfig] = None,
                 weights: Optional[Dict[str, torch.Tensor]] = None,
                 engine_config: Optional[EngineConfig] = None, ops=None):
        """Either model_dir (config.json + safetensors) or config + weights (name -> tensor)."""
        self.engine_config = ec = engine_config or EngineConfig()
        import return_amd.models  # noqa: F401  (fills the architecture registry)
        if model_dir is not None:
            config = load_config(model_dir)
        if config is None:
            raise ValueError("ModelRunner needs a model folder or a configuration")
        self.config = config
        _, build_spec = lookup_architecture(config.architecture)
        self.spec = build_spec(config)
        self.rt = Runtime(ec.device, ec.dtype, ops=ops)
        if hasattr(self.rt.ops, "defer_norms"):
            self.rt.ops.defer_norms = bool(ec.defer_norms)
        if weights is None:
            if model_dir is None:
                raise ValueError("ModelRunner got a configuration but no weights")
            weights = load_weights(model_dir, self.spec, device=self.rt.device)
        self.model = Decoder(self.spec, weights, self.rt)
        del weights
        if ec.tune_products and self.rt.dtype == torch.bfloat16 and hasattr(self.rt.ops, "tune_products"):
            self.rt.ops.tune_products(self.rt.products, max_rows=ec.max_reside,
                                      max_rows_residual=ec.max_reside + min(ec.max_step_tokens, ec.prefill_chunk))
            if ec.defer_norms and hasattr(self.rt.ops, "tune_norm_pairs"):
                self.rt.ops.tune_norm_pairs(self.rt.norm_pairs, max_rows=ec.max_reside)
        self._check_cache_fits()
        self.cache = CacheManager(self.model.cache_layers(), ec.page_size, ec.max_token,
                                  ec.max_reside, self.rt.dtype, self.rt.device)
        needs = self.model.step_needs()
        self.builder = StepBuilder(self.cache, ec.max_step_tokens, ec.max_reside, self.rt.device,
                                   tile_rows=needs["prefill_tile_rows"], token_columns=needs["token_columns"])
        self.vocab_size = self.spec.vocab_size
        self.max_position = self.spec.max_position
        # decode-only steps replayed from captured HIP graphs (rollout/model.py:346-407 captures one
        # graph per batch size; here one per (batch size, context bucket))
        self._graphs = {}
        self._graph_pool = None
        n = ec.max_reside
        pin = self.rt.device.type == "cuda"
        self._samp_host_f = torch.zeros(3, n, dtype=torch.float32, pin_memory=pin)
        self._samp_host_k = torch.zeros(n, dtype=torch.int32, pin_memory=pin)
        self._samp_dev_f = torch.zeros(3, n, dtype=torch.float32, device=self.rt.device)
        self._samp_dev_k = torch.zeros(n, dtype=torch.int32, device=self.rt.device)
        self._samp_copied = torch.cuda.Event() if pin else None      # the staging above has left for the device
        # Launch and collection of a decode step are two calls, so that the next step can be
        # launched before this one's tokens are read: two pinned result buffers, the tokens of
        # the last launch kept on the device for the next one to pick up.
        self._picked_host = [torch.zeros(n, 2, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._picked_ready = [torch.cuda.Event() if pin else None for _ in range(2)]
        self._feed_host = torch.zeros(n, dtype=torch.int64, pin_memory=pin)
        self._feed_dev = torch.zeros(n, dtype=torch.int64, device=self.rt.device)
        self._feed_at_host = torch.zeros(n, dtype=torch.int64, pin_memory=pin)
        self._feed_at_dev = torch.zeros(n, dtype=torch.int64, device=self.rt.device)
        self._launches = 0
        self._last_picked: Optional[torch.Tensor] = None

    def _check_cache_fits(self) -> None:
        """One clear error, before anything is allocated, when the cache asked for cannot fit beside the weights."""
        if self.rt.device.type != "cuda":
            return
        ec = self.engine_config
        layers = self.model.cache_layers()
        need = CacheManager.pool_bytes(layers, ec.page_size, ec.max_token, ec.max_reside, self.rt.dtype)
        torch.cuda.empty_cache()
        free, _ = torch.cuda.mem_get_info(self.rt.device)
        if need > free:
            per_token = CacheManager.pool_bytes(layers, 1, 1, 0, self.rt.dtype) // 2 or 1
            fits = max(0, free // per_token // ec.page_size - 1) * ec.page_size
            raise ValueError(
                f"the cache for max_token={ec.max_token} takes {need / 2 ** 30:.1f} GiB, but {free / 2 ** 30:.1f} GiB "
                f"of device memory are free beside the weights: about max_token={fits} would fit")

    # ------------------------------------------------------------------ requests
    def add_request(self, request_id) -> None:
        self.cache.add_request(request_id)

    def free_request(self, request_id) -> None:
        self.cache.free_request(request_id)
        if self.engine_config.check_invariants:
            self.cache.check_invariants()

    def _end_step(self) -> None:
        self.cache.end_step()
        if self.engine_config.check_invariants:
            self.cache.check_invariants()

    def is_live(self, request_id) -> bool:
        return request_id in self.cache.live

    def _flat_columns(self, per_entry, tables):
        """name -> the step's T integers of every token column the model reads, from what the entries
        bring (per_entry[i]: name -> one integer per token of entry i, or None); the rest are positions.
        None when no entry brings any."""
        if not any(per_entry):
            return None
        out = {}
        for i, cols in enumerate(per_entry):
            for name, values in (cols or {}).items():
                if name not in self.builder.token_columns:
                    raise ValueError(f"request {tables.request_ids[i]!r} brings token column {name!r}; the model "
                                     f"reads {list(self.builder.token_columns)}")
                a, b = int(tables.cu_q[i]), int(tables.cu_q[i + 1])
                if len(values) != b - a:
                    raise ValueError(f"request {tables.request_ids[i]!r}: token column {name!r} has {len(values)} "
                                     f"entries for {b - a} tokens")
                out.setdefault(name, tables.positions.copy())[a:b] = values
        return out

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run exactly the tokens the entries bring, as one batch, on top of the cache.

        Returns fp32 logits [number of wanted places, vocab] on the device, in the order
        of the entries and of each entry's ``want``; None if nothing is wanted.
        """
        if not entries:
            return None
        return self._run(entries, None)[0]

    def _run(self, entries: Sequence[StepEntry], after_build):
        """Checks, cache tables, device tables, forward. after_build(batch) runs between the copy
        of the tables and the model. Returns (logits or None, batch)."""
        rows: List[int] = []
        at = 0
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.request_id!r} brings no tokens")
            for t in e.tokens:
                if t is not None and not 0 <= int(t) < self.vocab_size:
                    raise ValueError(f"request {e.request_id!r}: token {t} outside the vocabulary of {self.vocab_size}")
            if e.request_id in self.cache.live and self.cache.seq_len(e.request_id) + n > self.max_position:
                raise ValueError(
                    f"request {e.request_id!r} would reach {self.cache.seq_len(e.request_id) + n} tokens, "
                    f"the model's max_position_embeddings is {self.max_position}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise ValueError(f"request {e.request_id!r}: wanted place {w} is not among its {n} tokens")
                rows.append(at + int(w))
            at += n
        tables = self.cache.begin_step([(e.request_id, len(e.tokens)) for e in entries])
        try:
            batch = self.builder.build(tables, [[0 if t is None else t for t in e.tokens] for e in entries], rows,
                                       self._flat_columns([e.columns for e in entries], tables))
            if after_build is not None:
                after_build(batch)
            with torch.no_grad():
                logits = self.model.forward(batch, self.cache)
        finally:
            self._end_step()
        return logits, batch

    def step_launch(self, entries: Sequence[StepEntry], temperature, top_k, top_p, uniforms, feed=None):
        """Start a step of any kind whose wanted places are all sampled, and return a ticket for
        decode_collect. Nothing here waits for the device.

        A token may be None in an entry of one token: then feed lists (entry number, row of the
        previous launch's sampled tokens) and the token is taken from there on the device, so
        that this step can be launched before the previous one's tokens have been read.
        temperature, top_k, top_p, uniforms: one per wanted place, in the entries' order.
        """
        m = sum(len(e.want) for e in entries)
        if m == 0 or m > self.engine_config.max_reside or len(temperature) != m:
            raise ValueError(f"step_launch: {m} sampled places, {len(temperature)} sampling options, "
                             f"at most {self.engine_config.max_reside}")
        feed = list(feed or [])
        fed = {i for i, _ in feed}
        for i, e in enumerate(entries):
            if (None in e.tokens) != (i in fed) or (i in fed and len(e.tokens) != 1):
                raise ValueError("step_launch: tokens that are None and the list of rows to take them from do not match")
        if feed and (self._last_picked is None or
                     any(not 0 <= int(r) < self._last_picked.shape[0] for _, r in feed)):
            raise ValueError("step_launch: a row to take a token from is not a row of the previous launch")

        def take_tokens(batch):
            if feed:
                if self._samp_copied is not None:
                    self._samp_copied.synchronize()      # the last launch's copies have left the staging buffers
                k = len(feed)
                starts = batch.cu_q_host
                self._feed_host[:k] = torch.as_tensor([int(r) for _, r in feed], dtype=torch.int64)
                self._feed_at_host[:k] = torch.as_tensor([starts[i] for i, _ in feed], dtype=torch.int64)
                self._feed_dev[:k].copy_(self._feed_host[:k], non_blocking=True)
                self._feed_at_dev[:k].copy_(self._feed_at_host[:k], non_blocking=True)
                batch.token_ids.index_copy_(0, self._feed_at_dev[:k],
                                            self._last_picked[:, 0].index_select(0, self._feed_dev[:k]))
            self._put_sampling(m, temperature, top_k, top_p, uniforms)

        logits, _ = self._run(entries, take_tokens)
        with torch.no_grad():
            picked = self.rt.ops.sample(logits, self._samp_dev_f[0, :m], self._samp_dev_k[:m],
                                        self._samp_dev_f[1, :m], self._samp_dev_f[2, :m])
        return self._ticket(picked, m, logits)

    def _ticket(self, picked, n, logits):
        slot = self._launches & 1
        self._launches += 1
        self._last_picked = picked
        self._picked_host[slot][:n].copy_(picked[:n], non_blocking=True)
        if self._picked_ready[slot] is not None:
            self._picked_ready[slot].record()
        return (slot, n, logits[:n])

    # ------------------------------------------------------------------ decode from a graph
    def _put_sampling(self, m, temperature, top_k, top_p, uniforms):
        if self._samp_copied is not None:
            self._samp_copied.synchronize()          # the last launch's options have left the staging buffer
        self._samp_host_f[0, :m] = torch.as_tensor(temperature, dtype=torch.float32)
        self._samp_host_f[1, :m] = torch.as_tensor(top_p, dtype=torch.float32)
        self._samp_host_f[2, :m] = torch.as_tensor(uniforms, dtype=torch.float32)
        self._samp_host_k[:m] = torch.as_tensor(top_k, dtype=torch.int32)
        self._samp_dev_f.copy_(self._samp_host_f, non_blocking=True)
        self._samp_dev_k.copy_(self._samp_host_k, non_blocking=True)
        if self._samp_copied is not None:
            self._samp_copied.record()

    def _decode_body(self, batch):
        logits = self.model.forward(batch, self.cache)
        m = batch.n_logit_rows
        picked = self.rt.ops.sample(logits, self._samp_dev_f[0, :m], self._samp_dev_k[:m],
                                    self._samp_dev_f[1, :m], self._samp_dev_f[2, :m])
        return logits, picked

    def decode_launch(self, request_ids, tokens, temperature, top_k, top_p, uniforms, feed_rows=None,
                      columns=None):
        """Start one decode step (one token per request, logits sampled at once) and return a
        ticket for decode_collect. Nothing here waits for the device.

        tokens: the requests' next tokens, or None: then request i takes the token that the
        previous launch sampled in its row feed_rows[i], straight from the device, so that
        this step can be launched before the previous one's tokens have been read.
        With use_graphs the whole step (model and sampler) is one captured HIP graph per
        (batch size, context bucket); tables and sampling options go into fixed buffers first.
        columns: per request, name -> [integer] for the token columns the model reads (or None).
        """
        n = len(request_ids)
        if n == 0:
            raise ValueError("decode_launch: a decode step needs at least one request")
        if tokens is None:
            if self._last_picked is None or feed_rows is None or len(feed_rows) != n:
                raise ValueError("decode_launch without tokens needs a previous launch and its rows to take them from")
            if any(not 0 <= int(r) < self._last_picked.shape[0] for r in feed_rows):
                raise ValueError("decode_launch: a row to take a token from is not a row of the previous launch")
        else:
            for rid, t in zip(request_ids, tokens):
                if not 0 <= int(t) < self.vocab_size:
                    raise ValueError(f"request {rid!r}: token {t} outside the vocabulary of {self.vocab_size}")
        for rid in request_ids:
            if self.cache.seq_len(rid) + 1 > self.max_position:
                raise ValueError(f"request {rid!r} would pass max_position_embeddings {self.max_position}")
        graphs = self.engine_config.use_graphs and self.rt.device.type == "cuda"
        rows = self.graph_batch_size(n) if graphs else n
        pad = rows - n
        # the step's class: what a graph for it is keyed by, with or without graphs
        key = self._graph_key(self.graph_batch_size(n), max(self.cache.seq_len(rid) for rid in request_ids) + 1)
        if graphs and key not in self._graphs:
            self._capture(key)
        tables = self.cache.begin_step([(rid, 1) for rid in request_ids])
        try:
            tables = self.cache.pad_tables(tables, pad)
            host_tokens = [[0]] * rows if tokens is None else [[int(t)] for t in tokens] + [[0]] * pad
            batch = self.builder.build(tables, host_tokens, list(range(rows)),
                                       self._flat_columns(list(columns) + [None] * pad, tables) if columns else None)
            batch.decode_rule = key
            if tokens is None:
                # after the tables' copy and before the step: the sampled tokens become the new tokens
                if self._samp_copied is not None:
                    self._samp_copied.synchronize()      # the last launch's copies have left the staging buffers
                self._feed_host[:n] = torch.as_tensor(list(feed_rows), dtype=torch.int64)
                self._feed_dev[:n].copy_(self._feed_host[:n], non_blocking=True)
                batch.token_ids[:n].copy_(self._last_picked[:, 0].index_select(0, self._feed_dev[:n]))
            # rows that only fill the batch up are chosen greedily and thrown away
            self._put_sampling(rows, list(temperature) + [0.0] * pad, list(top_k) + [0] * pad,
                               list(top_p) + [1.0] * pad, list(uniforms) + [0.0] * pad)
            with torch.no_grad():
                if graphs:
                    logits, picked = self._replay(key)
                else:
                    logits, picked = self._decode_body(batch)
        finally:
            self._end_step()
        return self._ticket(picked, n, logits)

    def decode_collect(self, ticket):
        """Wait for a launched decode step; returns (tokens, logprobs) as Python lists."""
        slot, n, _ = ticket
        if self._picked_ready[slot] is not None:
            self._picked_ready[slot].synchronize()
        host = self._picked_host[slot][:n]
        return host[:, 0].tolist(), host[:, 1].contiguous().view(torch.float32).tolist()

    def decode_and_sample(self, request_ids, tokens, temperature, top_k, top_p, uniforms):
        """decode_launch and decode_collect in one call. Returns (tokens, logprobs, logits); logits
        stay on the device and hold until the next launch."""
        ticket = self.decode_launch(request_ids, tokens, temperature, top_k, top_p, uniforms)
        toks, logps = self.decode_collect(ticket)
        return toks, logps, ticket[2]

    def graph_batch_size(self, n: int) -> int:
        """The batch size whose graph serves n decoding requests: n itself up to 8, then the
        next multiple of 8 (never more than max_reside), so that a batch that shrinks one
        request at a time does not capture a graph per size."""
        if n <= 8:
            return n
        return min(-(-n // 8) * 8, max(n, self.engine_config.max_reside))

    def _graph_key(self, rows: int, longest: int):
        """(batch size, context bucket) of the graph that serves `rows` decoding rows whose longest
        request holds `longest` tokens after the step."""
        bucket = 256
        while bucket < longest:
            bucket *= 2
        return rows, bucket

    def _capture(self, key) -> None:
        """Warms the decode step up and captures it for one (batch size, context bucket), on rows that
        belong to no request: every row sits on the spare page and the spare state slot. A step is
        not idempotent in general (a mixer with state of fixed size advances it), so nothing that a
        request holds may be touched by the warm-up; the first real step of this shape is a replay
        like every later one. What a launch derives from the context length (grid, split size,
        scratch) derives from the bucket here, and so holds for every replay."""
        rows, bucket = key
        dev = self.rt.device
        tables = self.cache.pad_tables(self.cache.begin_step([]), rows)
        try:
            batch = self.builder.build(tables, [[0]] * rows, list(range(rows)))
            batch.max_decode_seq_len = bucket
            batch.decode_len_is_bound = True
            batch.decode_rule = key
            with torch.no_grad():
                side = torch.cuda.Stream(dev)
                side.wait_stream(torch.cuda.current_stream(dev))
                with torch.cuda.stream(side):
                    self._decode_body(batch)                      # warm-up outside the capture
                torch.cuda.current_stream(dev).wait_stream(side)
                torch.cuda.synchronize(dev)
                graph = torch.cuda.CUDAGraph()
                if self._graph_pool is None:
                    self._graph_pool = torch.cuda.graph_pool_handle()
                with torch.cuda.graph(graph, pool=self._graph_pool):
                    logits, picked = self._decode_body(batch)
        finally:
            self._end_step()
        self._graphs[key] = (graph, logits, picked)

    def _replay(self, key):
        graph, logits, picked = self._graphs[key]
        graph.replay()
        return logits, picked

    def sample(self, logits: torch.Tensor, temperature, top_k, top_p, uniforms):
        """Choose a token per logits row on the device; returns (tokens, logprobs) as Python lists."""
        dev = self.rt.device
        m = logits.shape[0]
        packed = torch.tensor([list(map(float, temperature)), list(map(float, top_p)),
                               list(map(float, uniforms))], dtype=torch.float32).to(dev, non_blocking=True)
        ks = torch.tensor(list(map(int, top_k)), dtype=torch.int32).to(dev, non_blocking=True)
        out = self.rt.ops.sample(logits, packed[0].contiguous(), ks, packed[1].contiguous(),
                                 packed[2].contiguous())
        host = out.cpu()
        return host[:, 0].tolist(), host[:, 1].contiguous().view(torch.float32).tolist()
