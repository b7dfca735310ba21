"""The batch of one step as the parts see it, and the builder that puts the cache
manager's host tables on the device.

The reference fills pinned host arrays and copies them into persistent device
tensors so that captured graphs replay on fixed addresses (rollout/cache.py:42-70,
274-328). Here all integer tables of a step live in ONE pinned staging buffer and
ONE device buffer of fixed layout; a step costs one host-to-device copy for the
small tables and one per cache group for its page table, and the latter only when a
page list has changed or other requests take part (rollout/cache.py:286-306).
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, StepTables


@dataclasses.dataclass
class GroupOnDevice:
    slot_mapping: torch.Tensor   # int32 [T]
    page_table: torch.Tensor     # int32 [tp]
    cu_pages: torch.Tensor       # int32 [n+1]
    kv_start: torch.Tensor       # int32 [n]
    n_pages: List[int]           # host: pages listed per request
    max_pages: int               # host: most pages listed for one request


@dataclasses.dataclass
class StepBatch:
    """One step: n requests with q_lens[i] new tokens each, T tokens in all.

    Device tensors are int32 views into the builder's fixed buffer. Host lists carry
    the same numbers for decisions that must not wait for the device.
    """
    n_seqs: int
    n_tokens: int
    token_ids: torch.Tensor      # [T]
    positions: torch.Tensor      # [T]   position of each new token in its sequence
    cu_q: torch.Tensor           # [n+1] where each request's tokens start
    q_start: torch.Tensor        # [n]   position of each request's first new token
    seq_lens: torch.Tensor       # [n]   tokens held after this step
    slot_ids: torch.Tensor       # [n]   row of each request in per-request state tensors
    logit_rows: torch.Tensor     # [m]   token rows whose logits are wanted
    n_logit_rows: int
    groups: List[GroupOnDevice]
    # host copies
    request_ids: List
    q_lens: List[int]
    q_starts: List[int]
    cu_q_host: List[int]
    slot_ids_host: List[int]
    all_decode: bool             # every request brings exactly one token
    max_q_len: int
    max_seq_len: int
    # requests that bring one token go to the decode kernels, the others to the prefill kernels
    n_decode: int = 0
    decode_segs: Optional[torch.Tensor] = None     # int32 [n_decode] request numbers; None: all of them
    max_decode_seq_len: int = 0
    decode_len_is_bound: bool = False              # max_decode_seq_len is an upper bound (a graph's bucket), not the longest length
    # (requests, longest length) that the kernel set bases its choice of splits on, when these are not the step's
    # own: the runner names a decode step's class (the batch size and context bucket of the graph that serves or
    # would serve it), so that a step run eagerly and the same step replayed from a graph take the same splits
    # and with them the same order of sums
    decode_rule: Optional[tuple] = None
    n_prefill_tokens: int = 0
    prefill_toks: Optional[torch.Tensor] = None    # int32 token rows of the others; None: all rows
    prefill_segs: List[int] = dataclasses.field(default_factory=list)   # host: their request numbers
    # q tiles of the prefill attention kernel, by rows per tile: rows -> int32 [tiles, 2] of
    # (request number, first row of the tile among the request's new tokens)
    prefill_tiles: dict = dataclasses.field(default_factory=dict)
    # further integers per token that a part of the model asked for (step_needs()["token_columns"]), by name:
    # int32 [T] each; what a request does not bring for its tokens is their position
    token_columns: dict = dataclasses.field(default_factory=dict)



def prefill_tiles(q_lens, q_starts=None, rows=64):
    """(request number, first row) of every tile of ``rows`` rows, for requests with more than
    one token; tiles that read the most keys come first, so the longest work starts earliest."""
    tiles = [(i, off) for i, q in enumerate(q_lens) if q != 1 for off in range(0, q, rows)]
    if q_starts is not None:
        tiles.sort(key=lambda t: -(int(q_starts[t[0]]) + t[1]))
    return tiles


class StepBuilder:
    """Fixed device buffers for the tables of a step, sized for the worst case."""

    def __init__(self, cache: CacheManager, max_step_tokens: int, max_requests: int, device, tile_rows=(),
                 token_columns=()):
        """tile_rows: heights of the q tiles that the model's mixers want listed for the requests that
        bring more than one token (what their attention kernels' grids run over); none: no lists.
        token_columns: names of further integers per token that parts of the model read beside the
        position (a position encoding with more than one axis, say)."""
        self.cache = cache
        self.tile_rows = tuple(sorted(int(r) for r in tile_rows))
        self.token_columns = tuple(sorted(str(c) for c in token_columns))
        self.device = torch.device(device)
        self.max_tokens = int(max_step_tokens)
        self.max_requests = int(max_requests)
        T, N, G = self.max_tokens, self.max_requests, len(cache.groups)
        layout = [("token_ids", T), ("positions", T), ("logit_rows", T), ("cu_q", N + 1),
                  ("q_start", N), ("seq_lens", N), ("slot_ids", N), ("decode_segs", N),
                  ("prefill_toks", T)]
        layout += [(f"prefill_tiles{rows}", 2 * (T // rows + N)) for rows in self.tile_rows]
        layout += [(f"column_{name}", T) for name in self.token_columns]
        for g in range(G):
            layout += [(f"slot_mapping{g}", T), (f"cu_pages{g}", N + 1), (f"kv_start{g}", N)]
        self._small_end = None
        self._off = {}
        off = 0
        for name, size in layout:
            self._off[name] = (off, size)
            off += -(-size // 4) * 4          # keep every table 16-byte aligned
        self._small_end = off
        # a windowed request lists at most its held pages; the sum over a step never exceeds the
        # pool, plus the spare page once for every row that only fills the batch up
        for g in range(G):
            size = cache.groups[g].num_pages + N
            self._off[f"page_table{g}"] = (off, size)
            off += -(-size // 4) * 4
        self._total = off
        pin = self.device.type == "cuda"
        self._host = torch.zeros(self._total, dtype=torch.int32, pin_memory=pin)
        self._host_np = self._host.numpy()
        self._dev = torch.zeros(self._total, dtype=torch.int32, device=self.device)
        # the staging buffer is written again only after the last step's copies have left it
        self._copied = torch.cuda.Event() if pin else None
        self._copy_pending = False
        # the cache manager's page_key of the page tables that the device buffer holds: a step with
        # the same key (no page list changed since, the same requests) finds them there
        self._tables_on_device = None
        self.page_table_copies = 0

    def _put(self, name: str, values) -> int:
        off, size = self._off[name]
        k = len(values)
        if k > size:
            raise ValueError(f"{name}: {k} entries exceed the step builder's limit of {size}")
        self._host_np[off:off + k] = values
        return k

    def _view(self, name: str, k: int) -> torch.Tensor:
        off, _ = self._off[name]
        return self._dev[off:off + k]

    def build(self, tables: StepTables, tokens: Sequence[Sequence[int]],
              logit_rows: Sequence[int], columns: Optional[dict] = None) -> StepBatch:
        """tokens[i] are the new tokens of request i; logit_rows index the step's flat token rows;
        columns: name -> T integers for the token columns the builder was made with (a name that is
        missing gets the tokens' positions)."""
        n = len(tables.request_ids)
        T = int(tables.cu_q[-1])
        if T > self.max_tokens:
            raise ValueError(f"step of {T} tokens exceeds max_step_tokens {self.max_tokens}")
        if n > self.max_requests:
            raise ValueError(f"step of {n} requests exceeds max_reside {self.max_requests}")
        if self._copy_pending:
            self._copied.synchronize()
            self._copy_pending = False
        flat = np.fromiter((t for seq in tokens for t in seq), dtype=np.int64, count=T)
        if len(tokens) != n or any(len(seq) != q for seq, q in zip(tokens, tables.q_lens)):
            raise ValueError("tokens do not match the step's q_lens")
        self._put("token_ids", flat)
        self._put("positions", tables.positions)
        for name in self.token_columns:
            col = (columns or {}).get(name)
            col = tables.positions if col is None else np.asarray(col, dtype=np.int32)
            if len(col) != T:
                raise ValueError(f"token column {name!r} has {len(col)} entries for {T} tokens")
            self._put(f"column_{name}", col)
        unknown = set(columns or ()) - set(self.token_columns)
        if unknown:
            raise ValueError(f"token column(s) {sorted(unknown)} are not among those the model reads: "
                             f"{list(self.token_columns)}")
        m = self._put("logit_rows", np.asarray(logit_rows, dtype=np.int32))
        self._put("cu_q", tables.cu_q)
        self._put("q_start", tables.q_start)
        self._put("seq_lens", tables.seq_lens)
        self._put("slot_ids", tables.slot_ids)
        dec = [i for i, q in enumerate(tables.q_lens) if q == 1]
        pre = [i for i, q in enumerate(tables.q_lens) if q != 1]
        mixed_kinds = bool(dec) and bool(pre)
        n_pre_tok = T - len(dec)
        if mixed_kinds:
            self._put("decode_segs", np.asarray(dec, dtype=np.int32))
            self._put("prefill_toks", np.concatenate(
                [np.arange(tables.cu_q[i], tables.cu_q[i + 1], dtype=np.int32) for i in pre]))
        for g, gt in enumerate(tables.groups):
            self._put(f"slot_mapping{g}", gt.slot_mapping)
            self._put(f"cu_pages{g}", gt.cu_pages)
            self._put(f"kv_start{g}", gt.kv_start)
        tables_there = tables.page_key is not None and tables.page_key == self._tables_on_device
        if not tables_there:
            for g, gt in enumerate(tables.groups):
                self._put(f"page_table{g}", gt.page_table)
        tiles = {}
        if pre:
            for rows in self.tile_rows:
                tiles[rows] = prefill_tiles(tables.q_lens, tables.q_start, rows)
                self._put(f"prefill_tiles{rows}", np.asarray(tiles[rows], dtype=np.int32).reshape(-1))
        # one copy for the small tables, one per group for the used part of its page table
        self._dev[:self._small_end].copy_(self._host[:self._small_end], non_blocking=True)
        groups = []
        for g, gt in enumerate(tables.groups):
            off, _ = self._off[f"page_table{g}"]
            k = len(gt.page_table)
            if k and not tables_there:
                self._dev[off:off + k].copy_(self._host[off:off + k], non_blocking=True)
                self.page_table_copies += 1
            n_pages = np.diff(gt.cu_pages).tolist()
            groups.append(GroupOnDevice(
                self._view(f"slot_mapping{g}", T), self._view(f"page_table{g}", k),
                self._view(f"cu_pages{g}", n + 1), self._view(f"kv_start{g}", n),
                n_pages, max(n_pages) if n_pages else 0))
        self._tables_on_device = tables.page_key
        if self._copied is not None:
            self._copied.record()
            self._copy_pending = True
        return StepBatch(
            n_seqs=n, n_tokens=T,
            token_ids=self._view("token_ids", T), positions=self._view("positions", T),
            cu_q=self._view("cu_q", n + 1), q_start=self._view("q_start", n),
            seq_lens=self._view("seq_lens", n), slot_ids=self._view("slot_ids", n),
            logit_rows=self._view("logit_rows", m), n_logit_rows=m, groups=groups,
            request_ids=list(tables.request_ids), q_lens=list(tables.q_lens),
            q_starts=tables.q_start.tolist(), cu_q_host=tables.cu_q.tolist(),
            slot_ids_host=tables.slot_ids.tolist(),
            all_decode=all(q == 1 for q in tables.q_lens),
            max_q_len=max(tables.q_lens) if tables.q_lens else 0,
            max_seq_len=int(tables.seq_lens.max()) if n else 0,
            n_decode=len(dec), decode_segs=self._view("decode_segs", len(dec)) if mixed_kinds else None,
            max_decode_seq_len=max((int(tables.seq_lens[i]) for i in dec), default=0),
            n_prefill_tokens=n_pre_tok,
            prefill_toks=self._view("prefill_toks", n_pre_tok) if mixed_kinds else None,
            prefill_segs=pre,
            prefill_tiles={rows: self._view(f"prefill_tiles{rows}", 2 * len(t)).view(-1, 2)
                           for rows, t in tiles.items()},
            token_columns={name: self._view(f"column_{name}", T) for name in self.token_columns})
