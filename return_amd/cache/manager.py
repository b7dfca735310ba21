"""The cache manager: pages of keys and values with a block table per request, one
pool per group of layers with the same needs, and slots for per-request state of
fixed size.

What it restates of the reference: pools of pages per layer (rollout/cache.py:16-24, there
[pages, P, Hkv, D]; here [pages, Hkv, P, D]), the append planner that fills the tail page and then
takes new pages and yields flat write positions page*P + offset (cache.py:132-162,
266-272), the concatenated tables page_table / cu_pages / cu_q / qpos
(cache.py:282-328), freeing a session's pages (cache.py:94-106), and a place for
state of fixed size that is allocated and freed along with the pages
(LinearStateCache, cache.py:340-472; rollout/engine.py:149-157). Paragraph
operations of the reference are not here. New here: groups of layers (one pool
and one free list per distinct PagedKVSpec), windows that give pages back while
the request runs, and a capacity check that is made for the whole step before
anything is changed.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .pages import FreeList, KVCapacityError
from .spec import PagedKVSpec, StateSpec

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32,
           "float16": torch.float16}


@dataclasses.dataclass
class GroupTables:
    """Tables of one paged group for one step (host arrays, int32)."""
    slot_mapping: np.ndarray    # [T]   flat row page*P + offset where each new token is written
    page_table: np.ndarray      # [tp]  pages of all requests of the step, one after the other
    cu_pages: np.ndarray        # [n+1] where each request's pages start in page_table
    kv_start: np.ndarray        # [n]   position of the first row of the request's first listed page


@dataclasses.dataclass
class StepTables:
    """What one step needs to know of the cache (host side)."""
    request_ids: List
    q_lens: List[int]
    q_start: np.ndarray         # [n]   position of the first new token = tokens held before
    cu_q: np.ndarray            # [n+1]
    positions: np.ndarray       # [T]
    seq_lens: np.ndarray        # [n]   tokens held after this step
    slot_ids: np.ndarray        # [n]   the request's state slot
    groups: List[GroupTables]
    # (version of the page lists, request ids[, rows that fill the batch up]): two steps with the same
    # key have the same page_table, cu_pages and kv_start in every group, so whoever copies them to
    # the device may skip that (rollout/cache.py:286-306 skips its table rebuild on the same test)
    page_key: Optional[tuple] = None


class PagedGroup:
    """Layers that keep the same kind of keys and values: one pool, one free list."""

    def __init__(self, spec: PagedKVSpec, layers: List[int], num_pages: int, page_size: int,
                 dtype: torch.dtype, device):
        self.spec = spec
        self.layers = list(layers)
        self.local = {layer: i for i, layer in enumerate(self.layers)}
        self.num_pages = num_pages
        self.page_size = page_size
        # [layer, k|v, page, kv head, row in page, D]: the rows that one kv head has in a page lie
        # side by side (a kernel that walks the keys of one kv head reads runs of P rows: measured,
        # the decode attention is 4 to 10 % faster than with the kv heads of a token side by side),
        # a page of one layer is one contiguous run of Hkv*P*D elements. One page beyond the
        # num_pages that requests can hold is the spare page: rows that only fill a batch up
        # to a fixed size (pad_tables) write and read there.
        if (num_pages + 1) * page_size * spec.num_kv_heads >= 2 ** 31:
            raise ValueError(f"{num_pages} pages of {page_size} rows for {spec.num_kv_heads} kv heads: the kernels "
                             "count a layer's head rows in 32 bits")
        self.pool = torch.zeros(len(self.layers), 2, num_pages + 1, spec.num_kv_heads, page_size,
                                spec.head_dim, dtype=dtype, device=device)
        self.spare_page = num_pages
        self.pages = FreeList(num_pages, "page")

    def layer_pools(self, cache_layer: int) -> Tuple[torch.Tensor, torch.Tensor]:
        i = self.local[cache_layer]
        return self.pool[i, 0], self.pool[i, 1]


class _Live:
    __slots__ = ("slot", "seq_len", "pages", "first_pos", "_pages_np")

    def __init__(self, slot: int, n_groups: int):
        self.slot = slot
        self.seq_len = 0
        self.pages: List[List[int]] = [[] for _ in range(n_groups)]
        self.first_pos: List[int] = [0] * n_groups
        self._pages_np: List[Optional[np.ndarray]] = [None] * n_groups

    def pages_array(self, g: int) -> np.ndarray:
        """pages[g] as an int32 array, made again only after pages_changed(g)."""
        a = self._pages_np[g]
        if a is None:
            a = np.asarray(self.pages[g], dtype=np.int32)
            self._pages_np[g] = a
        return a

    def pages_changed(self, g: int) -> None:
        self._pages_np[g] = None


class CacheManager:
    """Owns every byte that lives between steps.

    cache_layers: cache layer number -> PagedKVSpec | StateSpec, as the mixers declare.
    max_token:    tokens each paged pool can hold (pages = max_token // page_size).
    max_requests: most requests live at a time (= number of state slots).
    """

    def __init__(self, cache_layers: Dict[int, object], page_size: int, max_token: int,
                 max_requests: int, dtype: torch.dtype, device="cpu"):
        self.page_size = int(page_size)
        self.num_pages = int(max_token) // self.page_size
        if self.num_pages < 1:
            raise ValueError(f"max_token {max_token} is less than one page of {page_size}")
        if self.num_pages * self.page_size >= 2 ** 31:
            raise ValueError("cache pool rows must stay below 2^31")
        self.max_requests = int(max_requests)
        self.device = device
        self.dtype = dtype

        by_spec: Dict[PagedKVSpec, List[int]] = {}
        self.state_layers: Dict[int, StateSpec] = {}
        for layer in sorted(cache_layers):
            spec = cache_layers[layer]
            if isinstance(spec, PagedKVSpec):
                if spec.window is not None and spec.window < 1:
                    raise ValueError(f"cache layer {layer}: window must be at least 1")
                by_spec.setdefault(spec, []).append(layer)
            elif isinstance(spec, StateSpec):
                self.state_layers[layer] = spec
            else:
                raise TypeError(f"cache layer {layer}: {spec!r} is neither PagedKVSpec nor StateSpec")
        self.groups: List[PagedGroup] = [
            PagedGroup(spec, layers, self.num_pages, self.page_size, dtype, device)
            for spec, layers in by_spec.items()]
        self.group_of: Dict[int, int] = {layer: g for g, grp in enumerate(self.groups)
                                         for layer in grp.layers}

        self.slots = FreeList(self.max_requests, "request slot")
        self.spare_slot = self.max_requests      # the state row of rows that only fill a batch up
        self.state: Dict[int, Dict[str, torch.Tensor]] = {}
        for layer, spec in self.state_layers.items():
            self.state[layer] = {
                name: torch.zeros((self.max_requests + 1,) + tuple(shape), dtype=_DTYPES[dt], device=device)
                for name, shape, dt in spec.tensors}

        self.live: Dict[object, _Live] = {}
        self._step_requests: List = []
        self.version = 0            # changes whenever any request's page list changes
        self._memo_key = None       # page_key of the last step and its groups' (page_table, cu_pages, kv_start)
        self._memo_tables: List = []
        self._pad_key = None        # the same for the last step that was filled up
        self._pad_tables: List = []
        self.table_builds = 0       # steps whose page tables were put together anew

    @staticmethod
    def pool_bytes(cache_layers: Dict[int, object], page_size: int, max_token: int, max_requests: int,
                   dtype: torch.dtype) -> int:
        """Bytes of device memory that a manager with these arguments allocates (pools with their
        spare page, state with its spare slot)."""
        item = torch.empty((), dtype=dtype).element_size()
        pages = int(max_token) // int(page_size) + 1
        total = 0
        for spec in cache_layers.values():
            if isinstance(spec, PagedKVSpec):
                total += 2 * pages * int(page_size) * spec.num_kv_heads * spec.head_dim * item
            elif isinstance(spec, StateSpec):
                for _, shape, dt in spec.tensors:
                    n = 1
                    for d in shape:
                        n *= int(d)
                    total += (int(max_requests) + 1) * n * torch.empty((), dtype=_DTYPES[dt]).element_size()
        return total

    # ------------------------------------------------------------------ requests
    def add_request(self, rid) -> int:
        if rid in self.live:
            raise ValueError(f"request {rid!r} is already live")
        slot = self.slots.take()
        self.live[rid] = _Live(slot, len(self.groups))
        for tensors in self.state.values():
            for t in tensors.values():
                t[slot].zero_()
        self.version += 1
        return slot

    def free_request(self, rid) -> None:
        if rid not in self.live:
            raise ValueError(f"request {rid!r} is not live (freed twice?)")
        r = self.live.pop(rid)
        for g, grp in enumerate(self.groups):
            grp.pages.give_back(r.pages[g])
        self.slots.give_back([r.slot])
        self.version += 1

    def seq_len(self, rid) -> int:
        return self.live[rid].seq_len

    def slot_of(self, rid) -> int:
        return self.live[rid].slot

    def free_pages(self) -> List[int]:
        """Free pages of every group."""
        return [grp.pages.available() for grp in self.groups]

    def free_slots(self) -> int:
        return self.slots.available()

    # ------------------------------------------------------------------ accounting
    def _need(self, r: _Live, g: int, n_new: int) -> int:
        P = self.page_size
        held_end = r.first_pos[g] + len(r.pages[g]) * P
        return max(0, -(-(r.seq_len + n_new - held_end) // P))

    def pages_needed(self, rid, n_new: int) -> List[int]:
        """Pages each group has to take to append n_new tokens to a request (live or not yet)."""
        r = self.live.get(rid)
        if r is None:
            return [-(-n_new // self.page_size)] * len(self.groups)
        return [self._need(r, g, n_new) for g in range(len(self.groups))]

    def pages_for_tokens(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def max_pages(self, total_tokens: int, max_portion: int) -> List[int]:
        """Most pages of each group that a request of total_tokens can hold at any time,
        when no step brings it more than max_portion tokens."""
        P = self.page_size
        full = -(-total_tokens // P)
        out = []
        for grp in self.groups:
            w = grp.spec.window
            if w is None:
                out.append(full)
            else:
                # before a step the held pages start at most P-1 rows before the window;
                # the step then adds max_portion rows
                out.append(min(full, -(-(w + max_portion + P - 1) // P) + 1))
        return out

    def held_pages(self, rid) -> List[int]:
        r = self.live.get(rid)
        return [len(p) for p in r.pages] if r is not None else [0] * len(self.groups)

    # ------------------------------------------------------------------ one step
    def begin_step(self, entries: Sequence[Tuple[object, int]]) -> StepTables:
        """Make room for (request, number of new tokens) of one step and say where things are.

        Either every entry gets its pages or KVCapacityError is raised and nothing changed.
        """
        P = self.page_size
        n = len(entries)
        seen = set()
        for rid, n_new in entries:
            if rid not in self.live:
                raise ValueError(f"request {rid!r} is not live")
            if rid in seen:
                raise ValueError(f"request {rid!r} appears twice in one step")
            if n_new < 1:
                raise ValueError(f"request {rid!r}: a step brings at least one token, got {n_new}")
            seen.add(rid)
        for g, grp in enumerate(self.groups):
            want = sum(self._need(self.live[rid], g, n_new) for rid, n_new in entries)
            if want > grp.pages.available():
                raise KVCapacityError(
                    f"step needs {want} pages of cache group {g}, {grp.pages.available()} "
                    f"of {grp.num_pages} are free")

        q_lens = [int(n_new) for _, n_new in entries]
        lives = [self.live[rid] for rid, _ in entries]
        total = sum(q_lens)
        cu_q = np.zeros(n + 1, dtype=np.int32)
        cu_q[1:] = np.cumsum(q_lens)
        q_start = np.array([r.seq_len for r in lives], dtype=np.int32)
        single = total == n                                   # one token each: a decode step
        if single:
            positions = q_start.copy()
        else:
            positions = np.empty(total, dtype=np.int32)
            for i in range(n):
                positions[cu_q[i]:cu_q[i + 1]] = np.arange(q_start[i], q_start[i] + q_lens[i])
        slot_ids = np.array([r.slot for r in lives], dtype=np.int32)

        for g, grp in enumerate(self.groups):
            for i, r in enumerate(lives):
                need = self._need(r, g, q_lens[i])
                if need:
                    r.pages[g].extend(grp.pages.take_many(need))
                    r.pages_changed(g)
                    self.version += 1
        # the page lists are final now: the same (version, requests) as the last step means the same tables
        ids = [rid for rid, _ in entries]
        page_key = (self.version, tuple(ids))
        same = page_key == self._memo_key
        if not same:
            self.table_builds += 1
            self._memo_tables = []

        groups = []
        for g, grp in enumerate(self.groups):
            slot_mapping = np.empty(total, dtype=np.int32)
            for i, r in enumerate(lives):
                if single:
                    rel = r.seq_len - r.first_pos[g]
                    slot_mapping[i] = r.pages[g][rel // P] * P + rel % P
                else:
                    rel = positions[cu_q[i]:cu_q[i + 1]] - r.first_pos[g]
                    slot_mapping[cu_q[i]:cu_q[i + 1]] = r.pages_array(g)[rel // P] * P + rel % P
            if same:
                page_table, cu_pages, kv_start = self._memo_tables[g]
            else:
                tables = [r.pages_array(g) for r in lives]
                cu_pages = np.zeros(n + 1, dtype=np.int32)
                cu_pages[1:] = np.cumsum([len(t) for t in tables])
                kv_start = np.array([r.first_pos[g] for r in lives], dtype=np.int32)
                page_table = np.concatenate(tables) if tables else np.zeros(0, dtype=np.int32)
                self._memo_tables.append((page_table, cu_pages, kv_start))
            groups.append(GroupTables(slot_mapping, page_table, cu_pages, kv_start))
        self._memo_key = page_key

        for rid, n_new in entries:
            self.live[rid].seq_len += n_new
        seq_lens = np.array([self.live[rid].seq_len for rid, _ in entries], dtype=np.int32)
        self._step_requests = [rid for rid, _ in entries]
        return StepTables(ids, q_lens, q_start, cu_q, positions, seq_lens, slot_ids, groups, page_key)

    def pad_tables(self, tables: StepTables, n_pad: int) -> StepTables:
        """The same step with n_pad more one-token sequences that belong to no request: token
        at position 0, written to and read from the spare page (state: the spare slot). A
        decode step of a few fixed sizes can be replayed from a few captured graphs; what the
        added rows compute is thrown away and touches nothing that a request holds."""
        if n_pad <= 0:
            return tables
        P = self.page_size
        one = np.ones(n_pad, dtype=np.int32)
        last = int(tables.cu_q[-1])
        page_key = None if tables.page_key is None else tables.page_key + (n_pad,)
        same = page_key is not None and page_key == self._pad_key
        if not same:
            self._pad_tables = []
        groups = []
        for g, (grp, gt) in enumerate(zip(self.groups, tables.groups)):
            if same:
                page_table, cu_pages, kv_start = self._pad_tables[g]
            else:
                page_table = np.concatenate([gt.page_table, one * grp.spare_page]).astype(np.int32)
                cu_pages = np.concatenate([gt.cu_pages, gt.cu_pages[-1] + np.arange(1, n_pad + 1)]).astype(np.int32)
                kv_start = np.concatenate([gt.kv_start, 0 * one]).astype(np.int32)
                self._pad_tables.append((page_table, cu_pages, kv_start))
            groups.append(GroupTables(
                np.concatenate([gt.slot_mapping, one * (grp.spare_page * P)]).astype(np.int32),
                page_table, cu_pages, kv_start))
        self._pad_key = page_key
        return StepTables(
            list(tables.request_ids) + [None] * n_pad, list(tables.q_lens) + [1] * n_pad,
            np.concatenate([tables.q_start, 0 * one]).astype(np.int32),
            np.concatenate([tables.cu_q, last + np.arange(1, n_pad + 1)]).astype(np.int32),
            np.concatenate([tables.positions, 0 * one]).astype(np.int32),
            np.concatenate([tables.seq_lens, one]).astype(np.int32),
            np.concatenate([tables.slot_ids, one * self.spare_slot]).astype(np.int32), groups, page_key)

    def end_step(self) -> None:
        """After the step ran: give back pages that every later query's window has passed."""
        P = self.page_size
        for rid in self._step_requests:
            r = self.live.get(rid)
            if r is None:
                continue
            for g, grp in enumerate(self.groups):
                w = grp.spec.window
                if w is None:
                    continue
                # the next query sits at position seq_len and reads keys >= seq_len - w + 1
                first_needed = r.seq_len - w + 1
                drop = 0
                while drop < len(r.pages[g]) and r.first_pos[g] + (drop + 1) * P <= first_needed:
                    drop += 1
                if drop:
                    grp.pages.give_back(r.pages[g][:drop])
                    del r.pages[g][:drop]
                    r.pages_changed(g)
                    r.first_pos[g] += drop * P
                    self.version += 1
        self._step_requests = []

    # ------------------------------------------------------------------ views for mixers
    def view(self, cache_layer: int):
        """What a mixer gets for its cache layer: (group number, k pool, v pool) or the state tensors."""
        if cache_layer in self.group_of:
            g = self.group_of[cache_layer]
            k, v = self.groups[g].layer_pools(cache_layer)
            return PagedView(g, k, v, self.page_size, self.groups[g].spec)
        if cache_layer in self.state:
            return StateView(self.state[cache_layer])
        raise KeyError(f"no cache layer {cache_layer}")

    # ------------------------------------------------------------------ checks
    def check_invariants(self) -> None:
        """No page lost, held twice, or both free and held; slots likewise; lengths fit the pages."""
        P = self.page_size
        for g, grp in enumerate(self.groups):
            free = grp.pages.free_ids()
            held = [p for r in self.live.values() for p in r.pages[g]]
            assert len(set(free)) == len(free), f"group {g}: a page is twice in the free list"
            assert len(set(held)) == len(held), f"group {g}: a page is held twice"
            assert not set(free) & set(held), f"group {g}: a page is both free and held"
            assert set(free) | set(held) == set(range(grp.num_pages)), f"group {g}: a page is lost"
            for rid, r in self.live.items():
                assert r._pages_np[g] is None or r._pages_np[g].tolist() == r.pages[g], f"{rid!r}: stale page array"
                assert r.first_pos[g] % P == 0
                end = r.first_pos[g] + len(r.pages[g]) * P
                assert r.seq_len <= end, f"{rid!r}: {r.seq_len} tokens but pages end at {end}"
                if grp.spec.window is None:
                    assert r.first_pos[g] == 0
                    assert len(r.pages[g]) == -(-r.seq_len // P), f"{rid!r}: page count off"
        slots = [r.slot for r in self.live.values()]
        free = self.slots.free_ids()
        assert len(set(slots)) == len(slots) and not set(slots) & set(free)
        assert set(slots) | set(free) == set(range(self.max_requests))


@dataclasses.dataclass
class PagedView:
    group: int                  # index into StepBatch.groups
    k_pool: torch.Tensor        # [pages, Hkv, P, D] of this cache layer
    v_pool: torch.Tensor
    page_size: int
    spec: PagedKVSpec


@dataclasses.dataclass
class StateView:
    tensors: Dict[str, torch.Tensor]    # name -> [max_requests + 1, ...]; row = StepBatch.slot_ids
