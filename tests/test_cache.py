"""The cache manager on the CPU: no page lost, held twice or freed twice, under random orders
of requests; tables against a brute-force builder; windows give pages back; reuse is immediate."""
import random

import numpy as np
import pytest
import torch

from return_amd.cache import CacheManager, FreeList, KVCapacityError, PagedKVSpec, StateSpec


def manager(page=4, max_token=64, max_requests=4, window=None, extra=None):
    layers = {0: PagedKVSpec(2, 8), 1: PagedKVSpec(2, 8)}
    if window:
        layers[2] = PagedKVSpec(2, 8, window)
    if extra:
        layers.update(extra)
    return CacheManager(layers, page, max_token, max_requests, torch.float32, "cpu")


def test_free_list_refuses_double_free_and_strangers():
    f = FreeList(3)
    a, b = f.take(), f.take()
    f.give_back([a])
    with pytest.raises(ValueError, match="twice"):
        f.give_back([a])
    with pytest.raises(ValueError, match="exist"):
        f.give_back([7])
    assert f.take() == a                      # last freed, first reused (rollout/cache.py:153)
    f.take()
    with pytest.raises(KVCapacityError):
        f.take()
    with pytest.raises(KVCapacityError):
        FreeList(2).take_many(3)


def brute_tables(cm, entries, before):
    """Tables from the manager's page lists alone (after check_tables.py:11-31 of the reference)."""
    P = cm.page_size
    out = []
    for g in range(len(cm.groups)):
        slot, table, cu, starts = [], [], [0], []
        for rid, n in entries:
            r = cm.live[rid]
            for pos in range(before[rid], before[rid] + n):
                rel = pos - r.first_pos[g]
                slot.append(r.pages[g][rel // P] * P + rel % P)
            table += r.pages[g]
            cu.append(len(table))
            starts.append(r.first_pos[g])
        out.append((slot, table, cu, starts))
    return out


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("window", [None, 6])
def test_random_requests_keep_every_page_accounted(seed, window):
    rng = random.Random(seed)
    cm = manager(page=4, max_token=96, max_requests=4, window=window)
    live, next_id, refused = {}, 0, 0
    for _ in range(300):
        op = rng.random()
        if op < 0.25 and len(live) < 4:
            cm.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.35 and live:
            rid = rng.choice(list(live))
            cm.free_request(rid)
            del live[rid]
        elif live:
            ids = rng.sample(list(live), rng.randint(1, len(live)))
            entries = [(rid, rng.choice([1, 1, 1, 2, 3, 7, 13])) for rid in ids]
            before = dict(live)
            free_before = cm.free_pages()
            try:
                t = cm.begin_step(entries)
            except KVCapacityError:
                refused += 1
                assert cm.free_pages() == free_before          # nothing changed
                assert all(cm.seq_len(r) == before[r] for r in live)
                cm.check_invariants()
                continue
            for rid, n in entries:
                live[rid] += n
            want = brute_tables(cm, entries, before)
            for g, (slot, table, cu, starts) in enumerate(want):
                assert t.groups[g].slot_mapping.tolist() == slot
                assert t.groups[g].page_table.tolist() == table
                assert t.groups[g].cu_pages.tolist() == cu
                assert t.groups[g].kv_start.tolist() == starts
            assert t.q_start.tolist() == [before[r] for r, _ in entries]      # tokens held before
            assert t.seq_lens.tolist() == [live[r] for r, _ in entries]
            assert t.positions.tolist() == [p for r, n in entries for p in range(before[r], before[r] + n)]
            assert len(set(t.groups[0].slot_mapping.tolist())) == len(t.groups[0].slot_mapping)
            cm.end_step()
        cm.check_invariants()
    assert refused > 0                                      # the pool was small enough to run out
    for rid in list(live):
        cm.free_request(rid)
    cm.check_invariants()
    assert all(g.pages.in_use() == 0 for g in cm.groups) and cm.slots.in_use() == 0


def test_positions_follow_the_reference_layout():
    """65 tokens, then 3 more: the second portion starts at position 65 on the second page
    (qpos = seqlen - q_len, rollout/cache.py:293; vector [0, 65, ...] of opd/test_parallel.py:113)."""
    cm = CacheManager({0: PagedKVSpec(1, 8)}, 64, 64 * 4, 2, torch.float32, "cpu")
    cm.add_request("u")
    t = cm.begin_step([("u", 65)])
    assert t.q_start.tolist() == [0] and len(cm.live["u"].pages[0]) == 2
    cm.end_step()
    t = cm.begin_step([("u", 3)])
    assert t.q_start.tolist() == [65] and t.positions.tolist() == [65, 66, 67]
    p = cm.live["u"].pages[0]
    assert t.groups[0].slot_mapping.tolist() == [p[1] * 64 + 1, p[1] * 64 + 2, p[1] * 64 + 3]


def test_pages_are_reused_at_once():
    cm = manager(page=4, max_token=16, max_requests=2)
    cm.add_request("a")
    cm.begin_step([("a", 16)]); cm.end_step()
    held = list(cm.live["a"].pages[0])
    cm.add_request("b")
    with pytest.raises(KVCapacityError):
        cm.begin_step([("b", 1)])
    cm.free_request("a")
    cm.begin_step([("b", 16)]); cm.end_step()
    assert sorted(cm.live["b"].pages[0]) == sorted(held)
    with pytest.raises(ValueError, match="not live"):
        cm.free_request("a")


def test_window_gives_pages_back_while_running():
    cm = manager(page=4, max_token=64, max_requests=2, window=6)
    g = [i for i, grp in enumerate(cm.groups) if grp.spec.window == 6][0]
    full = 1 - g
    cm.add_request("w")
    held = []
    for _ in range(40):
        cm.begin_step([("w", 1)]); cm.end_step()
        r = cm.live["w"]
        held.append(len(r.pages[g]))
        # every key a later query may read is still there
        assert r.first_pos[g] <= max(0, r.seq_len - 6 + 1)
        assert r.first_pos[g] + len(r.pages[g]) * 4 >= r.seq_len
        cm.check_invariants()
    assert max(held) <= 3 and len(cm.live["w"].pages[full]) == 10
    cm.add_request("x")
    cm.begin_step([("x", 24)]); cm.end_step()          # a long portion, then the window trims it
    assert len(cm.live["x"].pages[g]) <= 3 and cm.live["x"].first_pos[g] == 16
    assert cm.max_pages(40, 24)[g] >= 24 // 4


def test_state_slots():
    spec = StateSpec((("conv", (3, 2), "bfloat16"), ("rec", (2, 4, 4), "float32")))
    cm = manager(extra={5: spec}, max_requests=2)
    s0 = cm.add_request("a")
    view = cm.view(5)
    assert view.tensors["rec"].shape == (2 + 1, 2, 4, 4)       # one row per slot and the spare row
    assert view.tensors["conv"].dtype == torch.bfloat16
    view.tensors["rec"][s0] += 3.0
    cm.add_request("b")
    with pytest.raises(KVCapacityError):
        cm.add_request("c")
    cm.free_request("a")
    s2 = cm.add_request("c")
    assert s2 == s0 and float(cm.view(5).tensors["rec"][s2].abs().sum()) == 0.0    # zero at the start
    t = cm.begin_step([("c", 2), ("b", 1)])
    assert t.slot_ids.tolist() == [cm.slot_of("c"), cm.slot_of("b")]


def test_step_rules():
    cm = manager()
    cm.add_request("a")
    with pytest.raises(ValueError, match="twice"):
        cm.begin_step([("a", 1), ("a", 1)])
    with pytest.raises(ValueError, match="not live"):
        cm.begin_step([("zz", 1)])
    with pytest.raises(ValueError, match="at least one"):
        cm.begin_step([("a", 0)])
    with pytest.raises(ValueError, match="already live"):
        cm.add_request("a")


def test_groups_have_pools_of_their_own():
    cm = CacheManager({0: PagedKVSpec(2, 8), 1: PagedKVSpec(2, 8, 4), 2: PagedKVSpec(1, 16), 3: PagedKVSpec(2, 8)},
                      4, 32, 2, torch.float32, "cpu")
    assert len(cm.groups) == 3
    assert sorted(map(tuple, (g.layers for g in cm.groups))) == [(0, 3), (1,), (2,)]
    v0, v3 = cm.view(0), cm.view(3)
    assert v0.group == v3.group and v0.k_pool.data_ptr() != v3.k_pool.data_ptr()
    # 32 tokens in pages of 4, and the spare page; [pages, kv heads, rows in a page, D]
    assert v0.k_pool.shape == (8 + 1, 2, 4, 8) and cm.view(2).k_pool.shape == (8 + 1, 1, 4, 16)


def test_pad_tables_adds_rows_on_the_spare_page_only():
    """Rows that fill a batch up belong to no request: they sit at position 0 of the spare page
    and of the spare state slot, and change nothing the manager keeps."""
    from return_amd.cache import StateSpec
    cm = CacheManager({0: PagedKVSpec(2, 8, None), 1: PagedKVSpec(1, 8, 4), 2: StateSpec((("s", (3,), "float32"),))},
                      page_size=4, max_token=64, max_requests=3, dtype=torch.float32)
    cm.add_request("a"); cm.add_request("b")
    cm.begin_step([("a", 6), ("b", 3)]); cm.end_step()
    t = cm.begin_step([("a", 1), ("b", 1)])
    before = (cm.free_pages(), cm.free_slots(), {k: (v.seq_len, [list(p) for p in v.pages]) for k, v in cm.live.items()})
    p = cm.pad_tables(t, 3)
    after = (cm.free_pages(), cm.free_slots(), {k: (v.seq_len, [list(p) for p in v.pages]) for k, v in cm.live.items()})
    assert before == after
    assert cm.pad_tables(t, 0) is t
    assert p.request_ids == ["a", "b", None, None, None] and p.q_lens == [1, 1, 1, 1, 1]
    assert p.cu_q.tolist() == [0, 1, 2, 3, 4, 5]
    assert p.positions.tolist() == t.positions.tolist() + [0, 0, 0]
    assert p.q_start.tolist()[2:] == [0, 0, 0] and p.seq_lens.tolist()[2:] == [1, 1, 1]
    assert p.slot_ids.tolist()[2:] == [cm.spare_slot] * 3 and cm.spare_slot == 3
    for grp, g0, g1 in zip(cm.groups, t.groups, p.groups):
        assert grp.spare_page == grp.num_pages and grp.pool.shape[2] == grp.num_pages + 1
        assert g1.slot_mapping.tolist() == g0.slot_mapping.tolist() + [grp.spare_page * 4] * 3
        assert g1.page_table.tolist() == g0.page_table.tolist() + [grp.spare_page] * 3
        assert g1.cu_pages.tolist() == g0.cu_pages.tolist() + [g0.cu_pages[-1] + i for i in (1, 2, 3)]
        assert g1.kv_start.tolist()[2:] == [0, 0, 0]
        assert grp.spare_page not in grp.pages.free_ids()
    assert cm.state[2]["s"].shape[0] == 4
    cm.end_step()
    cm.check_invariants()


def test_pool_bytes_is_what_the_manager_allocates():
    layers = {0: PagedKVSpec(2, 8, None), 1: PagedKVSpec(2, 8, None), 2: PagedKVSpec(1, 24, 5),
              3: StateSpec((("conv", (3, 2), "bfloat16"), ("rec", (2, 4, 4), "float32")))}
    for dtype in (torch.bfloat16, torch.float32):
        cm = CacheManager(layers, page_size=4, max_token=50, max_requests=3, dtype=dtype)
        held = sum(g.pool.numel() * g.pool.element_size() for g in cm.groups)
        held += sum(t.numel() * t.element_size() for ts in cm.state.values() for t in ts.values())
        assert CacheManager.pool_bytes(layers, 4, 50, 3, dtype) == held


def test_a_pool_whose_head_rows_do_not_fit_32_bits_is_refused():
    with pytest.raises(ValueError, match="32 bits"):
        CacheManager({0: PagedKVSpec(8, 128)}, page_size=16, max_token=2 ** 28, max_requests=1, dtype=torch.bfloat16,
                     device="meta")


def test_page_tables_are_copied_only_when_a_page_list_changed():
    """100 decode steps of three requests: the page tables are put together and go to the device
    again only in steps in which a request starts a new page or a window lets one go
    (rollout/cache.py:286-306 skips its rebuild the same way); what the device buffer holds is right
    in every step, also after other requests took part and in steps filled up for a graph."""
    from return_amd.engine.batch import StepBuilder
    P = 4

    def check(cm, batch, ids):
        for g in range(len(cm.groups)):
            want = [p for rid in ids for p in cm.live[rid].pages[g]]
            assert batch.groups[g].page_table.tolist()[:len(want)] == want
            assert batch.groups[g].cu_pages.tolist()[:len(ids) + 1] == \
                np.cumsum([0] + [len(cm.live[rid].pages[g]) for rid in ids]).tolist()
            assert batch.groups[g].kv_start.tolist()[:len(ids)] == [cm.live[rid].first_pos[g] for rid in ids]

    for window in (None, 6):
        cm = manager(page=P, max_token=800, max_requests=4, window=window)
        sb = StepBuilder(cm, 64, 4, "cpu")
        prompts = {"a": 5, "b": 9, "c": 13}                # all one token into a page: they cross together
        for rid in prompts:
            cm.add_request(rid)
        t = cm.begin_step(list(prompts.items()))
        sb.build(t, [[0] * n for n in prompts.values()], [])
        cm.end_step()
        ids = list(prompts)
        steps_that_copied = 0
        version_at_last_tables = cm.version if window is None else None     # (a window may have let pages go)
        for step in range(100):
            copies, builds, version = sb.page_table_copies, cm.table_builds, cm.version
            t = cm.begin_step([(r, 1) for r in ids])
            batch = sb.build(t, [[0]] * 3, [0, 1, 2])
            check(cm, batch, ids)
            copied = sb.page_table_copies - copies
            assert copied in (0, len(cm.groups))
            assert (cm.table_builds - builds) == (1 if copied else 0)
            # nothing changed since the last step's tables were made: nothing is made or copied
            assert bool(copied) == (cm.version != version_at_last_tables)
            version_at_last_tables = cm.version
            steps_that_copied += bool(copied)
            cm.end_step()
        if window is None:
            assert steps_that_copied == 25                 # every fourth
        else:
            assert 25 < steps_that_copied <= 51            # the window gives pages back in steps of its own
        # other requests, then a filled-up step and its repeat
        t = cm.begin_step([("a", 1), ("c", 1)])
        check(cm, sb.build(t, [[0]] * 2, [0, 1]), ["a", "c"])
        cm.end_step()
        for _ in range(3):
            t = cm.pad_tables(cm.begin_step([("a", 1), ("c", 1)]), 2)
            batch = sb.build(t, [[0]] * 4, [0, 1, 2, 3])
            check(cm, batch, ["a", "c"])
            assert batch.groups[0].page_table.tolist()[-2:] == [cm.groups[0].spare_page] * 2
            assert batch.groups[0].cu_pages.tolist()[-1] == len(batch.groups[0].page_table)
            cm.end_step()
        cm.check_invariants()
