"""The cache manager: no page lost, none held twice, none freed twice, under random orders of
requests; pages come back at the end of a request and when a window has passed them."""
import random

import numpy as np
import pytest
import torch

from sparseengine_amd.cache.manager import CacheManager, OutOfRows
from sparseengine_amd.cache.page_pool import OutOfPages, PageOwnershipError, PagePool
from sparseengine_amd.parts.base import PagedKVRequest, StateRequest

FULL = PagedKVRequest(2, 16, None)
WINDOW = PagedKVRequest(2, 16, 40)


def manager(requests, pages, rows=4, page_size=16, max_len=512, tensors=False):
    return CacheManager(requests, max_rows=rows, max_model_len=max_len, page_size=page_size, num_pages=pages,
                        dtype=torch.float32, device="cpu", allocate_tensors=tensors)


def test_page_pool_ownership():
    pool = PagePool(4)
    a = pool.allocate(3, owner=0)
    assert sorted(a) == [0, 1, 2] and pool.free_count == 1
    with pytest.raises(OutOfPages):
        pool.allocate(2, owner=1)
    assert pool.free_count == 1                                 # a refused allocation changes nothing
    with pytest.raises(PageOwnershipError, match="owned by row 0"):
        pool.release([a[0]], owner=1)
    pool.release(a[:2], owner=0)
    with pytest.raises(PageOwnershipError, match="freed twice"):
        pool.release([a[0]], owner=0)
    with pytest.raises(PageOwnershipError, match="twice in one release"):
        pool.release([a[2], a[2]], owner=0)
    assert pool.allocate(1, owner=5) == [a[1]]                  # the page given back last is used again first
    pool.check()


def test_append_is_all_or_nothing_and_slots_follow_the_table():
    m = manager({0: FULL, 1: FULL}, pages=6)
    r0, r1 = m.admit("a"), m.admit("b")
    alloc = m.append([(r0, 20), (r1, 5)])
    group = m.groups[0]
    assert m.group_of_position == {0: 0, 1: 0} and len(m.groups) == 1     # same geometry: one group, one table
    slots = alloc.slots[0]
    pages0 = group.table[r0, :2]
    assert slots[:16].tolist() == [pages0[0] * 16 + i for i in range(16)]
    assert slots[16:20].tolist() == [pages0[1] * 16 + i for i in range(4)]
    assert slots[20:].tolist() == [group.table[r1, 0] * 16 + i for i in range(5)]
    before = (group.table.copy(), m.row_len.copy(), group.pool.free_count)
    with pytest.raises(OutOfPages):
        m.append([(r0, 12), (r1, 60)])                          # 0 + 4 pages wanted, 3 free
    assert (group.table == before[0]).all() and (m.row_len == before[1]).all() and group.pool.free_count == before[2]
    assert m.can_append([(r0, 12), (r1, 43)]) and not m.can_append([(r0, 13), (r1, 43 + 16)])
    m.append([(r0, 12), (r1, 43)])                              # exactly fills what is left
    m.check_invariants()
    with pytest.raises(ValueError, match="twice"):
        m.append([(r0, 1), (r0, 1)])
    m.free("a")
    with pytest.raises(PageOwnershipError, match="holds no row"):
        m.free("a")
    m.free("b")
    assert group.pool.free_count == 6 and m.num_free_rows == 4
    m.check_invariants()


def test_rows_run_out_and_come_back():
    m = manager({0: FULL}, pages=8, rows=2)
    m.admit(1); m.admit(2)
    with pytest.raises(OutOfRows):
        m.admit(3)
    with pytest.raises(ValueError, match="already holds"):
        m.admit(1)
    m.free(1)
    assert m.admit(3) in (0, 1)
    short = manager({0: FULL}, pages=100, max_len=32)
    with pytest.raises(ValueError, match="max_model_len"):
        short.append([(short.admit("x"), 33)])


def test_groups_have_pools_of_their_own_and_windows_give_pages_back():
    m = manager({0: FULL, 1: WINDOW, 2: FULL, 3: WINDOW}, pages={0: 40, 1: 6})
    assert [g.positions for g in m.groups] == [[0, 2], [1, 3]]
    row = m.admit("r")
    held = []
    for step in range(30):                                      # 300 tokens through a window of 40
        m.append([(row, 10)])
        m.check_invariants()
        held.append(6 - m.groups[1].pool.free_count)
    assert m.groups[0].pool.free_count == 40 - 19               # the full group keeps ceil(300 / 16) pages
    assert max(held) <= 4                                       # window 40 + step 10 never needs more than 4 pages of 16
    table = m.groups[1].table[row]
    live = np.nonzero(table >= 0)[0]
    assert live.tolist() == list(range(int(m.groups[1].first_live[row]), 19))
    # every key a coming query may still read is held: the next query sits at 300 and reads keys >= 261
    assert int(m.groups[1].first_live[row]) * 16 <= 261
    m.free("r")
    assert m.groups[1].pool.free_count == 6


def test_state_slots_are_zeroed_on_admission():
    m = manager({0: FULL, 1: StateRequest((("s", (3, 2), None), ("count", (1,), torch.int32)))}, pages=4, tensors=True)
    row = m.admit("a")
    m.state[1]["s"][row] += 5
    m.state[1]["count"][row] += 2
    m.free("a")
    m.admit("b")
    assert float(m.state[1]["s"][m.row_of("b")].abs().sum()) == 0 and int(m.state[1]["count"][m.row_of("b")]) == 0
    assert m.state[1]["s"].shape == (4, 3, 2) and m.state[1]["count"].dtype == torch.int32


def test_groups_may_have_pages_of_different_sizes_and_the_oracle_counts_tokens():
    """A group's request may name its own page size; tables, slots and window release follow it, and the
    scheduler's oracle answers in tokens of cache (whole pages of the tightest group), pages being no
    common unit."""
    from sparseengine_amd.engine.llm import CacheOracle
    small = PagedKVRequest(2, 16, 40, page_size=8)
    m = CacheManager({0: FULL, 1: small}, max_rows=3, max_model_len=256, page_size=32, num_tokens=192,
                     dtype=torch.float32, device="cpu", allocate_tensors=True)
    full, windowed = m.groups
    assert (full.page_size, windowed.page_size) == (32, 8) and (full.pool.num_pages, windowed.pool.num_pages) == (6, 24)
    assert m.kv_layer(0).shape == (6, 2, 2, 32, 16) and m.kv_layer(1).shape == (24, 2, 2, 8, 16)
    assert full.table.shape[1] == 8 and windowed.table.shape[1] == 32
    oracle = CacheOracle(m)
    assert oracle.free_tokens() == 192 and oracle.total_tokens() == 192
    assert oracle.cost_of_new(33) == 64 and oracle.cost_of_new(5) == 32          # the pages of 32 are the tighter ones
    row = m.admit("a")
    alloc = m.append([(row, 37)])
    assert alloc.slots[0][36] == full.table[row, 1] * 32 + 4 and alloc.slots[1][36] == windowed.table[row, 4] * 8 + 4
    assert oracle.free_tokens() == min(4 * 32, 19 * 8) == 128
    assert oracle.cost_to_append("a", 27) == 24 and oracle.cost_to_append("a", 28) == 32    # three pages of 8; one of 32
    assert oracle.tokens_that_fit("a", 40) == 3 + 40        # the rest of the last page of 8, and five more
    assert oracle.tokens_that_fit("a", 8) == 3 + 8
    for _ in range(7):                                       # through the window of 40: the small pages come back
        m.append([(row, 20)])
        m.check_invariants()
    # 177 tokens: all six pages of 32; the last step's first query sat at 157 and read the keys from 118 on
    assert int(m.row_len[row]) == 177 and full.pool.free_count == 0
    assert int(windowed.first_live[row]) == 118 // 8 and windowed.pool.free_count == 24 - (23 - 14)
    assert oracle.free_tokens() == 0 and oracle.cost_to_append("a", 15) == 0 and oracle.cost_to_append("a", 16) == 32
    m.free("a")
    assert oracle.free_tokens() == 192
    with pytest.raises(ValueError, match="multiple of 8"):
        CacheManager({0: PagedKVRequest(2, 16, None, page_size=12)}, max_rows=1, max_model_len=64, page_size=16,
                     num_tokens=64, dtype=torch.float32, device="cpu", allocate_tensors=False)


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    windowed = seed % 2 == 1
    second = (PagedKVRequest(2, 16, 40, page_size=8) if seed >= 6 else WINDOW) if windowed else \
        (PagedKVRequest(2, 16, None, page_size=32) if seed >= 6 else FULL)
    requests = {0: FULL, 1: second, 2: StateRequest((("h", (4,), None),))}
    m = manager(requests, pages={0: 24, 1: 9 if seed < 6 else 18} if len({FULL, second}) > 1 else 24, rows=5, max_len=200,
                tensors=False)
    live, next_id, reference = {}, 0, {}
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.num_free_rows:
            live[next_id] = m.admit(next_id)
            reference[next_id] = 0
            next_id += 1
        elif action < 0.85 and live:
            chosen = rng.sample(sorted(live), rng.randint(1, len(live)))
            items = [(live[r], rng.choice([1, 1, 2, 7, 16, 33])) for r in chosen]
            items = [(row, n) for (row, n), r in zip(items, chosen) if reference[r] + n <= 200]
            if not items:
                continue
            if m.can_append(items):
                alloc = m.append(items)
                for row, n in items:
                    rid = m.row_owner[row]
                    reference[rid] += n
                for slots in alloc.slots.values():
                    assert len(set(slots.tolist())) == len(slots)          # no two tokens share a slot
            else:
                with pytest.raises(OutOfPages):
                    m.append(items)
        elif live:
            rid = rng.choice(sorted(live))
            m.free(rid)
            del live[rid], reference[rid]
        m.check_invariants()
        for rid, row in live.items():
            assert int(m.row_len[row]) == reference[rid]
    for rid in list(live):
        m.free(rid)
    m.check_invariants()
    assert all(g.pool.free_count == g.pool.num_pages for g in m.groups) and m.num_free_rows == 5


def test_truncate_undoes_an_append():
    m = manager({0: FULL}, pages=5)
    row = m.admit("a")
    m.append([(row, 20)])
    m.append([(row, 30)])
    m.truncate(row, 20)
    m.check_invariants()
    assert m.groups[0].pool.free_count == 3 and int(m.row_len[row]) == 20


@pytest.mark.parametrize("seed", range(4))
def test_a_step_of_single_tokens_takes_the_short_way_to_the_same_state(seed):
    """Decode steps (one token per item, no windowed group) are appended by a vectorised routine; it leaves the
    tables, the pools, the lengths and the slots that the general routine leaves, and refuses what that refuses."""
    rng = random.Random(seed)
    requests = {0: PagedKVRequest(2, 16), 1: PagedKVRequest(2, 16), 2: PagedKVRequest(1, 32, page_size=8)}
    fast, slow = (manager(requests, pages={0: 24, 1: 40}, rows=6, page_size=16, max_len=150) for _ in range(2))
    slow._no_window = False                     # the general routine
    live = []
    for step in range(400):
        action = rng.random()
        if (action < 0.15 or not live) and len(live) < 6:
            name = f"r{step}"
            rows = [m.admit(name) for m in (fast, slow)]
            assert rows[0] == rows[1]
            prompt = rng.randrange(1, 40)
            outcome = []
            for m in (fast, slow):
                try:
                    outcome.append(m.append([(rows[0], prompt)]).slots)
                except OutOfPages:
                    outcome.append(None)
                    m.free(name)
            assert (outcome[0] is None) == (outcome[1] is None)
            if outcome[0] is not None:
                live.append(name)
        elif action < 0.25 and live:
            name = live.pop(rng.randrange(len(live)))
            fast.free(name); slow.free(name)
        else:
            chosen = rng.sample(live, rng.randrange(1, len(live) + 1))
            results = []
            for m in (fast, slow):
                try:
                    results.append(m.append([(m.row_of(name), 1) for name in chosen]).slots)
                except (OutOfPages, ValueError) as exc:
                    results.append(type(exc))
            if isinstance(results[0], dict):
                assert isinstance(results[1], dict)
                for gi in results[0]:
                    assert results[0][gi].dtype == results[1][gi].dtype == np.int32
                    assert np.array_equal(results[0][gi], results[1][gi])
            else:
                assert results[0] is results[1]
                if results[0] is ValueError:            # a request at its longest: it ends
                    for name in [n for n in chosen if fast.row_len[fast.row_of(n)] + 1 > fast.max_model_len]:
                        live.remove(name); fast.free(name); slow.free(name)
        assert np.array_equal(fast.row_len, slow.row_len)
        for a, b in zip(fast.groups, slow.groups):
            assert np.array_equal(a.table, b.table) and a.pool._free == b.pool._free and a.pool._owner == b.pool._owner
        fast.check_invariants()
