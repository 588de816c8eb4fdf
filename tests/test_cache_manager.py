"""The cache manager's bookkeeping (no GPU): no page lost, held twice or freed twice."""
import random

import pytest

from sharpinference_amd.cache.manager import CacheError, CacheManager, PagePool
from sharpinference_amd.cache.spec import KVSpec, StateSpec, WINDOW_CHUNK, WINDOW_NONE, WINDOW_SLIDING


def _mgr(num_pages=32, max_requests=4, chunk=24, page_size=16):
    specs = [KVSpec(2, 16, WINDOW_CHUNK, chunk), KVSpec(2, 16, WINDOW_NONE, 0), KVSpec(2, 16, WINDOW_CHUNK, chunk),
             StateSpec((3,)), None]
    return CacheManager(specs, page_size, num_pages, max_requests, allocate=False)


def test_groups_follow_the_windows():
    m = _mgr()
    assert [g.key for g in m.groups] == [("kv", 1, 24), ("kv", 0, 0)]
    assert m.group_of_slot == [0, 1, 0, -1, -1]
    assert m.groups[0].slots == [0, 2]


def test_pool_refuses_double_free_and_runs_dry():
    p = PagePool(2)
    a, b = p.alloc(), p.alloc()
    assert p.alloc() is None
    p.release(a)
    with pytest.raises(CacheError):
        p.release(a)
    assert p.alloc() == a                     # the page just released is handed out next
    with pytest.raises(CacheError):
        p.release(7)
    assert b != a


def test_append_commit_and_window_release():
    m = _mgr()
    m.add_request("r")
    assert m.append("r", 40)                  # positions 0..39: 3 blocks in both groups
    assert m.block_table("r", 0)[:3] == m.block_table("r", 0)[:3] and len(m.block_table("r", 1)) == 3
    released = m.commit("r")
    # next query sits at 40: chunk starts at 24, so block 0 (0..15) of the chunk group is gone
    assert released == 1 and m.block_table("r", 0)[0] == -1 and m.block_table("r", 0)[1] >= 0
    assert all(p >= 0 for p in m.block_table("r", 1))
    assert m.append("r", 8) and m.commit("r") == 2      # length 48: chunk starts at 48, blocks 1 and 2 go too
    assert m.block_table("r", 0)[:3] == [-1, -1, -1]
    m.check_invariants()
    assert m.slots_for("r", 1, 30, 3) == [m.block_table("r", 1)[1] * 16 + 14, m.block_table("r", 1)[1] * 16 + 15,
                                          m.block_table("r", 1)[2] * 16]
    with pytest.raises(CacheError):
        m.slots_for("r", 1, 47, 2)            # position 48 is beyond what was appended
    with pytest.raises(CacheError):
        m.slots_for("r", 0, 10, 1)            # a released position has no slot
    m.free_request("r")
    m.check_invariants()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups)
    with pytest.raises(CacheError):
        m.free_request("r")


def test_sliding_window_releases_behind_the_window():
    m = CacheManager([KVSpec(1, 16, WINDOW_SLIDING, 20)], 16, 8, 2, allocate=False)
    m.add_request("s")
    for _ in range(5):
        assert m.append("s", 16)
        m.commit("s")
        m.check_invariants()
    # length 80: the next query (80) sees keys from 61: blocks 0..2 released
    assert m.block_table("s", 0) == [-1, -1, -1] + m.block_table("s", 0)[3:]
    assert m.groups[0].pool.num_free == 8 - 2


def test_exhaustion_changes_nothing_and_rollback_returns_pages():
    m = _mgr(num_pages=4)
    m.add_request("a")
    m.add_request("b")
    assert m.append("a", 48)
    before = [g.pool.num_free for g in m.groups]
    assert not m.append("b", 40)              # needs 3 pages, one left
    assert [g.pool.num_free for g in m.groups] == before and m.requests["b"].pending == 0
    assert m.append("b", 10)
    m.rollback("b")
    assert [g.pool.num_free for g in m.groups] == before and m.block_table("b", 1) == []
    m.check_invariants()


def test_state_slots_and_reservations():
    m = _mgr(num_pages=8, max_requests=2)
    assert m.can_admit(100, 16) and not m.can_admit(16 * 9, 16)
    assert not m.fits_alone(16 * 9, 16) and m.fits_alone(128, 16)
    m.add_request("a", reserve_tokens=100, max_step_tokens=16)
    assert not m.can_admit(100, 16)           # 7 of 8 pages of the all-keys group are promised
    m.add_request("b")
    with pytest.raises(CacheError):
        m.add_request("c")                    # no state slot left
    assert m.requests["a"].state_slot != m.requests["b"].state_slot
    m.free_request("a")
    assert m.can_admit(100, 16)
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_a_page(seed):
    rng = random.Random(seed)
    m = _mgr(num_pages=rng.choice([6, 12, 40]), max_requests=4, chunk=rng.choice([16, 24, 40]), page_size=rng.choice([16, 32]))
    live, next_id, reuse = {}, 0, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 4:
            m.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 17, 33])
            free_before = [g.pool.num_free for g in m.groups]
            if m.append(rid, n):
                if rng.random() < 0.1:
                    m.rollback(rid)
                    assert [g.pool.num_free for g in m.groups] == free_before
                else:
                    m.commit(rid)
                    live[rid] += n
                    assert m.length(rid) == live[rid]
            else:
                assert [g.pool.num_free for g in m.groups] == free_before
        elif live:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
        m.check_invariants()
        # every position a later query can see has a page
        for rid, L in live.items():
            for g, grp in enumerate(m.groups):
                first = grp.spec.first_visible(L)
                tbl = m.block_table(rid, g)
                assert all(tbl[b] >= 0 for b in range(first // m.page_size, (L + m.page_size - 1) // m.page_size))
                # pages behind the window are all given back (none is kept by a step that skipped them), and
                # the table as an array, which is made anew only when the table changed, is the table
                if grp.spec.window_kind != 0:
                    assert all(tbl[b] < 0 for b in range(min(first // m.page_size, len(tbl))))
                assert m.block_table_array(rid, g).tolist() == list(tbl)
    reuse = sum(g.pool.total_allocs > g.pool.num_pages for g in m.groups)
    for rid in list(live):
        m.free_request(rid)
    m.check_invariants()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups)
    assert reuse >= 1 or m.groups[0].pool.num_pages >= 40


def test_keys_and_values_of_different_widths():
    """A mixer may ask for values of another width than its keys: the value tensor and the bytes of
    a page follow."""
    import torch

    spec = KVSpec(2, 48, WINDOW_NONE, 0, v_head_dim=32)
    m = CacheManager([spec, KVSpec(2, 16)], 16, 4, 2, dtype=torch.float32)
    assert m.k[0].shape == (4, 2, 16, 48) and m.v[0].shape == (4, 2, 32, 16)
    assert m.k[1].shape == (4, 2, 16, 16) and m.v[1].shape == (4, 2, 16, 16)
    assert m.bytes_per_page() == [2 * (48 + 32) * 16 * 4 + 2 * (16 + 16) * 16 * 4]
    assert spec.value_dim == 32 and KVSpec(2, 16).value_dim == 16
