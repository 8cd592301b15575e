"""Cache manager bookkeeping on the host: pages, block tables, windows, state slots (CPU)."""

import random

import pytest
import torch

from llm_runtime_study_amd.cache import CacheManager, PagePool
from llm_runtime_study_amd.errors import KVCacheError
from llm_runtime_study_amd.parts import PagedKVNeed, StateNeed

FULL = PagedKVNeed(2, 16)


def manager(needs=(FULL, FULL), page_size=4, num_pages=8, max_requests=3, max_seq_len=32, storage=False):
    return CacheManager(list(needs), page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                        max_seq_len=max_seq_len, dtype=torch.float32, device="cpu", allocate_storage=storage)


def test_page_pool_lowest_first_and_reuse_order():
    # reference tests/test_cache.py:268-281
    pool = PagePool(4)
    assert pool.allocate(3) == [0, 1, 2]
    with pytest.raises(KVCacheError, match="need 2 blocks but only 1 are free"):
        pool.allocate(2)
    pool.free([1])
    pool.free([0])
    assert pool.allocate(2) == [0, 1]
    with pytest.raises(KVCacheError, match="not held"):
        pool.free([3])
    pool.free([2])
    with pytest.raises(KVCacheError, match="not held"):
        pool.free([2])   # freed twice


def test_block_table_grows_page_by_page_across_edges():
    m = manager()
    a = m.admit("a")
    m.extend(a, 3)
    assert a.tables == [[0]] and a.length == 3
    m.extend(a, 1)            # exactly fills the page
    assert a.tables == [[0]]
    m.extend(a, 1)            # first token of the next page
    assert a.tables == [[0, 1]]
    m.extend(a, 6)
    assert a.tables == [[0, 1, 2]] and a.length == 11
    assert m.slot_of_position(a, 0, 0) == 0 and m.slot_of_position(a, 0, 5) == 1 * 4 + 1
    assert list(m.groups[0].host_table[a.slot, :4]) == [0, 1, 2, -1]
    m.check_invariants()
    assert m.used_pages() == 3 and m.used_tokens == 12 and m.active_requests == 1


def test_rollback_gives_back_only_the_pages_past_the_length():
    m = manager()
    a = m.admit("a")
    m.extend(a, 5)
    m.extend(a, 7)
    assert m.used_pages() == 3
    m.rollback(a, 5)
    assert a.length == 5 and a.tables == [[0, 1]] and m.used_pages() == 2
    m.rollback(a, 0)
    assert m.used_pages() == 0 and a.tables == [[]]
    with pytest.raises(KVCacheError, match="cannot roll cache back"):
        m.rollback(a, 1)
    m.check_invariants()


def test_exhaustion_leaves_everything_untouched():
    m = manager(num_pages=3)
    a, b = m.admit("a"), m.admit("b")
    m.extend(a, 8)
    with pytest.raises(KVCacheError, match="KV block pool exhausted: need 2 blocks but only 1 are free"):
        m.extend(b, 5)
    assert b.length == 0 and b.tables == [[]] and m.free_pages() == 1
    with pytest.raises(KVCacheError, match="capacity exceeded: need 33 positions but capacity is 32"):
        m.extend(a, 25)
    m.check_invariants()


def test_release_is_idempotent_and_a_released_cache_is_unusable():
    m = manager()
    a = m.admit("a")
    m.extend(a, 9)
    m.release(a)
    m.release(a)
    assert m.used_pages() == 0 and m.active_requests == 0 and m.free_slots == 3
    with pytest.raises(KVCacheError, match="released"):
        m.extend(a, 1)
    b = m.admit("b")
    m.extend(b, 9)
    assert b.tables == [[0, 1, 2]] and b.slot == a.slot   # pages and slot are used again, lowest first
    m.check_invariants()


def test_slots_run_out_and_reservations_gate_admission():
    m = manager(num_pages=8, max_requests=2)
    assert m.can_admit(20) and not m.can_admit(33)
    a = m.admit("a", reserve_tokens=20)      # 5 pages promised
    assert m.can_admit(12) and not m.can_admit(13)
    b = m.admit("b", reserve_tokens=12)
    assert not m.can_admit(1)                # no slot left
    with pytest.raises(KVCacheError, match="request slots are in use"):
        m.admit("c")
    m.release(a)
    assert m.can_admit(20)
    with pytest.raises(KVCacheError, match="only 5 are unreserved"):
        m.admit("c", reserve_tokens=24)
    m.release(b)


def test_window_group_gives_pages_back_as_the_window_passes():
    window = PagedKVNeed(2, 16, window=6)
    m = manager(needs=(FULL, window), page_size=4, num_pages=10, max_seq_len=40)
    assert len(m.groups) == 2
    a = m.admit("a")
    m.extend(a, 9)
    assert m.trim(a) == 1                     # next query (pos 9) sees keys > 3: page 0 (0..3) is dead
    assert a.tables[1] == [-1, 1, 2] and a.tables[0] == [0, 1, 2]
    m.extend(a, 1)
    assert m.trim(a) == 0                     # pos 10 sees keys > 4: page 1 (4..7) still holds 5, 6, 7
    m.extend(a, 6)
    assert m.trim(a) == 1                     # pos 16 sees keys > 10: pages 0 and 1 dead
    assert a.tables[1] == [-1, -1, 2, 0] and a.first_live[1] == 2   # the freed page 0 is used again
    m.check_invariants()
    with pytest.raises(KVCacheError, match="given back"):
        m.slot_of_position(a, 1, 5)
    with pytest.raises(KVCacheError, match="left the window"):
        m.rollback(a, 4)
    m.release(a)
    assert m.used_pages(0) == 0 and m.used_pages(1) == 0


def test_groups_share_needs_and_follow_cache_sources():
    window = PagedKVNeed(2, 16, window=8)
    state = StateNeed((3, 5))
    m = manager(needs=(FULL, window, FULL, ("from", 0), state, None, window), storage=True, page_size=4, num_pages=4)
    assert [g.entries for g in m.groups] == [[0, 2], [1, 6]]
    caches = m.layer_caches
    assert caches[3] is caches[0] and caches[0].group == 0 and caches[1].group == 1 and caches[5].group is None
    assert caches[0].k_pages.shape == (5, 2, 4, 16)          # one extra page for padding rows
    assert caches[0].v_pages.shape == (5, 2, 16, 4)          # values are transposed inside a page
    assert caches[0].k_pages.data_ptr() != caches[2].k_pages.data_ptr()
    assert caches[4].state.shape == (3 + 1, 3, 5) and m.trash_slot == 3   # one row beyond the requests' slots: the trash slot
    a = m.admit("a")
    caches[4].state[a.slot] += 1.0
    m.release(a)
    b = m.admit("b")
    assert b.slot == a.slot and caches[4].state[b.slot].abs().sum() == 0   # zeroed at admission
    with pytest.raises(KVCacheError, match="keeps no pages"):
        manager(needs=(state, ("from", 0)))
    with pytest.raises(KVCacheError, match="unknown cache need"):
        manager(needs=("pages",))


def test_state_rows_are_put_back_after_a_failed_step():
    state = StateNeed((4,))
    m = manager(needs=(FULL, state, state), storage=True, page_size=4, num_pages=8)
    a, b, c = m.admit("a"), m.admit("b"), m.admit("c")
    for position in (1, 2):
        m.layer_caches[position].state[:] = torch.arange(4 * 4, dtype=torch.float32).view(4, 4) + 100 * position
    kept = m.snapshot_state([a, c])
    before = [m.layer_caches[position].state.clone() for position in (1, 2)]
    for position in (1, 2):
        m.layer_caches[position].state[[a.slot, c.slot]] -= 7.0          # what a step's mixers did before the step failed
        m.layer_caches[position].state[b.slot] += 1.0                    # another request's row: not the failed step's business
    m.restore_state(kept)
    for position, old in zip((1, 2), before):
        now = m.layer_caches[position].state
        assert torch.equal(now[[a.slot, c.slot]], old[[a.slot, c.slot]]) and torch.equal(now[b.slot], old[b.slot] + 1.0)
    assert manager(needs=(FULL,)).snapshot_state([]) == []               # a model without state pays nothing


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_or_double_a_page(seed):
    rng = random.Random(seed)
    needs = (FULL, PagedKVNeed(1, 8, window=5), StateNeed((2,)))
    m = manager(needs=needs, page_size=4, num_pages=12, max_requests=4, max_seq_len=40)
    live, counter = [], 0
    for _ in range(400):
        action = rng.random()
        if action < 0.2 and m.free_slots:
            live.append(m.admit(counter))
            counter += 1
        elif action < 0.7 and live:
            request = rng.choice(live)
            before = (request.length, [list(t) for t in request.tables])
            try:
                m.extend(request, rng.randint(1, 9))
                if rng.random() < 0.2:         # a failed forward
                    m.rollback(request, before[0])
                else:
                    m.trim(request)
            except KVCacheError:
                assert (request.length, [list(t) for t in request.tables]) == before
        elif action < 0.85 and live:
            request = live.pop(rng.randrange(len(live)))
            m.release(request)
        m.check_invariants()
        for request in live:
            for group, table in enumerate(request.tables):
                assert len(table) == -(-request.length // 4)
                window = m.groups[group].need.window
                for block, page in enumerate(table):
                    last = (block + 1) * 4 - 1
                    visible = window is None or last > request.length - window
                    assert page >= 0 or not visible   # every position a future query may see is held
    for request in live:
        m.release(request)
    m.check_invariants()
    assert all(g.pool.used_pages == 0 and g.reserved_pages == 0 for g in m.groups) and m.free_slots == 4
