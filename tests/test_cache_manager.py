"""The cache manager (no GPU): pool behaviour, tables, windows, state slots, and random request orders.

Scenarios of the reference's tests/kv/test_block_pool.cpp and test_paged_kv_cache.cpp, plus groups with
windows and fixed-size state, which the reference does not have.
"""

import random

import pytest

from tie_amd.cache.block_pool import BlockPool
from tie_amd.cache.manager import FREED, CacheManager
from tie_amd.cache.spec import FixedState, PagedKV, plan_cache
from tie_amd.errors import CapacityError, InvalidArgument


def test_block_pool_hands_out_low_ids_and_reuses_the_last_freed():
    pool = BlockPool(3)                                  # tests/kv/test_block_pool.cpp:8-17
    assert (pool.allocate(), pool.allocate()) == (0, 1)
    pool.release(0)
    assert pool.allocate() == 0
    assert pool.allocate() == 2
    with pytest.raises(CapacityError):
        pool.allocate()
    pool.retain(1)
    pool.release(1)
    assert pool.ref_count(1) == 1 and pool.num_free == 0
    pool.release(1)
    assert pool.num_free == 1
    for bad in (lambda: pool.release(1), lambda: pool.retain(1), lambda: pool.release(7), lambda: BlockPool(0)):
        with pytest.raises(InvalidArgument):
            bad()


def full_plan(layers=2, kvh=2, dh=16):
    return plan_cache([PagedKV(kvh, dh)] * layers, [None] * layers)


def test_pool_sizing_from_a_byte_budget():
    # 28 layers x 8 KV heads x 128 x 2 bytes x 16 tokens = 1 835 008 bytes a page; 2340 pages in 4 GiB
    # (tests/kv/test_paged_kv_cache.cpp:26-35)
    plan = full_plan(28, 8, 128)
    cache = CacheManager(plan, block_size=16, budget_bytes=4 << 30, dtype="bfloat16")
    assert cache.bytes_per_block == 1835008 and cache.num_blocks == 2340
    with pytest.raises(CapacityError):
        CacheManager(plan, block_size=16, budget_bytes=1000, dtype="bfloat16")
    with pytest.raises(InvalidArgument):
        CacheManager(plan, block_size=16, dtype="bfloat16")
    with pytest.raises(InvalidArgument):
        CacheManager(plan, block_size=16, num_blocks=4, dtype="int8")


def test_a_budget_pays_for_state_slots_first_and_gives_a_windowed_group_its_share_of_pages():
    """A model of three kinds of layers: 4 that keep every key, 6 with a window of 256 keys, 2 with a state of
    1024 floats a request. The budget covers all three; with a context hint the windowed group gets only the
    pages its requests can hold at a time and the others get what that frees."""
    needs = [PagedKV(2, 64)] * 4 + [PagedKV(2, 64, window=256)] * 6 + [FixedState((1024,))] * 2
    plan = plan_cache(needs, [None] * len(needs))
    full_page, window_page = 2 * 4 * 2 * 16 * 64 * 2, 2 * 6 * 2 * 16 * 64 * 2
    state = 2 * 8 * 1024 * 4
    budget = 64 << 20
    even = CacheManager(plan, block_size=16, budget_bytes=budget, dtype="bfloat16", max_state_slots=8)
    assert even.state_bytes == state and even.page_bytes == {0: full_page, 1: window_page}
    assert even.pool_blocks == {0: even.num_blocks, 1: even.num_blocks}
    assert even.num_blocks == (budget - state) // (full_page + window_page) and even.total_bytes() <= budget
    hinted = CacheManager(plan, block_size=16, budget_bytes=budget, dtype="bfloat16", max_state_slots=8,
                          context_hint=8192, step_tokens=512)
    share = (256 + 512 + 32) / 8192
    assert hinted.num_blocks == int((budget - state) // (full_page + share * window_page))
    assert hinted.num_blocks > 2 * even.num_blocks                       # what the windows do not need goes to the rest
    assert hinted.pool_blocks[1] == -(-int(share * hinted.num_blocks * 1e6) // int(1e6)) or \
        abs(hinted.pool_blocks[1] - share * hinted.num_blocks) < 1
    assert hinted.total_bytes() <= budget + window_page                   # (the share is rounded up to a page)
    assert hinted.capacity_tokens == hinted.num_blocks * 16               # a request's length: the full groups' pages
    # a long request runs through the small windowed pool, giving pages back as it goes
    req = hinted.new_request()
    length, chunk = 0, 512
    while length < 8192 and hinted.reserve(req, length + chunk):
        length += chunk
        hinted.trim(req, length)
    assert length == 8192 and hinted.pools[1].num_free > 0
    hinted.release(req)
    assert hinted.all_free()
    with pytest.raises(CapacityError, match="state slots"):
        CacheManager(plan, block_size=16, budget_bytes=state + 1000, dtype="bfloat16", max_state_slots=8)


def test_reserve_is_all_or_nothing_and_slots_follow_the_table():
    cache = CacheManager(full_plan(), block_size=4, num_blocks=4)
    a, b = cache.new_request(), cache.new_request()
    assert cache.reserve(a, 9) and a.tables[0] == [0, 1, 2]
    assert not cache.reserve(b, 8) and b.tables[0] == [] and cache.num_free() == 1   # nothing changed
    assert cache.reserve(b, 4)
    assert cache.reserve(a, 5) and len(a.tables[0]) == 3                              # never shrinks
    assert cache.slots(a, 0, 3, 9) == [3, 4, 5, 6, 7, 8, 9, 10][:6]
    assert cache.slots(b, 0, 0, 4) == [12, 13, 14, 15]
    with pytest.raises(InvalidArgument):
        cache.slots(a, 0, 0, 13)
    with pytest.raises(InvalidArgument):
        cache.slots(a, 0, 5, 3)
    cache.truncate(a, 4)
    assert a.tables[0] == [0] and cache.num_free() == 2
    cache.truncate(a, 4)                                                              # idempotent
    assert cache.num_free() == 2
    cache.release(a)
    cache.release(b)
    assert cache.num_free() == 4 and a.tables[0] == []
    c = cache.new_request()
    assert cache.reserve(c, 1) and c.tables[0] == [3]                                 # the page freed last comes first
    cache.audit([c])


def test_fit_counts_held_and_free_pages():
    cache = CacheManager(full_plan(), block_size=4, num_blocks=4)
    a = cache.new_request()
    cache.reserve(a, 6)
    assert cache.fit(a, 6, 100) == 10 and cache.fit(a, 6, 3) == 3
    b = cache.new_request()
    cache.reserve(b, 8)
    assert cache.fit(a, 6, 100) == 2 and cache.fit(a, 8, 1) == 0
    assert cache.can_admit(4, 0) is False


def test_groups_have_pages_of_their_own_and_windows_give_pages_back():
    needs = [PagedKV(2, 16), PagedKV(2, 16, window=6), PagedKV(2, 16), PagedKV(1, 32, window=6), PagedKV(2, 16, window=6)]
    plan = plan_cache(needs, [None] * 5)
    assert [g.num_planes for g in plan.groups] == [2, 2, 1]
    assert [(c.group, c.plane) for c in plan.calls] == [(0, 0), (1, 0), (0, 1), (2, 0), (1, 1)]
    cache = CacheManager(plan, block_size=4, num_blocks=8)
    r = cache.new_request()
    assert cache.reserve(r, 18)
    assert [len(t) for t in r.tables] == [5, 5, 5]
    # queries from position 18 on read keys from 13 on: pages 0..2 (positions 0..11) of windowed groups go back
    assert cache.trim(r, 18) == 6
    assert r.tables[0] == [0, 1, 2, 3, 4] and r.tables[1][:3] == [FREED] * 3 and r.tables[2][:3] == [FREED] * 3
    assert cache.num_free(0) == 3 and cache.num_free(1) == 6 and cache.num_free(2) == 6
    assert cache.trim(r, 18) == 0
    cache.audit([r])
    with pytest.raises(InvalidArgument):
        cache.slots(r, 1, 10, 12)                       # a position whose page was given back
    assert cache.slots(r, 1, 12, 14) == [r.tables[1][3] * 4, r.tables[1][3] * 4 + 1]
    assert cache.reserve(r, 30)                          # a table keeps growing by position
    assert len(r.tables[1]) == 8 and cache.fit(r, 30, 100) == 2   # the all-keys group is the narrow one
    cache.release(r)
    assert all(cache.num_free(g) == 8 for g in range(3))


def test_a_call_may_read_another_calls_cache():
    need = PagedKV(2, 16)
    plan = plan_cache([need, need, need], [None, 0, None])
    assert [(c.group, c.plane, c.writes) for c in plan.calls] == [(0, 0, True), (0, 0, False), (0, 1, True)]
    assert plan.groups[0].num_planes == 2
    with pytest.raises(InvalidArgument):
        plan_cache([need, PagedKV(1, 16)], [None, 0])   # the shared cache must have the same geometry
    with pytest.raises(InvalidArgument):
        plan_cache([need, need, need], [None, 0, 1])    # entry 1 owns none


def test_state_slots():
    plan = plan_cache([FixedState((3, 4)), PagedKV(1, 8), None], [None, None, None])
    assert plan.calls[2] is None and plan.state_groups == [0] and plan.paged_groups == [1]
    cache = CacheManager(plan, block_size=4, num_blocks=8, device="cpu", max_state_slots=2, dtype="float32")
    assert cache.state[0].shape == (1, 2, 3, 4) and cache.kv[1].shape == (1, 2, 8, 1, 4, 8)
    a, b, c = cache.new_request(), cache.new_request(), cache.new_request()
    assert cache.reserve(a, 3) and cache.reserve(b, 3) and {a.state_slot, b.state_slot} == {0, 1}
    cache.state[0][:, b.state_slot] = 7.0
    assert not cache.reserve(c, 3) and c.tables[1] == [] and cache.fit(c, 0, 5) == 0   # no slot free
    assert not cache.can_admit(1, 0)
    slot = b.state_slot
    cache.release(b)
    assert cache.reserve(c, 3) and c.state_slot == slot
    assert float(cache.state[0][:, slot].abs().sum()) == 0.0                            # cleared when assigned
    cache.audit([a, c])
    cache.release(a)
    cache.release(c)
    assert cache.num_free_state_slots == 2


def test_a_model_without_state_has_slots_but_no_memory_behind_them():
    cache = CacheManager(full_plan(), block_size=4, num_blocks=4, device="cpu", dtype="float32")
    assert cache.state == {} and cache.num_free_state_slots == 64
    r = cache.new_request()
    cache.reserve(r, 4)
    assert r.state_slot == -1


@pytest.mark.parametrize("seed", range(40))
def test_random_orders_never_lose_or_share_a_page(seed):
    rng = random.Random(seed)
    needs = [PagedKV(2, 16), PagedKV(2, 16, window=rng.choice([3, 8, 17]))]
    if seed % 3 == 0:
        needs.append(FixedState((4,)))
    plan = plan_cache(needs, [None] * len(needs))
    blocks = rng.randint(3, 12)
    cache = CacheManager(plan, block_size=4, num_blocks=blocks, max_state_slots=3)
    live = {}
    for _ in range(400):
        action = rng.random()
        if action < 0.35 and len(live) < 6:
            live[len(live) + rng.randrange(10 ** 6)] = [cache.new_request(), 0]
        elif live:
            key = rng.choice(list(live))
            req, length = live[key]
            if action < 0.75:
                new_len = length + rng.randint(1, 9)
                before = (cache.num_free(0), cache.num_free(1), [list(t) for t in req.tables], req.state_slot)
                if cache.reserve(req, new_len):
                    if rng.random() < 0.15:              # the step failed: roll back
                        cache.truncate(req, length)
                    else:
                        for g in plan.paged_groups:
                            assert len(cache.slots(req, g, length, new_len)) == new_len - length
                        live[key][1] = new_len
                        cache.trim(req, new_len)
                else:                                    # all or nothing
                    assert before == (cache.num_free(0), cache.num_free(1), [list(t) for t in req.tables], req.state_slot)
            else:
                cache.release(req)
                del live[key]
        cache.audit([r for r, _ in live.values()])
        for req, length in live.values():
            if length:
                assert len(req.tables[0]) == cache.blocks_for(length)
    for req, _ in live.values():
        cache.release(req)
    assert cache.num_free(0) == blocks and cache.num_free(1) == blocks
    with pytest.raises(InvalidArgument):
        r = cache.new_request()
        cache.reserve(r, 1)
        page = r.tables[0][0]
        cache.release(r)
        cache.pools[0].release(page)                     # freed twice
