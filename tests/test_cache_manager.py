"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of
requests; windows give pages back; prefix pages are shared and evicted oldest-first; state slots."""
import random

import pytest

from llmserver_amd.cache import CacheExhaustedError, CacheManager, CacheStateError, PagePool, PageState
from llmserver_amd.parts import PagedKVSpec, StateSpec

FULL = PagedKVSpec(2, 16)
WINDOW = PagedKVSpec(2, 16, window=10)


def manager(specs, page_size=4, pages=8, slots=0):
    return CacheManager(specs, page_size, pages, num_state_slots=slots, allocate_storage=False)


def test_pool_hands_out_pages_in_order_and_reuses_freed_ones_last():
    pool = PagePool(4, 2)
    assert [pool.allocate() for _ in range(3)] == [0, 1, 2]
    pool.release(1)
    assert [pool.allocate(), pool.allocate()] == [3, 1]         # freed page goes to the back of the queue
    with pytest.raises(CacheExhaustedError):
        pool.allocate()
    pool.check_invariants()


def test_pool_rejects_bad_ids_and_double_frees():
    pool = PagePool(2, 2)
    page = pool.allocate()
    with pytest.raises(ValueError):
        pool.release(7)
    with pytest.raises(CacheStateError):
        pool.release(1)                  # never allocated
    pool.release(page)
    with pytest.raises(CacheStateError):
        pool.release(page)               # freed twice
    with pytest.raises(CacheStateError):
        pool.hold(page)
    with pytest.raises(ValueError):
        PagePool(0, 2)


def test_release_all_validates_before_it_frees_anything():
    pool = PagePool(4, 2)
    table = [pool.allocate(), pool.allocate()]
    with pytest.raises(ValueError):
        pool.release_all(table + [table[0]])
    with pytest.raises(CacheStateError):
        pool.release_all(table + [3])          # page 3 was never handed out
    assert pool.num_free == 2
    table.insert(1, -1)                        # an entry a window has passed was given back earlier
    pool.release_all(table)
    assert table == [] and pool.num_free == 4
    pool.check_invariants()


def test_every_page_is_in_one_state():
    pool = PagePool(3, 2)
    a, b = pool.allocate(), pool.allocate()
    pool.publish(a, "ha")
    pool.release(a)
    assert [pool.state[p] for p in range(3)] == [PageState.IDLE, PageState.HELD, PageState.FREE]
    pool.hold(a)                               # an idle page can be taken up again: its tokens are still there
    pool.hold(a)
    assert pool.state[a] == PageState.HELD and pool.holders[a] == 2 and pool.num_idle == 0
    pool.release(a)
    pool.release(a)
    pool.publish(b, "ha")                      # a second page with the same tokens: the first stays the one to adopt
    pool.release(b)
    assert pool.state[b] == PageState.FREE and pool.lookup("ha") == a
    pool.check_invariants()


def test_registered_pages_idle_then_are_evicted_oldest_first():
    pool = PagePool(3, 2)
    a, b, c = pool.allocate(), pool.allocate(), pool.allocate()
    pool.publish(a, "ha")
    pool.publish(b, "hb")
    pool.release(b)
    pool.release(a)
    pool.release(c)
    assert (pool.num_free, pool.num_idle, pool.num_available) == (1, 2, 3)
    table = []
    assert pool.adopt("ha", table) == a and pool.holders[a] == 1 and pool.num_idle == 1
    assert pool.allocate() == c
    assert pool.allocate() == b and pool.lookup("hb") is None    # b was the oldest idle page: recycled, digest forgotten
    with pytest.raises(CacheExhaustedError):
        pool.allocate()
    with pytest.raises(ValueError):
        pool.adopt("ha", table)          # same page twice in one table
    pool.check_invariants()


def test_groups_by_need_have_pages_of_their_own():
    m = manager({0: FULL, 1: WINDOW, 2: FULL, 3: WINDOW}, pages=[6, 4])
    assert [g.caches for g in m.groups] == [[0, 2], [1, 3]] and [g.pool.num_pages for g in m.groups] == [6, 4]
    assert not m.prefix_caching_possible
    m.open("a")
    m.ensure("a", 9)
    assert [len(t) for t in m.record("a").tables] == [3, 3]
    assert m.available_pages() == [3, 1]


def test_window_gives_pages_back_once_every_query_has_passed_them():
    m = manager({0: WINDOW}, page_size=4, pages=5)
    m.open("a")
    total = 0
    for chunk in (6, 5, 1, 1, 7, 1, 1, 1, 9):
        total += chunk
        m.ensure("a", total)
        m.advance("a", total)
        table = m.record("a").tables[0]
        first_visible = max(0, total - 10 + 1)                    # a query at position `total` sees keys from here
        for block, page in enumerate(table):
            assert (page < 0) == ((block + 1) * 4 <= first_visible), (total, table)
        m.check_invariants()
    assert total == 32 and m.groups[0].pool.num_pages == 5         # 32 tokens ran through 5 pages of 4
    m.close("a")
    assert m.available_pages() == [5]


def test_ensure_is_all_or_nothing():
    m = manager({0: FULL, 1: WINDOW}, pages=[8, 2])
    m.open("a")
    with pytest.raises(CacheExhaustedError):
        m.ensure("a", 12)                # needs 3 pages in both groups; the window group has 2
    assert m.available_pages() == [8, 2] and m.record("a").tables == [[], []]
    m.check_invariants()


def test_state_slots_are_acquired_zeroed_and_released():
    m = manager({0: FULL, 1: StateSpec((3,))}, slots=2)
    a, b = m.open("a"), m.open("b")
    assert {a.state_slot, b.state_slot} == {0, 1} and m.state_slots_free() == 0
    with pytest.raises(CacheExhaustedError):
        m.open("c")
    assert not m.has("c")
    freed = a.state_slot
    m.close("a")
    assert m.open("c").state_slot == freed
    m.check_invariants()


def test_a_record_can_wait_without_a_slot_and_take_one_when_it_computes():
    m = manager({0: FULL, 1: StateSpec((3,))}, slots=1)
    waiting = [m.open(name, state=False) for name in ("a", "b", "c")]        # more records than slots: nobody computes yet
    assert [r.state_slot for r in waiting] == [-1, -1, -1] and m.state_slots_free() == 1
    assert not m.holds_anything("a")
    assert m.acquire_state("a") == 0 and m.acquire_state("a") == 0            # asked twice, one slot
    assert m.holds_anything("a") and m.state_slots_free() == 0
    with pytest.raises(CacheExhaustedError):
        m.acquire_state("b")
    m.close("a")
    assert m.acquire_state("b") == 0
    m.check_invariants()
    assert manager({0: FULL}).state_slots_free() is None                      # no mixer keeps state: nothing to run out of


def test_what_a_plan_would_cost_is_answered_per_group():
    m = manager({0: FULL, 1: WINDOW}, page_size=4, pages=[8, 3])
    assert m.pages_needed("nobody", 9) == [3, 3] and m.token_room("nobody", [2, 1]) == 4
    m.open("a")
    m.ensure("a", 6)
    assert m.pages_needed("a", 6) == [0, 0] and m.pages_needed("a", 13) == [2, 2]
    assert m.available_pages() == [6, 1]
    assert m.token_room("a", [6, 1]) == 12 and m.token_room("a", [0, 0]) == 8    # the scarcer group bounds it
    assert m.holds_anything("a") and not m.holds_anything("nobody")
    with pytest.raises(CacheStateError):
        m.open("a")                      # a request has one record
    with pytest.raises(KeyError):
        m.close("nobody")


def test_prefix_pages_are_shared_leaving_one_token_to_compute():
    m = manager({0: FULL, 1: FULL}, page_size=4, pages=6)          # both caches in one group
    prompt = list(range(10, 20))
    m.open("a")
    m.ensure("a", 10)
    m.register_prefix("a", prompt, 0, 10)
    assert len(m.groups[0].pool.published_pages()) == 2                     # 10 tokens: two complete pages
    for length, shared in ((4, 0), (8, 1), (10, 2)):
        rid = f"r{length}"
        m.open(rid)
        assert m.share_prefix(rid, prompt[:length]) == shared * 4
        assert m.record(rid).tables[0] == m.record("a").tables[0][:shared]
        m.close(rid)
    m.open("other")
    assert m.share_prefix("other", [99] + prompt[1:]) == 0          # a different first page breaks the chain
    assert m.share_prefix("other", prompt[:4] + [0] * 6) == 4
    m.check_invariants()
    m.close("a")
    assert m.groups[0].pool.num_idle == 1 and m.groups[0].pool.num_free == 4   # page 1 idles, page 0 is still shared


def test_digest_depends_on_parent_tokens_and_model():
    m = manager({0: FULL})
    d = m.digest("root", [1, 2, 3, 4])
    assert len(d) == 64 and d == m.digest("root", [1, 2, 3, 4])
    assert d != m.digest("other", [1, 2, 3, 4]) and d != m.digest("root", [1, 2, 3, 5])
    other = CacheManager({0: FULL}, 4, 8, allocate_storage=False, model_identity="another")
    assert d != other.digest("root", [1, 2, 3, 4])


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_lose_nothing(seed):
    rng = random.Random(seed)
    specs = {0: FULL, 1: WINDOW, 2: StateSpec((2,))} if seed % 2 else {0: FULL, 1: FULL}
    m = manager(specs, page_size=4, pages=12, slots=4)
    live, lengths, prompts = [], {}, {}
    for step in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            rid = f"r{step}"
            m.open(rid)
            prompts[rid] = [rng.randrange(3) for _ in range(rng.randrange(1, 30))]
            lengths[rid] = m.share_prefix(rid, prompts[rid]) if m.prefix_caching_possible else 0
            live.append(rid)
        elif action < 0.85 and live:
            rid = rng.choice(live)
            grown = lengths[rid] + rng.choice((1, 1, 1, 2, 5, 9))
            try:
                m.ensure(rid, grown)
            except CacheExhaustedError:
                victim = rng.choice(live)
                m.close(victim)
                live.remove(victim)
                continue
            m.advance(rid, grown)
            m.register_prefix(rid, prompts[rid], lengths[rid], grown)
            lengths[rid] = grown
            if rng.random() < 0.5:       # the array a step copies into its block table mirrors the list, whatever changed it
                for group in m.groups:
                    assert m.record(rid).table_array(group.index).tolist() == m.record(rid).tables[group.index]
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            m.close(rid)
        m.check_invariants()
    for rid in live:
        for group in m.groups:
            assert m.record(rid).table_array(group.index).tolist() == m.record(rid).tables[group.index]
        m.close(rid)
    m.check_invariants()
    for group in m.groups:
        assert group.pool.num_available == group.pool.num_pages
