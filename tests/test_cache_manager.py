"""The cache manager on the host: the vectors that the reference's own allocator tests hold, windows, and
random orders of requests with the invariants checked after every operation."""
import random

import pytest

from vt_transformer_amd.cache import NO_PAGE, CacheError, CacheManager, GroupSpec, PagePool, SlotPool


def manager(num_pages=8, page_size=1, windows=(0,), max_requests=4, max_seq_len=4096):
    return CacheManager([GroupSpec(i, w, num_pages) for i, w in enumerate(windows)], page_size, max_requests, max_seq_len)


def test_pages_come_lowest_first_and_last_freed_first():
    """vt-transformer/test/vt_cache_test.cpp:72-78: the first allocation of three tokens gets ids 0, 1, 2."""
    m = manager(num_pages=8, page_size=1)
    m.admit("a")
    assert m.reserve([("a", 3)])
    assert m.get("a").tables[0] == [0, 1, 2]
    pool = PagePool(4)
    assert pool.alloc(2) == [0, 1]
    pool.free([0])
    assert pool.alloc(2) == [0, 2]         # last in, first out


def test_page_size_two():
    """vt_cache_test.cpp:108-116: page_size 2, four tokens -> the first two pages (the reference names them by
    their first slot, 0 and 2, and repeats each id per token: 0,0,2,2; here one entry per page: 0, 1)."""
    m = manager(num_pages=8, page_size=2)
    m.admit("a")
    assert m.reserve([("a", 4)])
    assert m.get("a").tables[0] == [0, 1]
    assert [p * 2 for p in m.get("a").tables[0]] == [0, 2]      # the reference's slot-numbered ids


def test_a_half_full_page_is_not_allocated_again():
    """vt_cache_test.cpp:168-207: after [0,6) with pages of 4, extending to 9 takes exactly one more page."""
    m = manager(num_pages=8, page_size=4)
    m.admit("a")
    assert m.reserve([("a", 6)])
    m.commit("a", 6)
    assert m.get("a").tables[0] == [0, 1]
    assert m.pages_needed(m.get("a"), 8) == [0]
    assert m.pages_needed(m.get("a"), 9) == [1]
    assert m.reserve([("a", 9)])
    assert m.get("a").tables[0] == [0, 1, 2] and m.pools[0].available == 5


def test_all_or_nothing():
    m = manager(num_pages=4, page_size=2)
    m.admit("a"); m.admit("b")
    assert m.reserve([("a", 4)])
    before = (list(m.get("a").tables[0]), list(m.get("b").tables[0]), m.pools[0].available)
    assert not m.reserve([("a", 6), ("b", 4)])                  # needs 1 + 2 pages, 2 are free
    assert (m.get("a").tables[0], m.get("b").tables[0], m.pools[0].available) == before
    assert m.reserve([("a", 6), ("b", 2)])
    m.check()


def test_available_is_counted_in_tokens():
    """vt_cache_test.cpp:254-262: available size = free pages x page size."""
    m = manager(num_pages=5, page_size=4)
    assert m.available_tokens() == 20
    m.admit("a")
    m.reserve([("a", 5)])
    assert m.available_tokens() == 12


def test_release_returns_everything_and_errors_are_loud():
    m = manager(num_pages=4, page_size=2, max_requests=2)
    m.admit("a"); m.admit("b")
    assert m.admit("c") is None                                  # no slot left
    m.reserve([("a", 3), ("b", 1)])
    slot_a = m.get("a").slot
    m.release("a")
    assert m.pools[0].available == 3 and m.slots.available == 1
    assert m.admit("c").slot == slot_a                           # the slot is used again
    with pytest.raises(CacheError):
        m.release("a")
    with pytest.raises(CacheError):
        m.admit("b")
    with pytest.raises(CacheError):
        m.reserve([("b", 2), ("b", 3)])
    with pytest.raises(CacheError):
        m.pools[0].free([3])                                     # never handed out
    with pytest.raises(CacheError):
        manager(max_seq_len=8).reserve([("x", 2)])
    m2 = manager(max_seq_len=8)
    m2.admit("x")
    with pytest.raises(CacheError):
        m2.reserve([("x", 9)])


def test_shrinking_is_refused():
    m = manager(num_pages=4, page_size=2)
    m.admit("b")
    m.reserve([("b", 3)])
    m.commit("b", 3)
    with pytest.raises(CacheError):
        m.reserve([("b", 2)])


def test_window_gives_pages_back_once_passed():
    """Group 0 keeps every key, group 1 the last 5.  With pages of 4, a page is dead when its last key is."""
    m = manager(num_pages=16, page_size=4, windows=(0, 5))
    m.admit("a")
    assert m.reserve([("a", 10)])
    assert m.get("a").tables == [[0, 1, 2], [0, 1, 2]]           # a long portion needs all its pages while it runs
    m.commit("a", 10)
    # the next token (position 10) sees keys 6..10: block 0 (keys 0-3) is dead, block 1 (4-7) is not
    assert m.get("a").tables == [[0, 1, 2], [NO_PAGE, 1, 2]]
    assert m.pools[1].available == 14 and m.pools[0].available == 13
    for n in range(11, 14):
        assert m.reserve([("a", n)])
        m.commit("a", n)
        m.check()
    # length 13: next token sees keys 9..13, blocks 0 and 1 dead
    assert m.get("a").tables[1][:2] == [NO_PAGE, NO_PAGE] and m.get("a").tables[0][:2] == [0, 1]
    held = [p for p in m.get("a").tables[1] if p != NO_PAGE]
    assert len(held) == 2
    m.release("a")
    assert m.pools[1].available == 16 and m.pools[0].available == 16
    m.check()


def test_freed_window_page_is_used_again():
    m = manager(num_pages=3, page_size=2, windows=(2,))
    m.admit("a")
    seen = set()
    for n in range(1, 40):
        assert m.reserve([("a", n)]), n                           # three pages carry a sequence of any length
        m.commit("a", n)
        seen.update(p for p in m.get("a").tables[0] if p != NO_PAGE)
        m.check()
    assert seen <= {0, 1, 2} and len(seen) >= 2      # freed pages came back; no fourth page was ever needed


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_invariants(seed):
    """No page lost, held twice or freed twice, whatever the order of admissions, portions and ends."""
    rng = random.Random(seed)
    page_size = rng.choice([1, 2, 4, 16])
    m = manager(num_pages=rng.randint(6, 40), page_size=page_size, windows=(0, rng.choice([3, 17, 64])),
                max_requests=5, max_seq_len=200)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and len(live) < 5:
            rp = m.admit(next_id)
            if rp is not None:
                live[next_id] = 0
                next_id += 1
        elif op < 0.85 and live:
            chosen = rng.sample(sorted(live), rng.randint(1, len(live)))
            items = [(r, min(200, live[r] + rng.choice([1, 1, 1, 2, 7, 30]))) for r in chosen]
            items = [(r, n) for r, n in items if n > live[r]]
            before = m.available_pages()
            if items and m.reserve(items):
                for r, n in items:
                    m.commit(r, n)
                    live[r] = n
            else:
                assert m.available_pages() == before               # a refused step changes nothing
        elif live:
            r = rng.choice(sorted(live))
            m.release(r)
            del live[r]
        m.check()
        for r, n in live.items():
            rp = m.get(r)
            assert rp.length == n
            # every key that a later token can still see has a page
            for gi, g in enumerate(m.groups):
                lo = max(0, n - g.window + 1) if g.window else 0
                for pos in range(lo, n):
                    assert rp.tables[gi][pos // page_size] != NO_PAGE
    for r in list(live):
        m.release(r)
    m.check()
    assert m.held_pages() == [0, 0] and m.slots.available == 5


def test_slot_pool():
    s = SlotPool(2)
    a, b = s.alloc(), s.alloc()
    assert (a, b) == (0, 1) and s.alloc() is None
    s.free(a)
    with pytest.raises(CacheError):
        s.free(a)
    assert s.alloc() == 0


def _kv_need(kv, d, window=0):
    from vt_transformer_amd.parts.base import CacheNeed, PageTensor
    return CacheNeed((PageTensor("k", (kv, d), 1), PageTensor("v", (kv, d), 2)), window=window)


def _fake_model(needs):
    from types import SimpleNamespace

    from vt_transformer_amd.config.base import ScheduleEntry
    mixers = [SimpleNamespace(cache_need=lambda n=n: n, state_need=lambda: None) for n in needs]
    return SimpleNamespace(schedule=[ScheduleEntry(i) for i in range(len(needs))],
                           layers=[SimpleNamespace(mixer=m) for m in mixers], spec=SimpleNamespace(vocab_size=10))


def test_a_byte_budget_is_shared_by_the_groups_of_layers_by_their_needs():
    """The reference sizes its one pool as budget // (block size x bytes per token)
    (vt-transformer/models/qwen3-0.6b/init.vt:109-113).  Here groups of layers have pages of their own.  A group with
    a window gets what its requests can hold at a time (window + a portion, per request) and no more; the rest of the
    budget is divided by the bytes of one page of each group that keeps every key."""
    import pytest
    import torch

    from vt_transformer_amd.cache.storage import CacheStorage
    from vt_transformer_amd.parts.base import Runtime

    # three layers keep every key of 2 heads x 16; two keep a window of 8 keys of 1 head x 32
    needs = [_kv_need(2, 16), _kv_need(1, 32, 8), _kv_need(2, 16), _kv_need(1, 32, 8), _kv_need(2, 16)]
    model = _fake_model(needs)
    rt = Runtime(torch.device("cpu"), torch.float32)
    page = 4
    whole_page = 2 * 4 * page * 3 * 2 * 16          # keys and values, float32, three layers
    window_page = 2 * 4 * page * 2 * 1 * 32         # two layers
    # 4 requests, portions of 8 tokens: a request holds (8 + 8) / 4 + 1 = 5 pages of the windowed group at most, and
    # the scheduler keeps one more free for each: 24 pages, however large the budget
    budget = 24 * window_page + 10 * whole_page + whole_page // 2
    st = CacheStorage(rt, model, page, None, 4, 64, kv_bytes=budget, max_portion=8)
    assert st.page_bytes == [whole_page, window_page]
    assert [p.num_pages for p in st.manager.pools] == [10, 24] and st.num_pages == 10
    assert st.kv_bytes == 24 * window_page + 10 * whole_page <= budget
    held = sum(t.numel() * t.element_size() for g in st.pages for t in g.values())
    assert held == st.kv_bytes
    assert st.pages[0]["k"].shape == (3, 10, 2, page, 16) and st.pages[0]["v"].shape == (3, 10, 2, 16, page)
    assert st.pages[1]["k"].shape == (2, 24, 1, page, 32)
    assert st.manager.max_held_pages(1, 8) == 5 and st.manager.max_held_pages(0, 8) == 16
    # ten times the budget: the windowed group stays, the other takes everything
    big = CacheStorage(rt, model, page, None, 4, 64, kv_bytes=24 * window_page + 100 * whole_page, max_portion=8)
    assert [p.num_pages for p in big.manager.pools] == [100, 24]
    # as it was before the groups were sized by need, every group would have had budget // (both pages) = the same
    assert budget // (whole_page + window_page) < 24
    # whole sequences in one step (no portion given): the windowed group's requests may hold a whole sequence
    assert CacheStorage(rt, model, page, None, 4, 64, kv_bytes=budget * 4).manager.pools[1].num_pages == 4 * 17
    with pytest.raises(ValueError, match="does not hold one page"):
        CacheStorage(rt, model, page, None, 4, 64, kv_bytes=whole_page - 1, max_portion=8)
    with pytest.raises(ValueError, match="not both"):
        CacheStorage(rt, model, page, 64, 4, 64, kv_bytes=budget)
    # the same pool given in tokens: every group holds that many
    assert [p.num_pages for p in CacheStorage(rt, model, page, 40, 4, 64).manager.pools] == [10, 10]


def test_what_a_page_holds_is_what_the_mixers_declare():
    """The storage allocates the tensors that a mixer's CacheNeed lists and nothing else: one latent vector per token
    in a dtype of its own, beside keys and values of another shape; layers whose needs are equal share a group."""
    import torch

    from vt_transformer_amd.cache.storage import CacheStorage
    from vt_transformer_amd.parts.base import CacheNeed, PageTensor, Runtime

    latent = CacheNeed((PageTensor("latent", (24,), 0, torch.float32),), page_multiple=1)
    needs = [_kv_need(2, 16), latent, _kv_need(2, 16), latent, None]
    st = CacheStorage(Runtime(torch.device("cpu"), torch.bfloat16), _fake_model(needs), 8, 64, 2, 64)
    assert st.n_groups == 2 and st.entry_group == [0, 1, 0, 1, None] and st.entry_index == [0, 0, 1, 1, None]
    assert set(st.pages[0]) == {"k", "v"} and set(st.pages[1]) == {"latent"}
    assert st.pages[1]["latent"].shape == (2, 8, 8, 24) and st.pages[1]["latent"].dtype == torch.float32
    assert st.pages[0]["k"].dtype == torch.bfloat16
    assert st.page_bytes == [2 * 2 * 8 * 2 * 2 * 16, 2 * 8 * 24 * 4]
    caches = st.layer_caches([torch.zeros(1, 8, dtype=torch.int32)] * 2)
    assert caches[4] is None and caches[3]["latent"].shape == (8, 8, 24) and caches[2]["v"].shape == (8, 2, 16, 8)
    # an entry that reads another's pages must lay them out alike
    import pytest
    from types import SimpleNamespace
    from vt_transformer_amd.config.base import ScheduleEntry
    m = _fake_model([_kv_need(2, 16), latent])
    m.schedule = [ScheduleEntry(0), ScheduleEntry(1, cache_from=0)]
    with pytest.raises(ValueError, match="pages differ"):
        CacheStorage(Runtime(torch.device("cpu"), torch.float32), m, 8, 64, 2, 64)


def test_pages_a_request_will_hold_on_its_way_through_a_window():
    m = manager(num_pages=64, page_size=4, windows=(0, 8), max_seq_len=256)
    rp = m.admit("a")
    # in one step of 40 tokens both groups need all ten pages; on the way there in portions of 8 the windowed group
    # never holds more than (8 + 8) / 4 + 1 = 5
    assert m.pages_needed(rp, 40) == [10, 10]
    assert m.pages_needed(rp, 40, portion=8) == [10, 5]
    assert m.reserve([("a", 8)])
    m.commit("a", 8)
    assert m.pages_needed(rp, 40, portion=8) == [8, 3]        # it holds two of the five already
    for n in range(16, 41, 8):
        assert m.reserve([("a", n)])
        m.commit("a", n)
        assert sum(1 for p in rp.tables[1] if p >= 0) <= 5
    m.check()
