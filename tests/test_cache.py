"""The cache manager's bookkeeping: no page lost, held twice or freed twice, under random orders."""
import numpy as np
import pytest
import torch

from transformers_neuronx_amd.cache import CacheManager, OutOfPages, OutOfSlots, PagePool, SlotPool
from transformers_neuronx_amd.parts.base import CacheNeed


def test_page_pool_basics():
    pool = PagePool(5)
    a = pool.allocate(3, "a")
    assert len(set(a)) == 3 and pool.num_free == 2
    with pytest.raises(OutOfPages):
        pool.allocate(3, "b")
    assert pool.num_free == 2                       # all or none
    b = pool.allocate(2, "b")
    assert not set(a) & set(b)
    with pytest.raises(ValueError, match="held by"):
        pool.free(a, "b")
    pool.free(a, "a")
    with pytest.raises(ValueError, match="twice"):
        pool.free(a[:1], "a")
    # LIFO: what was just given back is handed out next
    assert pool.allocate(1, "c")[0] == a[-1]
    pool.check()
    with pytest.raises(ValueError):
        PagePool(0)


def test_slot_pool():
    s = SlotPool(2)
    x, y = s.allocate("x"), s.allocate("y")
    assert x != y
    with pytest.raises(OutOfSlots):
        s.allocate("z")
    with pytest.raises(ValueError):
        s.free(x, "y")
    s.free(x, "x")
    assert s.allocate("z") == x


def _manager(num_pages=12, page=16, window=None, max_seqs=4):
    needs = {0: CacheNeed("paged", kv_heads=2, head_size=16), 1: CacheNeed("paged", kv_heads=2, head_size=16)}
    if window:
        needs[2] = CacheNeed("paged", kv_heads=1, head_size=16, window=window)
    return CacheManager(needs, page, num_pages, max_seqs, torch.float32, "cpu", allocate=False)


def test_groups_and_tables():
    m = _manager(window=40)
    assert set(m.groups) == {"full", "window40"}
    assert m.groups["full"].cache_ids == [0, 1] and m.groups["window40"].cache_ids == [2]
    m.add_request("a")
    m.grow("a", 33)
    assert len(m.requests["a"].tables["full"]) == 3 and len(m.requests["a"].tables["window40"]) == 3
    m.advance("a", 33)
    t = m.block_table(["a"], "full")
    assert t.shape == (1, 3) and t.dtype == np.int32 and (t >= 0).all()
    m.grow("a", 33)                                  # nothing more needed
    assert len(m.requests["a"].tables["full"]) == 3
    with pytest.raises(ValueError, match="already live"):
        m.add_request("a")
    m.free_request("a")
    m.check()
    assert m.groups["full"].pool.num_free == 12


def test_window_gives_pages_back():
    m = _manager(num_pages=8, window=40)
    m.add_request("a")
    n = 0
    for step in (16, 16, 16, 16, 16, 16, 16, 7):
        m.grow("a", n + step)
        m.advance("a", n + step - n)
        n += step
        win = m.requests["a"].tables["window40"]
        first_needed = n - 40 + 1
        for i, p in enumerate(win):
            # a page is given back exactly when every position in it is before the window of later queries
            assert (p < 0) == ((i + 1) * 16 <= first_needed), (n, i, p)
        assert all(p >= 0 for p in m.requests["a"].tables["full"])
        m.check()
    held = sum(p >= 0 for p in m.requests["a"].tables["window40"])
    assert held <= 40 // 16 + 2
    m.free_request("a")
    m.check()


def test_grow_is_all_or_nothing_across_groups():
    m = CacheManager({0: CacheNeed("paged", kv_heads=1, head_size=16),
                      1: CacheNeed("paged", kv_heads=1, head_size=16, window=1000)},
                     16, {"full": 4, "window1000": 2}, 4, torch.float32, "cpu", allocate=False)
    m.add_request("a")
    with pytest.raises(OutOfPages):
        m.grow("a", 48)                              # the window group has 2 pages only
    assert m.groups["full"].pool.num_free == 4 and m.groups["window1000"].pool.num_free == 2
    assert not m.can_grow("a", 48) and m.can_grow("a", 32)


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_nothing(seed):
    rng = np.random.default_rng(seed)
    m = _manager(num_pages=20, page=16, window=48, max_seqs=5)
    live = {}
    for _ in range(400):
        op = rng.integers(0, 4)
        if op == 0 and len(live) < 5:
            rid = f"r{rng.integers(0, 10**9)}"
            m.add_request(rid)
            live[rid] = 0
        elif op in (1, 2) and live:
            rid = list(live)[rng.integers(0, len(live))]
            n = int(rng.integers(1, 50))
            try:
                m.grow(rid, live[rid] + n)
            except OutOfPages:
                before = {g: grp.pool.num_free for g, grp in m.groups.items()}
                m.check()
                assert before == {g: grp.pool.num_free for g, grp in m.groups.items()}
                continue
            m.advance(rid, n)
            live[rid] += n
            assert m.num_tokens(rid) == live[rid]
        elif op == 3 and live:
            rid = list(live)[rng.integers(0, len(live))]
            m.free_request(rid)
            del live[rid]
            with pytest.raises(KeyError):
                m.free_request(rid)
        m.check()
    m.reset()
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups.values()) and m.slots.num_free == 5


def test_state_slots_are_cleared_on_allocation():
    needs = {0: CacheNeed("state", state_shapes=(("s", (3,)),))}
    m = CacheManager(needs, 16, 4, 2, torch.float32, "cpu")
    slot = m.add_request("a")
    m.caches[0].state["s"][slot] = 7.0
    m.free_request("a")
    assert m.add_request("b") == slot
    assert float(m.caches[0].state["s"][slot].abs().sum()) == 0.0


def test_storage_shapes():
    needs = {0: CacheNeed("paged", kv_heads=3, head_size=32)}
    m = CacheManager(needs, 16, 5, 2, torch.bfloat16, "cpu")
    assert m.caches[0].k_pages.shape == (5, 3, 16, 32) and m.caches[0].v_pages.shape == (5, 3, 32, 16)
    assert CacheManager.bytes_per_page(needs, 16, torch.bfloat16) == 2 * 3 * 32 * 16 * 2
