"""The cache manager: no page lost, held twice or freed twice, under random orders of requests (CPU)."""
import random

import pytest

from infinicore_infer_amd.cache import (CacheError, CacheManager, GroupSpec, OutOfPages, PagePool,
                                        PositionOverflow)

FULL = GroupSpec("full", 2, 16, None, (0, 1))
WIN = GroupSpec("window", 2, 16, 40, (2,))


def test_pool_basics_and_double_free():
    p = PagePool(3)
    a, b, c = p.alloc(), p.alloc(), p.alloc()
    assert sorted([a, b, c]) == [0, 1, 2] and p.n_free == 0
    with pytest.raises(OutOfPages):
        p.alloc()
    p.free(b)
    assert p.alloc() == b                      # last freed, first reused
    p.free(a)
    with pytest.raises(CacheError):
        p.free(a)
    with pytest.raises(CacheError):
        p.free(7)


def test_append_block_tables_and_slots():
    m = CacheManager([FULL], 8, 16, max_requests=2, max_positions=100)
    m.admit("a")
    assert m.append("a", 17) == 0
    assert len(m.block_table("a", 0)) == 2 and m.length("a") == 17
    assert m.append("a", 15) == 17 and len(m.block_table("a", 0)) == 2
    assert m.append("a", 1) == 32 and len(m.block_table("a", 0)) == 3
    t = m.block_table("a", 0)
    assert m.slot_of("a", 0, 16) == t[1] * 16 and m.slot_of("a", 0, 32) == t[2] * 16
    with pytest.raises(PositionOverflow):
        m.append("a", 100)
    m.admit("b")
    with pytest.raises(OutOfPages):
        m.admit("c")
    with pytest.raises(OutOfPages):
        m.append("b", 16 * 6)                    # 5 pages left
    assert m.length("b") == 0 and m.free_pages() == 5
    assert not m.can_append("b", 16 * 5, reserve=[1]) and m.can_append("b", 16 * 5)
    m.release("a")
    m.release("b")
    assert m.free_pages() == 8 and m.slots.n_free == 2
    m.check_invariants()


def test_window_group_gives_pages_back_early():
    m = CacheManager([FULL, WIN], [16, 16], 16, max_requests=2)
    m.admit("a")
    m.append("a", 100)
    assert m.trim("a") == 3                      # next query 100 reads keys >= 61: pages 0..2 are dead
    assert m.block_table("a", 1)[:4] == [-1, -1, -1, m.block_table("a", 1)[3]]
    assert m.free_pages(1) == 16 - 7 + 3 and m.free_pages(0) == 16 - 7
    with pytest.raises(CacheError):
        m.slot_of("a", 1, 5)
    m.append("a", 28)
    assert m.trim("a") == 2                      # next query 128 reads keys >= 89: pages 3, 4 go too
    assert m.trim("a") == 0
    m.check_invariants()
    m.release("a")
    assert m.free_pages(0) == 16 and m.free_pages(1) == 16
    m.check_invariants()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_conserve_pages(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN], [24, 24], 16, max_requests=5, max_positions=400)
    live, n = [], 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.can_admit():
            n += 1
            m.admit(n)
            live.append(n)
        elif op < 0.8 and live:
            r = rng.choice(live)
            k = rng.choice([1, 1, 1, 2, 7, 16, 33])
            before = (m.length(r), m.free_pages(0), m.free_pages(1), [list(t) for t in m.requests[r].tables])
            try:
                m.append(r, k)
            except (OutOfPages, PositionOverflow):       # a refused append changes nothing
                assert before == (m.length(r), m.free_pages(0), m.free_pages(1),
                                  [list(t) for t in m.requests[r].tables])
            else:
                if rng.random() < 0.15:                  # a step that failed after its appends is undone
                    m.truncate(r, before[0])
                    assert before == (m.length(r), m.free_pages(0), m.free_pages(1),
                                      [list(t) for t in m.requests[r].tables])
                else:
                    m.trim(r)
        elif op < 0.86 and live and m.can_admit():          # a copy of a request's first tokens in pages of its own
            r = rng.choice(live)
            n += 1
            try:
                _, pairs = m.fork(r, n, rng.randint(0, m.length(r)))
                live.append(n)
                assert len({(g, d) for g, _, d in pairs}) == len(pairs)
            except OutOfPages:
                assert not m.has_request(n)
        elif op < 0.9 and live:                              # a request's cache under a new name, cut back
            r = live.pop(rng.randrange(len(live)))
            n += 1
            if any(g.kind == "window" for g in m.groups):
                m.rename(r, n)
            else:
                m.rename(r, n)
                m.truncate(n, rng.randint(0, m.length(n)))
            live.append(n)
        elif live:
            r = live.pop(rng.randrange(len(live)))
            m.release(r)
            with pytest.raises(KeyError):
                m.release(r)
        m.check_invariants()
    for r in live:
        m.release(r)
    m.check_invariants()
    assert m.free_pages(0) == 24 and m.free_pages(1) == 24 and m.slots.n_free == 5


def test_truncate_gives_back_exactly_what_the_appends_took():
    m = CacheManager([FULL], [8], 16, max_requests=2, max_positions=200)
    m.admit("a")
    m.append("a", 20)
    table = list(m.block_table("a", 0))
    m.append("a", 30)
    m.append("a", 1)
    assert m.free_pages(0) == 8 - 4
    m.truncate("a", 20)
    assert m.length("a") == 20 and m.block_table("a", 0) == table and m.free_pages(0) == 6
    m.check_invariants()
    m.truncate("a", 0)
    assert m.block_table("a", 0) == [] and m.free_pages(0) == 8
    with pytest.raises(Exception):
        m.truncate("a", 5)                      # it cannot grow a request
    m.check_invariants()


def test_fork_copies_the_first_tokens_into_pages_of_its_own():
    m = CacheManager([FULL, WIN], [16, 16], 16, max_requests=3, max_positions=400)
    m.admit("a")
    m.append("a", 100)
    m.trim("a")                                   # the window group gave its first pages back
    slot, pairs = m.fork("a", "b", 70)
    assert m.length("b") == 70 and slot == m.state_slot("b") != m.state_slot("a")
    full = [(s, d) for g, s, d in pairs if g == 0]
    assert [s for s, _ in full] == m.block_table("a", 0)[:5] and [d for _, d in full] == m.block_table("b", 0)
    assert not set(m.block_table("b", 0)) & set(m.block_table("a", 0))
    win_b = m.block_table("b", 1)
    assert len(win_b) == 5 and [p < 0 for p in win_b] == [p < 0 for p in m.block_table("a", 1)[:5]]
    m.check_invariants()
    with pytest.raises(Exception):
        m.fork("a", "c", 101)                      # more than the source holds
    with pytest.raises(OutOfPages):
        m.fork("a", "c", 100) or m.fork("a", "d", 100)      # the second one finds no state slot
    m.release("a")
    m.append("b", 20)                              # the copy goes on by itself
    m.check_invariants()


def test_a_cache_need_names_planes_pages_and_state_together():
    """A mixer may ask for paged memory of any number of planes, for a fixed-size state, or for both."""
    import torch
    from infinicore_infer_amd.cache import CacheStorage
    from infinicore_infer_amd.parts import CacheNeed
    kv = CacheNeed("kv", 2, 16)
    assert kv.paged and not kv.has_state and kv.planes == 2
    latent = CacheNeed("kv+state", n_kv_heads=1, head_dim=24, planes=1, state_shape=(5,))
    assert latent.paged and latent.has_state
    assert CacheNeed("state", state_shape=(3, 2)).has_state and not CacheNeed("state", state_shape=(3,)).paged
    assert not CacheNeed().paged and not CacheNeed().has_state
    for bad in (dict(kind="pages"), dict(kind="kv", n_kv_heads=0, head_dim=8), dict(kind="kv", n_kv_heads=1, head_dim=8, planes=0),
                dict(kind="state"), dict(kind="kv+state", n_kv_heads=1, head_dim=8)):
        with pytest.raises(ValueError):
            CacheNeed(**bad)
    with pytest.raises(CacheError):
        GroupSpec("full", 1, 8, planes=0)
    groups = [GroupSpec("full", 1, 24, None, (0, 2), planes=1), GroupSpec("full", 2, 16, None, (1,))]
    st = CacheStorage(groups, [3, 3], 4, torch.float32, "cpu")
    assert tuple(st.group_planes[0].shape) == (2, 1, 3, 1, 4, 24) and tuple(st.group_planes[1].shape) == (1, 2, 3, 2, 4, 16)
    assert len(st.planes(2)) == 1 and len(st.planes(1)) == 2 and len(st.kv(1)) == 2
    assert st.planes(2)[0].data_ptr() == st.group_planes[0][1, 0].data_ptr()
    with pytest.raises(ValueError):
        st.kv(0)
