"""The cache manager on its own: no page is lost, held twice or freed twice, under random orders of requests."""
import random

import pytest
import torch

from tiny_inference_server_amd.cache import CacheError, CacheManager, OutOfPages, PagePool
from tiny_inference_server_amd.parts.spec import PagedKvNeed, StateNeed


def manager(n_pages=12, page_size=4, max_requests=5, window=0, allocate=False):
    needs = {"trunk.0": PagedKvNeed(2, 8, 0), "trunk.1": PagedKvNeed(2, 8, 0), "mtp0.0": PagedKvNeed(2, 8, 0),
             "mtp0.input": StateNeed((16,), "compute")}
    if window:
        needs["local.0"] = PagedKvNeed(2, 8, window)
    return CacheManager(needs, page_size, n_pages, max_requests, torch.float32, "cpu", allocate=allocate)


def test_pool_fifo_and_double_free():
    p = PagePool(3)
    a, b = p.take(), p.take()
    assert (a, b) == (0, 1) and p.n_free == 1
    p.give_back(a)
    assert p.take() == 2 and p.take() == 0          # first in, first out: a page comes back after the untouched ones
    with pytest.raises(OutOfPages):
        p.take()
    p.give_back(1)
    with pytest.raises(CacheError, match="twice"):
        p.give_back(1)
    with pytest.raises(CacheError, match="outside"):
        p.give_back(7)
    p.check()


def test_groups_planes_and_states():
    m = manager(allocate=True, window=6)
    assert set(m.groups) == {"kv2x8", "kv2x8w6"}
    g = m.groups["kv2x8"]
    assert g.spec.keys == ["trunk.0", "trunk.1", "mtp0.0"] and g.storage.shape == (3, 12, 2, 2, 4, 8)
    assert g.plane("mtp0.0").data_ptr() == g.storage[2].data_ptr()
    assert m.groups["kv2x8w6"].storage.shape[0] == 1
    assert m.states["mtp0.input"].shape == (5, 16)
    s = m.open_request()
    m.states["mtp0.input"][s] = 3.0
    m.close_request(s)
    for _ in range(5):                   # the slot comes round again and is zeroed when it is taken
        t = m.open_request()
    assert t == s and float(m.states["mtp0.input"][s].abs().sum()) == 0.0


def test_grow_is_all_or_nothing():
    m = manager(n_pages=4, page_size=4)
    a, b = m.open_request(), m.open_request()
    m.grow(a, 9)                                      # 3 pages
    assert m.block_table("kv2x8", a) == [0, 1, 2] and m.free_pages() == {"kv2x8": 1}
    assert m.pages_needed(b, 5) == {"kv2x8": 2} and not m.can_grow({b: 5}) and m.can_grow({b: 4, a: 12})
    with pytest.raises(OutOfPages):
        m.grow(b, 5)
    assert m.block_table("kv2x8", b) == [] and m.free_pages() == {"kv2x8": 1}
    m.grow(a, 9)                                      # nothing to add
    m.close_request(a)
    m.grow(b, 16)
    assert m.block_table("kv2x8", b) == [3, 0, 1, 2]  # given-back pages are used again, in FIFO order
    with pytest.raises(CacheError, match="not live"):
        m.close_request(a)
    m.check()


def test_window_pages_are_given_back_as_the_window_passes():
    m = manager(n_pages=6, page_size=4, window=6)
    s = m.open_request()
    full, local = m.groups["kv2x8"], m.groups["kv2x8w6"]
    for n in range(1, 25):
        if not m.can_grow({s: n}):
            break
        m.grow(s, n)
        m.release_behind(s, n, max_lag=1)            # next row is n, the lagging stage's next row n-1
        # a row at position p reads keys (p-6, p]; the lowest future row is n-1, so keys from n-6 stay
        first_needed = n - 1 - 6 + 1
        held = [i for i, p in enumerate(local.tables[s]) if p >= 0]
        assert all((i + 1) * 4 > first_needed for i in held)
        assert all(p >= 0 for p in full.tables[s])
        m.check()
    assert local.held(s) <= 3 and full.held(s) == 6
    assert local.pool.n_free >= 3 and full.pool.n_free == 0
    m.close_request(s)
    assert m.free_pages() == m.total_pages()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    m = manager(n_pages=rng.choice([5, 9, 17]), page_size=rng.choice([2, 4, 16]), max_requests=4,
                window=rng.choice([0, 5]))
    live = {}
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and m.n_live < 4:
            live[m.open_request()] = 0
        elif op < 0.45 and live:
            s = rng.choice(list(live))
            m.close_request(s)
            del live[s]
        elif live:
            s = rng.choice(list(live))
            n = live[s] + rng.randint(1, 9)
            if m.can_grow({s: n}):
                m.grow(s, n)
                live[s] = n
                m.release_behind(s, n, max_lag=rng.randint(0, 2))
            else:
                with pytest.raises(OutOfPages):
                    m.grow(s, n)
        m.check()
        for name, g in m.groups.items():
            held = sum(g.held(s) for s in live)
            assert held + g.pool.n_free == g.pool.n_pages
            for s in live:                            # the array form of a table follows every change of the table
                assert g.line(s).tolist() == g.tables[s]
    for s in list(live):
        m.close_request(s)
    assert m.free_pages() == m.total_pages() and m.n_live == 0
    with pytest.raises(CacheError):
        m.close_request(0)


def test_slots_run_out_with_a_clear_error():
    m = manager(max_requests=2)
    m.open_request(), m.open_request()
    with pytest.raises(CacheError, match="all 2 request slots"):
        m.open_request()


def test_the_spare_request_lives_beside_what_was_asked_for():
    """A manager with a spare request: its slot, state line and pages come on top of the slots and pages asked for and
    are counted by nobody; it cannot be closed; everything else behaves as without it."""
    needs = {"a": PagedKvNeed(2, 8), "b": PagedKvNeed(2, 8, window=6), "s": StateNeed((4,), "float32")}
    m = CacheManager(needs, 4, 5, 2, torch.float32, "cpu", spare_positions=3)
    assert m.spare_slot == 2 and m.n_live == 0
    assert m.free_pages() == m.total_pages() == {"kv2x8": 5, "kv2x8w6": 5}
    assert m.states["s"].shape == (3, 4) and all(g.storage.shape[1] == 6 for g in m.groups.values())
    assert [len(g.tables[2]) for g in m.groups.values()] == [1, 1]
    a, b = m.open_request(), m.open_request()
    assert {a, b} == {0, 1}
    with pytest.raises(CacheError, match="all 2 request slots"):
        m.open_request()
    m.grow(a, 12), m.grow(b, 8)                       # all five pages of the full group
    assert m.free_pages()["kv2x8"] == 0 and not m.can_grow({b: 9})
    spare_pages = {name: list(g.tables[2]) for name, g in m.groups.items()}
    assert all(p not in g.tables[a] + g.tables[b] for name, g in m.groups.items() for p in spare_pages[name])
    with pytest.raises(CacheError, match="spare"):
        m.close_request(2)
    m.check()
    m.close_request(a), m.close_request(b)
    assert m.free_pages() == m.total_pages() and m.n_live == 0
    m.check()
