"""The cache manager's bookkeeping: no page lost, held twice or freed twice, under random
orders of requests; groups with a window give back the pages the window has passed; slots."""
import random

import pytest

from lucciola_amd.cache.manager import CacheManager
from lucciola_amd.cache.page_pool import OutOfPages, PagePool, SlotPool
from lucciola_amd.cache.specs import FixedState, PagedKV

FULL = PagedKV(2, 16)
WINDOW = PagedKV(2, 16, window=10)


def test_pool_is_first_in_first_out():
    # src/block_manager.cc:26-40: allocate pops the front, free pushes to the back
    pool = PagePool(4, scatter=False)
    assert [pool.allocate() for _ in range(4)] == [0, 1, 2, 3]
    with pytest.raises(OutOfPages):
        pool.allocate()
    pool.free(2)
    pool.free(0)
    assert [pool.allocate(), pool.allocate()] == [2, 0]
    with pytest.raises(ValueError, match="not held"):
        pool.free(7)
    pool.free(1)
    with pytest.raises(ValueError, match="freed twice"):
        pool.free(1)
    pool.check()


def test_pool_scatters_its_first_round():
    """By default the first round of pages comes in a fixed shuffled order (a function of the
    pool's size), every page once; after that the pool is first in, first out as above."""
    first = [PagePool(64).allocate() for _ in range(1)]
    pool = PagePool(64)
    order = [pool.allocate() for _ in range(64)]
    assert sorted(order) == list(range(64)) and order != list(range(64)) and order[:1] == first
    again = PagePool(64)
    assert [again.allocate() for _ in range(64)] == order
    for page in (order[5], order[2], order[40]):
        pool.free(page)
    assert [pool.allocate() for _ in range(3)] == [order[5], order[2], order[40]]
    pool.check()


def test_slots():
    slots = SlotPool(3)
    a, b, c = slots.allocate(), slots.allocate(), slots.allocate()
    assert (a, b, c) == (0, 1, 2)
    with pytest.raises(OutOfPages):
        slots.allocate()
    slots.free(b)
    assert slots.allocate() == 1
    with pytest.raises(ValueError):
        slots.free(5)
    slots.check()


def test_groups_are_formed_by_equal_needs():
    cm = CacheManager([FULL, WINDOW, FULL, None, FixedState((3,)), WINDOW], 4, 20, 4)
    assert [g.sites for g in cm.groups] == [[0, 2], [1, 5]]
    assert cm.has_fixed_state and [i for i, n in enumerate(cm.site_needs) if n and not n[0].paged] == [4]
    assert cm.need_group == {(0, 0): 0, (2, 0): 0, (1, 0): 1, (5, 0): 1}


def test_pages_follow_the_length():
    cm = CacheManager([FULL], 4, 10, 2, scatter_pages=False)
    cm.admit("a")
    cm.reserve("a", 5)
    assert cm.block_table(0, "a") == [0, 1] and cm.length("a") == 0
    cm.commit("a")
    assert cm.length("a") == 5
    for expect in ([0, 1], [0, 1], [0, 1], [0, 1, 2]):     # lengths 6, 7, 8, 9
        cm.reserve("a", 1)
        cm.commit("a")
        assert cm.block_table(0, "a") == expect
    assert cm.slot_of_token(0, "a", 8) == 2 * 4 + 0
    cm.release("a")
    assert cm.groups[0].pool.num_free() == 10
    cm.check()


def test_reserve_takes_all_or_nothing():
    cm = CacheManager([FULL, WINDOW], 4, 3, 2)
    cm.admit("a")
    cm.reserve("a", 8)                      # two pages in each group
    cm.admit("b")
    assert not cm.can_reserve("b", 5)       # needs two, one is free
    with pytest.raises(OutOfPages):
        cm.reserve("b", 5)
    assert cm.block_table(0, "b") == [] and cm.block_table(1, "b") == []
    assert cm.can_reserve("b", 4) and not cm.can_reserve("b", 4, {0: 1})
    assert cm.can_reserve(None, 4) and not cm.can_reserve(None, 5)
    cm.check()


def test_window_gives_pages_back():
    cm = CacheManager([FULL, WINDOW], 4, 50, 2)      # window of 10 positions
    cm.admit("a")
    cm.reserve("a", 30)
    cm.commit("a")
    # the next query is at position 30 and reads keys 21..30: pages 0..4 (keys 0..19) are passed
    assert cm.block_table(1, "a")[:5] == [-1] * 5 and all(p >= 0 for p in cm.block_table(1, "a")[5:])
    assert all(p >= 0 for p in cm.block_table(0, "a"))
    assert cm.groups[1].pool.num_free() == 50 - 3 and cm.groups[0].pool.num_free() == 50 - 8
    with pytest.raises(RuntimeError, match="given back"):
        cm.slot_of_token(1, "a", 3)
    for _ in range(40):
        cm.reserve("a", 1)
        cm.commit("a")
        held = [p for p in cm.block_table(1, "a") if p >= 0]
        assert len(held) <= 4                    # ceil(10 / 4) + 1
        cm.check()
    cm.release("a")
    assert all(g.pool.num_free() == 50 for g in cm.groups)


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_of_requests(seed):
    rng = random.Random(seed)
    bs = rng.choice([1, 4, 16])
    cm = CacheManager([FULL, WINDOW, FixedState((2,))], bs, 40, 5)
    lengths = {}
    for step in range(600):
        action = rng.random()
        if action < 0.2 and cm.can_admit():
            name = f"r{step}"
            cm.admit(name)
            lengths[name] = 0
        elif action < 0.85 and lengths:
            name = rng.choice(list(lengths))
            n = rng.choice([1, 1, 1, 2, 7, 20])
            if cm.can_reserve(name, n):
                cm.reserve(name, n)
                if rng.random() < 0.9:
                    cm.commit(name)
                    lengths[name] += n
                else:               # a step that is given up before it ran
                    cm.release(name)
                    del lengths[name]
            else:
                with pytest.raises(OutOfPages):
                    cm.reserve(name, n)
        elif lengths:
            name = rng.choice(list(lengths))
            cm.release(name)
            del lengths[name]
        cm.check()
        used = sum(-(-n // bs) for n in lengths.values())
        assert cm.groups[0].pool.num_free() == 40 - used
        for name, n in lengths.items():
            assert cm.length(name) == n
            table = cm.block_table(1, name)
            first_needed = max(0, n - 10 + 1)
            for idx, page in enumerate(table):
                assert (page < 0) == ((idx + 1) * bs <= first_needed)
    for name in list(lengths):
        cm.release(name)
    cm.check()
    assert all(g.pool.num_free() == 40 for g in cm.groups) and cm.slots.num_free() == 5


def test_a_need_of_another_layout_and_two_needs_at_one_site():
    """The manager only counts: a need that is no key/value pair (one tensor of latents per
    site, with a kernel page of its own) makes its own memory, and a site may hold several
    needs (a layer with two caching parts)."""
    from dataclasses import dataclass
    import torch
    from lucciola_amd.cache.specs import CacheNeed

    @dataclass(frozen=True)
    class Latents(CacheNeed):
        rank: int
        window: int = None
        paged = True

        def kernel_page(self, page_size):
            return 4 if page_size % 4 == 0 else page_size

        def bytes_per_page(self, page_size, dtype):
            return page_size * self.rank * 4

        def allocate(self, layout, dtype, device):
            return torch.zeros((layout.kernel_pages, layout.kernel_page, self.rank), device=device)

    class Ring(CacheNeed):
        def bytes_per_request(self, dtype):
            return 40

        def allocate(self, layout, dtype, device):
            return {"ring": torch.ones((layout.max_seqs, 10)), "started": []}

        def start(self, storage, slot):
            storage["started"].append(slot)
            storage["ring"][slot] = 0

    ring = Ring()
    cm = CacheManager([Latents(6), (Latents(6), FULL, ring), None, Latents(6, window=8)], 8, 10, 3)
    assert [g.sites for g in cm.groups] == [[0, 1], [1], [3]]
    assert [(g.kernel_page, g.pieces) for g in cm.groups] == [(4, 2), (8, 1), (4, 2)]
    assert cm.need_group == {(0, 0): 0, (1, 0): 0, (1, 1): 1, (3, 0): 2} and cm.has_fixed_state
    assert cm.bytes_per_block(torch.float32) == 3 * 8 * 6 * 4 + 2 * 2 * 8 * 16 * 4
    assert cm.state_bytes() == 3 * 40
    cm.allocate_tensors(torch.float32, "cpu")
    assert sorted(cm.storage) == [0, 1, 3] and len(cm.storage[1]) == 3
    assert cm.storage[0][0].shape == (20, 4, 6) and cm.storage[1][1][0].shape == (10, 2, 8, 16)
    slot = cm.admit("a")
    cm.start_slots([slot])
    assert cm.storage[1][2]["started"] == [slot] and float(cm.storage[1][2]["ring"][slot].sum()) == 0
    cm.reserve("a", 20)
    cm.commit("a")
    assert [len(g.tables["a"]) for g in cm.groups] == [3, 3, 3]
    assert list(cm.groups[2].tables["a"])[0] == -1        # the window of 8 has passed the first page
    cm.check()
    cm.release("a")
    assert all(g.pool.num_free() == 10 for g in cm.groups)
    with pytest.raises(TypeError, match="not a cache need"):
        CacheManager([object()], 8, 10, 3)
