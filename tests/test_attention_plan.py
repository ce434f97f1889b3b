"""The attention kernels' work lists of a step (``ops.plan_attention``): made on the host from the
batch's layout alone, so checked here without a GPU."""
import numpy as np

from lucciola_amd.engine.batch import HostLayout
from lucciola_amd.kernels import ops


def layout(new, cached, single=False):
    q_start = [0]
    for n in new:
        q_start.append(q_start[-1] + n)
    return HostLayout(len(new), q_start[-1], q_start, list(cached), 16, single)


def test_decode_rows_name_token_request_and_position():
    # requests 0 and 3 bring portions of a prompt, 1, 2 and 4 one token each after histories of
    # different length
    new, cached = [5, 1, 1, 130, 1], [0, 40, 7, 64, 300]
    arrays, info = ops.plan_attention(layout(new, cached))
    rows = arrays["decode_rows"]
    assert rows.dtype == np.int32 and rows.shape == (3, 4)
    assert info["num_decode"] == 3 and not info["all_decode"]
    # longest request first: 4 (301 tokens after the step), 1 (41), 2 (8)
    assert rows[:, :3].tolist() == [[137, 4, 300], [5, 1, 40], [6, 2, 7]]
    # the tiles of the two portions: request, first token row, rows, first position; most keys first
    tiles = arrays["prefill_tiles"].tolist()
    assert sorted(tiles) == sorted([[0, 0, 5, 0], [3, 7, 64, 64], [3, 71, 64, 128], [3, 135, 2, 192]])
    seen = [t[3] + t[2] for t in tiles]
    assert seen == sorted(seen, reverse=True)


def test_a_step_of_single_tokens_is_planned_the_same_either_way():
    cached = [12, 700, 3, 3, 64]
    fast, info_fast = ops.plan_attention(layout([1] * 5, cached, single=True))
    slow, info_slow = ops.plan_attention(layout([1] * 5, cached, single=False))
    assert np.array_equal(fast["decode_rows"], slow["decode_rows"])
    assert np.array_equal(fast["decode_items"], slow["decode_items"])
    assert fast["prefill_tiles"].shape == slow["prefill_tiles"].shape == (0, 4)
    assert info_fast == info_slow and info_fast["all_decode"] and info_fast["num_decode"] == 5
    # equal lengths keep their order (the sort is stable)
    assert fast["decode_rows"][:, 1].tolist() == [1, 4, 0, 2, 3]


def test_even_lengths_hint():
    # the longest within a tenth of the mean: even; one long request among short ones: not
    assert ops.plan_attention(layout([1] * 4, [1000, 1010, 990, 1023], single=True))[1]["even_lengths"]
    assert not ops.plan_attention(layout([1] * 4, [100, 100, 100, 2000], single=True))[1]["even_lengths"]
    assert ops.plan_attention(layout([1], [5], single=True))[1]["even_lengths"]
    # no decoding request at all
    arrays, info = ops.plan_attention(layout([3, 70], [0, 10]))
    assert arrays["decode_rows"].shape == (0, 4) and info["num_decode"] == 0 and not info["even_lengths"]


def check_items(new, cached, single=False):
    """What the decode kernel relies on: a row's items are neighbours, their page ranges follow
    one another from page 0 to the row's last page, every item names its row's token, request
    and position and its number of items, spare items have none, and the list's size follows
    from the number of rows alone."""
    arrays, info = ops.plan_attention(layout(new, cached, single))
    rows, items = arrays["decode_rows"], arrays["decode_items"]
    assert items.dtype == np.int32 and items.shape == (ops.decode_item_count(len(rows)), 8)
    used = 0
    for r, (t, req, p, packed) in enumerate(rows.tolist()):
        first, count = packed & 0xFFFFF, packed >> 20
        assert first == used and 1 <= count <= ops.ITEM_SHARES_MOST
        pages = p // 16 + 1
        at = 0
        for item in items[first:first + count].tolist():
            assert item[:4] == [t, req, p, r] and item[6] == count and item[7] == 0
            assert item[4] == at and item[5] > item[4]
            at = item[5]
        assert at == pages
        if count > 1:       # no item smaller than the least size, and sizes that differ by a page at most
            sizes = [i[5] - i[4] for i in items[first:first + count].tolist()]
            assert min(sizes) >= ops.ITEM_PAGES_MIN and max(sizes) - min(sizes) <= 1
        used += count
    assert not items[used:].any()
    assert info["decode_longest"] == (max(c + 1 for n, c in zip(new, cached) if n == 1) if len(rows) else 0)
    assert info["decode_total"] == sum(c + 1 for n, c in zip(new, cached) if n == 1)
    return rows, items


def test_decode_items_cover_every_row_once():
    import random
    rng = random.Random(11)
    check_items([1], [0], single=True)
    check_items([1] * 3, [8191, 15, 16], single=True)
    check_items([4, 1, 1, 70, 1], [0, 40, 7000, 64, 300])
    for _ in range(30):
        n = rng.randint(1, 70)
        check_items([1] * n, [rng.choice([0, 5, 127, 128, 500, 2000, 9000]) for _ in range(n)], single=True)
    # one long request among short ones gets the spare items, and its largest item is small
    rows, items = check_items([1] * 64, [8191] + [511] * 63, single=True)
    assert rows[0, 0] == 0 and rows[0, 3] >> 20 >= 16
    assert max(i[5] - i[4] for i in items.tolist()) <= 32
    # lengths so even that no launcher takes the list: every row its one item, the spare ones unused
    rows, items = check_items([1] * 8, [1023] * 8, single=True)
    assert (rows[:, 3] >> 20).tolist() == [1] * 8
    # few requests of uneven lengths: the spare items go where the pages are
    rows, items = check_items([1] * 4, [3999, 299, 199, 99], single=True)
    assert (rows[:, 3] >> 20).tolist() == [28, 2, 1, 1]       # 32 items for four rows
