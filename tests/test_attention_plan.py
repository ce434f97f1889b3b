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
    assert rows.tolist() == [[137, 4, 300, 0], [5, 1, 40, 0], [6, 2, 7, 0]]
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
