"""The step's arrays: the worked example of the reference's input layout."""

import pytest

from tokasaurus_amd.engine.batch import PlannedEntry, layout


def test_worked_example_page_size_4():
    # request A: 10-token prompt, 4 already in the cache, 6 more now, table [5, 2, 9];
    # request B: decoding at position 7, table [7, 1]  (input_building.py:176-297)
    a = PlannedEntry("A", [11, 12, 13, 14, 15, 16], [5], slot=0, start=4, tables=[[5, 2, 9]])
    b = PlannedEntry("B", None, [0], slot=3, start=7, tables=[[7, 1]])
    hb = layout([a, b], vocab_size=100, num_groups=1)
    assert hb.positions == [4, 5, 6, 7, 8, 9, 7]
    assert hb.token_ids == [11, 12, 13, 14, 15, 16, -4]  # B's token comes from slot 3
    assert hb.token_req == [0] * 6 + [1]
    assert hb.q_start == [0, 6, 7] and hb.kv_len == [10, 8] and hb.slots == [0, 3]
    assert hb.block_tables == [[[5, 2, 9], [7, 1, -1]]]
    assert hb.want_rows == [5, 6] and hb.num_portions == 1
    # cache rows these tokens are written to: table[pos // 4] * 4 + pos % 4 (input_building.py:138-148)
    idx = [hb.block_tables[0][r][p // 4] * 4 + p % 4 for r, p in zip(hb.token_req, hb.positions)]
    assert idx == [8, 9, 10, 11, 36, 37, 7]


def test_portions_come_first_but_wanted_rows_keep_the_callers_order():
    dec = PlannedEntry("d", [9], [0], slot=1, start=20, tables=[[4, 5, 6]])
    pre = PlannedEntry("p", [1, 2, 3], [0, 2], slot=0, start=0, tables=[[0]])
    hb = layout([dec, pre], 100, 1)
    assert hb.order == [1, 0] and hb.token_ids == [1, 2, 3, 9]
    assert hb.want_rows == [3, 0, 2]  # d's row first, as the caller listed it


def test_bad_entries_are_refused():
    ok = PlannedEntry("a", [1], [0], 0, 0, [[0]])
    with pytest.raises(ValueError, match="vocabulary"):
        layout([PlannedEntry("a", [100], [0], 0, 0, [[0]])], 100, 1)
    with pytest.raises(ValueError, match="wanted place"):
        layout([PlannedEntry("a", [1, 2], [2], 0, 0, [[0]])], 100, 1)
    with pytest.raises(ValueError, match="twice"):
        layout([ok, ok], 100, 1)
    with pytest.raises(ValueError, match="no tokens"):
        layout([PlannedEntry("a", [], [], 0, 0, [[0]])], 100, 1)
