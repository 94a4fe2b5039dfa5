"""The flat batch of a step on the host side: what is packed, and the in-place update of a
repeated decode step."""

import pytest
import torch

from atomserve_amd.cache.manager import RELEASED
from atomserve_amd.engine.batch import Row, StepBatch

BS = 4
ATTENTION = (8, 64)  # rows of up to 8 tokens as single queries, longer ones in tiles of 64


def pack(rows, **layout):
    return StepBatch(rows, BS, 2, 100, "cpu", **{"row_splits": [ATTENTION], **layout})


def decode_rows(tables, starts, tokens, filler):
    rows = [Row([t], s, tb, [0], -1) for tb, s, t in zip(tables, starts, tokens)]
    return rows + [Row([0], 0, filler, [0], -1, store=False)]


def test_rows_are_flattened_with_slots_tables_and_tiles():
    t0, t1 = [[5, 2], [7, 1]], [[3], [4]]
    b = pack([Row([11, 12, 13], 4, t0, [2]), Row([21], 2, t1, [0])])
    assert b.token_ids.tolist() == [11, 12, 13, 21] and b.positions.tolist() == [4, 5, 6, 2]
    assert b.tok_row.tolist() == [0, 0, 0, 1] and b.logits_rows.tolist() == [2, 3]
    assert b.group_slots[0].tolist() == [2 * BS + 0, 2 * BS + 1, 2 * BS + 2, 3 * BS + 2]
    assert b.group_slots[1].tolist() == [1 * BS + 0, 1 * BS + 1, 1 * BS + 2, 4 * BS + 2]
    assert b.group_tables[0].tolist() == [[5, 2], [3, 0]]
    assert b.split(ATTENTION).short_tokens.tolist() == [2, 1, 0, 3] and b.split(ATTENTION).num_long_tiles == 0  # those that see most keys first
    long = pack([Row(list(range(70)), 0, [list(range(20)), list(range(20))], []), Row([1] * 9, 64, [list(range(20, 40))] * 2, [])])
    # work items of the prefill kernel, the one that sees most keys first
    assert long.split(ATTENTION).long_tiles.tolist() == [[70, 9, 1, 64], [64, 6, 0, 64], [0, 64, 0, 0]]
    assert long.split(ATTENTION).tile_keys == 73 + 70 + 64  # the keys that each tile's last token sees, added up
    # a prompt's slots are computed as arrays: the same places as token by token, from the middle of a page on
    table = [(7 * i + 3) % 31 for i in range(30)]  # 30 different pages, in no order
    start = BS + 3
    prompt = pack([Row(list(range(100)), start, [table, table[::-1]], [99])])
    for g, tb in enumerate((table, table[::-1])):
        assert prompt.group_slots[g].tolist() == [tb[p // BS] * BS + p % BS for p in range(start, start + 100)]
    with pytest.raises(ValueError, match="outside the vocabulary"):
        pack([Row([1] * 80 + [-1], 0, [table, table], [])])


def test_a_repeated_decode_step_is_updated_in_place():
    """Same requests, one position further: `advance` leaves exactly what packing anew gives, also
    when a request has just received a new page; anything else is refused untouched."""
    filler = [[0], [0]]
    tables = [[[5, 2], [7, 1]], [[3], [4]]]  # request 0 at position 6, request 1 at position 3 (last slot of its page)
    layout = dict(table_width=3, max_context=12)
    first = pack(decode_rows(tables, [6, 3], [11, 21], filler), **layout)
    batch = pack(decode_rows(tables, [6, 3], [11, 21], filler), into=first, **layout)
    tables[1][0].append(8)  # request 1 crosses into a new page
    tables[1][1].append(9)
    rows = decode_rows(tables, [7, 4], [12, 22], filler)
    assert batch.advance(rows)
    fresh = pack(decode_rows(tables, [7, 4], [12, 22], filler), **layout)
    assert torch.equal(first.device_buffer, fresh.device_buffer)  # `first` owns the buffer both wrote to
    assert batch.host_rows is rows and batch.shared == {}
    before = first.device_buffer.clone()
    for bad in (
        decode_rows(tables, [9, 5], [1, 2], filler),                      # a position was skipped
        decode_rows([tables[1], tables[0]], [8, 5], [1, 2], filler),      # other requests in these rows
        decode_rows([[list(t) for t in tables[0]], tables[1]], [8, 5], [1, 2], filler),  # equal tables, another object
        decode_rows(tables, [8, 5], [1, 2], [[0], [0]]),                  # not the filler it was packed with
        decode_rows(tables, [8, 5], [1, 2], filler)[:2],                  # fewer rows
        [Row([1, 2], 8, tables[0], [0], -1), *decode_rows(tables, [8, 5], [1, 2], filler)[1:]],  # two tokens
        decode_rows(tables, [8, 5], [1, 200], filler),                    # a token outside the vocabulary
    ):
        assert not batch.advance(bad)
        assert torch.equal(first.device_buffer, before)
    tables[0][0].append(RELEASED)
    tables[0][1].append(6)
    assert not batch.advance(decode_rows(tables, [8, 5], [1, 2], filler))  # its page is not there
    tables[0][0][2] = 6
    assert batch.advance(decode_rows(tables, [8, 5], [1, 2], filler))
    assert not batch.advance(decode_rows(tables, [12, 6], [1, 2], filler))  # beyond the packed table width


def test_a_decode_step_lists_its_tokens_longest_context_first():
    """`all_tokens` of a step of single tokens is the order in which the attention kernel takes whole contexts:
    most keys first, equal ones as they come; a step with a prompt lists its tokens as they are."""
    filler = [[0], [0]]
    tables = [[[5, 2, 6], [7, 1, 3]]] * 4
    batch = pack(decode_rows(tables, [2, 9, 5, 9], [1, 2, 3, 4], filler), table_width=3, max_context=12)
    assert batch.decode_only and batch.all_tokens.tolist() == [1, 3, 2, 0, 4]
    mixed = pack([Row([1, 2, 3], 0, tables[0], [2]), Row([4], 9, tables[1], [0])])
    assert not mixed.decode_only and mixed.all_tokens.tolist() == [0, 1, 2, 3]


def test_rows_are_sorted_only_for_mixers_that_ask():
    """Short rows and tiles are what the attention kernels of this package want; a model whose
    mixers ask for nothing gets its rows as they come, another split gives other lists, and mixers
    that ask for different splits each find theirs in the same step."""
    rows = [Row([1, 2, 3], 0, [[2], [1]], [2]), Row(list(range(10)), 0, [[3, 0, 6], [4, 5, 7]], [9])]
    plain = StepBatch(rows, BS, 2, 100, "cpu")
    assert plain.splits == {} and plain.row_first.tolist() == [0, 3] and plain.row_len.tolist() == [3, 10]
    with pytest.raises(ValueError, match="sorted for"):
        plain.split(ATTENTION)
    both = StepBatch(rows, BS, 2, 100, "cpu", row_splits=[(2, 4), ATTENTION, (3, 8)])
    fine = both.split((2, 4))
    assert fine.num_short_tokens == 0 and fine.max_short_context == 0
    assert sorted(fine.long_tiles.tolist()) == [[0, 3, 0, 0], [3, 4, 1, 0], [7, 4, 1, 4], [11, 2, 1, 8]]
    coarse = both.split(ATTENTION)
    assert coarse.short_tokens.tolist() == [2, 1, 0] and coarse.long_tiles.tolist() == [[3, 10, 1, 0]] and coarse.max_short_context == 3
    third = both.split((3, 8))
    assert third.short_tokens.tolist() == [2, 1, 0] and sorted(third.long_tiles.tolist()) == [[3, 8, 1, 0], [11, 2, 1, 8]]
    alone = StepBatch(rows, BS, 2, 100, "cpu", row_splits=[(3, 8)]).split((3, 8))
    assert alone.long_tiles.tolist() == third.long_tiles.tolist()  # a split does not depend on its neighbours
    with pytest.raises(ValueError):
        StepBatch(rows, BS, 2, 100, "cpu", row_splits=[(2, 0)])
    # a split without single queries lists positions per tile: such a decode step is packed anew, not moved on
    tables = [[[5, 2], [7, 1]], [[3], [4]]]
    tiled = StepBatch([Row([1], 6, tables[0], [0]), Row([2], 2, tables[1], [0])], BS, 2, 100, "cpu", row_splits=[(0, 4)])
    assert tiled.split((0, 4)).num_long_tiles == 2
    assert not tiled.advance([Row([3], 7, tables[0], [0]), Row([4], 3, tables[1], [0])])


def test_pages_given_back_by_a_window_leave_the_captured_table():
    """A request of a windowed group decodes on; the pages its window passes are given back between
    steps.  The step updated in place holds 0 where packing anew holds 0, not the page's old id
    (which by then may belong to somebody else)."""
    filler = [[0]]
    table = [[5, 2, 7]]
    first = StepBatch([Row([1], 9, table, [0], -1), Row([0], 0, filler, [0], -1, store=False)], BS, 1, 100, "cpu",
                      table_width=4, max_context=16)  # fmt: skip
    table[0][0] = RELEASED
    table[0][1] = RELEASED
    rows = [Row([2], 10, table, [0], -1), Row([0], 0, filler, [0], -1, store=False)]
    assert first.advance(rows)
    fresh = StepBatch(rows, BS, 1, 100, "cpu", table_width=4, max_context=16)
    assert torch.equal(first.device_buffer, fresh.device_buffer)
    assert first.group_tables[0].tolist() == [[0, 0, 7, 0], [0, 0, 0, 0]]
