"""The attention part's planning of work items, on the CPU (no kernel runs)."""

import numpy as np

from clockwork_amd.parts.attention import MAX_PARTS, MIN_PART_KEYS, _share_long_key_ranges, portions_have_short_ranges


class _Step:
    def __init__(self, q_lens, ctx_lens, num_compute_units=256):
        self.h_q_lens, self.h_ctx_lens, self.num_compute_units = list(q_lens), list(ctx_lens), num_compute_units


def _items(q_lens, tokens_per_item):
    rows = []
    for r, q in enumerate(q_lens):
        for tok0 in range(0, q, tokens_per_item):
            rows.append((r, tok0, min(tokens_per_item, q - tok0), 0))
    return np.asarray(rows, dtype=np.int32).reshape(-1, 4)


def _unpack(flat):
    items = flat.reshape(-1, 4)
    return items, items[:, 3] & 255, (items[:, 3] >> 8) & 255


def test_a_launch_that_fills_the_card_is_left_alone():
    step = _Step([2048], [2048])
    items = _items(step.h_q_lens, 10)  # 205 items on 2 key/value heads: 410 workgroups
    flat, most = _share_long_key_ranges(items, step, workgroups_per_item=2)
    assert most == 1 and (flat.reshape(-1, 4) == items).all()


def test_a_short_portion_behind_a_long_prefix_is_cut_into_parts():
    step = _Step([200], [8392])
    items = _items(step.h_q_lens, 20)  # 10 items on 2 heads: 20 workgroups for 256 compute units
    flat, most = _share_long_key_ranges(items, step, workgroups_per_item=2)
    out, part, parts = _unpack(flat)
    assert most == 12 and len(out) == 120 and (parts == 12).all()
    for i in range(10):  # the parts of an item follow one another and keep its first three fields
        block = out[12 * i : 12 * i + 12]
        assert (block[:, :3] == items[i, :3]).all() and list(part[12 * i : 12 * i + 12]) == list(range(12))


def test_parts_are_bounded_by_the_keys_and_by_the_list_format():
    step = _Step([16], [30016])
    flat, most = _share_long_key_ranges(_items([16], 10), step, workgroups_per_item=2)
    assert most == MAX_PARTS and MAX_PARTS <= 255  # eight bits in the item's fourth field
    step = _Step([16], [600])  # 600 keys: two parts of at least MIN_PART_KEYS
    flat, most = _share_long_key_ranges(_items([16], 10), step, workgroups_per_item=2)
    assert most == 600 // MIN_PART_KEYS == 2
    step = _Step([100, 1, 1], [100, 500, 700])  # few workgroups, but of few keys: nothing to share
    flat, most = _share_long_key_ranges(_items([100], 10), step, workgroups_per_item=2)
    assert most == 1
    flat, most = _share_long_key_ranges(np.zeros((0, 4), dtype=np.int32), step, workgroups_per_item=2)
    assert most == 1 and flat.size == 0


def test_items_of_different_lengths_get_parts_of_their_own():
    step = _Step([10, 10], [300, 5000])  # two portions: one behind 290 keys, one behind 4990
    flat, most = _share_long_key_ranges(_items(step.h_q_lens, 10), step, workgroups_per_item=1)
    out, part, parts = _unpack(flat)
    assert list(parts[out[:, 0] == 0]) == [1] and most == 5000 // MIN_PART_KEYS
    assert (parts[out[:, 0] == 1] == most).all() and (out[:, 0] == 1).sum() == most


def test_short_and_long_key_ranges():
    assert portions_have_short_ranges([2048], [2048])
    assert not portions_have_short_ranges([2048], [8192])
    assert not portions_have_short_ranges([1, 1], [500, 600])  # no portion at all
