"""The host's cut of a step's rows into the attention kernels' work items: every row once, within the kernels' limits."""
import random

import numpy as np
import pytest

from tiny_inference_server_amd.ops.hip_ops import attention_items, tile_columns


@pytest.mark.parametrize("group", [1, 3, 4, 5, 8, 16, 40, 64])
@pytest.mark.parametrize("head_dim", [64, 256])
def test_every_row_lies_in_one_item_or_tile(group, head_dim):
    rng = random.Random(group * 1000 + head_dim)
    cols = tile_columns(head_dim)
    for _ in range(30):
        seq_rows, row = [], 0
        for _ in range(rng.randint(1, 6)):
            n = rng.choice([0, 1, 1, 2, 3, 17, 64, 130, 700])
            seq_rows.append((row, rng.randint(0, 5000), n))
            row += n
        nb, items, tiles, steps = attention_items(seq_rows, group, cols)
        assert group <= 16 * nb
        seen = np.zeros(row, dtype=np.int64)
        owner = np.full(row, -1)
        for i, (first, _, n) in enumerate(seq_rows):
            owner[first:first + n] = i
        for first, n in items:
            assert 1 <= n and n * group <= 16 * nb or n == 1
            assert len(set(owner[first:first + n])) == 1            # one request
            seen[first:first + n] += 1
        tile_rows = 4 * (cols // group)
        for first, n in tiles:
            assert 1 <= n <= tile_rows
            assert len(set(owner[first:first + n])) == 1
            seen[first:first + n] += 1
        assert (seen == 1).all()
        if all(n <= 1 for _, _, n in seq_rows):
            assert len(tiles) == 0 and [f for f, _ in items] == [f for f, _, n in seq_rows if n]


def test_longest_first():
    _, items, tiles, _ = attention_items([(0, 0, 1000), (1000, 3000, 1), (1001, 50, 5)], 4, 64)
    keys = [first for first, _ in tiles]
    assert keys == sorted(keys, reverse=True)         # a prompt's last rows see the most keys
    assert tuple(items[0]) == (1000, 1)               # the row deep into its request before the short portion


def test_decode_items_cover_every_step_once_in_waves_of_even_length():
    """Single rows of requests that differ widely in length: the planned list gives each row splits by its own
    length, every entry names its row's position and table line, the list's length depends on the number of rows
    alone, and no wave walks more than about an even share of all keys."""
    import random
    from tiny_inference_server_amd.ops.hip_ops import (decode_items, decode_items_capacity, decode_items_most_splits,
                                                       uneven_lengths)
    rng = random.Random(5)
    for n, kvh, heads, hd in [(64, 3, 12, 128), (5, 4, 16, 128), (17, 8, 32, 128), (2, 1, 3, 48), (300, 2, 4, 64)]:
        for trial in range(20):
            pos = [rng.choice([0, 3, 31, 32, 700, 4095, 8000]) if rng.random() < 0.5 else rng.randrange(8192)
                   for _ in range(n)]
            seq_rows = [(k + 100, p, 1) for k, p in enumerate(pos)]          # rows of the stage need not start at 0
            entries, most = decode_items(seq_rows, heads, kvh, hd)
            assert entries.shape == (decode_items_capacity(n, kvh), 4)
            assert most == decode_items_most_splits(n, heads, hd) >= 1
            live = entries[entries[:, 0] >= 0]
            assert (entries[len(live):, 0] == -1).all()                     # padding only at the end
            per_row = {}
            for row, packed, p, line in live.tolist():
                split, splits = packed & 0xffff, packed >> 16
                assert p == pos[line] and row == line + 100 and 0 <= split < splits <= most
                per_row.setdefault(line, []).append((split, splits))
            assert sorted(per_row) == list(range(n))
            steps = [(p + 32) // 32 for p in pos]
            longest = 0
            for line, got in per_row.items():
                splits = got[0][1]
                assert sorted(s for s, _ in got) == list(range(splits)) and splits <= steps[line]
                longest = max(longest, -(-steps[line] // splits))
            even = max(4, -(-sum(steps) * kvh // 512))
            # (a row may not be cut below the fewest steps of a split, nor into more splits than the workspace holds)
            bound = max(2 * even, max(-(-s // most) for s in steps))
            assert longest <= bound, (longest, even, most)
    assert not uneven_lengths([(0, 100, 1), (1, 120, 1), (2, 90, 1)])
    assert uneven_lengths([(0, 100, 1), (1, 4000, 1), (2, 90, 1)])
    assert not uneven_lengths([(0, 100, 2), (2, 4000, 1)]) and not uneven_lengths([(0, 4000, 1)])


def test_decoded_tokens_get_a_whole_multiple_of_the_chips_units_in_waves_where_few_more_splits_reach_one():
    """Equal waves spread evenly over 256 compute units only if their number is a multiple of 256. Where up to twice
    the splits that the target asks for reach one, that count is taken; where none does, the target's count stays;
    a context too short for more splits caps it; rows of prompts are not touched."""
    from tiny_inference_server_amd.ops.hip_ops import attention_launch_plan as plan

    def splits(requests, kv_heads, keys, single=True):
        return plan(requests, requests, 0, (0, 0), single, keys, kv_heads * 4, kv_heads, 128).n_splits
    assert splits(64, 3, 4096) == 4          # 768 waves instead of 576
    assert splits(32, 3, 4096) == 8          # 768 instead of 576
    assert splits(16, 3, 4096) == 16         # 768 instead of 528
    assert splits(8, 3, 4096) == 32          # 768 instead of 528
    assert splits(24, 3, 4096) == 8          # 72 waves a split: no multiple of 256 within 16 splits
    assert splits(64, 8, 4096) == 1          # 512 waves without any split
    assert splits(32, 4, 4096) == 4          # 512: the target's count is one already
    assert splits(64, 3, 300) == 2           # splits of at least 128 keys
    for requests, kv_heads, keys in ((64, 3, 4096), (16, 3, 4096), (5, 2, 1000), (48, 3, 8192), (7, 1, 70)):
        s = splits(requests, kv_heads, keys)
        assert 1 <= s <= max(1, keys // 64) and s < 2 * 512 // (requests * kv_heads) + 2
    assert splits(64, 3, 4096, single=False) == 11     # 2,048 waves offered to rows of prompts; 12 would be the multiple
