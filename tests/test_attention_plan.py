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
