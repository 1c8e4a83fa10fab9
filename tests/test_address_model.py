"""Where the attention and rotary kernels reach, worked out on the host for the model sizes and steps that are run.

The kernels index the cache plane, the block tables, LDS and the partial-result workspace with arithmetic that the
host never sees. This file repeats that arithmetic in numpy, statement for statement, from csrc/attention_mfma.hip
and csrc/rope_cache.hip, for the three size presets (12 heads over 3, 16 over 4, 32 over 8; head size 128) and the
steps a benchmark or a serving run brings (a 2,048-token portion at the start of a request and behind 2,048 or
6,144 others, decoded tokens at batch 1, 8 and 64 near contexts of 4,096 and 8,192, a 512-token portion beside
decoded tokens), and asserts that every offset stays inside what it indexes. The planner and the split arithmetic are
the product's own (`attention_items`, `attention_launch_plan`), so the cases are the launches the engine makes.
"""
import json
import os

import numpy as np
import pytest

from tiny_inference_server_amd.ops import hip_ops
from tiny_inference_server_amd.ops.hip_ops import (attention_items, attention_launch_plan, decode_items, tile_columns,
                                                   uneven_lengths)

PRESETS = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tiny_inference_server_amd",
                       "config", "presets")
PAGE = 16
TW = 4                                   # waves of a tile (attention_mfma.hip: TW)


def geometry(size):
    with open(os.path.join(PRESETS, size + ".json")) as f:
        raw = json.load(f)
    nh = raw["N_HEAD"]
    return nh, nh // raw["NUM_GROUPS"], raw["D_MODEL"] // nh


def steps_of(batch_rows):
    """seq_rows (first row, first position, rows) of a step from (first position, rows) per request."""
    out, first = [], 0
    for p0, n in batch_rows:
        out.append((first, p0, n))
        first += n
    return out


CASES = {
    "prompt 2048": [(0, 2048)],
    "prompt 2048 behind 2048": [(2048, 2048)],
    "prompt 2048 behind 6144": [(6144, 2048)],
    "prompt 2027 behind 2048": [(2048, 2027)],
    "decode b1 ctx 4096": [(4095, 1)],
    "decode b8 ctx 4096": [(4080 + i, 1) for i in range(8)],
    "decode b64 ctx 4096": [(4032 + i, 1) for i in range(64)],
    "decode b64 ctx 8192": [(8128 + i, 1) for i in range(64)],
    "decode b64 of uneven lengths": [(17 + 127 * i, 1) for i in range(64)],
    "decode b5, one long": [(8000, 1), (3, 1), (40, 1), (700, 1), (0, 1)],
    "prompt 512 beside 8 decoding": [(4000 + i, 1) for i in range(8)] + [(1000, 512)],
    "4 prompts of 512": [(0, 512)] * 4,
    "prompt 31 behind 100": [(100, 31)],
    # steps of a scheduler that feeds prompts of 4,006 tokens under a budget of 2,056 beside decoded tokens
    "portion 2056": [(0, 2056)],
    "rest 1950 and next 106": [(2056, 1950), (0, 106)],
    "1 decoding, portion 2055": [(4006, 1), (106, 2055)],
    "2 decoding, rest 1845, next 209": [(4008, 1), (4006, 1), (2161, 1845), (0, 209)],
    "7 decoding, rest 700": [(4020 - i, 1) for i in range(7)] + [(3306, 700)],
}


def tile_extents(HD, kvh_count, tiles, positions, lp, table_width):
    """Largest page index, piece offset (elements inside a page) and LDS element that attention_tile_kernel reaches."""
    DB, NCH, TCH = HD // 16, HD // 8, 4 * HD
    TPT = (TCH + TW * 64 - 1) // (TW * 64)
    page_stride = 2 * kvh_count * PAGE * HD
    tid = np.arange(TW * 64)
    worst_page_index, worst_piece_end, worst_lds_end = 0, 0, 0
    for kvh in (0, kvh_count - 1):
        k_head, v_head = kvh * PAGE * HD, (kvh_count + kvh) * PAGE * HD
        for j in range(TPT):
            c = tid + j * TW * 64
            live = (tid // 64) * 64 + j * TW * 64 < TCH          # the kernel's break for pieces past the step's last
            key_in_tile = (c & 3) | ((c & 4) << 1) | ((c & 8) >> 1)
            k_off = k_head + key_in_tile * HD + ((c >> 4) % NCH) * 8
            v_off = v_head + (((c >> 5) % DB) * 16 + (c & 15)) * PAGE + ((c >> 4) & 1) * 8
            worst_piece_end = max(worst_piece_end, int((k_off[live] + 8).max()), int((v_off[live] + 8).max()))
            lds = ((tid // 64) + j * TW) * 512 + (tid % 64) * 8 + 8      # elements: base of the wave's fetch + lane * 16 B
            worst_lds_end = max(worst_lds_end, int(lds[live].max()))
    for row0, rows in tiles:
        p_first = int(positions[row0])
        k_hi = p_first + rows
        n_steps = (k_hi + 31) // 32
        splits = max(1, min(lp.tile_splits, -(-n_steps // lp.tile_max_steps)))
        per = -(-n_steps // splits)
        for split in range(splits):
            s_begin, s_end = split * per, min(n_steps, split * per + per)
            # load_run: lane l of a run that starts at step s0 reads the table at key (2 s0 + l) * 16 if that is a key
            for s0 in range(s_begin, max(s_end, s_begin + 1), 32):
                key0 = (2 * s0 + np.arange(64)) * 16
                idx = np.where(key0 < k_hi, key0 >> 4, 0)
                worst_page_index = max(worst_page_index, int(idx.max()))
                assert 2 * (min(s_end, s0 + 32) - 1 - s0) + 1 < 64           # what `stage` reads of the run
    assert worst_page_index < table_width
    assert worst_piece_end <= page_stride
    return worst_page_index, worst_piece_end, worst_lds_end, TCH * 8


# The statements of the kernel source that the functions here repeat. If one of them is edited there, the test below
# fails until the model has been brought in step with it (and this list with the source).
MIRRORED = {
    "attention_mfma.hip": [
        "const int key_in_tile = (c & 3) | ((c & 4) << 1) | ((c & 8) >> 1);",
        "k_off[j] = (unsigned)k_head + key_in_tile * HD + ((c >> 4) % NCH) * 8;",
        "v_off[j] = (unsigned)v_head + (((c >> 5) % DB) * 16 + (c & 15)) * page_size + ((c >> 4) & 1) * 8;",
        "const int key0 = k_lo + (2 * s0 + lane) * 16;",
        "const int pg = bt[key0 < k_hi ? (PS16 ? key0 >> 4 : key0 / page_size) : 0];",
        "const TileAddress* at = &run_tiles[wave][2 * (s - run_first)];",
        "if (s - run_first >= 32) load_run(s);",
        "const int item_splits = max(1, min(n_splits, (n_steps + max_steps - 1) / max_steps));",
        "static constexpr int TPT = (TCH + TW * 64 - 1) / (TW * 64);",
        "&k_lds[buf][(wave + j * TW) * 512]",
        # the one-wave kernel
        "const bf16* kp = base + k_head + (long)(slot0 + c16) * HD;",
        "const bf16* vp = base + v_head + (long)c16 * page_size + slot0 + g * 4;",
        "const long page_stride = 2L * n_kv_heads * page_size * HD;",
        "const long v_head = ((long)n_kv_heads + kvh) * page_size * HD;",
    ],
}


def test_the_model_mirrors_the_kernel_source_as_it_is():
    csrc = os.path.join(os.path.dirname(PRESETS), os.pardir, "csrc")
    for name, statements in MIRRORED.items():
        with open(os.path.join(csrc, name)) as f:
            text = " ".join(f.read().split())
        for st in statements:
            assert " ".join(st.split()) in text, f"{name} no longer holds `{st}`: bring tests/test_address_model.py in step"


def wave_extents(HD, kvh_count, items, positions, lp, single, table_width):
    """Largest table index and in-page offset that attention_mfma_kernel reaches (PS16 path)."""
    page_stride = 2 * kvh_count * PAGE * HD
    lanes = np.arange(64)
    c16, g = lanes & 15, lanes >> 4
    kvh = kvh_count - 1
    k_end = kvh * PAGE * HD + c16 * HD + ((HD + 31) // 32 - 1) * 32 + g * 8 + 8
    v_end = (kvh_count + kvh) * PAGE * HD + c16 * PAGE + g * 4 + (HD // 16 - 1) * 16 * PAGE + 4
    assert int(k_end.max()) <= kvh_count * PAGE * HD or HD % 32           # keys stay in the key half of the page
    assert int(v_end.max()) <= page_stride
    worst = 0
    for row0, rows in items:
        k_hi = int(positions[row0]) + rows
        n_steps = (k_hi + 31) // 32
        splits = lp.n_splits if lp.min_steps == 0 else max(1, min(lp.n_splits, n_steps // lp.min_steps))
        per = -(-n_steps // splits)
        for split in range(splits):
            s_begin, s_end = split * per, min(n_steps, split * per + per)
            for s in range(s_begin, s_end + 4):                         # the loop asks for page ids up to 3 steps ahead
                for t in range(2):
                    key0 = s * 32 + t * 16
                    ok = s < s_end and key0 < k_hi
                    worst = max(worst, key0 >> 4 if ok else 0)
    assert worst < table_width
    return worst


@pytest.mark.parametrize("size", ["0.9B", "2.1B", "7B"])
@pytest.mark.parametrize("case", list(CASES))
def test_attention_kernels_stay_inside_their_buffers(size, case):
    nh, kvh, HD = geometry(size)
    group = nh // kvh
    seq_rows = steps_of(CASES[case])
    n = sum(r for _, _, r in seq_rows)
    positions = np.concatenate([np.arange(p0, p0 + r) for _, p0, r in seq_rows])
    max_kv = max(p0 + r for _, p0, r in seq_rows)
    # the engine pads captured steps' tables to 64 pages; an eager step's table is as wide as its longest request
    table_width = -(-max_kv // PAGE)
    nb, items, tiles, tile_steps = attention_items(seq_rows, group, tile_columns(HD), kvh)
    assert nb in (1, 2, 4) and group <= 16 * nb
    covered = np.zeros(n, dtype=int)
    for r0, cnt in list(items) + list(tiles):
        covered[r0:r0 + cnt] += 1
    assert (covered == 1).all()                                          # every row in exactly one item or tile
    assert all(cnt * group <= 16 * nb for _, cnt in items)
    assert all(cnt <= TW * (tile_columns(HD) // group) for _, cnt in tiles)
    single = all(r <= 1 for _, _, r in seq_rows)
    if uneven_lengths(seq_rows):
        # single rows of very different lengths: the list planned row by row, one entry per wave
        entries, most = decode_items(seq_rows, nh, kvh, HD)
        lp = attention_launch_plan(n, len(entries), 0, (0, 0), False, max_kv, nh, kvh, HD, planned_splits=most)
        assert lp.min_steps == -1 and lp.n_splits == lp.stride == most
        assert lp.need_floats == lp.row_splits_offset + n <= hip_ops._ATTN_WORKSPACE_FLOATS or lp.stride == 1
        for row, packed, p, line in entries[entries[:, 0] >= 0].tolist():
            split, splits = packed & 0xffff, packed >> 16
            assert 0 <= row < n and p == int(positions[row]) and 0 <= line < len(seq_rows) and split < splits <= most
            n_steps = (p + 1 + 31) // 32
            per = -(-n_steps // splits)
            s_begin, s_end = split * per, min(n_steps, split * per + per)
            for st in range(s_begin, s_end + 4):
                for t in range(2):
                    key0 = st * 32 + t * 16
                    if st < s_end and key0 < p + 1:
                        assert key0 >> 4 < table_width
            slot = (row * nh + nh - 1) * lp.stride + split
            assert (slot + 1) * HD <= lp.ml_offset or lp.stride == 1
        return
    for kv_capacity in (max_kv, -(-table_width // 64) * 64 * PAGE):      # eager, and as a captured step sees it
        lp = attention_launch_plan(n, len(items), len(tiles), tile_steps, single, kv_capacity, nh, kvh, HD)
        # workspace: outputs, (maximum, sum) pairs and per-row counts lie one after the other inside it
        if lp.stride > 1:
            assert lp.ml_offset == n * nh * lp.stride * HD and lp.ml_offset % 2 == 0
            assert lp.row_splits_offset == lp.ml_offset + 2 * n * nh * lp.stride
            assert lp.need_floats == lp.row_splits_offset + n <= hip_ops._ATTN_WORKSPACE_FLOATS
            # the merge's largest reads: slot = (row * heads + head) * stride + split
            last_slot = ((n - 1) * nh + nh - 1) * lp.stride + lp.stride - 1
            assert (last_slot + 1) * HD <= lp.ml_offset and 2 * (last_slot + 1) <= lp.row_splits_offset - lp.ml_offset
        assert 1 <= lp.n_splits <= 65535 and 1 <= lp.tile_splits <= 65535
        if len(tiles):
            _, _, lds_end, lds_size = tile_extents(HD, kvh, tiles, positions, lp, table_width)
            assert lds_end <= lds_size
        if len(items):
            wave_extents(HD, kvh, items, positions, lp, single, table_width)


@pytest.mark.parametrize("size", ["0.9B", "2.1B", "7B"])
@pytest.mark.parametrize("rows,p0", [(2048, 0), (2027, 2048), (64, 5), (100, 4000)])
def test_rotary_rows_kernel_stays_inside_its_buffers(size, rows, p0):
    """rope_write_kv_rows_kernel (rope_cache.hip): sixteen rows a workgroup, four pairs a lane, values through LDS."""
    nh, kvh, HD = geometry(size)
    RB, THREADS = 16, 256
    half, pieces = HD // 2, HD // 8
    ld = (nh + 2 * kvh) * HD
    n_pages = -(-(p0 + rows) // PAGE) + 3
    plane_elems = n_pages * 2 * kvh * PAGE * HD
    slots = np.arange(p0, p0 + rows) + 3 * PAGE                 # some pages of this request, in order
    assert HD % 8 == 0 and HD <= 256 and ld % 8 == 0
    worst_in, worst_table, worst_plane, worst_tile = 0, 0, 0, 0
    for block in (0, (rows + RB - 1) // RB - 1):                # the first and the last (possibly short) workgroup
        r0 = block * RB
        n_rows = min(RB, rows - r0)
        i = np.arange(n_rows * pieces)                          # every (row, piece) the workgroup's threads take in turn
        row, piece = i // pieces, i % pieces
        r = r0 + row
        for hh in (0, nh + kvh - 1):
            worst_in = max(worst_in, int((r * ld + hh * HD + piece * 8 + 8).max()))
            worst_table = max(worst_table, int(((p0 + r) * half + piece * 4 + 4).max()))      # float2 entries
            if hh >= nh:
                s = slots[r]
                dst = ((s // PAGE) * 2 * kvh + (hh - nh)) * PAGE * HD + (s % PAGE) * HD
                worst_plane = max(worst_plane, int((dst + half + piece * 4 + 4).max()))
        # values: tile[row][piece * 8 .. + 8), then out along the rows
        worst_tile = max(worst_tile, int((row * (256 + 8) + piece * 8 + 8).max()))
        row_t = np.arange(THREADS) % RB
        live = row_t < n_rows
        s = slots[np.minimum(r0 + row_t, rows - 1)]
        v_dst = ((s // PAGE) * 2 + 1) * kvh * PAGE * HD + s % PAGE
        d = HD - 1
        worst_plane = max(worst_plane, int((v_dst[live] + ((kvh - 1) * HD + d) * PAGE + 1).max()))
        worst_in = max(worst_in, int(((r0 + n_rows - 1) * ld + (nh + 2 * kvh - 1) * HD + (pieces - 1) * 8 + 8)))
    assert worst_in <= rows * ld
    assert worst_table <= (p0 + rows) * half                   # the table has max_context >= p0 + rows positions
    assert worst_plane <= plane_elems
    assert worst_tile <= RB * (256 + 8)
