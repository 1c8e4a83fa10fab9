"""The kernels as Python calls on torch tensors: what the parts and the engine compute with.

Every method checks on the host that shapes, dtypes and strides are what the kernel and its grid assume,
then launches on torch's current stream. There is no CPU path: without a GPU or without the compiled
libraries construction fails. Matrix products in bfloat16 of a few rows go to the fused few-row kernel
(csrc/gemm_skinny.hip), those of many rows to hipBLASLt through csrc/gemm_library.hip, as the reference's go to
a library (main_models_new.py:19-20); in 32-bit they go to the plain multiply-add kernel so that no
reduced-precision matrix mode can take part.

The library is only ever asked for products whose widths (output columns, input columns) stand in
ops/library_widths.json, the list of widths that this repository's GPU tests and benchmarks run, and only at row
counts from one family (library_rows): a library kernel differs from shape to shape, and a shape that nothing has
run is a kernel that nothing has tested. Any other product runs on this repository's own kernels: right at every
size, slower where there are many rows.
"""
from __future__ import annotations

import ctypes
import json
import os
from ctypes import c_float, c_int, c_long, c_void_p
from typing import NamedTuple, Optional

import numpy as np
import torch

from . import build as _build

_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def _ptr(t: Optional[torch.Tensor]):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


class _Lib:
    """One compiled library with typed entry points that raise on failure."""

    def __init__(self, name: str, prefix: str, signatures: dict):
        self.name = name
        self.cdll = _build.load(name)
        self._err = getattr(self.cdll, f"{prefix}_last_error")
        self._err.restype = ctypes.c_char_p
        for fn, argtypes in signatures.items():
            f = getattr(self.cdll, fn)
            f.argtypes = argtypes
            f.restype = c_int
            setattr(self, fn, self._wrap(f))

    def _wrap(self, f):
        def call(*args):
            if f(*args) != 0:
                raise KernelError(self._err().decode(errors="replace"))
        return call


_P, _I, _L, _F = c_void_p, c_int, c_long, c_float

_SIGNATURES = {
    "rowwise": ("tis_rowwise", {
        "tis_rmsnorm": [_I, _P, _L, _P, _P, _L, _I, _I, _F, _P],
        "tis_embedding": [_I, _P, _P, _P, _L, _I, _I, _P],
        "tis_embedding_rmsnorm": [_I, _P, _P, _P, _P, _L, _I, _I, _F, _P],
        "tis_gather_rows": [_I, _P, _L, _P, _L, _P, _P, _L, _I, _I, _P],
        "tis_copy_rows": [_I, _P, _L, _P, _P, _L, _P, _I, _I, _P],
        "tis_swiglu": [_I, _P, _L, _P, _L, _I, _I, _P],
    }),
    "rope_cache": ("tis_rope_cache", {
        "tis_rope_write_kv": [_I, _P, _L, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _L, _P],
    }),
    "attention_generic": ("tis_attention_generic", {
        "tis_attention_generic": [_I, _P, _L, _P, _P, _I, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _F, _P, _P],
    }),
    "gemm_plain": ("tis_gemm_plain", {
        "tis_gemm_plain": [_I, _I, _P, _L, _P, _L, _P, _L, _P, _L, _I, _I, _I, _P],
    }),
    "sampling": ("tis_sampling", {
        "tis_sample": [_P, _L, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P],
        "tis_argmax": [_P, _L, _I, _I, _P, _P],
    }),
}

_SIGNATURES["gemm_skinny"] = ("tis_gemm_skinny", {
    "tis_gemm_skinny": [_P, _L, _P, _P, _F, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P],
    "tis_gemm_skinny_qkv_rope": [_P, _L, _P, _P, _F, _P, _L, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
})
_SIGNATURES["gemm_tiles"] = ("tis_gemm_tiles", {
    "tis_gemm_tiles": [_P, _L, _P, _P, _L, _P, _L, _I, _I, _I, _I, _P],
})
_SIGNATURES["gemm_library"] = ("tis_gemm_library", {
    "tis_gemm_library_init": [],
    "tis_gemm_library": [_P, _L, _P, _P, _L, _P, _L, _I, _I, _I, _I, _P],
})
_SIGNATURES["attention_mfma"] = ("tis_attention_mfma", {
    "tis_attention_mfma_side_stream": [_P],
    "tis_attention_mfma": [_P, _L, _P, _P, _I, _P, _P, _P, _I, _I, _P, _I, _P, _L, _P, _P, _I, _I, _I, _I, _I, _I, _F,
                           _I, _I, _I, _I, _P, _P],
})

_libs = {}


def library(name: str) -> _Lib:
    """`name` may carry a variant: 'attention_mfma@128'."""
    lib = _libs.get(name)
    if lib is None:
        prefix, sigs = _SIGNATURES[name.split("@")[0]]
        lib = _libs[name] = _Lib(name, prefix, sigs)
    return lib


_FEW_ROWS = 128                 # up to this many rows a product goes to the few-row kernels whatever its widths

_WIDTHS_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "library_widths.json")


def library_widths(path: str = _WIDTHS_FILE):
    """The (output columns, input columns) pairs that may go to the library's product: a data file, not code."""
    with open(path) as f:
        return frozenset((int(n), int(k)) for n, k in json.load(f)["widths"])


def library_rows(m: int) -> int:
    """The row count the library is asked for when a product has `m` rows: the next multiple of 64 up to 256 rows,
    of 256 beyond. A serving run's steps bring row counts that nobody chose (a portion beside some decoded tokens, a
    prediction head's rows one short of the trunk's); rounded up, they all become the few shapes that every
    benchmark and test of a width has already run. The extra rows are computed on whatever lies behind the operands'
    rows and are never read."""
    step = 64 if m <= 256 else 256
    return -(-m // step) * step


def product_route(M: int, N: int, K: int, aligned: bool, out_f32: bool, widths, few_rows: int = _FEW_ROWS):
    """Which kernel takes a bfloat16 product of M rows, N output and K input columns: "few_rows" (the fused few-row
    kernel, in panels of rows beyond its own height), "library" (at library_rows(M) rows, at the widths of its
    list), "tiles" (this repository's tiled product, for many rows at any other width and for 32-bit results at any
    width) or "plain" (multiply-adds, for operands that do not lie as the others need them). Pure: the decision can be checked without a device."""
    if not aligned:
        return "plain"
    if M <= few_rows:
        return "few_rows"
    if (N, K) in widths and not out_f32:
        return "library"
    return "tiles" if N % 4 == 0 else "few_rows"


# wavefronts the attention launch aims for, so that short batches still spread over the chip
_ATTN_TARGET_WAVES = 512
_CHIP_UNITS = 256               # compute units of an MI355X: the default where no device is asked (host-only tests)
_ATTN_PROMPT_TARGET_WAVES = 2048  # what the grid offers where rows of prompts are in the batch ...
_ATTN_PROMPT_SPLIT_MAX_ROWS = 512 # ... and the batch is small; a long portion fills the chip by its rows alone
_ATTN_PROMPT_MIN_STEPS = 8         # steps of 32 keys below which a prompt item's split is not worth its merge
_ATTN_UNEVEN = 1.5              # decoded tokens: from this ratio of the longest request to the mean on, splits are planned
                                # request by request on the host instead of being the same for all
_ATTN_DECODE_MAX_SPLITS = 64    # ... and the most that one request may get
_ATTN_PLANNED_MIN_ROWS = 16     # ... where there are at least this many requests (8: as fast either way) ...
_ATTN_PLANNED_MAX_WAVES = 384   # ... and requests x key/value heads are at most this: beyond, there are too few splits
                                # to shift between requests and the plain grid is as fast or faster. A planned list
                                # aims at one entry (a wave per key/value head) per compute unit, and at
                                # _ATTN_TARGET_WAVES waves at least. Uneven requests of 128 to 4,200 keys, planned /
                                # same splits for all, us: 3 kv heads, 96 requests 72 / 87, 64: 43 / 47, 24: 20.5 /
                                # 24.6; 4 heads, 96: 100 / 103, 48: 39 / 43; 8 heads, 64: 126 / 124, 32: 53.5 / 60.6;
                                # 1 head, 64: 19.8 / 21.0; with 8 requests 13.2 / 12.4 (3 heads), 23.6 / 21.8 (8)
_ATTN_DECODE_BYTES_PER_US = 5.0e6   # keys and values a step of decoded tokens streams: 5 TB/s
_ATTN_PLANNED_BESIDE_FROM = 1.15   # single rows beside tiles get a planned list if they take this much longer than the tiles
_ATTN_PLANNED_WAVES_BESIDE_TILES = 1.5   # ... and at this many waves per compute unit, over all key/value heads, where
                                # the list runs beside a portion's tiles, whose workgroups need room on every unit
_ATTN_MIN_SPLIT_KEYS = 128      # a split shorter than this costs more in merging than it gains in spreading
_ATTN_TILE_WAVES = 4            # waves of the workgroup that takes a tile of a long portion
_ATTN_TILE_GROUPS = 512         # workgroups of the tile kernel that the chip runs side by side
_ATTN_TILE_MIN_STEPS = 8        # steps of 32 keys below which a tile's split is not worth its merge
_ATTN_TILE_SPLIT_SLACK = 1.4    # a split may be this much longer than an even share of all steps
_ATTN_TILE_STEP_US = (0.72, 1.3)   # what a tile's step of 32 keys takes while a workgroup has a compute unit to itself,
                                # and once two share one (12 heads of 128 over 3; other geometries differ little)
_ATTN_TILE_MERGE_US = (10.0, 4.0, 6e6)   # what cutting tiles into key splits costs beyond the tiles' own time: the
                                # merge's launch and the per-row counts (less where the items' splits are merged anyway),
                                # and microseconds per byte of 32-bit partial results. Tiles are cut only where, by
                                # these figures, the shorter chains save more than that. 12 heads of 128 over 3, us,
                                # cut / uncut / one-wave kernel: 4 prompts of 512 tokens 28.8 / 18.8 / 22.8, 8 of 512
                                # 40.8 / 25.4 / 33.2, 4 of 1,024 50.6 / 39.5 / 57.2, one of 1,024 29.2 / 28.6 / 29.2; but
                                # one of 1,536 35.3 / 39.9 / 47.7, of 2,048 42.4 / 51.3 / 69.5, 512 tokens behind 3,000
                                # others 41.5 / 82.5 / 60.0
_ATTN_TILE_PARTIAL_BYTES = 40 << 20   # partial results (32-bit, per split) beyond which the merge costs more than
                                      # shorter chains save; at least two splits are always allowed
_ATTN_TILE_MIN_WORK_MIXED = 1500   # tile steps times key/value heads below which the one-wave kernel is the faster
                                   # beside decoded tokens deep in their requests (few tiles with long chains: the
                                   # one-wave kernel spreads them over more waves, and its splits are merged anyway)
_ATTN_WORKSPACE_FLOATS = 16 << 20


def tile_columns(head_dim: int) -> int:
    """Columns (row, query head of a group) of one wave of the tile kernel, as the kernel source sets them."""
    return 32


def attention_items(seq_rows, group_size: int, tile_cols: int = 0, n_kv_heads: int = 0):
    """Work items of the matrix-core attention kernels for the rows of one stage.

    seq_rows: (first row, first position, rows) per request. Returns (column blocks per item, items, tiles, steps):
    items and tiles are int32 arrays of (first row, rows) lines that together hold every row once, steps is
    (the number of 32-key steps that all tiles walk together, the most that one tile walks): the kernel's work, by
    which its key splits are sized.
    An item (one wave) holds consecutive rows of one request, rows * group_size <= 16 * blocks. When no request has
    more than one row the list is simply every row in order, which the kernel knows without being given a list.
    A tile (a workgroup of four waves, `tile_cols` columns each; 0: no tiles) takes up to 4 * (tile_cols // group_size)
    consecutive rows of a portion that fills at least half of one. Beside decoded tokens deep in their requests, tiles
    are made only where their steps times `n_kv_heads` (the workgroups' work; 0: always) reach
    _ATTN_TILE_MIN_WORK_MIXED. Measured at 12 heads of 128 over 3 (tiles / one-wave kernel, us): one prompt of 256
    rows 12.1 / 13.3, of 512 rows 17.5 / 22.3, of 1,024 rows 28.6 / 29.2, 8 of 512 rows 25.4 / 33.2; a portion of 512
    rows at 1,000 beside 8 decoded tokens at 4,095: 54.9 / 64.7, one of 256 rows 40.6 / 30.1, one of 128 35.9 / 23.9.
    """
    none = np.zeros((0, 2), dtype=np.int32)
    # (arrays over all requests at once: a step may hold hundreds, and this runs for every stage of every step that
    # is not replayed from a graph)
    rows = np.asarray(seq_rows, dtype=np.int64).reshape(-1, 3)
    first, p0, n = rows[:, 0], rows[:, 1], rows[:, 2]
    if not (n > 1).any():
        nb = 1
        while group_size > 16 * nb:
            nb *= 2
        live = n > 0
        return nb, np.stack((first[live], n[live]), axis=1).astype(np.int32), none, (0, 0)

    def cut(which, per_item):
        if not which.any():
            return none, (0, 0)
        f, q0, m = first[which], p0[which], n[which]
        k = -(-m // per_item)                                          # items of each segment
        r = (np.arange(int(k.sum())) - np.repeat(np.cumsum(k) - k, k)) * per_item    # an item's first row in its segment
        counts = np.minimum(per_item, np.repeat(m, k) - r)
        firsts = np.repeat(f, k) + r
        keys = np.repeat(q0, k) + r + counts
        # those with the most keys first: under a causal mask the last rows of a prompt are the longest, and
        # started last they would run on alone while the rest of the chip idles
        order = np.argsort(-keys, kind="stable")
        steps = (keys + 31) // 32
        return np.stack((firsts[order], counts[order]), axis=1).astype(np.int32), (int(steps.sum()), int(steps.max()))

    tile_rows = _ATTN_TILE_WAVES * (tile_cols // group_size)
    tiled = (n >= max(2, tile_rows // 2)) if tile_rows else np.zeros(len(n), dtype=bool)
    tiles, steps = cut(tiled, tile_rows) if tile_rows else (none, (0, 0))
    if len(tiles) and n_kv_heads and steps[0] * n_kv_heads < _ATTN_TILE_MIN_WORK_MIXED \
            and ((n == 1) & (p0 >= 512)).any():
        # beside decoded tokens deep in their requests: too little work for tiles
        tiled, tiles, steps = np.zeros(len(n), dtype=bool), none, (0, 0)
    rest = (n > 0) & ~tiled
    nb = 2
    # 64-column items halve what a portion reads of its keys and values; they pay once there are enough of them
    # to fill the chip, and cost where a few long chains of steps set the time
    if group_size <= 64 and int((-(-n[rest] // max(1, 64 // group_size))).sum()) >= 384:
        nb = 4
    while group_size > 16 * nb:
        nb *= 2
    return nb, cut(rest, max(1, (16 * nb) // group_size))[0], tiles, steps


def uneven_lengths(seq_rows, window: int = 0) -> bool:
    """Whether a step of single rows holds requests of such different lengths that equal split counts would leave the
    longest request's waves running on alone: then the splits are planned request by request (decode_items). With a
    window a row's length is what it sees of its request."""
    n = len(seq_rows)
    if n < 2:
        return False
    longest = total = 0
    for _, p0, rows in seq_rows:            # (one pass: this runs for every step of decoded tokens)
        if rows != 1:
            return False
        steps = (p0 + 32) >> 5 if window <= 0 or p0 < window else (p0 + 32 - ((p0 - window + 1) & ~31)) >> 5
        total += steps
        if steps > longest:
            longest = steps
    return longest * n > _ATTN_UNEVEN * total + 2 * n


def planned_list_pays(n_rows: int, n_kv_heads: int) -> bool:
    """Whether single rows of uneven lengths get a planned list rather than the same splits for all."""
    return n_rows >= _ATTN_PLANNED_MIN_ROWS and n_rows * n_kv_heads <= _ATTN_PLANNED_MAX_WAVES


def planned_target_waves(n_kv_heads: int, units: int = _CHIP_UNITS) -> int:
    return max(_ATTN_TARGET_WAVES, units * n_kv_heads)


def decode_items_capacity(n_rows: int, n_kv_heads: int, units: int = _CHIP_UNITS) -> int:
    """Entries of a planned list for `n_rows` single rows: what the splits can add up to, whatever the lengths."""
    # (a multiple of the eight XCDs: workgroups go to them in turn, so the waves of an entry's key/value heads, which
    # read the same pages, then meet in one L2: 162 against 183 us at 8 key/value heads)
    return -(-(planned_target_waves(n_kv_heads, units) // n_kv_heads + n_rows + 1) // 8) * 8


def decode_items_most_splits(n_rows: int, n_heads: int, head_dim: int, workspace_floats=None) -> int:
    """The most splits one row of such a list may have: bounded by the workspace for partial results."""
    workspace_floats = _ATTN_WORKSPACE_FLOATS if workspace_floats is None else workspace_floats
    return int(max(1, min(_ATTN_DECODE_MAX_SPLITS, (workspace_floats - n_rows) // (n_rows * n_heads * (head_dim + 2)))))


def decode_items(seq_rows, n_heads: int, n_kv_heads: int, head_dim: int, workspace_floats=None, window: int = 0,
                 units: int = _CHIP_UNITS, table_lines=None, all_rows: int = 0, share: float = 1.0):
    """The work list of a step of single rows whose requests differ widely in length: one entry per wave (and
    key/value head), (row, split + 65536 * splits of the row, position, block-table line), so that every wave walks
    about the same number of keys; longest first; padded with row -1 to a length that depends on the number of rows
    alone (a captured launch keeps its grid while the lengths change). Returns (int32 [capacity, 4], most splits).
    table_lines: the rows' lines of the block table where they are not simply 0, 1, ... (single rows beside portions
    of other requests); all_rows: the rows of the whole step then (they share the workspace for partial results)."""
    n = len(seq_rows)
    rows = np.fromiter((f for f, _, _ in seq_rows), dtype=np.int64, count=n)
    pos = np.fromiter((p0 for _, p0, _ in seq_rows), dtype=np.int64, count=n)
    # a row at position p sees p + 1 keys, or the last `window` of them; the kernel walks them in steps of 32 from a
    # multiple of 32
    first = np.maximum(0, pos - window + 1) & ~31 if window > 0 else 0
    steps = (pos + 32 - first) // 32
    fewest = max(1, _ATTN_MIN_SPLIT_KEYS // 32)
    even = max(fewest, -(-int(steps.sum()) * n_kv_heads // max(1, int(planned_target_waves(n_kv_heads, units) * share))))
    most = decode_items_most_splits(max(n, all_rows), n_heads, head_dim, workspace_floats)
    splits = np.clip((steps + even // 2) // even, 1, np.minimum(steps, most))
    cap = decode_items_capacity(n, n_kv_heads, units)
    total = int(splits.sum())
    if total > cap:
        raise KernelError(f"attention: {total} planned splits for a list of {cap}")
    # one entry per (row, split); those with the most steps first, and among equals split by split over all rows, so
    # that waves that start together read different requests' pages (the order a grid of rows x splits would have)
    who = np.repeat(np.arange(n), splits)
    which = np.arange(total) - np.repeat(np.cumsum(splits) - splits, splits)
    per_split = -(-steps // splits)
    by = np.lexsort((who, which, -per_split[who]))
    who, which = who[by], which[by]
    out = np.full((cap, 4), -1, dtype=np.int32)
    out[:total, 0] = rows[who]
    out[:total, 1] = which + (splits[who] << 16)
    out[:total, 2] = pos[who]
    out[:total, 3] = who if table_lines is None else np.asarray(table_lines, dtype=np.int64)[who]
    return out, most


def planned_beside_tiles(seq_rows, items, tiles, tile_steps, n_heads: int, n_kv_heads: int, head_dim: int,
                         window: int = 0, units: int = _CHIP_UNITS):
    """For a step whose portions all go to tiles and whose other rows are single rows of requests that differ widely
    in length (decoded tokens beside a prompt's portion): the planned list of decode_items for those rows, or None.
    With the same number of splits for every row the longest request's waves would run on alone, here beside the
    tiles' workgroups. It pays where the single rows are the longer half of the pair: beside tiles that take as long as
    they do or longer (a portion deep in a long prompt) the rows are done first either way, and the list only costs the
    host its making. 64 decoded tokens at 512 to 8,000 keys, us a layer, planned / same splits for all, 12 heads over 3:
    beside a 2,048-token prompt 125 / 151, beside 1,024 tokens behind 1,000 others 126 / 151, beside 2,048 behind
    2,048 others 143 / 154; 16 over 4: 158 / 191, 164 / 195 and 197 / 186."""
    n_items = len(items)
    if not len(tiles) or n_items < _ATTN_PLANNED_MIN_ROWS or n_items * n_kv_heads > _ATTN_PLANNED_MAX_WAVES \
            or n_heads // n_kv_heads > 64 or int(items[:, 1].max()) != 1:
        return None
    singles, lines, all_rows = [], [], 0
    for i, (f, p0, n) in enumerate(seq_rows):
        all_rows += n
        if n == 1:
            singles.append((f, p0, 1))
            lines.append(i)
    if len(singles) != n_items or not uneven_lengths(singles, window):
        return None
    # what the rows take at the rate a step of decoded tokens streams keys and values, against the tiles' estimate
    row_steps = sum((p0 + 32) >> 5 if window <= 0 or p0 < window else (p0 + 32 - ((p0 - window + 1) & ~31)) >> 5
                    for _, p0, _ in singles)
    rows_us = row_steps * n_kv_heads * 64 * head_dim * 2 / _ATTN_DECODE_BYTES_PER_US
    cut, cut_steps = _tiles_cut(all_rows, len(tiles), tile_steps, n_heads, n_kv_heads, head_dim)
    tiles_us = min(_tiles_us(all_rows, len(tiles), tile_steps[0], tile_steps[1], cut, cut_steps, n_heads, n_kv_heads,
                             head_dim, True, units))
    if rows_us < _ATTN_PLANNED_BESIDE_FROM * tiles_us:
        return None
    return decode_items(singles, n_heads, n_kv_heads, head_dim, window=window, units=units, table_lines=lines,
                        all_rows=all_rows, share=min(1.0, _ATTN_PLANNED_WAVES_BESIDE_TILES / n_kv_heads))


class AttentionLaunch(NamedTuple):
    """How one call of the matrix-core attention cuts its keys, and where its partial results lie in the workspace
    (offsets in floats): [rows][heads][stride][head size] outputs, then [rows][heads][stride] (maximum, sum) pairs,
    then [rows] split counts."""
    n_splits: int
    min_steps: int
    tile_splits: int
    tile_max_steps: int
    stride: int
    ml_offset: int
    row_splits_offset: int
    need_floats: int


def _tiles_us(n, n_tiles, all_steps, longest, cut, cut_steps, n_heads, n_kv_heads, head_dim, merged_anyway, units):
    """Estimated microseconds of a call's tiles left whole, and cut into `cut` key splits of at most `cut_steps` steps:
    the longest chain of steps sets the time (a step takes longer once two workgroups share a compute unit, and no
    less than all steps spread evenly take), and the cut adds the merge."""
    alone, shared = _ATTN_TILE_STEP_US

    def chain_us(steps, workgroups):
        return max(steps * min(shared, alone * max(1.0, workgroups / units)), all_steps * n_kv_heads / (2 * units) * shared)
    whole = chain_us(longest, n_tiles * n_kv_heads)
    launch, launch_merged, bytes_per_us = _ATTN_TILE_MERGE_US
    merge = (launch_merged if merged_anyway else launch) + n * n_heads * head_dim * 4 * cut / bytes_per_us
    parts = chain_us(cut_steps, n_kv_heads * (all_steps / cut_steps + n_tiles / 2)) + merge
    return whole, parts


def _tiles_cut_pays(*args) -> bool:
    """Whether cutting the tiles of a call into key splits is estimated to be faster than leaving them whole."""
    whole, parts = _tiles_us(*args)
    return parts < whole


def _tiles_cut(n, n_tiles, tile_steps, n_heads, n_kv_heads, head_dim):
    """Into how many key splits, of at most how many steps, a call's tiles would be cut if they are cut."""
    all_steps, longest = tile_steps
    share = all_steps * n_kv_heads / _ATTN_TILE_GROUPS
    cut_steps = max(_ATTN_TILE_MIN_STEPS, int(share * _ATTN_TILE_SPLIT_SLACK) + 1)
    most_splits = max(2, _ATTN_TILE_PARTIAL_BYTES // (n * n_heads * head_dim * 4))
    cut = max(1, min(most_splits, -(-longest // cut_steps)))
    return cut, max(cut_steps, -(-longest // cut))


def attention_launch_plan(n, n_items, n_tiles, tile_steps, single, max_kv_len, n_heads, n_kv_heads, head_dim,
                          workspace_floats=None, planned_splits=0, units: int = _CHIP_UNITS) -> AttentionLaunch:
    """Split counts of one attention call over `n` rows, from the planner's items and tiles; pure host arithmetic.
    planned_splits > 0: the items are a list planned by decode_items, whose rows have at most that many splits."""
    workspace_floats = _ATTN_WORKSPACE_FLOATS if workspace_floats is None else workspace_floats
    n_splits, min_steps, tile_splits, tile_max_steps = 1, 0, 1, 1 << 20
    if planned_splits:
        n_splits, min_steps = planned_splits, -1
    elif n_items:
        # decoded tokens: every request's keys are cut into the same number of splits, enough to spread a
        # short batch over the chip. Prompt rows: the grid offers more splits than the chip needs and every
        # item takes as many as its own length deserves (the kernel decides, from _ATTN_PROMPT_MIN_STEPS),
        # because the last rows of a long prompt would otherwise run on alone long after the first have finished.
        target = _ATTN_PROMPT_TARGET_WAVES if (not single and n <= _ATTN_PROMPT_SPLIT_MAX_ROWS) else _ATTN_TARGET_WAVES
        # a lone request or two: shorter splits still pay, because so few waves would leave most of the chip idle
        min_keys = _ATTN_MIN_SPLIT_KEYS // 2 if n_items * n_kv_heads <= 8 else _ATTN_MIN_SPLIT_KEYS
        n_splits = max(1, min(-(-target // (n_items * n_kv_heads)), max_kv_len // min_keys))
        if single and n_splits > 1:
            # equal waves spread evenly only if their number is a whole multiple of the chip's compute units: a few
            # more splits that reach one beat the target's count (64 requests over 3 heads at 4,096 keys: 4 splits
            # 79 us, 3 splits 82; 32 requests: 8 splits 37, 6 splits 40; at 8,192 keys 146 against 163)
            waves = n_items * n_kv_heads
            for s in range(n_splits, min(2 * n_splits, max_kv_len // min_keys) + 1):
                if waves * s % units == 0:
                    n_splits = s
                    break
        min_steps = 0 if single else _ATTN_PROMPT_MIN_STEPS
    if n_tiles:
        # a tile's keys are cut so that no workgroup walks a chain of steps much longer than an even share of
        # all tiles' steps: the last rows of a long prompt would otherwise run on alone. Measured at 12 heads
        # of 128 (tiles / one-wave kernel, us): 2,048 rows from 0: 54 / 69; from 2,048: 99 / 134; from 6,144:
        # 196 / 260; 4,096 rows: 146 / 202.
        all_steps, longest = tile_steps
        cut, cut_steps = _tiles_cut(n, n_tiles, tile_steps, n_heads, n_kv_heads, head_dim)
        if cut > 1 and _tiles_cut_pays(n, n_tiles, all_steps, longest, cut, cut_steps, n_heads, n_kv_heads, head_dim,
                                       n_splits > 1, units):
            tile_splits, tile_max_steps = cut, cut_steps
    # partial results of split key ranges live in one workspace of fixed size; fewer splits where it
    # would not suffice
    most = max(1, (workspace_floats - n) // (n * n_heads * (head_dim + 2)))
    n_splits, tile_splits = min(n_splits, most), min(tile_splits, most)
    stride = max(n_splits, tile_splits)
    ml_offset = n * n_heads * stride * head_dim
    rs_offset = n * n_heads * stride * (head_dim + 2)
    return AttentionLaunch(n_splits, min_steps, tile_splits, tile_max_steps, stride, ml_offset, rs_offset,
                           rs_offset + n if stride > 1 else 0)


_side_streams = {}


def _side_stream(device_index: int):
    """The device's second stream (default priority), on which the attention library runs a step's tiles beside its
    items. One per device for the life of the process: the library keeps its handle."""
    s = _side_streams.get(device_index)
    if s is None:
        s = _side_streams[device_index] = torch.cuda.Stream(torch.device("cuda", device_index))
    return s


def _rows_view(t: torch.Tensor, what: str):
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what}: expected a 2-d tensor with unit column stride, got shape {tuple(t.shape)} "
                          f"strides {t.stride()}")
    return t


class HipOps:
    """The operations of one engine instance: a device, a compute dtype, and the kernels for them."""
    supports_graphs = True      # every launch goes to torch's current stream, so a stream capture records it

    def __init__(self, device="cuda:0", dtype=torch.bfloat16):
        if dtype not in _DT:
            raise KernelError(f"unsupported compute dtype {dtype}; use torch.bfloat16 or torch.float32")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: this engine runs on HIP kernels only and has no CPU path")
        self.device = torch.device(device)
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.dtype = dtype
        self.code = _DT[dtype]
        # whatever is not built yet is compiled side by side, not one after the other
        _build.build(["rowwise", "rope_cache", "attention_generic", "gemm_plain", "sampling"] +
                     (["gemm_skinny", "gemm_library", "gemm_tiles"] if dtype == torch.bfloat16 else []))
        self.rowwise = library("rowwise")
        self.rope = library("rope_cache")
        self.attn_generic = library("attention_generic")
        self.gemm_plain = library("gemm_plain")
        self.sampling = library("sampling")
        self.gemm_skinny = library("gemm_skinny") if dtype == torch.bfloat16 else None
        self.gemm_library = None
        self.few_rows = _FEW_ROWS
        self.library_widths = library_widths()
        self._warned_widths = set()
        # compute units of this device: what the attention planner spreads waves over
        self.units = int(torch.cuda.get_device_properties(self.device).multi_processor_count) or _CHIP_UNITS
        if dtype == torch.bfloat16:
            self.gemm_skinny.cdll.tis_gemm_skinny_units(self.units)
            self.gemm_tiles = library("gemm_tiles")
            self.gemm_tiles.cdll.tis_gemm_tiles_units(self.units)
            self.gemm_library = library("gemm_library")
            with torch.cuda.device(self.device):
                self.gemm_library.tis_gemm_library_init()
        self._attn_mfma = {}               # head size -> library
        # partial results of split key ranges: one buffer of fixed size that never moves (captured graphs hold its address)
        self._workspace = torch.empty(_ATTN_WORKSPACE_FLOATS, dtype=torch.float32, device=self.device) \
            if dtype == torch.bfloat16 else None

    # ---- planning on the host --------------------------------------------------------------------------
    def plan_attention_mode(self, seq_rows, window: int = 0):
        """What kind of plan a step gets, from its first stage's rows: two steps may share a captured graph only if
        this is equal. "uneven": single rows of requests that differ widely in length (in what a row sees of its
        request, where the mixer has a window)."""
        return "uneven" if self.dtype == torch.bfloat16 and uneven_lengths(seq_rows, window) else None

    def plan_attention(self, n_heads: int, n_kv_heads: int, head_dim: int, seq_rows, add, mode=None, window: int = 0):
        """An attention mixer's host planning, called while a step's arrays are packed: the work items of the
        matrix-core kernels for the step's rows. Returns {name: (packed array id, host values...)}."""
        plans = {}
        if self.dtype == torch.bfloat16:
            group, cols = n_heads // n_kv_heads, tile_columns(head_dim)
            if (mode == "uneven" and group <= 64 and planned_list_pays(len(seq_rows), n_kv_heads)
                    and all(n == 1 for _, _, n in seq_rows)):
                entries, most = decode_items(seq_rows, n_heads, n_kv_heads, head_dim, window=window, units=self.units)
                return {("attention_decode_items", group, cols, n_kv_heads, window): (add(entries), len(entries), most)}
            nb, items, tiles, steps = attention_items(seq_rows, group, cols, n_kv_heads)
            beside = planned_beside_tiles(seq_rows, items, tiles, steps, n_heads, n_kv_heads, head_dim, window, self.units)
            if beside is not None:
                # one array: the planned entries of four integers, then the tiles' lines of two
                entries, most = beside
                plans[("attention_items", group, cols, n_kv_heads, window)] = (
                    add(np.concatenate((entries.reshape(-1), tiles.reshape(-1)))), len(entries), 1, len(tiles), steps, most)
            elif nb <= 4 and (len(items) or len(tiles)):
                # one array: the items' lines, then the tiles'
                # (a mixer with a window plans for itself: its lists are the same, its keys are its own)
                plans[("attention_items", group, cols, n_kv_heads, window)] = (add(np.concatenate((items, tiles))), len(items),
                                                                       nb, len(tiles), steps, 0)
        return plans

    # ---- helpers -------------------------------------------------------------------------------------
    def _stream(self):
        # torch's current stream of the device (under a graph capture: the capturing stream), by the short way:
        # a kernel launch asks for it, and the public accessor builds a stream object each time (4 us)
        return c_void_p(torch._C._cuda_getCurrentRawStream(self._device_index))

    def _check(self, t: torch.Tensor, what: str, dtype=None):
        dtype = dtype or self.dtype
        if t.device != self.device and not (t.device.type == self.device.type and
                                            (t.device.index or 0) == (self.device.index or 0)):
            raise KernelError(f"{what}: tensor is on {t.device}, engine on {self.device}")
        if t.dtype != dtype:
            raise KernelError(f"{what}: dtype {t.dtype}, expected {dtype}")
        return t

    def _index(self, t: torch.Tensor, what: str, n: Optional[int] = None):
        self._check(t, what, torch.int32)
        if not t.is_contiguous():
            raise KernelError(f"{what}: index tensor must be contiguous")
        if n is not None and t.numel() < n:
            raise KernelError(f"{what}: {t.numel()} entries for {n} rows")
        return t

    def empty(self, *shape, dtype=None):
        """An uninitialised tensor. Rows of bfloat16 activations that may go into the library's product are allocated
        up to the row count the library is asked for (library_rows), so that the product can run on them as they
        lie; the tensor that comes back shows the rows asked for."""
        dtype = dtype or self.dtype
        if len(shape) == 2 and dtype == torch.bfloat16 and shape[0] > self.few_rows:
            rows = library_rows(shape[0])
            if rows != shape[0]:
                return torch.empty(rows, shape[1], dtype=dtype, device=self.device)[:shape[0]]
        return torch.empty(*shape, dtype=dtype, device=self.device)

    # ---- row-wise ------------------------------------------------------------------------------------
    def embedding(self, table, tokens, out=None):
        self._check(table, "embedding table")
        n = tokens.numel()
        self._index(tokens, "tokens")
        D = table.shape[1]
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "embedding out"), "embedding out")
        if out.shape[0] < n or out.shape[1] != D or not table.is_contiguous():
            raise KernelError(f"embedding: out {tuple(out.shape)} does not fit {n} rows of {D}")
        self.rowwise.tis_embedding(self.code, _ptr(table), _ptr(tokens), _ptr(out), out.stride(0), n, D,
                                   self._stream())
        return out

    def rmsnorm(self, x, gain, eps: float, out=None):
        _rows_view(self._check(x, "rmsnorm x"), "rmsnorm x")
        self._check(gain, "rmsnorm gain", torch.float32)
        n, D = x.shape
        if gain.numel() != D or not gain.is_contiguous():
            raise KernelError(f"rmsnorm: gain has {gain.numel()} entries for width {D}")
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "rmsnorm out"), "rmsnorm out")
        if tuple(out.shape) != (n, D):
            raise KernelError(f"rmsnorm: out {tuple(out.shape)} vs x {tuple(x.shape)}")
        self.rowwise.tis_rmsnorm(self.code, _ptr(x), x.stride(0), _ptr(gain), _ptr(out), out.stride(0), n, D,
                                 float(eps), self._stream())
        return out

    def embedding_rmsnorm(self, table, tokens, gain, eps: float, out=None):
        self._check(table, "embedding table")
        self._check(gain, "rmsnorm gain", torch.float32)
        self._index(tokens, "tokens")
        n, D = tokens.numel(), table.shape[1]
        if gain.numel() != D or not gain.is_contiguous() or not table.is_contiguous():
            raise KernelError(f"embedding_rmsnorm: gain has {gain.numel()} entries for width {D}")
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "embedding_rmsnorm out"), "embedding_rmsnorm out")
        if out.shape[0] < n or out.shape[1] != D:
            raise KernelError(f"embedding_rmsnorm: out {tuple(out.shape)} does not fit {n} rows of {D}")
        self.rowwise.tis_embedding_rmsnorm(self.code, _ptr(table), _ptr(tokens), _ptr(gain), _ptr(out),
                                           out.stride(0), n, D, float(eps), self._stream())
        return out

    def gather_rows(self, src, state, index, out=None):
        """out[r] = src[index[r]] if index[r] >= 0 else state[-index[r]-1]."""
        _rows_view(self._check(src, "gather src"), "gather src")
        _rows_view(self._check(state, "gather state"), "gather state")
        n = index.numel()
        self._index(index, "gather index")
        D = src.shape[1]
        if state.shape[1] != D:
            raise KernelError(f"gather_rows: src width {D}, state width {state.shape[1]}")
        if out is None:
            out = self.empty(n, D)
        _rows_view(self._check(out, "gather out"), "gather out")
        if out.shape[0] < n or out.shape[1] != D:
            raise KernelError(f"gather_rows: out {tuple(out.shape)} does not fit {n} rows of {D}")
        self.rowwise.tis_gather_rows(self.code, _ptr(src), src.stride(0), _ptr(state), state.stride(0), _ptr(index),
                                     _ptr(out), out.stride(0), n, D, self._stream())
        return out

    def copy_rows(self, src, src_index, dst, dst_index):
        """dst[dst_index[i]] = src[src_index[i]]."""
        _rows_view(self._check(src, "copy src"), "copy src")
        _rows_view(self._check(dst, "copy dst"), "copy dst")
        n = src_index.numel()
        self._index(src_index, "copy src_index")
        self._index(dst_index, "copy dst_index", n)
        if src.shape[1] != dst.shape[1]:
            raise KernelError(f"copy_rows: widths {src.shape[1]} and {dst.shape[1]}")
        self.rowwise.tis_copy_rows(self.code, _ptr(src), src.stride(0), _ptr(src_index), _ptr(dst), dst.stride(0),
                                   _ptr(dst_index), n, src.shape[1], self._stream())

    def swiglu(self, gu, out=None):
        """out[:, f] = silu(gu[:, 2f]) * gu[:, 2f + 1]: gate and up columns interleaved."""
        _rows_view(self._check(gu, "swiglu in"), "swiglu in")
        n, F2 = gu.shape
        if F2 % 2:
            raise KernelError(f"swiglu: input width {F2} is odd")
        F = F2 // 2
        if out is None:
            out = self.empty(n, F)
        _rows_view(self._check(out, "swiglu out"), "swiglu out")
        if tuple(out.shape) != (n, F):
            raise KernelError(f"swiglu: out {tuple(out.shape)} for {n} rows of {F}")
        self.rowwise.tis_swiglu(self.code, _ptr(gu), gu.stride(0), _ptr(out), out.stride(0), n, F, self._stream())
        return out

    # ---- matrix products -----------------------------------------------------------------------------
    def linear(self, x, w, residual=None, out_dtype=None, rms=None, reuse_residual=False):
        """f(x)[M,K] . w[N,K]^T (+ residual[M,N]); `out_dtype` float32 gives 32-bit results from bfloat16 inputs.

        rms = (gain, eps): f is the RMSNorm of the rows, fused into the product where the kernel allows.
        reuse_residual: the caller has no further use for `residual`; an operations object may then write the result
        over it. This one never does: every product's result has memory of its own.
        """
        _rows_view(self._check(x, "linear x"), "linear x")
        self._check(w, "linear w")
        out_dtype = out_dtype or self.dtype
        M, K = x.shape
        if w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
            raise KernelError(f"linear: x {tuple(x.shape)} against w {tuple(w.shape)} (w is [out, in], contiguous)")
        N = w.shape[0]
        if residual is not None:
            _rows_view(self._check(residual, "linear residual", out_dtype), "linear residual")
            if tuple(residual.shape) != (M, N):
                raise KernelError(f"linear: residual {tuple(residual.shape)} for result {(M, N)}")
        if rms is not None:
            self._check(rms[0], "rmsnorm gain", torch.float32)
            if rms[0].numel() != K or not rms[0].is_contiguous():
                raise KernelError(f"linear: norm gain has {rms[0].numel()} entries for width {K}")
        if self.dtype == torch.float32:
            if rms is not None:
                x = self.rmsnorm(x, rms[0], rms[1])
            out = self.empty(M, N, dtype=torch.float32)
            self.gemm_plain.tis_gemm_plain(0, 0, _ptr(x), x.stride(0), _ptr(w), K, _ptr(residual),
                                           residual.stride(0) if residual is not None else 0, _ptr(out), N, M, N, K,
                                           self._stream())
            return out
        route = self._route(x, M, N, K, out_dtype, residual)
        if route == "few_rows":
            out = self.empty(M, N, dtype=out_dtype)
            if out_dtype == torch.float32 and residual is not None:
                raise KernelError("linear: a 32-bit result of bfloat16 operands takes no residual")
            self.gemm_skinny.tis_gemm_skinny(
                _ptr(x), x.stride(0), _ptr(w), _ptr(rms[0] if rms else None), float(rms[1]) if rms else 0.0,
                _ptr(residual), residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0), M, N, K,
                1 if residual is not None else 0, _DT[out_dtype], self._stream())
            return out
        if rms is not None:
            x = self.rmsnorm(x, rms[0], rms[1])
        if route == "library":
            return self._linear_library(x, w, residual)
        if route == "tiles":
            if out_dtype == torch.float32 and residual is not None:
                raise KernelError("linear: a 32-bit result of bfloat16 operands takes no residual")
            out = self.empty(M, N, dtype=out_dtype)
            self.gemm_tiles.tis_gemm_tiles(_ptr(x), x.stride(0), _ptr(w), _ptr(residual),
                                           residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0),
                                           M, N, K, 1 if out_dtype == torch.float32 else 0, self._stream())
            return out
        out = self.empty(M, N, dtype=out_dtype)
        self.gemm_plain.tis_gemm_plain(1, _DT[out_dtype], _ptr(x), x.stride(0), _ptr(w), K, _ptr(residual),
                                       residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0), M, N,
                                       K, self._stream())
        return out

    def _route(self, x, M, N, K, out_dtype=None, residual=None):
        """Which kernel takes this bfloat16 product (see product_route); says once per width that a product of many
        rows runs on the few-row kernel because the library's list does not hold its widths."""
        aligned = K % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
        route = product_route(M, N, K, aligned, out_dtype == torch.float32, self.library_widths, self.few_rows)
        if route == "library" and residual is not None and (residual.stride(0) % 8 or residual.data_ptr() % 16):
            route = "few_rows"
        if route == "tiles" and residual is not None and (residual.stride(0) % 4 or residual.data_ptr() % 8):
            route = "few_rows"
        if route == "few_rows" and M > 8 * self.few_rows and (N, K) not in self._warned_widths \
                and out_dtype != torch.float32:
            self._warned_widths.add((N, K))
            print(f"[tis-amd] a product of {M} rows with {N} output and {K} input columns runs on the few-row kernel: "
                  f"these widths are not in {os.path.basename(_WIDTHS_FILE)} (the widths the library's product has "
                  f"been tested at)", file=__import__("sys").stderr, flush=True)
        return route

    def _few_rows_ok(self, x, M, N, K):
        return self.dtype == torch.bfloat16 and M > 0 and self._route(x, M, N, K) == "few_rows"

    def linear_swiglu(self, x, w, rms=None):
        """silu(g) * u of the rows of f(x) . w^T, w holding gate and up rows interleaved: [M, N/2]."""
        _rows_view(self._check(x, "linear x"), "linear x")
        M, K = x.shape
        if w.dim() == 2 and w.shape[0] % 2 == 0 and self._few_rows_ok(x, M, w.shape[0], K):
            self._check(w, "linear w")
            if w.shape[1] != K or not w.is_contiguous():
                raise KernelError(f"linear: x {tuple(x.shape)} against w {tuple(w.shape)} (w is [out, in], contiguous)")
            if rms is not None and (rms[0].numel() != K or rms[0].dtype != torch.float32):
                raise KernelError(f"linear: norm gain has {rms[0].numel()} entries for width {K}")
            N = w.shape[0]
            out = self.empty(M, N // 2)
            self.gemm_skinny.tis_gemm_skinny(
                _ptr(x), x.stride(0), _ptr(w), _ptr(rms[0] if rms else None), float(rms[1]) if rms else 0.0,
                _ptr(None), 0, _ptr(out), out.stride(0), M, N, K, 2, 1, self._stream())
            return out
        return self.swiglu(self.linear(x, w, rms=rms))

    @staticmethod
    def _holds_rows(t, rows: int) -> bool:
        """Whether `rows` rows of t's stride lie inside the memory behind t."""
        last = t.storage_offset() + (rows - 1) * t.stride(0) + t.shape[1]
        return last * t.element_size() <= t.untyped_storage().nbytes()

    def _with_rows(self, t, rows: int):
        """t itself if the memory behind it holds `rows` rows (tensors from `empty` do), else a copy that does."""
        if self._holds_rows(t, rows):
            return t
        c = self.empty(t.shape[0], t.shape[1], dtype=t.dtype)
        c.copy_(t)
        return c

    def _linear_library(self, x, w, residual):
        """The library's product for many rows (reference main_models_new.py:19-20 uses one too), asked at
        library_rows(M) rows: the operands' memory reaches that far, and the rows beyond M are not looked at again.
        The result has memory of its own, also where the caller has no further use for the residual."""
        M, K = x.shape
        N = w.shape[0]
        rows = library_rows(M)
        if (N, K) not in self.library_widths:
            raise KernelError(f"linear: widths ({N}, {K}) are not among those the library's product is used at")
        x = self._with_rows(x, rows)
        if residual is not None:
            residual = self._with_rows(residual, rows)
        out = self.empty(M, N)
        if not self._holds_rows(out, rows):
            raise KernelError(f"linear: the result of {M} rows has no room for {rows}")
        self.gemm_library.tis_gemm_library(_ptr(x), x.stride(0), _ptr(w), _ptr(residual),
                                           residual.stride(0) if residual is not None else 0, _ptr(out), out.stride(0),
                                           rows, N, K, 0, self._stream())
        return out

    # ---- position encoding + cache write, attention --------------------------------------------------
    def rope_write_kv(self, qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                      interleaved=False, write_cache=True, paired=False, q_out=None):
        """Rotate q (in place, or into `q_out`) and write rotated k and v into the cache plane.

        paired: the q and k heads of `qkv` hold the members of each rotary pair side by side (pair j at columns
        2j, 2j+1), as a projection with pair-ordered weight rows leaves them; `q_out` then receives the queries
        in natural order.
        """
        _rows_view(self._check(qkv, "qkv"), "qkv")
        if paired and q_out is None:
            raise KernelError("rope_write_kv: paired input needs q_out")
        if q_out is not None:
            _rows_view(self._check(q_out, "q_out"), "q_out")
            if tuple(q_out.shape) != (qkv.shape[0], n_heads * head_dim):
                raise KernelError(f"rope_write_kv: q_out {tuple(q_out.shape)} for {qkv.shape[0]} rows of {n_heads * head_dim}")
        n = qkv.shape[0]
        if qkv.shape[1] != (n_heads + 2 * n_kv_heads) * head_dim:
            raise KernelError(f"rope_write_kv: row width {qkv.shape[1]} is not (heads {n_heads} + 2 x kv heads "
                              f"{n_kv_heads}) x head size {head_dim}")
        self._index(positions, "positions", n)
        if table is not None:
            self._check(table, "rotary table", torch.float32)
            if table.dim() != 3 or table.shape[1] != head_dim // 2 or table.shape[2] != 2 or not table.is_contiguous():
                raise KernelError(f"rope_write_kv: table {tuple(table.shape)} for head size {head_dim}")
        if write_cache:
            self._index(write_slots, "write_slots", n)
            self._check_plane(plane, n_kv_heads, head_dim, page_size)
        self.rope.tis_rope_write_kv(self.code, _ptr(qkv), qkv.stride(0), _ptr(positions),
                                    _ptr(write_slots if write_cache else None), _ptr(table),
                                    _ptr(plane if write_cache else None), n, n_heads, n_kv_heads, head_dim, page_size,
                                    int(bool(interleaved)), int(bool(write_cache)), int(bool(paired)), _ptr(q_out),
                                    q_out.stride(0) if q_out is not None else 0, self._stream())

    def qkv_rope(self, x, w, rms, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                 interleaved=False, write_cache=True):
        """Queries [rows, heads*head_dim], rotated, of f(x) . w^T; rotated keys and values go into the cache plane.

        w: [(heads + 2 kv heads) * head_dim, K] with the rows of every q and k head in pair order. For few rows in
        bfloat16 this is one kernel; otherwise the projection followed by the rotary/cache-write kernel.
        """
        _rows_view(self._check(x, "qkv x"), "qkv x")
        self._check(w, "qkv w")
        M, K = x.shape
        N = (n_heads + 2 * n_kv_heads) * head_dim
        if w.dim() != 2 or tuple(w.shape) != (N, K) or not w.is_contiguous():
            raise KernelError(f"qkv_rope: w {tuple(w.shape)} is not [{N}, {K}] contiguous")
        if self._few_rows_ok(x, M, N, K) and head_dim % 4 == 0:
            self._index(positions, "positions", M)
            if table is not None:
                self._check(table, "rotary table", torch.float32)
                if table.dim() != 3 or table.shape[1] != head_dim // 2 or table.shape[2] != 2 or not table.is_contiguous():
                    raise KernelError(f"qkv_rope: table {tuple(table.shape)} for head size {head_dim}")
            if write_cache:
                self._index(write_slots, "write_slots", M)
                self._check_plane(plane, n_kv_heads, head_dim, page_size)
            if rms is not None and (rms[0].numel() != K or rms[0].dtype != torch.float32):
                raise KernelError(f"qkv_rope: norm gain has {rms[0].numel()} entries for width {K}")
            q = self.empty(M, n_heads * head_dim)
            self.gemm_skinny.tis_gemm_skinny_qkv_rope(
                _ptr(x), x.stride(0), _ptr(w), _ptr(rms[0] if rms else None), float(rms[1]) if rms else 0.0, _ptr(q),
                q.stride(0), M, K, _ptr(positions), _ptr(write_slots if write_cache else None), _ptr(table),
                _ptr(plane if write_cache else None), n_heads, n_kv_heads, head_dim, page_size,
                int(bool(interleaved)), int(bool(write_cache)), self._stream())
            return q
        qkv = self.linear(x, w, rms=rms)
        q = self.empty(M, n_heads * head_dim)
        self.rope_write_kv(qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                           interleaved, write_cache, paired=True, q_out=q)
        return q

    def _check_plane(self, plane, n_kv_heads, head_dim, page_size):
        self._check(plane, "cache plane")
        if plane.dim() != 5 or tuple(plane.shape[1:]) != (2, n_kv_heads, page_size, head_dim) or \
                not plane.is_contiguous():
            raise KernelError(f"cache plane {tuple(plane.shape)} is not [pages, 2, {n_kv_heads}, {page_size}, "
                              f"{head_dim}] contiguous")

    def paged_attention(self, q, plane, batch, group, n_heads, n_kv_heads, head_dim, window=0, scale=None,
                        slopes=None):
        """Attention of the rows in `batch` over the cache plane; `q` is [rows, heads*head_dim] (a strided view is fine).

        `batch` brings positions, row_seq and the group's block tables; `group` names the page group. `slopes`
        ([heads] 32-bit, or None): a bias slope[h] * (key position - row position) on the scores; such calls go to
        the general kernel.
        """
        _rows_view(self._check(q, "q"), "q")
        n = q.shape[0]
        page_size = plane.shape[3]
        self._check_plane(plane, n_kv_heads, head_dim, page_size)
        if q.shape[1] != n_heads * head_dim:
            raise KernelError(f"attention: q width {q.shape[1]} is not heads {n_heads} x head size {head_dim}")
        tables = batch.block_tables[group]
        self._check(tables, "block tables", torch.int32)
        if tables.dim() != 2 or tables.stride(1) != 1:
            raise KernelError(f"attention: block tables {tuple(tables.shape)} must be 2-d")
        self._index(batch.positions, "positions", n)
        self._index(batch.row_seq, "row_seq", n)
        if batch.max_kv_len > tables.shape[1] * page_size:
            raise KernelError(f"attention: a row sees {batch.max_kv_len} keys but block tables cover "
                              f"{tables.shape[1] * page_size}")
        if scale is None:
            scale = head_dim ** -0.5
        out = self.empty(n, n_heads * head_dim)
        if n == 0:
            return out
        group = n_heads // n_kv_heads
        if slopes is not None:
            self._check(slopes, "score slopes", torch.float32)
            if slopes.numel() != n_heads or not slopes.is_contiguous():
                raise KernelError(f"attention: {slopes.numel()} score slopes for {n_heads} heads")
        if (slopes is None and self.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256 and page_size % 16 == 0
                and group <= 64 and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0):
            cols = tile_columns(head_dim)
            planned = batch.extras.get(("attention_decode_items", group, cols, n_kv_heads, int(window)))
            plan = batch.extras.get(("attention_items", group, cols, n_kv_heads, int(window)))
            if planned is None and plan is None:
                # a caller that did not plan (a kernel test): plan now, tiles wherever they fit
                if uneven_lengths(batch.seq_rows, int(window)) and planned_list_pays(n, n_kv_heads):
                    entries, most = decode_items(batch.seq_rows, n_heads, n_kv_heads, head_dim, window=int(window),
                                                 units=self.units)
                    planned = (torch.from_numpy(entries).reshape(-1).to(self.device), len(entries), most)
                else:
                    nb, host_items, host_tiles, steps = attention_items(batch.seq_rows, group, cols)
                    beside = planned_beside_tiles(batch.seq_rows, host_items, host_tiles, steps, n_heads, n_kv_heads,
                                                  head_dim, int(window), self.units)
                    if beside is not None:
                        both = np.concatenate((beside[0].reshape(-1), host_tiles.reshape(-1)))
                        plan = (torch.from_numpy(np.ascontiguousarray(both)).to(self.device), len(beside[0]), 1,
                                len(host_tiles), steps, beside[1])
                    else:
                        both = np.ascontiguousarray(np.concatenate((host_items, host_tiles)))
                        plan = (torch.from_numpy(both).reshape(-1).to(self.device), len(host_items), nb, len(host_tiles),
                                steps, 0)
            planned_splits = 0
            if planned is not None:
                # single rows with splits planned row by row: one entry of four integers per wave
                lines, n_items, planned_splits = planned
                lines = lines.reshape(-1)
                if batch.max_seq_rows > 1 or lines.numel() != 4 * n_items:
                    raise KernelError(f"attention: a planned list of {lines.numel()} integers for {n_items} entries "
                                      f"of single rows ({batch.max_seq_rows} rows a request)")
                items, tiles, n_tiles, tile_steps, nb = lines, None, 0, (0, 0), 1
                while group > 16 * nb:
                    nb *= 2
            else:
                lines, n_items, nb, n_tiles, tile_steps, planned_splits = plan
                lines = lines.reshape(-1)
                width = 4 if planned_splits else 2      # a planned entry, or an item's (first row, rows)
                if lines.numel() < width * n_items + 2 * n_tiles:
                    raise KernelError(f"attention: the work list holds {lines.numel()} integers for {n_items} items "
                                      f"and {n_tiles} tiles")
                items = lines[:width * n_items] if n_items else None
                tiles = lines[width * n_items:] if n_tiles else None
                if planned_splits:
                    while group > 16 * nb:
                        nb *= 2
                elif batch.max_seq_rows <= 1 and n_items == n:
                    items = None        # single rows in order: the kernel needs no list
            lib = self._attn_mfma.get(head_dim)
            if lib is None:
                lib = self._attn_mfma[head_dim] = library(f"attention_mfma@{head_dim}")
                with torch.cuda.device(self.device):
                    lib.tis_attention_mfma_side_stream(c_void_p(_side_stream(self._device_index).cuda_stream))
                built = lib.cdll.tis_attention_mfma_tile_columns()
                if built != cols:
                    raise KernelError(f"attention: the kernel's tiles hold {built} columns a wave, the planner "
                                      f"assumes {cols}")
            single = items is None and n_tiles == 0
            lp = attention_launch_plan(n, n_items, n_tiles, tile_steps, single, batch.max_kv_len, n_heads, n_kv_heads,
                                       head_dim, planned_splits=planned_splits, units=self.units)
            n_splits, min_steps, tile_splits, tile_max_steps = lp.n_splits, lp.min_steps, lp.tile_splits, lp.tile_max_steps
            part_o = part_ml = row_splits = None
            if lp.stride > 1:
                if lp.need_floats > self._workspace.numel():
                    raise KernelError(f"attention: {lp.need_floats} floats of partial results for a workspace of "
                                      f"{self._workspace.numel()}")
                part_o = self._workspace
                part_ml = self._workspace[lp.ml_offset:]
                if lp.min_steps != 0 or n_tiles:
                    row_splits = self._workspace[lp.row_splits_offset:]
            if lines.dtype != torch.int32 or not lines.is_contiguous():
                raise KernelError("attention: the work list must be contiguous 32-bit integers")
            lib.tis_attention_mfma(_ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0),
                                   _ptr(batch.row_seq), _ptr(batch.positions), _ptr(items), n_items, nb, _ptr(tiles),
                                   n_tiles, _ptr(out), out.stride(0), _ptr(part_o), _ptr(part_ml), n, n_heads,
                                   n_kv_heads, head_dim, page_size, int(window), float(scale), n_splits, min_steps,
                                   tile_splits, tile_max_steps, _ptr(row_splits), self._stream())
            return out
        self.attn_generic.tis_attention_generic(
            self.code, _ptr(q), q.stride(0), _ptr(plane), _ptr(tables), tables.stride(0), _ptr(batch.row_seq),
            _ptr(batch.positions), _ptr(out), out.stride(0), n, n_heads, n_kv_heads, head_dim, page_size, int(window),
            float(scale), _ptr(slopes), self._stream())
        return out

    # ---- sampling ------------------------------------------------------------------------------------
    def argmax(self, logits):
        _rows_view(self._check(logits, "logits", torch.float32), "logits")
        n, V = logits.shape
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        self.sampling.tis_argmax(_ptr(logits), logits.stride(0), n, V, _ptr(out), self._stream())
        return out

    def sample(self, logits, temperature, top_k, top_p, rep_penalty, uniform, ctx_tokens=None, ctx_offsets=None,
               seen=None, seen_row=None):
        """One token per row of 32-bit logits; per-row parameters are device tensors of length rows.

        A request's context for the repetition penalty comes as a flat token list with offsets, or as `seen`, a
        [requests, vocab] byte table (nonzero: occurred) with `seen_row[i]` naming row i's line (-1: none); the
        kernel then also marks the token it draws.
        """
        _rows_view(self._check(logits, "logits", torch.float32), "logits")
        n, V = logits.shape
        for t, what, dt in ((temperature, "temperature", torch.float32), (top_p, "top_p", torch.float32),
                            (uniform, "uniform", torch.float32), (top_k, "top_k", torch.int32)):
            self._check(t, what, dt)
            if t.numel() != n or not t.is_contiguous():
                raise KernelError(f"sample: {what} has {t.numel()} entries for {n} rows")
        if rep_penalty is not None:
            self._check(rep_penalty, "rep_penalty", torch.float32)
            if rep_penalty.numel() != n:
                raise KernelError(f"sample: rep_penalty has {rep_penalty.numel()} entries for {n} rows")
        if ctx_tokens is not None:
            self._index(ctx_tokens, "ctx_tokens")
            self._index(ctx_offsets, "ctx_offsets", n + 1)
        if seen is not None:
            self._check(seen, "seen", torch.uint8)
            if seen.dim() != 2 or seen.shape[1] != V or seen.stride(1) != 1:
                raise KernelError(f"sample: seen {tuple(seen.shape)} is not [requests, {V}]")
            self._index(seen_row, "seen_row", n)
        work = torch.empty(n, V, dtype=torch.float32, device=self.device)
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        self.sampling.tis_sample(_ptr(logits), logits.stride(0), _ptr(work), n, V, _ptr(temperature), _ptr(top_k),
                                 _ptr(top_p), _ptr(rep_penalty), _ptr(ctx_tokens), _ptr(ctx_offsets), _ptr(uniform),
                                 _ptr(out), _ptr(seen), seen.stride(0) if seen is not None else 0,
                                 _ptr(seen_row if seen is not None else None), self._stream())
        return out
