"""The rows of one step, as the kernels want them.

A step brings, for some live requests, their next tokens: a request that was fed positions [0, s) and
now brings n tokens contributes the rows of positions [s, s+n). A stage of lag j (stage 0 is the trunk)
runs, for the same entry, the positions [max(0, s-j), s+n-j): the same tokens, shifted. Every stage gets
its own row arrays; the block tables are the same for all stages because they describe the requests, not
the rows. All integer arrays of a step are packed into one host buffer and copied to the device once.

Per stage:
  tokens[r], positions[r]      the row's token and absolute position
  row_seq[r]                   index of the row's entry (its line in the block tables)
  cu_rows[k], cu_rows[k+1]     the rows of entry k
  write_slots[group][r]        page * page_size + offset where the row's key and value go
  source_index[r]              for stages that read the previous stage: its row index there, or -(slot+1)
                               for the row kept in the request's state slot
  keep_source[i], keep_slot[i] previous-stage rows to keep in state slots after the reads
  previous_rows                how many rows read the previous stage's rows of this step; with none, the stage
                               does not wait for the previous one
  want_index[i]                the rows whose outputs are asked for (-1 where this stage has no such row yet)
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch


@dataclass
class Entry:
    slot: int                  # request slot in the cache manager
    start: int                 # position of the first token
    tokens: Sequence[int]
    want: Sequence[int] = ()   # indices into `tokens`


@dataclass
class StageBatch:
    lag: int
    n_rows: int
    n_seqs: int
    tokens: torch.Tensor
    positions: torch.Tensor
    row_seq: torch.Tensor
    cu_rows: torch.Tensor
    seq_slots: torch.Tensor
    write_slots: Dict[str, torch.Tensor]
    block_tables: Dict[str, torch.Tensor]
    source_index: Optional[torch.Tensor]
    keep_source: Optional[torch.Tensor]
    keep_slot: Optional[torch.Tensor]
    keep_count: int
    previous_rows: int         # rows that read the previous stage's output of this very step (the others: state)
    want_index: torch.Tensor
    want_valid: List[bool]
    max_kv_len: int
    max_seq_rows: int
    seq_rows: List[Tuple[int, int, int]]      # host copy: (first row, first position, rows) per entry
    host_slots: List[int] = field(default_factory=list)       # host copy: state slot per entry
    extras: Dict[str, object] = field(default_factory=dict)   # what faster kernels plan on the host


@dataclass
class StepBatch:
    entries: List[Entry]
    stages: List[StageBatch]
    n_wanted: int


class _Packer:
    """Collects int32 arrays, uploads them in one copy, hands back device views."""

    def __init__(self):
        self.parts: List[np.ndarray] = []
        self.offsets: List[Tuple[int, Tuple[int, ...]]] = []
        self.total = 0

    def add(self, arr, shape=None) -> int:
        a = np.ascontiguousarray(arr, dtype=np.int32).reshape(-1)
        shape = tuple(shape) if shape is not None else (a.size,)
        self.parts.append(a)
        self.offsets.append((self.total, shape))
        self.total += (a.size + 3) // 4 * 4          # keep every array 16-byte aligned
        return len(self.offsets) - 1

    def layout(self):
        """What must be equal for two packings to share one device buffer."""
        return tuple(self.offsets)

    def fill(self, host: torch.Tensor) -> None:
        flat = host.numpy()
        for a, (off, _) in zip(self.parts, self.offsets):
            flat[off:off + a.size] = a

    def upload(self, device, host: Optional[torch.Tensor] = None, dev: Optional[torch.Tensor] = None):
        """Copy everything to the device in one transfer; `host` (pinned) and `dev` may be buffers to reuse."""
        if host is None:
            host = torch.zeros(max(self.total, 4), dtype=torch.int32,
                               pin_memory=(torch.device(device).type == "cuda"))
        self.fill(host)
        if dev is None:
            dev = host.to(device, non_blocking=True)
        else:
            dev.copy_(host, non_blocking=True)
        out = []
        for a, (off, shape) in zip(self.parts, self.offsets):
            out.append(dev[off:off + a.size].view(shape))
        return out


class StepPlan:
    """A step's arrays on the host, before they are copied to the device."""

    def __init__(self, entries, packer, bt_ids, slots_id, plans):
        self.entries, self.packer, self.bt_ids, self.slots_id, self.plans = entries, packer, bt_ids, slots_id, plans

    def layout(self):
        return (self.packer.layout(), tuple(pl["n_rows"] for pl in self.plans),
                tuple(tuple(sorted((k, v[1:]) for k, v in pl["extra"].items())) for pl in self.plans))


def build_step_batch(entries: Sequence[Entry], lags: Sequence[int], has_source: Sequence[bool], cache, device,
                     max_context: int, plan_rows=None, mode=None) -> StepBatch:
    """Row arrays for every stage of one step. `cache` is the CacheManager that already covers the new positions."""
    return materialize(plan_step_batch(entries, lags, has_source, cache, max_context, plan_rows, mode=mode), device)


def first_stage_rows(entries: Sequence[Entry]) -> List[Tuple[int, int, int]]:
    """(first row, first position, rows) per entry, as the first stage (lag 0) sees the step."""
    out, first = [], 0
    for e in entries:
        out.append((first, e.start, len(e.tokens)))
        first += len(e.tokens)
    return out


def plan_step_batch(entries: Sequence[Entry], lags: Sequence[int], has_source: Sequence[bool], cache,
                    max_context: int, plan_rows=None, table_width: Optional[int] = None, mode=None) -> StepPlan:
    """The host half: every array of the step, packed. `table_width` pads the block tables to a fixed width; `mode`
    is what the model's plan_mode said about the step and goes back to plan_rows with every stage's rows."""
    n_seqs = len(entries)
    pk = _Packer()
    page_size = cache.page_size

    # block tables: one line per entry, padded; shared by all stages
    bt_ids, tables = {}, {}
    for gname, g in cache.groups.items():
        lines = [g.line(e.slot) for e in entries]
        width = max(1, max(len(t) for t in lines))
        if table_width is not None:
            if width > table_width:
                raise ValueError(f"block tables of {width} pages do not fit the fixed width {table_width}")
            width = table_width
        tab = np.zeros((n_seqs, width), dtype=np.int32)
        for k, t in enumerate(lines):
            np.maximum(t, 0, out=tab[k, :len(t)], casting="unsafe")     # (-1: a page given back)
        tables[gname] = tab
        bt_ids[gname] = pk.add(tab, tab.shape)
    slots_id = pk.add([e.slot for e in entries])

    # everything below works on arrays over all entries at once: a step may hold hundreds of them
    starts = np.fromiter((e.start for e in entries), dtype=np.int64, count=n_seqs)
    n_toks = np.fromiter((len(e.tokens) for e in entries), dtype=np.int64, count=n_seqs)
    slots = np.fromiter((e.slot for e in entries), dtype=np.int64, count=n_seqs)
    ends = starts + n_toks
    if n_seqs and int(ends.max()) > max_context:
        k = int(np.argmax(ends))
        raise ValueError(f"request in slot {entries[k].slot} would reach position {int(ends[k]) - 1}, "
                         f"beyond the model's context of {max_context}")
    all_tokens = (np.concatenate([np.asarray(e.tokens, dtype=np.int64).reshape(-1) for e in entries])
                  if n_seqs else np.zeros(0, dtype=np.int64))
    tok_first = np.cumsum(n_toks) - n_toks                       # where an entry's tokens start in all_tokens
    for k, e in enumerate(entries):
        for i in e.want:
            if not (0 <= i < len(e.tokens)):
                raise ValueError(f"want index {i} is outside the entry's {len(e.tokens)} tokens")
    want_entry = np.fromiter((k for k, e in enumerate(entries) for _ in e.want), dtype=np.int64)
    want_at = np.fromiter((i for e in entries for i in e.want), dtype=np.int64)
    seq_index = np.arange(n_seqs)

    plans = []
    prev = None                 # the previous stage's (first rows, first positions, row counts)
    for j, lag in enumerate(lags):
        p0 = np.maximum(0, starts - lag)
        n = np.maximum(0, ends - lag - p0)
        first = np.cumsum(n) - n
        n_rows = int(n.sum())
        row_seq = np.repeat(seq_index, n)
        positions = np.arange(n_rows) - np.repeat(first - p0, n)
        # a stage that lags takes the last n of an entry's tokens
        tokens = all_tokens[np.repeat(tok_first + n_toks - n - p0, n) + positions]
        seq_rows = list(zip(first.tolist(), p0.tolist(), n.tolist()))
        source = keep_src = keep_slot = None
        if has_source[j]:
            pfirst, pp0, pn = prev
            # a row reads the previous stage's row at its position, or the request's kept row before the portion
            source = np.where(positions >= np.repeat(pp0, n), np.repeat(pfirst - pp0, n) + positions,
                              np.repeat(-(slots + 1), n))
            kept = pn > 0
            keep_src, keep_slot = (pfirst + pn - 1)[kept], slots[kept]
        ws = {}
        for gname in cache.groups:
            # (a new position never lies in a page that was given back, so the padded table serves)
            t = tables[gname]
            ws[gname] = pk.add(t[row_seq, positions // page_size].astype(np.int64) * page_size + positions % page_size)
        wp = starts[want_entry] + want_at - lag
        ok = (wp >= p0[want_entry]) & (n[want_entry] > 0)
        want = np.where(ok, first[want_entry] + wp - p0[want_entry], -1)
        extra = {}
        if plan_rows is not None:
            extra = plan_rows(seq_rows, pk.add, mode) if mode is not None else plan_rows(seq_rows, pk.add)
        live = n > 0
        plans.append(dict(
            extra=extra, lag=lag, n_rows=n_rows, tokens=pk.add(tokens), positions=pk.add(positions),
            row_seq=pk.add(row_seq), cu=pk.add(np.concatenate(([0], np.cumsum(n)))), ws=ws,
            source=pk.add(source) if has_source[j] else None,
            keep_src=pk.add(keep_src) if has_source[j] else None,
            keep_slot=pk.add(keep_slot) if has_source[j] else None,
            keep_count=int(len(keep_src)) if has_source[j] else 0,
            previous_rows=int((source >= 0).sum()) if has_source[j] else 0,
            want=pk.add(want), valid=ok.tolist(), seq_rows=seq_rows,
            max_kv=int((p0 + n)[live].max()) if live.any() else 0,
            max_rows=int(n.max()) if n_seqs else 0))
        prev = (first, p0, n)

    return StepPlan(list(entries), pk, bt_ids, slots_id, plans)


def materialize(plan: StepPlan, device, host: Optional[torch.Tensor] = None,
                dev_buffer: Optional[torch.Tensor] = None) -> StepBatch:
    """The device half: one copy, then views of the device buffer for every array."""
    entries, pk, bt_ids, slots_id, plans = plan.entries, plan.packer, plan.bt_ids, plan.slots_id, plan.plans
    n_seqs = len(entries)
    dev = pk.upload(device, host, dev_buffer)
    tables = {g: dev[i] for g, i in bt_ids.items()}
    stages = []
    for pl in plans:
        stages.append(StageBatch(
            lag=pl["lag"], n_rows=pl["n_rows"], n_seqs=n_seqs, tokens=dev[pl["tokens"]],
            positions=dev[pl["positions"]], row_seq=dev[pl["row_seq"]], cu_rows=dev[pl["cu"]],
            seq_slots=dev[slots_id], write_slots={g: dev[i] for g, i in pl["ws"].items()}, block_tables=tables,
            source_index=dev[pl["source"]] if pl["source"] is not None else None,
            keep_source=dev[pl["keep_src"]] if pl["keep_src"] is not None else None,
            keep_slot=dev[pl["keep_slot"]] if pl["keep_slot"] is not None else None,
            keep_count=pl["keep_count"], previous_rows=pl["previous_rows"], want_index=dev[pl["want"]], want_valid=pl["valid"],
            max_kv_len=pl["max_kv"], max_seq_rows=pl["max_rows"], seq_rows=pl["seq_rows"],
            host_slots=[e.slot for e in entries],
            extras={k: (dev[v[0]],) + tuple(v[1:]) for k, v in pl["extra"].items()}))
    return StepBatch(list(entries), stages, sum(len(e.want) for e in entries))
