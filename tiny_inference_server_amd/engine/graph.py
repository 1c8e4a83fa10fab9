"""Captured steps.

A step in which every request brings exactly one token, far enough into its sequence that every stage has
one row per request, always launches the same kernels on arrays of the same shapes. Such a step is
captured once per (number of requests, block-table width) as a HIP graph over a fixed device buffer that
holds the step's integer arrays; later steps of the same shape copy their arrays into that buffer and
replay the graph, which removes the launch cost of several hundred small kernels. Any other step is captured
the same way once its exact shape (row counts, wanted places, attention work) has come three times.

Nothing is cleared inside the graph with a memset, and the first steps of a shape run without a graph (the
library chooses its algorithms for the shape then), so a capture records kernel launches only.
"""
from __future__ import annotations

import gc

import numpy as np
import torch

from .batch import StepPlan, materialize


class _NoEvent:
    """Stands in for a device event where copies are synchronous (a host-only run)."""

    def record(self):
        pass

    def synchronize(self):
        pass


class DecodeGraph:
    """One captured step: a fixed buffer of the step's integer arrays, and the graph that runs on it.

    occupants: for every entry of the plan something that names the request itself and not merely its slot
    (the engine passes (slot, admission number)); the quick update below is only right while the buffer's
    lines belong to the very same requests.
    capture=False records nothing: a replay then runs the same calls again on the same buffers. That is how an
    operations object without a device (a test's stand-in) exercises this file's host logic.
    """

    def __init__(self, engine, plan: StepPlan, kv_capacity: int, occupants=None, capture: bool = True, mode=None):
        self.layout = plan.layout()
        self.mode = mode
        self.engine = engine
        self.capture = capture
        dev = engine.device
        on_gpu = torch.device(dev).type == "cuda"
        self.host = torch.zeros(max(plan.packer.total, 4), dtype=torch.int32, pin_memory=on_gpu)
        self.dev = torch.zeros(max(plan.packer.total, 4), dtype=torch.int32, device=dev)
        self.copied = torch.cuda.Event() if on_gpu else _NoEvent()
        self.step = materialize(plan, dev, self.host, self.dev)
        for st in self.step.stages:          # later steps of the shape may see more keys than this one
            st.max_kv_len = kv_capacity
        self.graph = None
        if capture:
            self.graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize(dev)
            # No garbage collection while the stream is capturing: a collection may finalise an engine that is no
            # longer used (engines and their captured steps refer to each other, so only the collector frees them),
            # and destroying its graphs in the middle of a capture aborts the process. The context below collects
            # once before the capture begins.
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(self.graph):
                    self._launch()
            finally:
                if collecting:
                    gc.enable()
        self.copied.record()
        # what the quick update needs: which requests, in which order, the buffer holds, and where their arrays lie
        self.slots = tuple(e.slot for e in plan.entries)
        self.occupants = tuple(occupants) if occupants is not None else None
        self.cache = engine.cache
        self.page_size = engine.page_size
        off = lambda i: plan.packer.offsets[i][0]
        self.table_at = {g: (off(i), plan.packer.offsets[i][1]) for g, i in plan.bt_ids.items()}
        self.stage_at = [dict(lag=pl["lag"], tokens=off(pl["tokens"]), positions=off(pl["positions"]),
                              ws={g: off(i) for g, i in pl["ws"].items()}) for pl in plan.plans]
        self.pages_held = {g: np.array([len(engine.cache.groups[g].tables[s]) for s in self.slots])
                           for g in self.table_at}
        # what the parts planned for each stage (work lists of their kernels): where each array lies, in the order
        # the planning added them, and the host values that the captured launches were made from
        self.extras_at = [[(off(i), plan.packer.offsets[i][1]) for i in sorted(v[0] for v in pl["extra"].values())]
                          for pl in plan.plans]
        self.extras_host = [tuple(sorted((k, v[1:]) for k, v in pl["extra"].items())) for pl in plan.plans]
        self._ahead = None       # (positions the buffer was filled for ahead of time, requests still to be filled)

    def _launch(self):
        engine, n = self.engine, self.step.n_wanted
        outs = engine.model.forward(self.step, engine.cache)
        self.logits = engine.logits_of(outs, self.step, n)

    def _replay(self):
        if self.graph is not None:
            self.graph.replay()
        else:
            self._launch()

    def holds(self, occupants) -> bool:
        """Whether the buffer's lines are those of exactly these requests, in this order."""
        return self.occupants is not None and self.occupants == tuple(occupants)

    def run_same_requests(self, entries) -> torch.Tensor:
        """The next step of the very requests whose arrays the buffer already holds, in the same order: only
        tokens, positions, write slots and newly taken pages change, and those are written in place.

        Everything but the tokens depends on the requests' positions alone, and after a step of single tokens the
        likeliest next step is the same requests one position on. So once a step has been launched, while the GPU
        runs it (the caller cannot go on before it has the step's tokens anyway), the buffer is filled for that next
        step; when it comes, only its tokens, and the lines of requests that have taken a page since, are left to
        write before the copy and the replay."""
        self.copied.synchronize()
        flat = self.host.numpy()
        n = len(entries)
        starts = np.fromiter((e.start for e in entries), dtype=np.int64, count=n)
        tokens = np.fromiter((e.tokens[0] for e in entries), dtype=np.int32, count=n)
        ahead, self._ahead = self._ahead, None
        if ahead is not None and len(ahead[0]) == n and np.array_equal(ahead[0], starts):
            if len(ahead[1]):
                self._fill_positions(flat, starts, only=ahead[1])
        else:
            self._fill_positions(flat, starts)
        for st in self.stage_at:
            flat[st["tokens"]:st["tokens"] + n] = tokens
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        self._replay()
        # the buffer for the step after this one, while this one runs (the copy above has to have left the buffer)
        self.copied.synchronize()
        nxt = starts + 1
        if self.cache.spare_slot is not None:       # (lines that fill the step up stay where they are)
            nxt = nxt - np.fromiter((s == self.cache.spare_slot for s in self.slots), dtype=np.int64, count=n)
        self._ahead = (nxt, self._fill_positions(flat, nxt, ahead=True))
        return self.logits

    def _fill_positions(self, flat, starts, only=None, ahead=False):
        """Positions, write slots, newly taken pages and the parts' work lists for requests that stand at `starts`.
        only: the indices of the requests whose lines are to be written (the others' are right already).
        ahead: the step has not come yet, so a request whose position opens a page may not have that page; such
        requests are skipped and their indices returned, to be filled when the step comes."""
        n = len(starts)
        ps = self.page_size
        late = np.zeros(0, dtype=np.int64)
        for g, (t_off, (rows, width)) in self.table_at.items():
            tables = self.cache.groups[g].tables
            need = starts // ps + 1
            for k in np.nonzero(need > self.pages_held[g])[0]:
                t = tables[self.slots[k]]
                if len(t) < need[k]:
                    if not ahead:
                        raise RuntimeError("a request's position lies beyond its pages")
                    late = np.union1d(late, [k])
                    continue
                if len(t) > width:
                    raise RuntimeError("a block table outgrew the captured width")
                flat[t_off + k * width:t_off + k * width + len(t)] = [p if p >= 0 else 0 for p in t]
                self.pages_held[g][k] = len(t)
        which = np.arange(n) if only is None else np.asarray(only, dtype=np.int64)
        if ahead and len(late):
            which = np.setdiff1d(which, late)
        for st in self.stage_at:
            pos = starts[which] - st["lag"]
            flat[st["positions"] + which] = pos
            for g, w_off in st["ws"].items():
                t_off, (rows, width) = self.table_at[g]
                table = flat[t_off:t_off + rows * width].reshape(rows, width)
                flat[w_off + which] = table[which, pos // ps] * ps + pos % ps
        if only is None and any(self.extras_at):
            # the parts plan again for the new positions, into the places their arrays have in the buffer
            for at, host_values, st in zip(self.extras_at, self.extras_host, self.stage_at):
                slots_left = list(at)

                def put(arr, shape=None, slots_left=slots_left):
                    a = np.ascontiguousarray(arr, dtype=np.int32).reshape(-1)
                    if not slots_left or int(np.prod(slots_left[0][1])) != a.size:
                        raise RuntimeError("a part planned an array that the captured step has no place for")
                    o, _ = slots_left.pop(0)
                    flat[o:o + a.size] = a
                    return -1

                pos = starts - st["lag"]
                extra = self.engine.model.plan_rows([(k, int(pos[k]), 1) for k in range(n)], put, self.mode)
                if slots_left or tuple(sorted((k, v[1:]) for k, v in extra.items())) != host_values:
                    raise RuntimeError("the parts' planning no longer fits the captured step")
        return late

    def run(self, plan: StepPlan, occupants=None) -> torch.Tensor:
        if plan.layout() != self.layout:
            raise RuntimeError("this step's arrays do not have the captured layout")
        self.copied.synchronize()            # the previous copy out of the pinned buffer has finished
        self._ahead = None
        plan.packer.fill(self.host)
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        self.slots = tuple(e.slot for e in plan.entries)
        self.occupants = tuple(occupants) if occupants is not None else None
        for g in self.table_at:
            self.pages_held[g] = np.array([len(self.cache.groups[g].tables[s]) for s in self.slots])
        self._replay()
        return self.logits
