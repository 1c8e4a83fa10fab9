"""The engine: a model, its cache, and the one step function that generation and replay both drive.

`step` takes a batch of (request, its next tokens): portions of prompts beside single decoded tokens,
cut anywhere. It runs only those tokens, as one batch, on top of what earlier steps left in the cache,
and returns 32-bit logits at the places asked for.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from collections import OrderedDict
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import architectures  # noqa: F401  (registers the built-in architectures)
from ..cache.manager import CacheManager, OutOfPages
from ..config.model_config import ARCHITECTURES, load_config
from ..weights.loader import load_tensors
from .batch import Entry, build_step_batch, first_stage_rows, materialize, plan_step_batch
from .model import Model

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


# Captured steps of single tokens: up to this many requests a step has its own shape, beyond it the next multiple of
# the step below (the filler lines cost a row of every product and a wave of attention over three keys each)
_EXACT_DECODE_SHAPES = 8
_DECODE_SHAPE_STEP = 8


def resolve_dtype(dtype):
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype {dtype!r}: use 'bfloat16' or 'float32'") from None


@dataclass
class StepOutput:
    logits: torch.Tensor                         # [wanted, vocab] float32, in the order of entries and want
    head_logits: Optional[List[torch.Tensor]]    # per prediction stage: [wanted, vocab]; rows not valid yet are NaN
    head_valid: Optional[List[List[bool]]]


class Engine:
    def __init__(self, model_dir: Optional[str] = None, *, config=None, tensors=None, dtype="bfloat16",
                 page_size: int = 16, max_tokens: Optional[int] = None, n_pages: Optional[int] = None,
                 pool_bytes: Optional[int] = None, max_requests: int = 64, device="cuda:0", ops=None,
                 use_graphs: bool = True, run_heads: bool = True):
        """The cache's size is given as tokens (`max_tokens`), pages (`n_pages`) or bytes (`pool_bytes`: as many
        pages as fit, whatever groups and planes the model's parts ask for)."""
        self.dtype = resolve_dtype(dtype)
        if model_dir is not None:
            config = load_config(model_dir)
        if config is None:
            raise ValueError("give a model folder or a configuration with tensors")
        self.config = config
        arch = ARCHITECTURES.get(config.architecture)
        self.spec = arch.build_spec(config)
        if tensors is None:
            if model_dir is None:
                raise ValueError("a configuration without a model folder needs its tensors")
            tensors = load_tensors(model_dir, self.spec)
        if ops is None:
            from ..ops.hip_ops import HipOps
            ops = HipOps(device, self.dtype)
        self.ops = ops
        self.device = ops.device
        # run_heads=False runs the first stage only, as the reference does with spec=False (server.py:118): the
        # prediction heads' weights are still loaded and checked, but they take no time and no cache
        self.run_spec = self.spec if run_heads else dataclasses.replace(self.spec, stages=self.spec.stages[:1])
        self.model = Model(self.run_spec, tensors, ops)
        if n_pages is None and pool_bytes is not None:
            per_page = CacheManager.page_bytes(self.model.cache_needs(), page_size, self.dtype)
            n_pages = max(1, int(pool_bytes) // per_page) if per_page else 1
        if n_pages is None:
            if max_tokens is None:
                if CacheManager.page_bytes(self.model.cache_needs(), page_size, self.dtype):
                    raise ValueError("give the cache's size as max_tokens, n_pages or pool_bytes")
                max_tokens = page_size          # no part keeps pages: the size is of no consequence
            n_pages = -(-int(max_tokens) // page_size)
        self.page_size = page_size
        # decode steps are replayed from captured graphs where the kernels allow it
        can = bool(use_graphs) and bool(getattr(ops, "supports_graphs", False))
        self.use_graphs = can and self.model.graph_safe                          # any step whose shape repeats
        self.use_decode_graphs = can and self.model.graph_safe_single_rows       # steps of single tokens
        # A captured step of single tokens has a fixed number of lines. Steps of nine requests and more are filled up
        # to the next multiple of eight with lines of a request of the cache manager's own (a token at a fixed
        # position, in a slot and a page beyond the ones that were asked for), so that a batch that shrinks request
        # by request meets a few shapes and not one per size.
        self.cache = CacheManager(self.model.cache_needs(), page_size, n_pages, max_requests, self.dtype, self.device,
                                  spare_positions=self.model.max_lag + 1 if self.use_decode_graphs else 0)
        self.max_requests = max_requests
        self.requests: Dict[Hashable, Tuple[int, int]] = {}      # id -> (slot, positions fed)
        # a slot is handed to request after request; what a captured step keeps about "the requests it holds" must
        # change when a slot changes hands, so every admission gets a number and a slot remembers its occupant's
        self._admissions = 0
        self._slot_admission: Dict[int, int] = {}
        if self.cache.spare_slot is not None:
            self._slot_admission[self.cache.spare_slot] = 0
        # an operations object without a device to capture on (a test's stand-in) may ask for the same host logic
        # with plain launches in place of replays
        self._capture_graphs = not getattr(ops, "emulates_graphs", False)
        self.graph_table_pages = 64          # block-table widths are rounded up to this many pages
        self._graphs: "OrderedDict[Tuple[int, int], object]" = OrderedDict()   # least recently used first
        # Each graph holds its step's activations; the least recently used one of its kind goes when there are more.
        # Steps of single tokens are small and a serving run meets one shape per number of live requests and table
        # width, so many of them are kept; other steps (prompt portions) hold a portion's activations each.
        self.max_graphs = 32
        self.max_decode_graphs = 192
        self._graph_seen: Dict[Tuple[int, int], int] = {}
        self._has_windows = any(g.spec.window > 0 for g in self.cache.groups.values())
        self.graph_replays = 0

    # ---- requests ------------------------------------------------------------------------------------
    def open(self, rid: Hashable) -> None:
        if rid in self.requests:
            raise ValueError(f"request {rid!r} is already live")
        slot = self.cache.open_request()
        self._admissions += 1
        self._slot_admission[slot] = self._admissions
        self.requests[rid] = (slot, 0)

    def close(self, rid: Hashable) -> None:
        slot, _ = self.requests.pop(rid)
        self._slot_admission.pop(slot, None)
        self.cache.close_request(slot)

    def _occupants(self, batch_entries):
        return tuple((e.slot, self._slot_admission[e.slot]) for e in batch_entries)

    def reserve(self, rid: Hashable, n_tokens: int) -> None:
        """Take now every page that `rid` needs to hold `n_tokens` positions (opening it if it is not live), the way
        the reference's static storage modes do at admission (server.py:163-166). All or nothing: OutOfPages."""
        opened = rid not in self.requests
        if opened:
            self.open(rid)
        slot, _ = self.requests[rid]
        n_tokens = min(int(n_tokens), self.spec.max_context)
        if not self.cache.can_grow({slot: n_tokens}):
            if opened:
                self.close(rid)
            raise OutOfPages(f"the cache cannot reserve {n_tokens} positions for request {rid!r}: free are "
                             f"{self.cache.free_pages()}")
        self.cache.grow(slot, n_tokens)

    def fed(self, rid: Hashable) -> int:
        return self.requests[rid][1]

    # Pages, as one number for whoever plans above the step function: every group has as many pages as every other,
    # so what binds is the group that needs the most. A model without paged groups (its mixers keep state of fixed
    # size only) needs none and never runs out.
    NO_PAGE_LIMIT = 1 << 40

    def pages_to_grow(self, rid: Hashable, n_tokens: int) -> int:
        """Most pages any group must take so that `rid` can be fed `n_tokens` more."""
        slot, fed = self.requests[rid]
        return max(self.cache.pages_needed(slot, fed + n_tokens).values(), default=0)

    def pages_to_hold(self, n_positions: int, step_positions: int = 0) -> int:
        """Most pages any group holds at a time for a request that grows to `n_positions`, fed at most
        `step_positions` a step (a window group gives pages back as it goes)."""
        return max(self.cache.pages_to_hold(n_positions, step_positions, self.model.max_lag).values(), default=0)

    def free_pages(self) -> int:
        return min(self.cache.free_pages().values(), default=self.NO_PAGE_LIMIT)

    def total_pages(self) -> int:
        return min(self.cache.total_pages().values(), default=self.NO_PAGE_LIMIT)

    # ---- the step ------------------------------------------------------------------------------------
    @torch.no_grad()
    def step(self, entries: Sequence[Tuple[Hashable, Sequence[int], Sequence[int]]], heads: bool = False) -> StepOutput:
        """entries: (request id, its next tokens, indices among them whose logits are wanted).

        A request that is not live yet is opened. Raises OutOfPages, before anything is run or taken, if
        the cache cannot hold the new tokens.
        """
        if not entries:
            raise ValueError("a step needs at least one entry")
        batch_entries = self._single_token_entries(entries)
        if batch_entries is None:
            batch_entries = self._checked_entries(entries)
        return self._run(entries, batch_entries, heads)

    def _single_token_entries(self, entries):
        """The step that serving is mostly made of: one token for each of some live requests. Returns its batch
        entries, pages taken, or None for any other step and for whatever is wrong with this one (the general path
        then says what). A request can only need a page when its next position opens one, so nothing is asked of the
        cache for the other fifteen of sixteen."""
        reqs, vocab, ctx, ps = self.requests, self.spec.vocab_size, self.spec.max_context, self.page_size
        out, opening, slots = [], {}, set()
        for rid, toks, want in entries:
            info = reqs.get(rid)
            if info is None or len(toks) != 1:
                return None
            t = toks[0]
            slot, fed = info
            if not isinstance(t, (int, np.integer)) or not (0 <= t < vocab) or fed >= ctx or slot in slots:
                return None
            slots.add(slot)
            if fed % ps == 0:
                opening[slot] = fed + 1
            out.append(Entry(slot, fed, [int(t)], list(want)))
        if opening:
            if not self.cache.can_grow(opening):
                return None
            for slot, n in opening.items():
                self.cache.grow(slot, n)
        return out

    def _checked_entries(self, entries):
        """Any step: its entries checked, new requests opened, pages taken for all of it or for none of it."""
        seen = set()
        arrays = {}
        for rid, toks, _ in entries:
            if rid in seen:
                raise ValueError(f"request {rid!r} appears twice in one step")
            seen.add(rid)
            if len(toks) == 0:
                raise ValueError(f"request {rid!r} brings no tokens")
            if len(toks) <= 16:          # a few decoded tokens: plain checks beat building an array
                for t in toks:
                    if not (0 <= int(t) < self.spec.vocab_size):
                        raise ValueError(f"token {t} of request {rid!r} is outside the vocabulary of {self.spec.vocab_size}")
                arrays[rid] = list(toks)
                continue
            arr = arrays[rid] = np.asarray(toks)
            if arr.dtype.kind not in "iu" or int(arr.min()) < 0 or int(arr.max()) >= self.spec.vocab_size:
                bad = [t for t in toks if not (isinstance(t, (int, np.integer)) and 0 <= int(t) < self.spec.vocab_size)]
                raise ValueError(f"token {bad[0] if bad else toks[0]!r} of request {rid!r} is outside the vocabulary "
                                 f"of {self.spec.vocab_size}")
        opened = []
        for rid, _, _ in entries:
            if rid not in self.requests:
                self.open(rid)
                opened.append(rid)
        wants = {self.requests[rid][0]: self.requests[rid][1] + len(toks) for rid, toks, _ in entries}
        too_long = [rid for rid, toks, _ in entries if self.requests[rid][1] + len(toks) > self.spec.max_context]
        if too_long or not self.cache.can_grow(wants):
            for rid in opened:
                self.close(rid)
            if too_long:
                raise ValueError(f"request {too_long[0]!r} would pass the model's context of {self.spec.max_context}")
            raise OutOfPages(f"the cache cannot take this step: it needs "
                             f"{ {g: sum(grp.pages_for(s, n) for s, n in wants.items()) for g, grp in self.cache.groups.items()} } "
                             f"pages, free are {self.cache.free_pages()}")
        batch_entries = []
        for rid, toks, want in entries:
            slot, fed = self.requests[rid]
            self.cache.grow(slot, fed + len(toks))
            batch_entries.append(Entry(slot, fed, arrays[rid], list(want)))
        return batch_entries

    def _run(self, entries, batch_entries, heads):
        logits = plan = None
        if self.use_decode_graphs and not heads:
            if all(len(e.tokens) == 1 and e.start >= self.model.max_lag and list(e.want) == [0] for e in batch_entries):
                logits = self._decode_step(batch_entries)
            elif self.use_graphs:
                logits, plan = self._repeated_step(batch_entries)
        if logits is None:
            if plan is not None:
                step = materialize(plan, self.device)
            else:
                step = build_step_batch(batch_entries, self.model.lags, self.model.reads_previous, self.cache,
                                        self.device, self.spec.max_context, self.model.plan_rows,
                                        mode=self.model.plan_mode(first_stage_rows(batch_entries)))
            outs = self.model.forward(step, self.cache)
        n = sum(len(e.want) for e in batch_entries)
        head_logits = head_valid = None
        if logits is None:
            if heads and len(outs) > 1:
                logits, head_logits, head_valid = self.model.logits_of_stages(outs, n)
            else:
                logits = self.logits_of(outs, step, n)
        windows = self._has_windows
        for (rid, _, _), e in zip(entries, batch_entries):
            fed = e.start + len(e.tokens)
            self.requests[rid] = (e.slot, fed)
            if windows:
                self.cache.release_behind(e.slot, fed, self.model.max_lag)
        return StepOutput(logits, head_logits, head_valid)

    def _sync(self):
        if torch.device(self.device).type == "cuda":
            torch.cuda.synchronize(self.device)

    def logits_of(self, outs, step, n):
        """32-bit logits [n, vocab] of the first stage's wanted rows."""
        if n:
            return self.model.logits(outs[0].hidden, step.stages[0].want_index, n)
        return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=self.device)

    def _make_room(self, of_kind, limit: int) -> None:
        """Drop the least recently used graphs of one kind until another fits under `limit`."""
        keys = [k for k in self._graphs if of_kind(k)]          # least recently used first
        while len(keys) >= max(1, limit):
            self._sync()              # no replay of the graph to be dropped is still running
            del self._graphs[keys.pop(0)]

    def _repeated_step(self, batch_entries):
        """Any other step whose shape has come before: the same requests' row counts, the same places wanted, the
        same work for the attention kernels (a batch of equal prompts, a benchmark's prefill). Returns (logits or
        None, the step's plan); from its third occurrence on a shape is replayed from a captured graph."""
        from .graph import DecodeGraph
        pages = max((max(len(g.tables[e.slot]) for e in batch_entries) for g in self.cache.groups.values()), default=1)
        width = -(-pages // self.graph_table_pages) * self.graph_table_pages
        plan = plan_step_batch(batch_entries, self.model.lags, self.model.reads_previous, self.cache,
                               self.spec.max_context, self.model.plan_rows, table_width=width,
                               mode=self.model.plan_mode(first_stage_rows(batch_entries)))
        # what the host decides from, beyond the arrays' shapes
        key = ("step", width, plan.layout(),
               tuple((pl["max_rows"], pl["keep_count"], pl["previous_rows"], tuple(pl["valid"])) for pl in plan.plans))
        graph = self._graphs.get(key)
        if graph is None:
            if len(self._graph_seen) > 4096:          # shapes that never came back
                self._graph_seen.clear()
            seen = self._graph_seen.get(key, 0)
            self._graph_seen[key] = seen + 1
            if seen < 2:
                return None, plan
            self._make_room(lambda k: k[0] == "step", self.max_graphs)
            graph = self._graphs[key] = DecodeGraph(self, plan, width * self.page_size, capture=self._capture_graphs)
        else:
            self._graphs.move_to_end(key)
        self.graph_replays += 1
        return graph.run(plan), plan

    def _decode_step(self, batch_entries):
        """A step of single tokens through a captured graph: logits [requests, vocab], valid until the next step."""
        from .graph import DecodeGraph
        pages = max((max(len(g.tables[e.slot]) for e in batch_entries) for g in self.cache.groups.values()), default=1)
        width = -(-pages // self.graph_table_pages) * self.graph_table_pages
        # (what the parts' planning says about the step, e.g. requests of very different lengths, changes the launches)
        mode = self.model.plan_mode(first_stage_rows(batch_entries))
        n_real = len(batch_entries)
        if n_real > _EXACT_DECODE_SHAPES and self.cache.spare_slot is not None:
            lines = -(-n_real // _DECODE_SHAPE_STEP) * _DECODE_SHAPE_STEP
            filler = Entry(self.cache.spare_slot, self.model.max_lag, [0], [0])
            batch_entries = list(batch_entries) + [filler] * (lines - n_real)
        key = (len(batch_entries), width, mode)
        graph = self._graphs.get(key)
        if graph is not None:
            self._graphs.move_to_end(key)
        occupants = self._occupants(batch_entries)
        if graph is not None and graph.holds(occupants):
            for e in batch_entries:
                if e.start + 1 > self.spec.max_context:
                    raise ValueError(f"request in slot {e.slot} would pass the model's context of {self.spec.max_context}")
            self.graph_replays += 1
            return graph.run_same_requests(batch_entries)[:n_real]
        plan = plan_step_batch(batch_entries, self.model.lags, self.model.reads_previous, self.cache,
                               self.spec.max_context, self.model.plan_rows, table_width=width, mode=mode)
        if graph is None:
            seen = self._graph_seen.get(key, 0)
            self._graph_seen[key] = seen + 1
            if seen == 0:
                # the first step of a shape runs as it is: it warms the library's choices for these shapes, so the
                # capture that follows records kernel launches only
                step = materialize(plan, self.device)
                for st in step.stages:
                    st.max_kv_len = width * self.page_size
                outs = self.model.forward(step, self.cache)
                return self.model.logits(outs[0].hidden, step.stages[0].want_index, len(batch_entries))[:n_real]
            self._make_room(lambda k: k[0] != "step", self.max_decode_graphs)
            graph = self._graphs[key] = DecodeGraph(self, plan, width * self.page_size, occupants,
                                                    capture=self._capture_graphs, mode=mode)
        self.graph_replays += 1
        return graph.run(plan, occupants)[:n_real]
