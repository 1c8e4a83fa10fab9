"""The cache manager: pages of keys and values with a block table per request, and slots of fixed-size state.

Layers whose mixers keep keys and values fall into *groups* by what they need: the geometry of a key
(heads, head size) and whether all positions or only a window of them stay readable. A group has its own
pool of pages, its own free list and, for every live request, its own block table; all cache users of a
group share the request's page ids and differ in the plane they write (the reference keeps one page id
across all layers too: block_table.py:31-63). Pages come from a FIFO free list, are taken on demand as a
request grows, and go back when the request ends, when it is preempted, or, in a window group, when the
window has passed them. A page that comes back is handed out again as it is: kernels never read a slot
that the reader's length or window masks, so nothing is cleared.

Beside the pages every live request owns one *slot*: an index into per-request arrays of fixed size, one
array per part that declared such a need (the hidden row a prediction head keeps between steps lives
there). A slot's state is zeroed when the slot is taken.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Tuple

import numpy as np
import torch

from ..parts.spec import PagedKvNeed, StateNeed


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """A request asked for more pages than its group has free."""


class PagePool:
    """Page ids of one group: a FIFO free list with checks against losing a page or freeing one twice."""

    def __init__(self, n_pages: int):
        if n_pages < 1:
            raise CacheError(f"a page pool needs at least one page, got {n_pages}")
        self.n_pages = n_pages
        self._free = deque(range(n_pages))
        self._held = [False] * n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfPages("no free page")
        page = self._free.popleft()
        self._held[page] = True
        return page

    def give_back(self, page: int) -> None:
        if not (0 <= page < self.n_pages):
            raise CacheError(f"page id {page} is outside the pool of {self.n_pages}")
        if not self._held[page]:
            raise CacheError(f"page {page} was given back twice")
        self._held[page] = False
        self._free.append(page)

    def check(self) -> None:
        """Every page is either free once or held, never both, never lost."""
        free = list(self._free)
        free_set = set(free)
        if len(free_set) != len(free):
            raise CacheError("a page is on the free list twice")
        for p in range(self.n_pages):
            if self._held[p] == (p in free_set):
                raise CacheError(f"page {p} is {'both held and free' if self._held[p] else 'neither held nor free'}")


@dataclass
class GroupSpec:
    name: str
    n_kv_heads: int
    head_dim: int
    window: int                      # 0: every position stays readable
    keys: List[str] = field(default_factory=list)    # cache keys of the users, in plane order


class PageGroup:
    """One group: its pool, its planes of storage, and the block tables of the live requests."""

    def __init__(self, spec: GroupSpec, n_pages: int, page_size: int, dtype, device, allocate: bool = True):
        self.spec = spec
        self.page_size = page_size
        self.pool = PagePool(n_pages)
        self.plane_of = {k: i for i, k in enumerate(spec.keys)}
        self.tables: Dict[int, List[int]] = {}           # slot -> page id per page index, -1 once released
        self.released: Dict[int, int] = {}               # slot -> number of leading pages already given back
        self._lines: Dict[int, np.ndarray] = {}          # slot -> its table as an array, until the table changes
        self.storage = None
        if allocate:
            # [plane][page][key or value][kv head][slot in page][head size]; within a page and head the values
            # lie transposed, [head size][slot]. Zeroed once, as the reference does (block_table.py:40), though no
            # kernel needs it: slots that a row may not see are read, but replaced before any arithmetic
            self.storage = torch.zeros((len(spec.keys), n_pages, 2, spec.n_kv_heads, page_size, spec.head_dim),
                                       dtype=dtype, device=device)

    def plane(self, key: str):
        return self.storage[self.plane_of[key]]

    def held(self, slot: int) -> int:
        return sum(1 for p in self.tables.get(slot, ()) if p >= 0)

    def line(self, slot: int) -> np.ndarray:
        """The slot's table as an int64 array (read only: the same array comes back until the table changes)."""
        table = self.tables[slot]
        a = self._lines.get(slot)
        if a is None or len(a) != len(table):
            a = self._lines[slot] = np.asarray(table, dtype=np.int64)
        return a

    def pages_for(self, slot: int, n_positions: int) -> int:
        """Pages to take so that positions [0, n_positions) of `slot` are covered."""
        have = len(self.tables.get(slot, ()))
        return max(0, -(-n_positions // self.page_size) - have)

    def grow(self, slot: int, n_positions: int) -> None:
        table = self.tables[slot]
        need = self.pages_for(slot, n_positions)
        if need > self.pool.n_free:
            raise OutOfPages(f"group {self.spec.name!r}: request needs {need} more pages, {self.pool.n_free} are free")
        for _ in range(need):
            table.append(self.pool.take())
        if need:
            self._lines.pop(slot, None)

    def release_behind(self, slot: int, first_needed: int) -> int:
        """Window groups: give back the pages that lie wholly before the position `first_needed`."""
        if self.spec.window <= 0:
            return 0
        table = self.tables[slot]
        upto = min(len(table), max(0, first_needed) // self.page_size)
        done = self.released.get(slot, 0)
        for i in range(done, upto):
            self.pool.give_back(table[i])
            table[i] = -1
        if upto > done:
            self._lines.pop(slot, None)
        self.released[slot] = max(done, upto)
        return max(0, upto - done)

    def close(self, slot: int) -> None:
        for p in self.tables.pop(slot):
            if p >= 0:
                self.pool.give_back(p)
        self.released.pop(slot, None)
        self._lines.pop(slot, None)


class CacheManager:
    """Pages for every group and state slots for every state key, for up to `max_requests` live requests.

    needs: {cache key: PagedKvNeed | StateNeed}, as the model's parts declared them.
    n_pages: pages per group (every group gets as many: they all follow the same positions).
    """

    def __init__(self, needs: Mapping[str, object], page_size: int, n_pages: int, max_requests: int, dtype,
                 device, allocate: bool = True, spare_positions: int = 0):
        """spare_positions > 0: beside the `max_requests` slots and `n_pages` pages there is one request of the
        manager's own, live from the start with that many positions covered (`spare_slot`; its slot, state and pages
        come on top and are not counted by free_pages, total_pages and n_live): what a step of a fixed shape is
        filled up with when fewer requests come than the shape has lines."""
        if page_size < 1:
            raise CacheError(f"page size must be at least 1, got {page_size}")
        if max_requests < 1:
            raise CacheError(f"max_requests must be at least 1, got {max_requests}")
        self.page_size = page_size
        self.max_requests = max_requests
        self.spare_slot: Optional[int] = max_requests if spare_positions > 0 else None
        self._spare_pages = -(-spare_positions // page_size) if spare_positions > 0 else 0
        n_slots = max_requests + (1 if spare_positions > 0 else 0)
        n_pages = n_pages + self._spare_pages
        self.dtype, self.device = dtype, device
        specs: Dict[Tuple[int, int, int], GroupSpec] = {}
        self.group_of: Dict[str, str] = {}
        self.states: Dict[str, Optional[torch.Tensor]] = {}
        self._state_needs: Dict[str, StateNeed] = {}
        for key, need in needs.items():
            if isinstance(need, PagedKvNeed):
                geom = (need.n_kv_heads, need.head_dim, need.window)
                if geom not in specs:
                    name = f"kv{need.n_kv_heads}x{need.head_dim}" + (f"w{need.window}" if need.window else "")
                    specs[geom] = GroupSpec(name, need.n_kv_heads, need.head_dim, need.window)
                specs[geom].keys.append(key)
                self.group_of[key] = specs[geom].name
            elif isinstance(need, StateNeed):
                self._state_needs[key] = need
                self.states[key] = None
                if allocate:
                    dt = {"compute": dtype, "float32": torch.float32, "int32": torch.int32}[need.dtype]
                    self.states[key] = torch.zeros((n_slots,) + tuple(need.shape), dtype=dt, device=device)
            elif need is not None:
                raise CacheError(f"cache key {key!r}: unknown kind of need {need!r}")
        self.groups: Dict[str, PageGroup] = {
            s.name: PageGroup(s, n_pages, page_size, dtype, device, allocate) for s in specs.values()}
        self._free_slots = deque(range(max_requests))
        self._live: Dict[int, bool] = {}
        if self.spare_slot is not None:
            self._live[self.spare_slot] = True
            for g in self.groups.values():
                g.tables[self.spare_slot] = []
                g.grow(self.spare_slot, spare_positions)

    # ---- requests ------------------------------------------------------------------------------------
    @property
    def n_live(self) -> int:
        return len(self._live) - (1 if self.spare_slot is not None else 0)

    def open_request(self) -> int:
        if not self._free_slots:
            raise CacheError(f"all {self.max_requests} request slots are taken")
        slot = self._free_slots.popleft()
        self._live[slot] = True
        for g in self.groups.values():
            g.tables[slot] = []
        for key, t in self.states.items():
            if t is not None:
                t[slot].zero_()
        return slot

    def close_request(self, slot: int) -> None:
        if slot == self.spare_slot:
            raise CacheError("the spare request stays live as long as the manager")
        if slot not in self._live:
            raise CacheError(f"request slot {slot} is not live (closed twice?)")
        del self._live[slot]
        for g in self.groups.values():
            g.close(slot)
        self._free_slots.append(slot)

    # ---- pages ---------------------------------------------------------------------------------------
    def pages_needed(self, slot: int, n_positions: int) -> Dict[str, int]:
        return {name: g.pages_for(slot, n_positions) for name, g in self.groups.items()}

    def can_grow(self, wants: Mapping[int, int]) -> bool:
        """Whether all the requests in {slot: n_positions} can be covered together."""
        for name, g in self.groups.items():
            if sum(g.pages_for(s, n) for s, n in wants.items()) > g.pool.n_free:
                return False
        return True

    def grow(self, slot: int, n_positions: int) -> None:
        """Cover positions [0, n_positions) of `slot` in every group, or take nothing and raise OutOfPages."""
        if slot not in self._live:
            raise CacheError(f"request slot {slot} is not live")
        for name, g in self.groups.items():
            if g.pages_for(slot, n_positions) > g.pool.n_free:
                raise OutOfPages(f"group {name!r}: request needs {g.pages_for(slot, n_positions)} more pages, "
                                 f"{g.pool.n_free} are free")
        for g in self.groups.values():
            g.grow(slot, n_positions)

    def release_behind(self, slot: int, next_position: int, max_lag: int = 0) -> None:
        """Tell window groups that no row before `next_position - max_lag` will be run for `slot` again."""
        for g in self.groups.values():
            if g.spec.window > 0:
                g.release_behind(slot, next_position - max_lag - g.spec.window + 1)

    def pages_to_hold(self, n_positions: int, step_positions: int = 0, max_lag: int = 0) -> Dict[str, int]:
        """Pages of each group that a request holds at the most while it grows to `n_positions`, fed at most
        `step_positions` a step: every page of its positions, or, in a window group, the pages of a window, of the
        stages' lag and of one step's positions (what is released behind a step is released after it)."""
        out = {}
        for name, g in self.groups.items():
            pages = -(-n_positions // self.page_size)
            if g.spec.window > 0:
                span = g.spec.window + max_lag + max(1, step_positions or n_positions)
                pages = min(pages, -(-span // self.page_size) + 1)
            out[name] = pages
        return out

    @staticmethod
    def page_bytes(needs: Mapping[str, object], page_size: int, dtype) -> int:
        """Bytes that one more page costs: every group gets as many pages as every other, and a page of a group has
        a plane for each of the group's cache users (the reference's one geometry: block_table.py:34-38)."""
        elem = torch.empty(0, dtype=dtype).element_size()
        return sum(2 * need.n_kv_heads * need.head_dim * page_size * elem
                   for need in needs.values() if isinstance(need, PagedKvNeed))

    def bytes_per_position(self) -> int:
        """Bytes of keys and values that one position of one request takes, over all groups and planes."""
        elem = torch.empty(0, dtype=self.dtype).element_size()
        return sum(len(g.spec.keys) * 2 * g.spec.n_kv_heads * g.spec.head_dim * elem for g in self.groups.values())

    def free_pages(self) -> Dict[str, int]:
        return {name: g.pool.n_free for name, g in self.groups.items()}

    def total_pages(self) -> Dict[str, int]:
        return {name: g.pool.n_pages - self._spare_pages for name, g in self.groups.items()}

    def block_table(self, group: str, slot: int) -> List[int]:
        return self.groups[group].tables[slot]

    def check(self) -> None:
        """Invariants: no page lost, held twice or free twice; no slot both live and free; no stale copy of a table."""
        for g in self.groups.values():
            g.pool.check()
            seen = set()
            for slot, table in g.tables.items():
                if slot not in self._live:
                    raise CacheError(f"group {g.spec.name!r} keeps a table for dead slot {slot}")
                for p in table:
                    if p < 0:
                        continue
                    if p in seen:
                        raise CacheError(f"page {p} of group {g.spec.name!r} is in two block tables")
                    seen.add(p)
            if len(seen) + g.pool.n_free != g.pool.n_pages:
                raise CacheError(f"group {g.spec.name!r}: {len(seen)} held + {g.pool.n_free} free != {g.pool.n_pages}")
            for slot, a in g._lines.items():
                if slot not in g.tables or a.tolist() != g.tables[slot]:
                    raise CacheError(f"group {g.spec.name!r}: the kept array of slot {slot}'s table is stale")
        if set(self._free_slots) & set(self._live) or len(self._free_slots) + self.n_live != self.max_requests:
            raise CacheError("request slots are inconsistent")
