"""The cache manager: pages, per-request block tables, groups, state slots.

A *cache* is what one run of a mixer keeps between steps.  Caches with the same
need (``CacheNeed.group_key``) form a *group*: one pool of pages with its own
page ids, and one block table per request, shared by all caches of the group
(as in the reference one block id addresses that block in every layer,
src/csrc/model/gpt/gpt_base.h:70-72).  A group whose need has a window gives
pages back as soon as every position in them is behind the window of the
request's next token; all groups give everything back when the request ends.
Besides pages every request holds a *state slot*: an index into fixed-size
per-request device state (``kind == "state"`` needs), assigned at admission.

This class is host-side bookkeeping only and runs without a GPU; the device
tensors live in ``cache.device.DeviceCache``.

Reference for what exists there: block tables are dense int64 rows rebuilt by the
driver (src/examples/lib/inference_batch.cc:71-85, :205-214), grown before each
decode step (:168-179) and never released."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence

import numpy as np

from ..parts.base import CacheNeed
from .page_pool import OutOfPages, PagePool


@dataclass
class CacheGroup:
    index: int
    need: CacheNeed
    cache_ids: List[int]
    pool: Optional[PagePool]          # None for state groups

    @property
    def paged(self) -> bool:
        return self.need.kind == "paged_kv"


@dataclass
class RequestCache:
    slot: int
    length: int = 0                                   # tokens whose keys are (being) cached
    tables: Dict[int, List[int]] = field(default_factory=dict)   # group -> pages (-1: given back)


class OutOfSlots(RuntimeError):
    pass


class CacheManager:
    def __init__(self, needs: Dict[int, CacheNeed], page_size: int, num_pages, max_seqs: int,
                 max_pages_per_seq: int):
        """``needs``: cache id -> need.  ``num_pages``: an int for every paged group, or a
        dict group index -> int."""
        self.page_size = page_size
        self.max_seqs = max_seqs
        self.max_pages_per_seq = max_pages_per_seq
        self.groups: List[CacheGroup] = []
        self.group_of_cache: Dict[int, int] = {}
        by_key: Dict[object, CacheGroup] = {}
        for cid in sorted(needs):
            need = needs[cid]
            if need.kind not in ("paged_kv", "state"):
                raise ValueError(f"cache {cid}: unknown need kind {need.kind!r}")
            key = need.group_key()
            if key not in by_key:
                gi = len(self.groups)
                pool = None
                if need.kind == "paged_kv":
                    n = num_pages[gi] if isinstance(num_pages, dict) else num_pages
                    pool = PagePool(int(n))
                g = CacheGroup(gi, need, [], pool)
                by_key[key] = g
                self.groups.append(g)
            by_key[key].cache_ids.append(cid)
            self.group_of_cache[cid] = by_key[key].index
        self._free_slots: List[int] = list(range(max_seqs - 1, -1, -1))
        self.requests: Dict[Hashable, RequestCache] = {}
        # called with the slot whenever a request takes one over, whoever admits it (a scheduler,
        # a replay, a test): the owner of the per-slot device state clears it there
        self.on_admit: List[Callable[[int], None]] = []
        # the block tables once more as arrays indexed by state slot, kept in step with the
        # lists: a batch's tables are then one gather instead of a loop over requests
        self.table_array: Dict[int, np.ndarray] = {
            g.index: np.full((max_seqs, max_pages_per_seq), -1, np.int32) for g in self.paged_groups}

    # ------------------------------------------------------------------ queries
    @property
    def paged_groups(self) -> List[CacheGroup]:
        return [g for g in self.groups if g.paged]

    def num_free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_free

    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def pages_needed(self, req_id: Hashable, new_length: int) -> Dict[int, int]:
        """Pages each paged group would have to hand out for ``req_id`` to reach ``new_length``."""
        rc = self.requests.get(req_id)
        have = {g.index: (len(rc.tables[g.index]) if rc else 0) for g in self.paged_groups}
        want = -(-new_length // self.page_size)
        return {gi: max(0, want - h) for gi, h in have.items()}

    def can_extend(self, req_id: Hashable, new_length: int) -> bool:
        need = self.pages_needed(req_id, new_length)
        return all(self.groups[gi].pool.num_free >= n for gi, n in need.items())

    # ---------------------------------------------------------------- lifecycle
    def admit(self, req_id: Hashable) -> RequestCache:
        if req_id in self.requests:
            raise KeyError(f"request {req_id!r} is already live")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.max_seqs} state slots are in use")
        rc = RequestCache(slot=self._free_slots.pop())
        for g in self.paged_groups:
            rc.tables[g.index] = []
        self.requests[req_id] = rc
        for hook in self.on_admit:
            hook(rc.slot)
        return rc

    def extend(self, req_id: Hashable, new_length: int) -> RequestCache:
        """Make room for positions < ``new_length``; all or nothing over the groups."""
        rc = self.requests[req_id]
        if new_length < rc.length:
            raise ValueError("a request's cache does not shrink")
        want = -(-new_length // self.page_size)
        if want > self.max_pages_per_seq:
            raise ValueError(f"{new_length} tokens need {want} pages; a request may hold "
                             f"{self.max_pages_per_seq}")
        need = self.pages_needed(req_id, new_length)
        for gi, n in need.items():
            if self.groups[gi].pool.num_free < n:
                raise OutOfPages(f"group {gi}: {n} pages wanted, "
                                 f"{self.groups[gi].pool.num_free} free")
        for gi, n in need.items():
            if n:
                have = len(rc.tables[gi])
                new = self.groups[gi].pool.alloc(n)
                rc.tables[gi].extend(new)
                self.table_array[gi][rc.slot, have:have + n] = new
        rc.length = new_length
        return rc

    def shrink(self, req_id: Hashable, length: int, pages_per_group: Dict[int, int]) -> None:
        """Undo an ``extend``: back to ``length`` tokens and the given number of table entries."""
        rc = self.requests[req_id]
        for gi, n in pages_per_group.items():
            extra = rc.tables[gi][n:]
            self.groups[gi].pool.free([p for p in extra if p >= 0])
            del rc.tables[gi][n:]
            self.table_array[gi][rc.slot, n:] = -1
        rc.length = length

    def release_behind_window(self, req_id: Hashable, next_position: int) -> int:
        """Give back the pages that no token at position >= ``next_position`` will read.
        Returns the number of pages released."""
        rc = self.requests[req_id]
        released = 0
        for g in self.paged_groups:
            w = g.need.window
            if w <= 0:
                continue
            first_needed = max(0, next_position - w + 1)      # oldest position still read
            table = rc.tables[g.index]
            for pi in range(min(first_needed // self.page_size, len(table))):
                if table[pi] >= 0:
                    g.pool.free([table[pi]])
                    table[pi] = -1
                    self.table_array[g.index][rc.slot, pi] = -1
                    released += 1
        return released

    def finish(self, req_id: Hashable) -> None:
        rc = self.requests.pop(req_id)
        for g in self.paged_groups:
            g.pool.free([p for p in rc.tables[g.index] if p >= 0])
            self.table_array[g.index][rc.slot, :] = -1
        self._free_slots.append(rc.slot)

    def reset_request(self, req_id: Hashable) -> None:
        """Drop what the request has cached but keep it live (pre-emption by recomputation)."""
        rc = self.requests[req_id]
        for g in self.paged_groups:
            g.pool.free([p for p in rc.tables[g.index] if p >= 0])
            rc.tables[g.index] = []
            self.table_array[g.index][rc.slot, :] = -1
        rc.length = 0

    # ----------------------------------------------------------------- checking
    def check_invariants(self) -> None:
        """No page lost, held twice or free while held (used by tests)."""
        for g in self.paged_groups:
            held = [p for rc in self.requests.values() for p in rc.tables[g.index] if p >= 0]
            if len(held) != len(set(held)):
                raise AssertionError(f"group {g.index}: a page is in two block tables")
            if len(held) + g.pool.num_free != g.pool.num_pages:
                raise AssertionError(f"group {g.index}: {len(held)} held + {g.pool.num_free} free "
                                     f"!= {g.pool.num_pages} pages")
            for p in held:
                if not g.pool.is_held(p):
                    raise AssertionError(f"group {g.index}: page {p} is in a table and on the free list")
            for rc in self.requests.values():
                row = self.table_array[g.index][rc.slot]
                t = rc.tables[g.index]
                if list(row[:len(t)]) != t or (row[len(t):] != -1).any():
                    raise AssertionError(f"group {g.index}: the table array differs from the table")
        slots = [rc.slot for rc in self.requests.values()]
        if len(slots) != len(set(slots)) or len(slots) + len(self._free_slots) != self.max_seqs:
            raise AssertionError("state slots are lost or shared")
