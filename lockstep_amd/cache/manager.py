"""The cache manager: pages of keys and values with a block table per request,
and slots for per-request state of fixed size.

Mixers declare what they keep between steps (``PagedKVSpec`` or
``StateSpec``), one declaration per *cache unit* of the model's schedule.
Units with the same page geometry and window form a *group*; a group has its
own page pool, its own block table per request, and one storage tensor in
which a page id is valid for every unit of the group.  Pages are taken
lowest-id-first from a min-heap, so placement is a pure function of the
sequence of calls (reference engine/kv/paged.py:76-101).  They are given back
when a request closes or, in a group with a window, as soon as the window has
passed them; a page whose count of holders drops to zero returns to the heap
(reference engine/kv/paged.py:103-113).  Holders are requests that map the
page and pins of the prefix index (reference engine/kv/paged.py:116-139).

Every request also owns a *slot*: its row in the block tables on the device
and its index into the state tensors of the units that keep a ``StateSpec``.
State is zeroed when the slot is taken and, like freed pages, poisoned when
the slot is given back (``poison_on_free``); the audit and the digest cover it.

The manager does its accounting on the host; with ``device=None`` it holds no
storage at all, which is how the tests without a GPU drive it.
"""

from __future__ import annotations

import heapq
from dataclasses import dataclass, field
from typing import Hashable, Optional, Sequence

import numpy as np

from ..parts.base import PagedKVSpec, StateSpec

SUPPORTED_PAGE_SIZES = (8, 16, 32, 64, 128)


class OutOfPages(RuntimeError):
    """A group's pool has no free page left."""


class CacheAuditError(AssertionError):
    """An internal invariant of the cache manager broke."""


class PagePool:
    """Free list and holder counts of one group's pages."""

    def __init__(self, num_pages: int):
        self.num_pages = num_pages
        self._free = list(range(num_pages))
        heapq.heapify(self._free)
        self.holders = [0] * num_pages
        self.taken_total = 0
        self.freed_total = 0

    @property
    def free_pages(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfPages(f"all {self.num_pages} pages are held")
        page = heapq.heappop(self._free)
        if self.holders[page] != 0:
            raise CacheAuditError(f"page {page} was free with {self.holders[page]} holders")
        self.holders[page] = 1
        self.taken_total += 1
        return page

    def retain(self, page: int) -> None:
        if self.holders[page] <= 0:
            raise CacheAuditError(f"retaining free page {page}")
        self.holders[page] += 1

    def release(self, page: int) -> bool:
        """Drop one holder; True if the page went back to the free list."""
        if self.holders[page] <= 0:
            raise CacheAuditError(f"page {page} released more often than it was taken")
        self.holders[page] -= 1
        if self.holders[page] == 0:
            heapq.heappush(self._free, page)
            self.freed_total += 1
            return True
        return False

    def free_set(self) -> list[int]:
        return sorted(self._free)


@dataclass
class _RequestPages:
    pages: list[int] = field(default_factory=list)  # logical -> physical, -1 once released
    first_held: int = 0                             # logical pages below were released


@dataclass
class _Request:
    slot: int
    length: int = 0
    groups: list[_RequestPages] = field(default_factory=list)


class CacheGroup:
    """Units that share page geometry: one pool, one table, one storage."""

    def __init__(self, index: int, spec: PagedKVSpec, units: list[int], num_pages: int, page_size: int,
                 max_requests: int, max_pages_per_request: int, torch_dtype, device):
        self.index = index
        self.spec = spec
        self.units = units
        self.page_size = page_size
        self.pool = PagePool(num_pages)
        self.pinned: dict[int, int] = {}
        self.table_host = np.full((max_requests, max_pages_per_request), -1, dtype=np.int32)
        self.dirty_rows: set[int] = set()
        self.device = device
        self.keys = self.values = self.table = None
        if device is not None:
            import torch

            n, h, d = len(units), spec.num_kv_heads, spec.head_dim
            # keys [unit][page][kv head][slot][d]; values transposed [unit][page][kv head][d][slot]
            self.keys = torch.zeros((n, num_pages, h, page_size, d), dtype=torch_dtype, device=device)
            self.values = torch.zeros((n, num_pages, h, d, page_size), dtype=torch_dtype, device=device)
            self.table = torch.full((max_requests, max_pages_per_request), -1, dtype=torch.int32, device=device)

    def poison(self, page: int) -> None:
        if self.keys is not None:
            self.keys[:, page].fill_(float("nan"))
            self.values[:, page].fill_(float("nan"))

    def bytes_per_token(self, element_size: int) -> int:
        return 2 * len(self.units) * self.spec.num_kv_heads * self.spec.head_dim * element_size


class GraphStore(dict):
    """Captured step graphs that point into one cache manager's storage, by step shape.  They
    belong to the model that captured them, live here because they are valid for this storage
    only, and die with the manager.  The least recently captured ones make room for new ones."""

    def __init__(self, capacity: int = 32):
        super().__init__()
        self.capacity = capacity

    def make_room(self) -> None:
        while len(self) >= self.capacity:
            del self[next(iter(self))]


class CacheManager:
    def __init__(self, unit_specs: Sequence[object], page_size: int, num_pages, max_requests: int,
                 max_tokens_per_request: int, torch_dtype=None, device=None, poison_on_free: bool = False):
        """``unit_specs[u]`` is what cache unit ``u`` keeps (``PagedKVSpec``,
        ``StateSpec`` or ``None``).  ``num_pages`` is the pool size of every
        group (an int) or one size per group (a list)."""
        if page_size not in SUPPORTED_PAGE_SIZES:
            raise ValueError(f"page size {page_size} is not one of {SUPPORTED_PAGE_SIZES}: "
                             "a page must divide the 128-key tile of the attention kernels")
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_pages_per_request = max(1, -(-max_tokens_per_request // page_size))
        self.poison_on_free = poison_on_free
        self.device = device

        keyed: dict[tuple, list[int]] = {}
        self.state_units: dict[int, StateSpec] = {}
        for unit, spec in enumerate(unit_specs):
            if isinstance(spec, PagedKVSpec):
                keyed.setdefault((spec.num_kv_heads, spec.head_dim, spec.window), []).append(unit)
            elif isinstance(spec, StateSpec):
                self.state_units[unit] = spec
            elif spec is not None:
                raise TypeError(f"cache unit {unit} declares {spec!r}; expected PagedKVSpec, StateSpec or None")
        sizes = list(num_pages) if isinstance(num_pages, (list, tuple)) else [num_pages] * len(keyed)
        if len(sizes) != len(keyed):
            raise ValueError(f"{len(keyed)} cache groups but {len(sizes)} pool sizes")
        self.groups: list[CacheGroup] = []
        self.unit_place: dict[int, tuple[int, int]] = {}
        for index, ((h, d, window), units) in enumerate(keyed.items()):
            group = CacheGroup(index, PagedKVSpec(h, d, window), units, sizes[index], page_size, max_requests,
                               self.max_pages_per_request, torch_dtype, device)
            self.groups.append(group)
            for position, unit in enumerate(units):
                self.unit_place[unit] = (index, position)

        self.state: dict[int, object] = {}
        if device is not None and self.state_units:
            import torch

            kinds = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}
            for unit, spec in self.state_units.items():
                if spec.dtype not in kinds:
                    raise TypeError(f"cache unit {unit} asks for state of dtype {spec.dtype!r}; known: {sorted(kinds)}")
                self.state[unit] = torch.zeros((max_requests, *spec.shape), dtype=kinds[spec.dtype], device=device)

        self.ever_shared = False     # set once a page got a second holder (prefix sharing)
        self.step_graphs = GraphStore()
        self._free_slots = list(range(max_requests))
        heapq.heapify(self._free_slots)
        self._ever_used: set[int] = set()
        self.requests: dict[Hashable, _Request] = {}

    # -- requests ---------------------------------------------------------------
    def open(self, request_id: Hashable) -> int:
        """Give the request a slot (lowest free first) with zeroed state."""
        if request_id in self.requests:
            raise KeyError(f"request {request_id!r} is already open")
        if not self._free_slots:
            raise OutOfPages(f"all {self.max_requests} request slots are taken")
        slot = heapq.heappop(self._free_slots)
        self._ever_used.add(slot)
        self.requests[request_id] = _Request(slot=slot, groups=[_RequestPages() for _ in self.groups])
        for tensor in self.state.values():
            tensor[slot].zero_()
        return slot

    def slot(self, request_id: Hashable) -> int:
        return self.requests[request_id].slot

    def length(self, request_id: Hashable) -> int:
        return self.requests[request_id].length

    def _first_needed(self, group: CacheGroup, next_position: int) -> int:
        """Logical page below which a query at ``next_position`` reads nothing."""
        if group.spec.window is None:
            return 0
        return max(0, next_position - group.spec.window + 1) // self.page_size

    def pages_to_reserve(self, request_id: Optional[Hashable], start: int, end: int) -> list[int]:
        """Pages each group must still take so positions ``< end`` are held for a
        step whose first query is at ``start``."""
        request = self.requests.get(request_id) if request_id is not None else None
        out = []
        for gi, group in enumerate(self.groups):
            needed_to = -(-end // self.page_size)
            have = len(request.groups[gi].pages) if request else 0
            first = max(have, self._first_needed(group, start))
            out.append(max(0, needed_to - first))
        return out

    def can_reserve(self, request_id: Optional[Hashable], start: int, end: int) -> bool:
        return all(n <= g.pool.free_pages for n, g in zip(self.pages_to_reserve(request_id, start, end), self.groups))

    def reserve(self, request_id: Hashable, end: int, start: Optional[int] = None) -> None:
        """Hold pages for all positions ``< end`` (that a window still needs).

        Either every group gets its pages or none does (``OutOfPages``).
        ``start`` is the position of the step's first query, by default the
        request's current length.
        """
        request = self.requests[request_id]
        start = request.length if start is None else start
        needed_to = -(-end // self.page_size)
        if all(len(mine.pages) >= needed_to for mine in request.groups):
            return  # the last page still has room: nothing to take
        if needed_to > self.max_pages_per_request:
            raise ValueError(f"{end} tokens exceed the {self.max_pages_per_request * self.page_size} "
                             "tokens a request may hold")
        need = self.pages_to_reserve(request_id, start, end)
        for n, group in zip(need, self.groups):
            if n > group.pool.free_pages:
                raise OutOfPages(f"group {group.index} needs {n} pages for request {request_id!r}, "
                                 f"{group.pool.free_pages} of {group.pool.num_pages} are free")
        for gi, group in enumerate(self.groups):
            mine = request.groups[gi]
            needed_to = -(-end // self.page_size)
            first = self._first_needed(group, start)
            while len(mine.pages) < needed_to:
                logical = len(mine.pages)
                if logical < first:
                    mine.pages.append(-1)  # never needed: the window starts above it
                    mine.first_held = max(mine.first_held, logical + 1)
                    continue
                page = group.pool.take()
                mine.pages.append(page)
                group.table_host[request.slot, logical] = page
                group.dirty_rows.add(request.slot)

    def commit(self, request_id: Hashable, length: int) -> None:
        """The request now holds ``length`` tokens; give back what windows passed."""
        request = self.requests[request_id]
        if length < request.length:
            raise ValueError(f"request {request_id!r} cannot shrink from {request.length} to {length}")
        request.length = length
        for gi, group in enumerate(self.groups):
            mine = request.groups[gi]
            first = min(self._first_needed(group, length), len(mine.pages))
            for logical in range(mine.first_held, first):
                page = mine.pages[logical]
                if page >= 0:
                    self._release_page(group, page)
                    mine.pages[logical] = -1
                    group.table_host[request.slot, logical] = -1
                    group.dirty_rows.add(request.slot)
            mine.first_held = max(mine.first_held, first)

    def close(self, request_id: Hashable) -> None:
        """Give back every page and the slot."""
        request = self.requests.pop(request_id)
        for gi, group in enumerate(self.groups):
            mine = request.groups[gi]
            for page in mine.pages:
                if page >= 0:
                    self._release_page(group, page)
            if mine.pages:
                group.table_host[request.slot, : len(mine.pages)] = -1
                group.dirty_rows.add(request.slot)
            mine.pages.clear()
        if self.poison_on_free:
            for tensor in self.state.values():      # a later reader of the slot's old state must notice
                tensor[request.slot].fill_(self._poison_value(tensor))
        heapq.heappush(self._free_slots, request.slot)

    @staticmethod
    def _poison_value(tensor):
        return float("nan") if tensor.dtype.is_floating_point else -(1 << 30)

    def _release_page(self, group: CacheGroup, page: int) -> None:
        if group.pool.release(page) and self.poison_on_free:
            group.poison(page)

    # -- sharing (prefix index) ---------------------------------------------------
    def shareable(self) -> bool:
        """Whole pages of a prefix can stand for the prefix only when every unit
        keeps all keys in pages: one group without a window and no state."""
        return self.why_not_shareable() is None

    def why_not_shareable(self):
        """None if pages can be shared between requests, else the reason in words."""
        if self.state_units:
            return "a mixer keeps per-request state, which no page of keys and values stands for"
        if len(self.groups) != 1:
            return f"the layers' caches form {len(self.groups)} groups with page tables of their own"
        if self.groups[0].spec.window is not None:
            return "the layers keep a window of keys only, so early pages of a prefix are gone"
        return None

    def adopt(self, request_id: Hashable, pages: Sequence[int]) -> None:
        """Map shared ``pages`` as the request's first logical pages."""
        if not self.shareable():
            raise CacheAuditError("pages cannot be shared in this cache layout")
        request = self.requests[request_id]
        group, mine = self.groups[0], request.groups[0]
        if mine.pages:
            raise CacheAuditError("adopt expects a request without pages")
        self.ever_shared = True
        for logical, page in enumerate(pages):
            group.pool.retain(page)
            mine.pages.append(page)
            group.table_host[request.slot, logical] = page
        if pages:
            group.dirty_rows.add(request.slot)

    def pin(self, page: int) -> None:
        self.ever_shared = True
        group = self.groups[0]
        group.pool.retain(page)
        group.pinned[page] = group.pinned.get(page, 0) + 1

    def unpin(self, page: int) -> None:
        group = self.groups[0]
        held = group.pinned.get(page, 0)
        if held <= 0:
            raise CacheAuditError(f"unpinning page {page}, which the index does not hold")
        if held == 1:
            del group.pinned[page]
        else:
            group.pinned[page] = held - 1
        self._release_page(group, page)

    def request_pages(self, request_id: Hashable, group: int = 0) -> list[int]:
        return list(self.requests[request_id].groups[group].pages)

    def assert_exclusive(self, request_id: Hashable, group_index: int, logical_page: int) -> None:
        """A write must land in a page no one else maps (reference
        engine/kv/paged.py:162-181): sharing is whole-page, without copy-on-write."""
        group = self.groups[group_index]
        page = self.requests[request_id].groups[group_index].pages[logical_page]
        if page < 0 or group.pool.holders[page] != 1:
            raise CacheAuditError(f"request {request_id!r} would write page {page} "
                                  f"(holders {group.pool.holders[page] if page >= 0 else 'released'})")

    # -- device side -----------------------------------------------------------------
    def sync_tables(self) -> None:
        """Upload the block-table rows that changed since the last call."""
        if self.device is None:
            return
        import torch

        for group in self.groups:
            if not group.dirty_rows:
                continue
            rows = sorted(group.dirty_rows)
            index = torch.as_tensor(rows, dtype=torch.long, device=self.device)
            data = torch.from_numpy(group.table_host[rows]).to(self.device, non_blocking=False)
            group.table.index_copy_(0, index, data)
            group.dirty_rows.clear()

    def unit_group(self, unit: int) -> CacheGroup:
        return self.groups[self.unit_place[unit][0]]

    def unit_pages(self, unit: int):
        """(group, key pages, value pages) of a paged unit."""
        gi, position = self.unit_place[unit]
        group = self.groups[gi]
        return group, group.keys[position], group.values[position]

    def unit_state(self, unit: int):
        """State tensor ``[slots, *shape]`` of a unit with a ``StateSpec``."""
        return self.state[unit]

    def unit_tensors(self, unit: int) -> tuple:
        """The device tensors that are this unit's own: (key pages, value pages), (state,) or ()."""
        if unit in self.unit_place:
            gi, position = self.unit_place[unit]
            return (self.groups[gi].keys[position], self.groups[gi].values[position])
        if unit in self.state:
            return (self.state[unit],)
        return ()

    # -- accounting -----------------------------------------------------------------
    @property
    def free_pages(self) -> list[int]:
        return [g.pool.free_pages for g in self.groups]

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def audit(self) -> None:
        """No page lost, held twice without a record, or free while held
        (reference engine/kv/paged.py:190-223)."""
        slots = [r.slot for r in self.requests.values()]
        if len(set(slots)) != len(slots):
            raise CacheAuditError("two requests share a slot")
        if sorted(slots + self._free_slots) != list(range(self.max_requests)):
            raise CacheAuditError("request slots are lost or duplicated")
        self._audit_state()
        for gi, group in enumerate(self.groups):
            expected = [0] * group.pool.num_pages
            for page, count in group.pinned.items():
                expected[page] += count
            for rid, request in self.requests.items():
                seen = set()
                mine = request.groups[gi]
                for logical, page in enumerate(mine.pages):
                    if page < 0:
                        if logical >= mine.first_held:
                            raise CacheAuditError(f"request {rid!r} lost page {logical} of group {gi}")
                        continue
                    if page in seen:
                        raise CacheAuditError(f"request {rid!r} maps page {page} twice in group {gi}")
                    seen.add(page)
                    expected[page] += 1
                    if group.table_host[request.slot, logical] != page:
                        raise CacheAuditError(f"block table of {rid!r} disagrees at logical page {logical}")
            free = group.pool.free_set()
            if len(set(free)) != len(free):
                raise CacheAuditError(f"a page of group {gi} is in the free list twice")
            free = set(free)
            for page in range(group.pool.num_pages):
                if group.pool.holders[page] != expected[page]:
                    raise CacheAuditError(f"group {gi} page {page}: {group.pool.holders[page]} holders counted, "
                                          f"{expected[page]} found")
                if (group.pool.holders[page] == 0) != (page in free):
                    raise CacheAuditError(f"group {gi} page {page} has {group.pool.holders[page]} holders but is "
                                          f"{'in' if page in free else 'not in'} the free list")

    def _audit_state(self) -> None:
        """State units: every unit has a row per slot; with poisoning on, the rows of free slots
        hold the poison and the rows of live requests hold none of it."""
        for unit, spec in self.state_units.items():
            tensor = self.state.get(unit)
            if self.device is None:
                continue
            if tensor is None or tuple(tensor.shape) != (self.max_requests, *spec.shape):
                raise CacheAuditError(f"state unit {unit} does not hold {self.max_requests} rows of {spec.shape}")
            if not self.poison_on_free:
                continue
            rows = tensor.reshape(self.max_requests, -1)
            bad = rows.isnan().any(dim=1) if tensor.dtype.is_floating_point else (rows == -(1 << 30)).any(dim=1)
            bad = bad.cpu().tolist()
            live = {r.slot: rid for rid, r in self.requests.items()}
            for slot, poisoned in enumerate(bad):
                if slot in live and poisoned:
                    raise CacheAuditError(f"state unit {unit}: request {live[slot]!r} (slot {slot}) holds poisoned state")
                if slot not in live and slot in self._ever_used and not poisoned:
                    raise CacheAuditError(f"state unit {unit}: free slot {slot} was not poisoned when it was given back")

    def state_digest(self, content: bool = False) -> tuple:
        """Allocator state as a comparable value (reference engine/kv/paged.py:225-237); the
        state units' declarations are part of it, and with ``content`` a hash of the state rows
        of the live requests (read back from the device)."""
        states = tuple((unit, tuple(spec.shape), spec.dtype) for unit, spec in sorted(self.state_units.items()))
        if content and self.state:
            import hashlib

            slots = sorted(r.slot for r in self.requests.values())
            rows = hashlib.sha256()
            for unit in sorted(self.state):
                if slots:
                    picked = self.state[unit][slots].contiguous().view(-1)
                    rows.update(picked.view(dtype=__import__("torch").uint8).cpu().numpy().tobytes())
            states += (rows.hexdigest(),)
        return states + tuple(
            (tuple(g.pool.holders), tuple(g.pool.free_set()), tuple(sorted(g.pinned.items())),
             tuple((repr(rid), r.slot, r.length, tuple(r.groups[gi].pages))
                   for rid, r in sorted(self.requests.items(), key=lambda kv: repr(kv[0]))))
            for gi, g in enumerate(self.groups)
        ) + (self.page_size,)
