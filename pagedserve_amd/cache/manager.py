"""Paged key/value cache and fixed-size state slots, one manager for both.

The reference keeps two pools ``[layers, pages, heads, page, head_dim]`` with a LIFO
free list and one block table per request (src/model/kv_manager.py:77-86,115-127,
9-16), allocates a page whenever a token lands on a page boundary (``:149-171``),
and gives everything back when a request finishes (``:425-442``).

This manager keeps those rules and adds what other layer kinds need:

* **Cache groups.**  Cache entries (one per caching call of the run order) with the
  same geometry and visibility form a group; each group has a pool, a free list and
  block tables of its own.  A group that only ever looks ``window`` keys back gives
  pages back as soon as the window has passed them.
* **Slots.**  Every live request holds one slot index.  Mixers with per-request state
  of fixed size get a tensor ``[max_slots, ...]`` per cache entry, zeroed when the
  slot is handed out.  GPT-2 has none; the slot then only carries the position.

Pages are taken *before* a step runs (``grow``), lengths move after it succeeded
(``commit``).  All bookkeeping is host-side Python and runs without a GPU; pools and
state tensors live on the device given at construction.
"""

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch


class CacheFull(RuntimeError):
    """No free page (or slot) is left (src/model/kv_manager.py:116-117)."""


@dataclass(frozen=True)
class CacheGroupSpec:
    """Cache entries that share page geometry and visibility."""

    entries: Tuple[int, ...]
    kv_heads: int
    head_dim: int
    window: int = 0  # 0: every earlier key stays visible
    value_dim: int = 0  # head size of the values where it differs from the keys' (0: the same)

    @property
    def value_head_dim(self) -> int:
        return self.value_dim or self.head_dim

    def geometry(self):
        return (self.kv_heads, self.head_dim, self.window, self.value_head_dim)


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size for one cache entry."""

    entry: int
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class PagePool:
    """Free list of one group.  LIFO: a page that was just freed is handed out next
    (src/model/kv_manager.py:118,127), so reuse happens immediately."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self.free_pages: List[int] = list(range(num_pages))
        self._held = [False] * num_pages
        self.peak_allocated = 0

    @property
    def num_free(self) -> int:
        return len(self.free_pages)

    @property
    def num_allocated(self) -> int:
        return self.num_pages - len(self.free_pages)

    def allocate(self) -> int:
        if not self.free_pages:
            raise CacheFull("KV cache full")
        page = self.free_pages.pop()
        if self._held[page]:
            raise AssertionError(f"page {page} was on the free list while held")
        self._held[page] = True
        self.peak_allocated = max(self.peak_allocated, self.num_allocated)
        return page

    def allocate_many(self, count: int) -> List[int]:
        """``count`` pages in the order that ``allocate`` would hand them out."""
        if count > len(self.free_pages):
            raise CacheFull("KV cache full")
        pages = self.free_pages[len(self.free_pages) - count:][::-1]
        del self.free_pages[len(self.free_pages) - count:]
        for page in pages:
            if self._held[page]:
                raise AssertionError(f"page {page} was on the free list while held")
            self._held[page] = True
        self.peak_allocated = max(self.peak_allocated, self.num_allocated)
        return pages

    def free(self, page: int):
        if not 0 <= page < self.num_pages:
            raise ValueError(f"page {page} does not exist")
        if not self._held[page]:
            raise RuntimeError(f"page {page} freed twice")
        self._held[page] = False
        self.free_pages.append(page)


@dataclass
class RequestCache:
    slot: int
    length: int = 0
    # per group: logical page index -> physical page, -1 once a window has passed it
    tables: List[List[int]] = field(default_factory=list)
    # positions that the pages held in every group have room for (``grow`` keeps it)
    capacity: int = 0


RELEASED = -1


class CacheManager:
    def __init__(self, groups: Sequence[CacheGroupSpec], num_pages, page_size: int,
                 max_slots: int, dtype: torch.dtype, device, states: Sequence[StateSpec] = (),
                 max_positions: Optional[int] = None, allocate_pools: bool = True):
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        if max_slots <= 0:
            raise ValueError("max_slots must be positive")
        self.groups = tuple(groups)
        seen = set()
        for group in self.groups:
            for entry in group.entries:
                if entry in seen:
                    raise ValueError(f"cache entry {entry} is in two groups")
                seen.add(entry)
        self.page_size = page_size
        self.max_slots = max_slots
        self._windowed = any(group.window > 0 for group in self.groups)
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_positions = max_positions
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(self.groups)
        if len(num_pages) != len(self.groups):
            raise ValueError("one page count per cache group is needed")
        self.pools = [PagePool(count) for count in num_pages]
        # entry -> (group index, index inside the group's pool tensor)
        self.entry_location: Dict[int, Tuple[int, int]] = {}
        for group_index, group in enumerate(self.groups):
            for local, entry in enumerate(group.entries):
                self.entry_location[entry] = (group_index, local)
        self.key_pools: List[Optional[torch.Tensor]] = []
        self.value_pools: List[Optional[torch.Tensor]] = []
        for group, pool in zip(self.groups, self.pools):
            if allocate_pools:
                shape = (len(group.entries), pool.num_pages, group.kv_heads, page_size)
                self.key_pools.append(torch.empty(shape + (group.head_dim,), dtype=dtype, device=self.device))
                self.value_pools.append(torch.empty(shape + (group.value_head_dim,), dtype=dtype,
                                                    device=self.device))
            else:
                self.key_pools.append(None)
                self.value_pools.append(None)
        self.state_specs = tuple(states)
        self.state_tensors: Dict[int, torch.Tensor] = {}
        for spec in self.state_specs:
            if spec.entry in self.state_tensors:
                raise ValueError(f"cache entry {spec.entry} has two state tensors")
            self.state_tensors[spec.entry] = torch.zeros(
                (max_slots,) + tuple(spec.shape), dtype=spec.dtype, device=self.device)
        self.free_slots: List[int] = list(range(max_slots - 1, -1, -1))
        self.requests: Dict[Hashable, RequestCache] = {}
        # Block tables as arrays [slot, logical page] (-1: no page), kept in step with the
        # lists, so that a step gathers its rows with one indexing operation.
        self.table_arrays: Optional[List[np.ndarray]] = None
        if max_positions is not None:
            width = -(-max_positions // page_size)
            self.table_arrays = [np.full((max_slots, width), RELEASED, dtype=np.int32)
                                 for _ in self.groups]

    # ------------------------------------------------------------------ sizes
    def bytes_per_page(self, group_index: int) -> int:
        group = self.groups[group_index]
        element = torch.empty(0, dtype=self.dtype).element_size()
        # src/model/kv_manager.py:55-58
        return (len(group.entries) * group.kv_heads * self.page_size
                * (group.head_dim + group.value_head_dim) * element)

    def pages_for_length(self, group_index: int, length: int, longest_step: Optional[int] = None) -> int:
        """Most pages that one request of ``length`` tokens holds in a group at any
        time, when no step brings more than ``longest_step`` tokens."""
        full = -(-length // self.page_size)
        window = self.groups[group_index].window
        if window <= 0:
            return full
        step = length if longest_step is None else min(longest_step, length)
        # keys of the step plus the window behind its first token, page-aligned slack
        span = window + step
        return min(full, -(-span // self.page_size) + 1)

    # --------------------------------------------------------------- requests
    def admit(self, request_id: Hashable) -> int:
        """Hand out a slot (zeroing its state) for a new request."""
        if request_id in self.requests:
            raise RuntimeError(f"request {request_id!r} is already live")
        if not self.free_slots:
            raise CacheFull("no free request slot")
        slot = self.free_slots.pop()
        for tensor in self.state_tensors.values():
            tensor[slot].zero_()
        record = RequestCache(slot=slot, tables=[[] for _ in self.groups])
        record.capacity = self._capacity(record)
        self.requests[request_id] = record
        return slot

    def _capacity(self, record) -> int:
        """Positions that the record's pages have room for in every group (no group: no limit)."""
        if not record.tables:
            return 1 << 62
        return min(len(table) for table in record.tables) * self.page_size

    def length(self, request_id: Hashable) -> int:
        return self.requests[request_id].length

    def slot(self, request_id: Hashable) -> int:
        return self.requests[request_id].slot

    def pages_missing(self, request_id: Optional[Hashable], new_length: int) -> List[int]:
        """Pages per group that ``grow`` would have to take."""
        out = []
        for group_index in range(len(self.groups)):
            have = 0
            if request_id is not None and request_id in self.requests:
                have = len(self.requests[request_id].tables[group_index])
            out.append(max(0, -(-new_length // self.page_size) - have))
        return out

    def can_grow(self, request_id: Optional[Hashable], new_length: int) -> bool:
        return all(missing <= pool.num_free
                   for missing, pool in zip(self.pages_missing(request_id, new_length), self.pools))

    def grow(self, request_id: Hashable, new_length: int):
        """Take the pages that positions ``< new_length`` need, in every group.

        All or nothing: on ``CacheFull`` the pages taken so far go back
        (src/model/kv_manager.py:264-275)."""
        record = self.requests[request_id]
        if new_length < record.length:
            raise ValueError("a request's cache cannot shrink")
        if self.max_positions is not None and new_length > self.max_positions:
            raise ValueError(
                f"request {request_id!r} would reach {new_length} positions, the model has {self.max_positions}")
        if new_length <= record.capacity:
            return      # (most decode steps: the last page still has room)
        missing = self.pages_missing(request_id, new_length)
        if not any(missing):
            return
        for group_index, count in enumerate(missing):
            if count > self.pools[group_index].num_free:
                raise CacheFull("KV cache full")      # nothing has been taken yet
        for group_index, count in enumerate(missing):
            if count == 0:
                continue
            pages = self.pools[group_index].allocate_many(count)
            table = record.tables[group_index]
            first = len(table)
            table.extend(pages)
            if self.table_arrays is not None:
                self.table_arrays[group_index][record.slot, first:first + count] = pages
        record.capacity = self._capacity(record)

    def commit(self, request_id: Hashable, new_length: int):
        """The step that wrote positions ``< new_length`` succeeded."""
        record = self.requests[request_id]
        if new_length < record.length:
            raise ValueError("a request's cache cannot shrink")
        if new_length > record.capacity:
            raise RuntimeError("commit beyond the pages that were taken")
        record.length = new_length
        if not self._windowed:
            return
        for group_index, group in enumerate(self.groups):
            if group.window <= 0:
                continue
            # The next query sits at position >= new_length and sees keys
            # > position - window; keys <= new_length - window are dead.
            last_dead = new_length - group.window
            table = record.tables[group_index]
            page = 0
            while page < len(table) and (page + 1) * self.page_size - 1 <= last_dead:
                if table[page] != RELEASED:
                    self.pools[group_index].free(table[page])
                    table[page] = RELEASED
                    if self.table_arrays is not None:
                        self.table_arrays[group_index][record.slot, page] = RELEASED
                page += 1

    def release(self, request_id: Hashable):
        """Give back every page and the slot (src/model/kv_manager.py:425-442)."""
        if request_id not in self.requests:
            raise RuntimeError(f"request {request_id!r} is not live")
        record = self.requests.pop(request_id)
        for group_index, table in enumerate(record.tables):
            live = [page for page in table if page != RELEASED]
            if len(live) != len(set(live)):
                raise RuntimeError("request holds a page twice")
            for page in live:
                self.pools[group_index].free(page)
            if self.table_arrays is not None:
                self.table_arrays[group_index][record.slot, :] = RELEASED
        self.free_slots.append(record.slot)

    def table(self, request_id: Hashable, group_index: int) -> List[int]:
        return self.requests[request_id].tables[group_index]

    # ------------------------------------------------------------------ views
    def entry_pools(self, entry: int):
        """(keys, values) of one cache entry: ``[pages, kv_heads, page, head_dim]`` (the values
        with their own head size where the group names one)."""
        group_index, local = self.entry_location[entry]
        return self.key_pools[group_index][local], self.value_pools[group_index][local]

    def entry_group(self, entry: int) -> int:
        return self.entry_location[entry][0]

    def state(self, entry: int) -> torch.Tensor:
        return self.state_tensors[entry]

    # ------------------------------------------------------------------ stats
    def usage_summary(self) -> dict:
        """Counters in the manner of src/model/kv_manager.py:134-147, per group."""
        groups = []
        for group_index, pool in enumerate(self.pools):
            per_page = self.bytes_per_page(group_index)
            groups.append({
                "total_blocks": pool.num_pages,
                "free_blocks_at_end": pool.num_free,
                "peak_allocated_blocks": pool.peak_allocated,
                "peak_allocated_tokens": pool.peak_allocated * self.page_size,
                "peak_allocated_bytes": pool.peak_allocated * per_page,
                "peak_utilization_percent": 100 * pool.peak_allocated / pool.num_pages,
                "bytes_per_block": per_page,
                "bytes_per_token": per_page // self.page_size,
            })
        return {"groups": groups, "live_requests": len(self.requests),
                "free_slots": len(self.free_slots)}

    def reset_usage_stats(self):
        for pool in self.pools:
            pool.peak_allocated = pool.num_allocated

    def check_invariants(self):
        """Every page is either free or held by exactly one request; same for slots."""
        for group_index, pool in enumerate(self.pools):
            held = []
            for record in self.requests.values():
                held.extend(page for page in record.tables[group_index] if page != RELEASED)
            free = pool.free_pages
            if len(set(held)) != len(held):
                raise AssertionError(f"group {group_index}: a page is held twice")
            if len(set(free)) != len(free):
                raise AssertionError(f"group {group_index}: a page is on the free list twice")
            if set(held) & set(free):
                raise AssertionError(f"group {group_index}: a page is both held and free")
            if len(held) + len(free) != pool.num_pages:
                raise AssertionError(
                    f"group {group_index}: {pool.num_pages - len(held) - len(free)} pages lost")
        for request_id, record in self.requests.items():
            if record.capacity != self._capacity(record) or record.length > record.capacity:
                raise AssertionError(f"request {request_id!r}: room for {record.capacity} positions "
                                     f"noted, {self._capacity(record)} held, {record.length} used")
        slots = [record.slot for record in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self.free_slots):
            raise AssertionError("a slot is held twice")
        if len(slots) + len(self.free_slots) != self.max_slots:
            raise AssertionError("a slot was lost")


def kv_cache_budget(free_memory: int, total_memory: int, memory_utilization: float = 0.90,
                    safety_memory: int = 3072 * 1024 * 1024) -> int:
    """Bytes for the cache from the device's free/total memory.

    The smaller of "fill the device up to ``memory_utilization``" and "leave
    ``safety_memory`` free" (main.py:48-73; defaults main.py:30-31)."""
    if not 0 < memory_utilization <= 1:
        raise ValueError("KV-cache memory utilization must be in (0, 1]")
    if safety_memory < 0:
        raise ValueError("KV-cache safety memory cannot be negative")
    if not 0 < free_memory <= total_memory:
        raise ValueError("device memory information is invalid")
    used = total_memory - free_memory
    budget = min(int(total_memory * memory_utilization) - used, free_memory - safety_memory)
    if budget <= 0:
        raise RuntimeError("no device memory remains for the KV cache after the utilization "
                           "target and the safety margin")
    return budget
