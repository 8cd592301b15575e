"""Cache manager: paged keys and values with a block table per request, and slots of
fixed-size per-request state.

What each schedule entry of the model keeps between steps is declared by its mixer:
  PagedKVNeed(nkv, d, window, dtype)  keys and values of every position, or of a sliding window, kept in `dtype`
                               (None: the run's activation dtype);
  StateNeed(shape, dtype)      a state of fixed size;
  ("from", j)                  nothing of its own: it reads the cache of entry j;
  None                         nothing.
Entries whose paged needs are equal form a group.  A group has a page pool of its own, one
K tensor [pages + 1, nkv, page_size, d] and one V tensor [pages + 1, nkv, d, page_size] per
entry (values are kept transposed inside a page, so that the keys of one value column are
contiguous, which is what the matrix-core kernels read; a page id addresses the same page
in every entry of the group; the extra last page absorbs the writes of padding rows),
and one block table per request.  Pages are taken when a request grows into them and given
back when the request ends, is rolled back, or (windowed groups) when every position in
the page has left the window of all future queries.

The block tables live on the device for good: one int32 array [groups, max_requests + 1, max_blocks] (row = the
request's slot; the last row, the trash row, points at the trash page), a copy of the host's.  Whatever changes an
entry on the host (extend, rollback, trim, release) writes the range down; the step function takes the ranges with
table_patches() and sends the changed entries along with its step's metadata, a few integers a step however long the
contexts may grow.  Kernels read the device array at a fixed address, with the slot of a token's request as the row.

Every admitted request also holds one state slot out of `max_requests`; StateNeed entries
keep a tensor [max_requests + 1, *shape], zeroed for the slot at admission.  The slot is also
the request's row in the per-group host block tables.  The extra last row is the trash slot:
rows that pad a batch (graph replays) point there, as their keys and values go to the trash
page, so no request's state is touched by them.  A step that fails must leave no trace:
snapshot_state() before the forward and restore_state() after a failure put the touched
rows back, as rollback() does for lengths and pages.

Lengths are host integers (reference mini_llm/cache/lengths.py:8-43): extend() before the
forward, rollback() if it fails.  The reference reserves a request's whole lifetime at
admission (mini_llm/cache/paged/cache.py:257-352); here pages are taken on demand and a
reservation count gives the scheduler the same guarantee.
"""

from __future__ import annotations

import heapq
from dataclasses import dataclass, field

import numpy as np
import torch

from ..errors import KVCacheError
from ..parts import PagedKVNeed, StateNeed
from .pages import PagePool


@dataclass
class LayerCache:
    """What a mixer is handed for one schedule entry."""

    group: int | None = None          # index of the paged group (ctx.group(i) has table and slots)
    k_pages: torch.Tensor | None = None
    v_pages: torch.Tensor | None = None
    state: torch.Tensor | None = None  # [max_requests + 1, *shape] for StateNeed entries (last row: trash slot)
    window: int | None = None


@dataclass
class RequestCache:
    """Pages, slot and length of one live request."""

    request_id: object
    slot: int
    length: int = 0
    tables: list = field(default_factory=list)      # per group: page id per logical block, -1 = given back
    first_live: list = field(default_factory=list)  # per group: first logical block still held
    reserved: list = field(default_factory=list)    # per group: pages promised to this request
    released: bool = False


class PagedGroup:
    def __init__(self, need: PagedKVNeed, entries: list[int], num_pages: int):
        self.need, self.entries = need, entries
        self.dtype: torch.dtype | None = None       # what its pages hold: the need's own dtype, else the manager's
        self.pool = PagePool(num_pages)
        self.reserved_pages = 0
        self.k: dict[int, torch.Tensor] = {}
        self.v: dict[int, torch.Tensor] = {}
        self.host_table: np.ndarray | None = None   # [max_requests, max_blocks] int32, a view of the manager's array of all groups


class CacheManager:
    def __init__(self, needs: list, *, page_size: int, num_pages: int, max_requests: int, max_seq_len: int,
                 dtype: torch.dtype = torch.float32, device="cpu", allocate_storage: bool = True):
        if page_size <= 0:
            raise KVCacheError(f"page_size must be positive, got {page_size}")
        if max_requests <= 0:
            raise KVCacheError(f"max_requests must be positive, got {max_requests}")
        if max_seq_len <= 0:
            raise KVCacheError(f"max_seq_len must be positive, got {max_seq_len}")
        self.page_size, self.max_requests, self.max_seq_len = page_size, max_requests, max_seq_len
        self.dtype, self.device = dtype, torch.device(device)
        self.max_blocks = -(-max_seq_len // page_size)
        self.groups: list[PagedGroup] = []
        self.layer_caches: list[LayerCache] = []
        self.state_entries: list[int] = []
        self._free_slots = list(range(max_requests))
        heapq.heapify(self._free_slots)
        self._active: dict[int, RequestCache] = {}   # slot -> request
        self.last_allocation_tokens = 0

        by_need: dict[PagedKVNeed, PagedGroup] = {}
        for position, need in enumerate(needs):
            cache = LayerCache()
            if isinstance(need, PagedKVNeed):
                if need not in by_need:
                    by_need[need] = PagedGroup(need, [], num_pages)
                    by_need[need].dtype = need.dtype if need.dtype is not None else dtype
                    self.groups.append(by_need[need])
                group = by_need[need]
                group.entries.append(position)
                cache.group, cache.window = self.groups.index(group), need.window
            elif isinstance(need, StateNeed):
                self.state_entries.append(position)
                if allocate_storage:
                    cache.state = torch.zeros((max_requests + 1, *need.shape), dtype=need.dtype, device=self.device)
            elif isinstance(need, tuple) and len(need) == 2 and need[0] == "from":
                source = need[1]
                if not 0 <= source < position or self.layer_caches[source].group is None:
                    raise KVCacheError(f"entry {position} reads the cache of entry {source}, which keeps no pages")
                cache = self.layer_caches[source]
            elif need is not None:
                raise KVCacheError(f"entry {position} declares an unknown cache need: {need!r}")
            self.layer_caches.append(cache)

        if allocate_storage and self.device.type == "cuda" and self.groups:
            # a pool the device cannot hold is refused before anything is allocated, with the numbers that decide it
            per_page = page_size * self.bytes_per_token()
            # free: what the device has left, and what torch's allocator holds without using it (an engine reserves
            # its memory as one segment before its weights are made: the pool comes out of that)
            free = torch.cuda.mem_get_info(self.device)[0] + torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)
            if (num_pages + 1) * per_page > free:
                fits = max(free // per_page - 1, 0)
                raise KVCacheError(f"a cache pool of {num_pages} pages of {page_size} tokens needs {(num_pages + 1) * per_page / 2**30:.1f} GiB, "
                                   f"{free / 2**30:.1f} GiB are free on {self.device}: {fits} pages ({fits * page_size} tokens) would fit")
        # block tables of all groups, host and device: [groups, max_requests + 1, max_blocks]; the last row of a group
        # is the trash row (rows that pad a batch read their one page there)
        self._tables_host = np.full((len(self.groups), max_requests + 1, self.max_blocks), -1, dtype=np.int32)
        self._dirty: list[tuple[int, int, int, int]] = []     # (group, slot, first block, end block) changed since table_patches()
        for index, group in enumerate(self.groups):
            self._tables_host[index, max_requests, 0] = group.pool.num_pages          # the trash page
            group.host_table = self._tables_host[index, :max_requests]
        self.device_tables = None
        if allocate_storage and self.groups:
            self.device_tables = torch.from_numpy(self._tables_host).to(self.device)
        for index, group in enumerate(self.groups):
            if allocate_storage:
                k_shape = (num_pages + 1, group.need.num_kv_heads, page_size, group.need.head_dim)
                v_shape = (num_pages + 1, group.need.num_kv_heads, group.need.head_dim, page_size)
                for position in group.entries:
                    group.k[position] = torch.zeros(k_shape, dtype=group.dtype, device=self.device)
                    group.v[position] = torch.zeros(v_shape, dtype=group.dtype, device=self.device)
                    self.layer_caches[position].k_pages = group.k[position]
                    self.layer_caches[position].v_pages = group.v[position]

    # ------------------------------------------------------------------ sizes
    @property
    def capacity(self) -> int:
        """Tokens the smallest pool can hold."""
        return min((g.pool.num_pages for g in self.groups), default=0) * self.page_size

    @property
    def active_requests(self) -> int:
        return len(self._active)

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.free_pages

    def used_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.used_pages

    @property
    def used_tokens(self) -> int:
        return max((g.pool.used_pages for g in self.groups), default=0) * self.page_size

    def bytes_per_token(self) -> int:
        return sum(2 * len(g.entries) * g.need.num_kv_heads * g.need.head_dim * torch.empty(0, dtype=g.dtype).element_size()
                   for g in self.groups)

    def trash_page(self, group: int = 0) -> int:
        """Page that no request owns; padding rows of a padded batch write there."""
        return self.groups[group].pool.num_pages

    @property
    def trash_slot(self) -> int:
        """State row that no request owns; padding rows of a padded batch point there."""
        return self.max_requests

    def snapshot_state(self, requests) -> list:
        """Copies of the state rows of `requests` (every StateNeed entry), to put back with restore_state()
        if the step that is about to run fails.  Empty, and free, for a model without such entries."""
        if not self.state_entries:
            return []
        slots = [request.slot for request in requests]
        kept = []
        for position in self.state_entries:
            state = self.layer_caches[position].state
            if state is not None:
                kept.append((state, slots, state[slots].clone()))
        return kept

    @staticmethod
    def restore_state(snapshot: list) -> None:
        for state, slots, rows in snapshot:
            state[slots] = rows

    def pages_for(self, group: int, tokens: int, max_step_tokens: int | None = None) -> int:
        """Pages a request of `tokens` positions can hold at once in `group`."""
        blocks = -(-tokens // self.page_size)
        window = self.groups[group].need.window
        if window is None:
            return blocks
        step = tokens if max_step_tokens is None else max_step_tokens
        return min(blocks, -(-window // self.page_size) + -(-step // self.page_size) + 2)

    # -------------------------------------------------------------- admission
    def can_admit(self, tokens: int, max_step_tokens: int | None = None) -> bool:
        """Whether a slot is free and every pool can promise the pages of a `tokens`-long request."""
        if not self._free_slots or tokens > self.max_seq_len:
            return False
        return all(g.reserved_pages + self.pages_for(i, tokens, max_step_tokens) <= g.pool.num_pages
                   for i, g in enumerate(self.groups))

    def admit(self, request_id=None, reserve_tokens: int = 0, max_step_tokens: int | None = None) -> RequestCache:
        """Give a new request a state slot (zeroed) and, if asked, a promise of pages."""
        if reserve_tokens < 0:
            raise KVCacheError(f"reserve_tokens must not be negative, got {reserve_tokens}")
        if reserve_tokens > self.max_seq_len:
            raise KVCacheError(f"cache capacity {reserve_tokens} exceeds the context length {self.max_seq_len}")
        if not self._free_slots:
            raise KVCacheError(f"all {self.max_requests} request slots are in use")
        reserved = [self.pages_for(i, reserve_tokens, max_step_tokens) if reserve_tokens else 0 for i in range(len(self.groups))]
        for group, pages in zip(self.groups, reserved):
            if group.reserved_pages + pages > group.pool.num_pages:
                raise KVCacheError(
                    f"KV block pool exhausted: need {pages} blocks but only "
                    f"{group.pool.num_pages - group.reserved_pages} are unreserved")
        slot = heapq.heappop(self._free_slots)
        for group, pages in zip(self.groups, reserved):
            group.reserved_pages += pages
            group.host_table[slot, :] = -1
        for position in self.state_entries:
            state = self.layer_caches[position].state
            if state is not None:
                state[slot].zero_()
        request = RequestCache(request_id, slot, 0, [[] for _ in self.groups], [0 for _ in self.groups], reserved)
        self._active[slot] = request
        self.last_allocation_tokens = reserve_tokens
        return request

    def _check_live(self, request: RequestCache) -> None:
        if request.released or self._active.get(request.slot) is not request:
            raise KVCacheError("cache has been released")

    # ----------------------------------------------------------------- growth
    def extend(self, request: RequestCache, tokens: int) -> None:
        """Make room for `tokens` more positions and count them in; call before the forward."""
        self._check_live(request)
        if tokens <= 0:
            raise KVCacheError(f"token_count must be positive, got {tokens}")
        required = request.length + tokens
        if required > self.max_seq_len:
            raise KVCacheError(f"KV cache capacity exceeded: need {required} positions but capacity is {self.max_seq_len}")
        blocks = -(-required // self.page_size)
        wanted = [blocks - len(table) for table in request.tables]
        for group, count in zip(self.groups, wanted):
            if count > group.pool.free_pages:
                raise KVCacheError(f"KV block pool exhausted: need {count} blocks but only {group.pool.free_pages} are free")
        for index, (group, count) in enumerate(zip(self.groups, wanted)):
            if count > 0:
                table = request.tables[index]
                pages = group.pool.allocate(count)
                group.host_table[request.slot, len(table):len(table) + count] = pages
                self._touch(index, request.slot, len(table), len(table) + count)
                table.extend(pages)
        request.length = required

    def rollback(self, request: RequestCache, length: int) -> None:
        """Forget positions from `length` on and give back the pages only they used."""
        self._check_live(request)
        if length < 0 or length > request.length:
            raise KVCacheError(f"cannot roll cache back to length {length}")
        blocks = -(-length // self.page_size)
        for index, group in enumerate(self.groups):
            table = request.tables[index]
            if blocks < request.first_live[index]:
                raise KVCacheError(f"cannot roll back to length {length}: its pages have left the window and were given back")
            extra = [page for page in table[blocks:] if page >= 0]
            group.pool.free(extra)
            self._touch(index, request.slot, blocks, len(table))
            del table[blocks:]
            group.host_table[request.slot, blocks:] = -1
        request.length = length

    def trim(self, request: RequestCache) -> int:
        """Give back pages whose every position is outside the window of all future queries."""
        self._check_live(request)
        freed = 0
        for index, group in enumerate(self.groups):
            window = group.need.window
            if window is None:
                continue
            # the next query sits at position `length` and sees keys j > length - window
            dead_blocks = max(0, (request.length - window + 1) // self.page_size)
            table = request.tables[index]
            dead_blocks = min(dead_blocks, len(table))
            pages = [table[b] for b in range(request.first_live[index], dead_blocks) if table[b] >= 0]
            for b in range(request.first_live[index], dead_blocks):
                table[b] = -1
            if dead_blocks > request.first_live[index]:
                group.host_table[request.slot, request.first_live[index]:dead_blocks] = -1
                self._touch(index, request.slot, request.first_live[index], dead_blocks)
                request.first_live[index] = dead_blocks
            group.pool.free(pages)
            freed += len(pages)
        return freed

    def release(self, request: RequestCache) -> None:
        """Give back everything the request holds; releasing twice is harmless."""
        if request.released:
            return
        if self._active.get(request.slot) is not request:
            raise KVCacheError("cache is not owned by this cache manager")
        for index, group in enumerate(self.groups):
            group.pool.free([page for page in request.tables[index] if page >= 0])
            group.reserved_pages -= request.reserved[index]
            group.host_table[request.slot, :] = -1
            self._touch(index, request.slot, 0, len(request.tables[index]))
            request.tables[index] = []
        request.released = True
        request.length = 0
        del self._active[request.slot]
        heapq.heappush(self._free_slots, request.slot)

    # ------------------------------------------------------------ step support
    def _touch(self, group: int, slot: int, first: int, end: int) -> None:
        if end > first and self.device_tables is not None:
            self._dirty.append((group, slot, first, end))

    def tables_with_trash_row(self, group: int) -> np.ndarray:
        """The group's host block table with the trash row behind the requests' rows: [max_requests + 1, max_blocks]."""
        return self._tables_host[group]

    def device_table(self, group: int) -> torch.Tensor:
        """The group's block table on the device, int32 [max_requests + 1, max_blocks]: row = a request's slot."""
        return self.device_tables[group]

    def table_patches(self) -> tuple[np.ndarray, np.ndarray] | None:
        """The block table entries that have changed on the host since the last call, as (offsets into the device
        array of all groups, values), or None if there are none.  The caller writes them into the device array
        before the next kernel reads it."""
        if not self._dirty:
            return None
        dirty, self._dirty = self._dirty, []
        rows, blocks = self.max_requests + 1, self.max_blocks
        flat: list[int] = []
        for g, slot, first, end in dirty:
            base = (g * rows + slot) * blocks
            flat.extend(range(base + first, base + end))
        if len(dirty) > 1:
            flat = sorted(set(flat))             # a page taken and given back again is sent once, with what the host holds now
        offsets = np.array(flat, dtype=np.int32)
        return offsets, self._tables_host.reshape(-1)[offsets]

    def upload_tables(self) -> None:
        """The whole host array to the device at once (for more changes than a step's metadata has room for)."""
        self._dirty = []
        self.device_tables.copy_(torch.from_numpy(self._tables_host))

    def tables_match_device(self) -> bool:
        """Whether the device's block tables equal the host's in every entry that is not waiting in table_patches()."""
        expected = self._tables_host.copy()
        got = self.device_tables.cpu().numpy().copy()
        for g, slot, first, end in self._dirty:
            expected[g, slot, first:end] = got[g, slot, first:end]
        return bool((expected == got).all())

    def slot_of_position(self, request: RequestCache, group: int, position: int) -> int:
        """Physical slot (page * page_size + offset) of a logical position."""
        page = request.tables[group][position // self.page_size]
        if page < 0:
            raise KVCacheError(f"position {position} lies in a page that was given back")
        return page * self.page_size + position % self.page_size

    def check_invariants(self) -> None:
        """No page lost, held twice or free while held; used by tests."""
        for index, group in enumerate(self.groups):
            held = [page for request in self._active.values() for page in request.tables[index] if page >= 0]
            if len(held) != len(set(held)):
                raise AssertionError(f"group {index}: a page is held twice")
            if len(held) != group.pool.used_pages:
                raise AssertionError(f"group {index}: {group.pool.used_pages} pages are out but requests hold {len(held)}")
            if set(held) & set(group.pool._free):
                raise AssertionError(f"group {index}: a held page is on the free list")
            for request in self._active.values():
                row = group.host_table[request.slot]
                table = request.tables[index]
                if list(row[:len(table)]) != table or (row[len(table):] != -1).any():
                    raise AssertionError(f"group {index}: host block table of slot {request.slot} is stale")
        slots = [request.slot for request in self._active.values()]
        if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots):
            raise AssertionError("a state slot is held twice or free while held")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise AssertionError("a state slot was lost")
