"""The cache manager: pages of keys and values with a page table per request, and slots of
fixed-size state.

Layers of the run order whose cache needs are equal (same key/value geometry, same window) form
a group.  A group owns a pool of pages, storage [layer][page][K|V][kv_head][place][head_dim]
and one page table per request slot: table[slot][i] is the page that holds positions
i*page_size .. (i+1)*page_size-1 of that request in every layer of the group, or -1.  A group
with a window gives pages back as soon as no later position can see them; a request that ends
gives back everything.  Requests also hold a slot in every fixed-size state tensor
[slot][...], zeroed when the request opens.

Behind the request slots lies one spare slot that no request ever holds, with one page of its own
in every group, outside the pool, for positions 0 .. page_size-1: rows that only fill a step up to
a size it was prepared for (a captured decode step) are computed there, at position 0, and touch
nothing a request can see.

The reference's pool is one group over all layers with per-sequence tables kept on the host
(src/model/kv_cache.h:4-13, 73-118); groups, windows and state slots have no counterpart there.
"""
from __future__ import annotations

from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .needs import PagedKvNeed, StateNeed
from .pages import OutOfPages, PagePool
from .prefix import PrefixIndex


class CacheError(RuntimeError):
    pass


class PageGroup:
    def __init__(self, need: PagedKvNeed, entries: List[int], n_pages: int, page_size: int, max_requests: int,
                 max_positions: int, dtype, device, allocate_storage: bool):
        self.need = need
        self.entries = list(entries)                 # run-order entries, in run order
        self.page_size = page_size
        self.pool = PagePool(n_pages)
        self.table_width = -(-max_positions // page_size)
        self.table_host = np.full((max_requests + 1, self.table_width), -1, dtype=np.int32)
        self.table_host[max_requests, 0] = n_pages                   # the spare slot's page, behind the pool's
        self.first_live = np.zeros(max_requests, dtype=np.int64)     # pages below this index were given back (windows)
        self.n_held = np.zeros(max_requests, dtype=np.int64)         # table entries in use, counted from 0
        self.dirty: set = set()                      # slots whose table row on the device is out of date
        self.dirty_from = np.zeros(max_requests, dtype=np.int64)     # ... from this entry on,
        self.on_device = np.zeros(max_requests, dtype=np.int64)      # ... and how many entries of the row the device copy may hold (the rest is -1 there)
        self.storage = None
        self.table_dev = None
        if allocate_storage:
            self.storage = torch.zeros((len(entries), n_pages + 1, 2, need.n_kv_heads, page_size, need.head_dim), dtype=dtype, device=device)
            self.table_dev = torch.tensor(self.table_host, dtype=torch.int32, device=device)

    def _changed(self, slot: int, first_entry: int) -> None:
        self.dirty_from[slot] = min(int(self.dirty_from[slot]), first_entry) if slot in self.dirty else first_entry
        self.dirty.add(slot)

    def pages_for(self, slot: int, new_length: int) -> int:
        """Pages to allocate so that positions below new_length have one."""
        return max(0, -(-new_length // self.page_size) - int(self.n_held[slot]))

    def grow(self, slot: int, new_length: int) -> None:
        first, count = int(self.n_held[slot]), self.pages_for(slot, new_length)
        if count > 0:
            self.table_host[slot, first:first + count] = self.pool.allocate_many(count)
            self.n_held[slot] = first + count
            self._changed(slot, first)

    def adopt(self, slot: int, pages: Sequence[int]) -> None:
        """The first pages of a request that has none yet: full pages another request computed (the caller has
        retained them for this request)."""
        if int(self.n_held[slot]) != 0:
            raise CacheError("only a request without pages can adopt shared ones")
        self.table_host[slot, :len(pages)] = np.asarray(pages, dtype=np.int32)
        self.n_held[slot] = len(pages)
        self._changed(slot, 0)

    def drop_behind_window(self, slot: int, length: int) -> None:
        """After `length` positions the next row is at position `length`; it sees keys from
        length - window + 1 on, so pages that end at or before that are given back."""
        if self.need.window is None:
            return
        keep_from = (length - self.need.window + 1) // self.page_size       # first page still visible
        first = i = int(self.first_live[slot])
        while i < min(keep_from, int(self.n_held[slot])):
            self.pool.release(int(self.table_host[slot, i]))
            self.table_host[slot, i] = -1
            i += 1
        if i > first:
            self._changed(slot, first)
        self.first_live[slot] = max(int(self.first_live[slot]), i)

    def release_all(self, slot: int) -> None:
        # last page first, as the reference's truncate (src/model/kv_cache.cpp:100-109): the request's
        # first page is then the next one handed out
        for i in range(int(self.n_held[slot]) - 1, int(self.first_live[slot]) - 1, -1):
            self.pool.release(int(self.table_host[slot, i]))
        self.table_host[slot, :int(self.n_held[slot])] = -1
        self.first_live[slot] = 0
        self.n_held[slot] = 0
        self._changed(slot, 0)

    def held_pages(self, slot: int) -> List[int]:
        return [int(p) for p in self.table_host[slot, int(self.first_live[slot]):int(self.n_held[slot])]]

    def can_rewind_to(self, slot: int, length: int) -> bool:
        """Whether the pages the row at position `length` sees are still held (a window may have given them back)."""
        if self.need.window is None or length == 0:
            return True
        return int(self.first_live[slot]) <= max(0, length - self.need.window + 1) // self.page_size

    def pages_freed_by_rewind(self, slot: int, length: int) -> int:
        first = max(-(-length // self.page_size), int(self.first_live[slot]))
        return sum(1 for i in range(first, int(self.n_held[slot])) if self.pool.ref_count(int(self.table_host[slot, i])) == 1)

    def shared_page_at(self, slot: int, length: int) -> bool:
        """Whether position `length` falls inside a held page that someone else holds too: it must be copied
        before the request writes there again."""
        i = length // self.page_size
        return length % self.page_size != 0 and i < int(self.n_held[slot]) and self.pool.ref_count(int(self.table_host[slot, i])) > 1

    def rewind(self, slot: int, length: int) -> None:
        """Gives back the pages that hold only positions from `length` on, last first (the reference's truncate,
        src/model/kv_cache.cpp:100-109), and makes the page that `length` falls into the request's own
        (its make_writable, src/model/kv_cache.cpp:116-141: a copy of the whole page, every layer)."""
        if length == 0:
            self.release_all(slot)
            return
        keep = max(-(-length // self.page_size), int(self.first_live[slot]))
        for i in range(int(self.n_held[slot]) - 1, keep - 1, -1):
            self.pool.release(int(self.table_host[slot, i]))
            self.table_host[slot, i] = -1
        self.n_held[slot] = min(int(self.n_held[slot]), keep)
        if self.shared_page_at(slot, length):
            i = length // self.page_size
            old, new = int(self.table_host[slot, i]), self.pool.allocate()
            if self.storage is not None:
                self.storage[:, new].copy_(self.storage[:, old])
            self.pool.release(old)
            self.table_host[slot, i] = new
        self._changed(slot, min(keep, length // self.page_size))

    def sync(self, upload=None, stage=None) -> None:
        """Brings the device's copy of the changed rows up to date.  Only the columns that changed go over: from the
        first changed entry of any dirty row to the last entry that a dirty row holds or held on the device (a request
        that crosses into a new page sends one column, not its whole row of max_positions / page_size entries).
        `upload(arrays...)`: int32 arrays -> device tensors without waiting for the device; `stage(array)`: the array in
        pinned memory, for a copy made here (one changed row, a prompt's usually, goes straight into its place so)."""
        if self.table_dev is None or not self.dirty:
            self.dirty.clear()
            return
        rows = sorted(self.dirty)
        self.dirty.clear()
        lo = int(self.dirty_from[rows].min())
        hi = int(max(self.n_held[rows].max(), self.on_device[rows].max()))
        self.on_device[rows] = self.n_held[rows]
        if hi <= lo:
            return
        if stage is not None and len(rows) == 1:
            self.table_dev[rows[0], lo:hi].copy_(stage(self.table_host[rows[0], lo:hi]), non_blocking=True)
            return
        block = self.table_host[rows, lo:hi]
        if upload is not None:                 # int32 array -> device tensor without waiting for the device
            # (both in one copy; the rows go as 64-bit numbers, which is what the copy by index wants: no kernel to widen them)
            idx, data = upload(np.asarray(rows, dtype=np.int64).view(np.int32), block)
            self.table_dev[:, lo:hi].index_copy_(0, idx.view(torch.int64), data.view(len(rows), hi - lo))
            return
        idx = torch.tensor(rows, dtype=torch.int64)
        self.table_dev[:, lo:hi].index_copy_(0, idx.to(self.table_dev.device), torch.from_numpy(np.ascontiguousarray(block)).to(self.table_dev.device))


class CacheManager:
    """`needs[i]` is the need of run-order entry i (PagedKvNeed, StateNeed or None); `reads_from[i]`
    is the entry whose pages entry i reads instead of keeping its own (or None)."""

    def __init__(self, needs: Sequence, reads_from: Sequence[Optional[int]], *, page_size: int, n_pages: int, max_requests: int,
                 max_positions: int, dtype=torch.float32, device="cpu", allocate_storage: bool = True):
        if page_size < 1 or n_pages < 1 or max_requests < 1 or max_positions < 1:
            raise ValueError("page_size, n_pages, max_requests and max_positions must be positive")
        self.page_size, self.max_requests, self.max_positions = int(page_size), int(max_requests), int(max_positions)
        self.spare_slot = self.max_requests          # a slot of tables and state that no request holds
        self.groups: List[PageGroup] = []
        self._entry_group: Dict[int, Tuple[int, int]] = {}          # entry -> (group index, layer index in group)
        self.states: Dict[int, torch.Tensor] = {}
        by_need: Dict[PagedKvNeed, List[int]] = {}
        for i, (need, src) in enumerate(zip(needs, reads_from)):
            if src is not None:
                if needs[src] != need or not isinstance(need, PagedKvNeed):
                    raise CacheError(f"run-order entry {i} reads the cache of entry {src}, whose need differs: {needs[src]} against {need}")
                continue
            if isinstance(need, PagedKvNeed):
                by_need.setdefault(need, []).append(i)
            elif isinstance(need, StateNeed):
                if allocate_storage:
                    self.states[i] = torch.zeros((max_requests + 1, *need.shape), dtype=need.dtype, device=device)
            elif need is not None:
                raise CacheError(f"run-order entry {i} has an unknown cache need {need!r}")
        self._state_needed = any(isinstance(need, StateNeed) for need in needs)
        for need, entries in by_need.items():
            g = PageGroup(need, entries, n_pages, page_size, max_requests, max_positions, dtype, device, allocate_storage)
            for li, e in enumerate(entries):
                self._entry_group[e] = (len(self.groups), li)
            self.groups.append(g)
        for i, src in enumerate(reads_from):
            if src is not None:
                self._entry_group[i] = self._entry_group[src]
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self._slot: Dict[Hashable, int] = {}
        self._length: Dict[Hashable, int] = {}
        self.prefix: Optional[PrefixIndex] = None
        self.evicted_pages = 0                       # pages taken back from the prefix index so far

    def enable_prefix_sharing(self) -> bool:
        """Lets requests share the pages of equal prompt prefixes (`self.prefix`).  Possible when pages without a
        window hold all of a request's past, in one group or in several: with a window, pages of a prefix are given
        back while it is still shared; with fixed-size state, the state after the prefix would have to be kept too."""
        if self.prefix is None and self.groups and all(g.need.window is None for g in self.groups) and not self._state_needed:
            self.prefix = PrefixIndex(self.groups[0].pool, self.page_size, [g.pool for g in self.groups[1:]])
        return self.prefix is not None

    # ------------------------------------------------------------------------------ requests
    def open(self, request: Hashable, shared_pages: Sequence[int] = ()) -> int:
        """shared_pages: full pages of an equal prompt prefix, retained for this request by `self.prefix.match`
        (the first group's; the index knows the other groups' pages for the same positions); the request starts with
        their positions in place."""
        if request in self._slot:
            raise CacheError(f"request {request!r} is already open")
        if not self._free_slots:
            raise CacheError(f"all {self.max_requests} request slots are in use")
        if shared_pages and self.prefix is None:
            raise CacheError("pages can be shared only after enable_prefix_sharing()")
        if len(shared_pages) * self.page_size > self.max_positions:
            raise CacheError("more shared pages than a request may hold")
        slot = self._free_slots.pop()
        self._slot[request] = slot
        self._length[request] = len(shared_pages) * self.page_size
        for s in self.states.values():
            s[slot].zero_()
        if shared_pages:
            self.groups[0].adopt(slot, shared_pages)
            others = [self.prefix.companions(int(p)) for p in shared_pages] if len(self.groups) > 1 else []
            for gi, g in enumerate(self.groups[1:]):
                g.adopt(slot, [pages[gi] for pages in others])
        return slot

    def pages_of(self, request: Hashable) -> List[int]:
        """The request's page table in the first group (what the prefix index names pages by)."""
        return self.groups[0].held_pages(self.slot(request))

    def page_row(self, request: Hashable):
        """The same as an array (a view of the table's row: read it now, do not keep it)."""
        g, slot = self.groups[0], self.slot(request)
        return g.table_host[slot, int(g.first_live[slot]):int(g.n_held[slot])]

    def index_prefix(self, request: Hashable, tokens: Sequence[int], n_tokens: int, after=None) -> int:
        """Names the request's full pages under its first `n_tokens` positions in the prefix index (`PrefixIndex.insert`, which
        says what `after` is): the pages of every group."""
        slot = self.slot(request)
        others = [g.table_host[slot, int(g.first_live[slot]):int(g.n_held[slot])] for g in self.groups[1:]]
        return self.prefix.insert(tokens, n_tokens, self.page_row(request), after=after, companions=others)

    def evictable_pages(self) -> int:
        return self.prefix.evictable() if self.prefix is not None else 0

    def evict(self, count: int) -> int:
        """Gives back up to `count` pages that only the prefix index still holds; returns how many."""
        freed = self.prefix.evict(count) if self.prefix is not None and count > 0 else 0
        self.evicted_pages += freed
        return freed

    def available_pages(self) -> List[int]:
        """Per group: free pages plus the pages that only the prefix index still holds, which a reservation takes back
        when it needs them.  Whoever reserves (a scheduler's step, a lone `generate`, a replay) gets them, whether or
        not it was the one that filled the index."""
        out = self.free_pages()
        if self.prefix is not None:                # (a page the index gives back is one page of every group)
            out = [n + self.prefix.evictable() for n in out]
        return out

    def _make_room(self, need: Sequence[int]) -> bool:
        """True if every group has `need[g]` free pages, after index-only pages were taken back where that helps."""
        if self.prefix is not None:
            short = max(n - g.pool.free_count for n, g in zip(need, self.groups))
            if 0 < short <= self.prefix.evictable():
                self.evict(short)
        return all(n <= g.pool.free_count for n, g in zip(need, self.groups))

    def close(self, request: Hashable) -> None:
        slot = self.slot(request)
        for g in self.groups:
            g.release_all(slot)
        del self._slot[request], self._length[request]
        self._free_slots.append(slot)

    def is_open(self, request: Hashable) -> bool:
        return request in self._slot

    def slot(self, request: Hashable) -> int:
        try:
            return self._slot[request]
        except KeyError:
            raise CacheError(f"request {request!r} is not open") from None

    def length(self, request: Hashable) -> int:
        self.slot(request)
        return self._length[request]

    def open_requests(self):
        return list(self._slot)

    def slots_and_lengths(self, requests: Sequence[Hashable]) -> Tuple[List[int], List[int]]:
        """The slots and the lengths of the named requests, in their order (what a decode step asks of every request
        of its batch, in one call); `CacheError` names the first request that is not open."""
        try:
            return [self._slot[r] for r in requests], [self._length[r] for r in requests]
        except KeyError as err:
            raise CacheError(f"request {err.args[0]!r} is not open") from None

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    # --------------------------------------------------------------------------------- pages
    def pages_needed(self, request: Hashable, n_new: int) -> List[int]:
        """New pages per group for n_new more positions of the request."""
        slot, length = self.slot(request), self._length[request]
        return [g.pages_for(slot, length + n_new) for g in self.groups]

    def free_pages(self) -> List[int]:
        return [g.pool.free_count for g in self.groups]

    def _pages_for(self, additions: Sequence[Tuple[Hashable, int]]) -> List[int]:
        need = [0] * len(self.groups)
        for request, n_new in additions:
            for gi, n in enumerate(self.pages_needed(request, n_new)):
                need[gi] += n
        return need

    def fits(self, additions: Sequence[Tuple[Hashable, int]]) -> bool:
        return all(n <= a for n, a in zip(self._pages_for(additions), self.available_pages()))

    def reserve(self, additions: Sequence[Tuple[Hashable, int]]) -> None:
        """Pages for n_new more positions of every named request, or `OutOfPages` with nothing changed."""
        seen = set()
        for request, n_new in additions:
            if request in seen:
                raise CacheError(f"request {request!r} is named twice in one reservation")
            seen.add(request)
            if n_new < 1:
                raise CacheError("a reservation must add at least one position")
            if self.length(request) + n_new > self.max_positions:
                raise CacheError(f"request {request!r} would reach position {self._length[request] + n_new}, beyond the limit {self.max_positions}")
        if not self._make_room(self._pages_for(additions)):
            raise OutOfPages(f"not enough free pages (free per group: {self.free_pages()})")
        for request, n_new in additions:
            slot, length = self._slot[request], self._length[request]
            for g in self.groups:
                g.grow(slot, length + n_new)

    def reserve_one_each(self, requests: Sequence[Hashable], slots: Sequence[int], lengths: Sequence[int]) -> None:
        """`reserve` for one more position of every named request (open, each named once, `slots` and
        `lengths` theirs): the common case of a decode step, without a Python loop over requests
        unless a request crosses into a new page."""
        slot_arr, next_len = np.asarray(slots, dtype=np.int64), np.asarray(lengths, dtype=np.int64) + 1
        if int(next_len.max()) > self.max_positions:
            raise CacheError(f"a request would pass the position limit {self.max_positions}")
        growing, counts = [], []
        for g in self.groups:
            need = (next_len + g.page_size - 1) // g.page_size > g.n_held[slot_arr]
            counts.append(int(need.sum()))
            growing.append(np.nonzero(need)[0] if counts[-1] else ())
        if any(counts) and not self._make_room(counts):
            raise OutOfPages(f"not enough free pages (free per group: {self.free_pages()})")
        for g, idx in zip(self.groups, growing):
            for i in idx:
                g.grow(slots[i], int(next_len[i]))

    def advance_one_each(self, requests: Sequence[Hashable], slots: Sequence[int], lengths: Sequence[int]) -> None:
        """`advance` by one position for every named request, after `reserve_one_each`."""
        for r, n in zip(requests, lengths):
            self._length[r] = n + 1
        for g in self.groups:
            if g.need.window is not None:
                for slot, n in zip(slots, lengths):
                    g.drop_behind_window(slot, n + 1)

    def advance(self, request: Hashable, n_new: int) -> None:
        """The reserved positions have been written: the request is n_new longer; pages behind a
        window are given back."""
        slot = self.slot(request)
        new_length = self._length[request] + n_new
        for g in self.groups:
            if new_length > int(g.n_held[slot]) * g.page_size:
                raise CacheError(f"request {request!r} advanced beyond its reserved pages")
        self._length[request] = new_length
        for g in self.groups:
            g.drop_behind_window(slot, new_length)

    def truncate(self, request: Hashable, length: int) -> None:
        """Rewind: the request keeps its first `length` positions and its next token goes to position `length`.
        Pages beyond are given back; a page that `length` falls into and that others hold too (a shared prefix,
        the prefix index) is copied first, so that what they see never changes.  Refused, with nothing changed,
        where the past cannot be restored: fixed-size state, or pages that a window has given back.
        Behaviour as the reference's rewind (src/model/transformer.cpp:545-552, src/model/kv_cache.cpp:100-141)."""
        slot, old = self.slot(request), self._length[request]
        if not 0 <= length <= old:
            raise CacheError(f"request {request!r} holds {old} positions; it cannot be cut to {length}")
        if length == old:
            return
        if self._state_needed:
            raise CacheError("a request with fixed-size state cannot be rewound: the state of earlier positions is gone")
        for g in self.groups:
            if not g.can_rewind_to(slot, length):
                raise CacheError(f"request {request!r} cannot be rewound to {length}: a window of {g.need.window} has given those pages back")
        for g in self.groups:
            if g.shared_page_at(slot, length) and g.pool.free_count + g.pages_freed_by_rewind(slot, length) < 1 and self.evict(1) < 1:
                raise OutOfPages("no free page to copy a shared page into")
        for g in self.groups:
            g.rewind(slot, length)
        self._length[request] = length

    def sync(self, upload=None, stage=None) -> None:
        """Brings the device copies of changed page tables up to date.  `upload(int32 arrays...) -> device tensors`
        is the caller's way of copying without waiting for the device (it must take a snapshot at once); `stage(array)
        -> the same in pinned memory`, if it has one, lets a single changed row go straight to its place."""
        for g in self.groups:
            g.sync(upload, stage)

    # --------------------------------------------------------------------------------- views
    def kv(self, entry: int):
        """(cache of the entry's layer [page, 2, kv_head, place, hd], device page table, window)."""
        gi, li = self._entry_group[entry]
        g = self.groups[gi]
        return g.storage[li], g.table_dev, g.need.window

    def state(self, entry: int) -> torch.Tensor:
        return self.states[entry]

    def check_consistency(self) -> None:
        """Every page is free, or held by the requests and the prefix index that its reference count says;
        without prefix sharing a page has at most one holder."""
        for gi, g in enumerate(self.groups):
            holders: Dict[int, List[Hashable]] = {}
            for request, slot in self._slot.items():
                for p in g.held_pages(slot):
                    if p < 0:
                        raise CacheError(f"group {gi}: request {request!r} holds no page at a live place")
                    holders.setdefault(p, []).append(request)
                    if len(holders[p]) > 1 and self.prefix is None:
                        raise CacheError(f"group {gi}: page {p} is held by {holders[p][0]!r} and {request!r}")
            indexed = set()
            if self.prefix is not None:
                indexed = set(self.prefix.pages()) if gi == 0 else {self.prefix.companions(p)[gi - 1] for p in self.prefix.pages()}
                if len(indexed) != len(self.prefix):
                    raise CacheError(f"group {gi}: the prefix index names a page twice")
            in_use = set(holders) | indexed
            free = set(g.pool._free)
            if len(free) != len(g.pool._free):
                raise CacheError(f"group {gi}: a page is twice in the free stack")
            if free & in_use:
                raise CacheError(f"group {gi}: pages {sorted(free & in_use)} are free and held")
            if len(free) + len(in_use) != g.pool.n_pages:
                raise CacheError(f"group {gi}: {g.pool.n_pages - len(free) - len(in_use)} pages are lost")
            for p in range(g.pool.n_pages):
                expected = len(holders.get(p, ())) + (1 if p in indexed else 0)
                if g.pool.ref_count(p) != expected:
                    raise CacheError(f"group {gi}: page {p} has reference count {g.pool.ref_count(p)}, {expected} holders")
